"""The Rufedra design without a GPU: the configuration reader and its errors, the tensors the model asks for, the
needs its layers declare to the cache manager, and pins on the plain implementation (``plain_rufedra``) that the
GPU tests compare against."""

import copy

import pytest
import torch

import plain_rufedra as PR
import tiny_rufedra
from rvllm_amd.cache.manager import CacheManager
from rvllm_amd.config.errors import ConfigError
from rvllm_amd.config.rufedra import RufedraConfig
from rvllm_amd.models import DecoderModel
from rvllm_amd.models.registry import architecture_of
from rvllm_amd.parts.base import KVNeed, StateNeed, atomic_needs


@pytest.mark.parametrize("name", list(tiny_rufedra.CONFIGS))
def test_the_reader_takes_every_size_from_the_file_and_writes_it_back(name):
    doc = tiny_rufedra.CONFIGS[name][0]
    arch = architecture_of(doc)
    cfg = arch.read_config(doc, "test")
    assert isinstance(cfg, RufedraConfig) and arch.write_config(cfg) == doc
    assert [layer.type for layer in cfg.layers] == [layer["type"] for layer in doc["layers"]]


def test_every_problem_of_a_file_is_reported_at_once():
    doc = copy.deepcopy(tiny_rufedra.CONFIG_A)
    doc["vocab"] = 0
    del doc["norm"]
    doc["layers"][0]["mixer"]["left"]["heads"] = 3          # not a multiple of kv_heads 2
    doc["layers"][1]["mixer"]["conv"] = "three"
    doc["layers"][2]["type"] = "conv"
    doc["layers"][3]["mixer"]["left"]["rot"]["dims"] = 7
    doc["layers"][4]["mlp"] = {"kind": "moe"}
    with pytest.raises(ConfigError) as e:
        RufedraConfig.from_dict(doc, "test")
    text = str(e.value)
    for piece in ("vocab", "norm", "layers[0]", "kv_heads", "layers[1]", "conv", "layers[2]", "unknown mixer type",
                  "layers[3]", "rot.dims", "layers[4]", "unknown kind"):
        assert piece in text, piece


def test_values_that_are_keys_need_equal_sizes():
    doc = copy.deepcopy(tiny_rufedra.CONFIG_A)
    doc["layers"][0]["mixer"]["left"]["vdim"] = 16
    with pytest.raises(ConfigError, match="vdim"):
        RufedraConfig.from_dict(doc, "test")


def test_the_model_asks_for_the_designs_tensors():
    doc = tiny_rufedra.CONFIG_A
    model = DecoderModel(architecture_of(doc).build_spec(RufedraConfig.from_dict(doc)))
    shapes = {s.name: tuple(s.shape) for s in model.param_specs()}
    assert shapes["embed"] == (211, 64) and shapes["head"] == (211, 64) and shapes["final.norm"] == (64,)
    # a parallel layer with a feed-forward: four norms, two scales, left without a value projection, right
    for name, shape in {"l0.norm1": (64,), "l0.norm1b": (64,), "l0.norm2": (64,), "l0.norm2b": (64,), "l0.ls1": (64,),
                        "l0.ls2": (64,), "l0.mix.left.q": (128, 64), "l0.mix.left.q.b": (128,),
                        "l0.mix.left.k": (64, 64), "l0.mix.left.k.b": (64,), "l0.mix.left.g": (128, 64),
                        "l0.mix.left.o": (64, 128), "l0.mix.right.in": (96, 64), "l0.mix.right.conv": (48, 3),
                        "l0.mix.right.conv.b": (48,), "l0.mix.right.x": (16, 48), "l0.mix.right.dt": (48, 4),
                        "l0.mix.right.dt.b": (48,), "l0.mix.right.A_log": (48, 6), "l0.mix.right.D": (48,),
                        "l0.mix.right.o": (64, 48), "l0.mlp.gate": (96, 64), "l0.mlp.down": (64, 96)}.items():
        assert shapes[name] == shape, name
    assert "l0.mix.left.v" not in shapes
    # a delta layer without a feed-forward: two norms, one scale
    for name, shape in {"l1.mix.q": (32, 64), "l1.mix.k": (32, 64), "l1.mix.v": (96, 64), "l1.mix.q.conv": (32, 3),
                        "l1.mix.v.conv": (96, 3), "l1.mix.b": (4, 64), "l1.mix.a": (4, 64), "l1.mix.A_log": (4,),
                        "l1.mix.dt_bias": (4,), "l1.mix.norm": (24,), "l1.mix.g": (96, 64), "l1.mix.o": (64, 96),
                        "l1.ls1": (64,)}.items():
        assert shapes[name] == shape, name
    assert not {"l1.norm2", "l1.norm2b", "l1.ls2", "l1.mlp.gate"} & set(shapes)


def test_a_layer_may_need_pages_and_a_state_at_once():
    doc = tiny_rufedra.CONFIG_A
    model = DecoderModel(architecture_of(doc).build_spec(RufedraConfig.from_dict(doc)))
    needs = model.cache_needs()
    assert isinstance(needs[0], tuple) and isinstance(needs[0][0], KVNeed) and isinstance(needs[0][1], StateNeed)
    assert needs[0][0] == KVNeed(2, 32, 21) and needs[3][0] == KVNeed(1, 16, 5)
    # convolution rows and the state: (3 - 1) * 48 + 48 * 6; (3 - 1) * (2 * 32 + 96) + 4 * 16 * 24
    assert needs[0][1].shape == (2 * 48 + 48 * 6,) and needs[1] == StateNeed((2 * 160 + 4 * 16 * 24,), torch.float32)
    assert atomic_needs(needs[0]) == needs[0] and atomic_needs(None) == () and atomic_needs(needs[1]) == (needs[1],)
    manager = CacheManager(needs, 16, 8, 3)
    assert set(manager.groups) == {"window21", "window5"} and manager.state_layers == [0, 1, 2, 3, 4]
    assert manager.layer_group == ["window21", None, None, "window5", None]
    a = manager.add_request("a")
    manager.extend("a", 40)
    manager.commit("a", 40)
    assert len(manager.table("a", "window21")) == 3 and manager.groups["window5"].pool.free_count == 8 - 1
    manager.release("a")
    assert manager.add_request("b").slot == a.slot  # the slot that was given back is the next to be used
    manager.check()


# ---- pins on the plain implementation ------------------------------------------------------------------------
def test_plain_convolution_sees_the_token_itself_last_and_zeros_before_the_start():
    x = torch.tensor([[1.0], [10.0], [100.0], [1000.0]], dtype=PR.F)
    w = torch.tensor([[3.0, 2.0, 1.0]], dtype=PR.F)  # the last tap is the token's own
    assert PR.causal_conv(x, w).flatten().tolist() == [1.0, 12.0, 123.0, 1230.0]
    cut = torch.cat([PR.causal_conv(x[:1], w), PR.causal_conv(x[1:], w, before=torch.tensor([[0.0], [1.0]], dtype=PR.F))])
    assert cut.flatten().tolist() == [1.0, 12.0, 123.0, 1230.0]


def test_plain_delta_rule_reads_its_own_write_and_forgets_by_its_decay():
    k = torch.tensor([[1.0, 0.0], [1.0, 0.0], [0.0, 1.0]], dtype=PR.F)
    v = torch.tensor([[2.0], [6.0], [5.0]], dtype=PR.F)
    one = torch.ones(3, dtype=PR.F)
    o, S = PR.delta_recurrence(k, k, v, one, one)
    # beta 1, no decay: a key's slot is overwritten by the newest value, and the read-out sees it at once
    assert o.flatten().tolist() == [2.0, 6.0, 5.0] and S.flatten().tolist() == [6.0, 5.0]
    o, S = PR.delta_recurrence(k, k, v, 0.5 * one, 0.5 * one)
    # S0 = 0.5 * 2 = 1; then decayed to 0.5, u = 0.5 * (6 - 0.5) = 2.75, S = 3.25
    assert o.flatten().tolist() == [1.0, 3.25, 2.5]
    # carrying S over a cut gives the same as the whole
    first, S1 = PR.delta_recurrence(k[:2], k[:2], v[:2], 0.5 * one[:2], 0.5 * one[:2])
    second, _ = PR.delta_recurrence(k[2:], k[2:], v[2:], 0.5 * one[2:], 0.5 * one[2:], S=S1)
    assert torch.equal(torch.cat([first, second]), o)


def test_plain_scan_is_a_decaying_sum():
    T = 4
    x = torch.ones(T, 1, dtype=PR.F)
    step = torch.full((T, 1), 0.5, dtype=PR.F)
    A = torch.tensor([[-2.0]], dtype=PR.F)
    B = C = torch.ones(T, 1, dtype=PR.F)
    y, S = PR.scan_recurrence(x, step, A, B, C, torch.tensor([10.0], dtype=PR.F))
    e = torch.exp(torch.tensor(-1.0, dtype=PR.F))
    want, s = [], 0.0
    for _ in range(T):
        s = e * s + 0.5
        want.append(s + 10.0)
    assert torch.allclose(y.flatten(), torch.stack(want)) and torch.allclose(S.flatten(), want[-1] - 10.0)


def test_plain_window_and_rotation():
    T, d = 9, 4
    g = torch.Generator().manual_seed(0)
    q = torch.randn(T, 1, d, generator=g, dtype=PR.F)
    k = torch.randn(T, 1, d, generator=g, dtype=PR.F)
    v = torch.eye(T, dtype=PR.F)[:, None, :]  # value j is the j-th unit vector: the output is the weights themselves
    w = PR.window_softmax_attention(q, k, v, 1.0, 3)[:, 0]
    for i in range(T):
        seen = [j for j in range(T) if w[i, j] > 0]
        assert seen == list(range(max(0, i - 2), i + 1)) and abs(float(w[i].sum()) - 1.0) < 1e-12
    assert torch.equal(PR.window_softmax_attention(q, k, v, 1.0, 1)[:, 0], torch.eye(T, dtype=PR.F))
    # a rotation keeps lengths, leaves the dimensions past `dims` alone, and turns pairs (i, i + dims/2)
    x = torch.randn(T, 2, 6, generator=g, dtype=PR.F)
    r = PR.rotate_halves(x, torch.arange(T), 4, 100.0)
    assert torch.equal(r[..., 4:], x[..., 4:]) and torch.allclose(r.norm(dim=-1), x.norm(dim=-1))
    assert torch.equal(r[0], x[0])  # position 0 turns nothing
    ang = 5 * 100.0 ** (-2.0 * 1 / 4)
    u, w2 = x[5, 0, 1], x[5, 0, 3]
    assert torch.allclose(r[5, 0, 1], u * torch.cos(torch.tensor(ang)) - w2 * torch.sin(torch.tensor(ang)))
    # scores depend on the distance alone
    a = PR.rotate_halves(x[:1].expand(T, 2, 6), torch.arange(T), 6, 50.0)
    assert torch.allclose((a[2, 0] * a[5, 0]).sum(), (a[4, 0] * a[7, 0]).sum())
