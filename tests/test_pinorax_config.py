"""Pinorax without a GPU: the reader of config.json, the description of the model that is built from it, the
random-weights mode, and pins on the plain implementation that the GPU tests compare the engine with."""

import copy
import json

import pytest
import torch

import plain_pinorax as PP
import tiny_pinorax
from rvllm_amd.config.errors import ConfigError
from rvllm_amd.config.pinorax import PinoraxConfig
from rvllm_amd.models import DecoderModel, load_config
from rvllm_amd.models.registry import architecture_of
from rvllm_amd.weights.random_init import random_tensors


@pytest.mark.parametrize("name", list(tiny_pinorax.CONFIGS))
def test_config_is_read_and_written_back(name):
    doc = tiny_pinorax.CONFIGS[name][0]
    arch = architecture_of(doc)
    assert arch.name == "Pinorax"
    cfg = arch.read_config(doc, "test")
    assert arch.write_config(cfg) == doc
    assert [layer.mixer.heads for layer in cfg.layers] == [l["mixer"]["heads"] for l in doc["layers"]]


def test_every_problem_of_a_config_is_reported_at_once():
    doc = copy.deepcopy(tiny_pinorax.CONFIG_P)
    doc["width"] = 0
    doc["norm"] = {}
    doc["layers"][0]["mlp"]["router"]["top"] = 9
    doc["layers"][1]["type"] = "convolution"
    doc["layers"][2]["mixer"].pop("kv_rank")
    doc["layers"][3]["mlp"]["kind"] = "sparse"
    with pytest.raises(ConfigError) as e:
        PinoraxConfig.from_dict(doc, "test")
    text = str(e.value)
    for piece in ("width", "norm: missing", "layers[0]: mlp: router: top=9", "layers[1]: unknown mixer type",
                  "layers[2]: mixer: missing or invalid required field kv_rank", "layers[3]: mlp: unknown kind"):
        assert piece in text, (piece, text)


def test_the_model_asks_for_the_designs_tensors(tmp_path):
    folder = tiny_pinorax.write_model(tmp_path / "P", "P")
    arch, cfg = load_config(folder)
    model = DecoderModel(arch.build_spec(cfg))
    asked = {s.name: tuple(s.shape) for s in model.param_specs()}
    held = {k: tuple(v.shape) for k, v in PP.load_weights(folder).items()}
    assert asked == held
    assert asked["l0.norm1"] == () and asked["l2.dwa"] == (4,) and asked["l0.mlp.table"] == (211, 2)
    assert "l2.mlp.gate" not in asked and "l3.mlp.shared.gate" not in asked and asked["l1.mlp.down.b"] == (64,)
    assert asked["l1.mix.uk"] == (3 * 8, 48) and asked["l1.mix.uv"] == (3 * 8, 48) and asked["l1.mix.sink"] == (3,)
    needs = model.cache_needs()
    assert [(n.num_kv_heads, n.head_dim, n.window) for n in needs] == [(1, 32, None), (1, 48, None), (1, 16, None), (1, 64, None)]
    assert model.spec.residual_float32 and model.capturable


def test_an_experts_table_names_different_experts_in_a_row():
    arch = architecture_of(tiny_pinorax.CONFIG_P)
    model = DecoderModel(arch.build_spec(arch.read_config(tiny_pinorax.CONFIG_P, "test")))
    tensors = random_tensors(model.param_specs(), 3)
    for name, experts in (("l0.mlp.table", 5), ("l3.mlp.table", 3)):
        table = tensors[name]
        assert table.dtype == torch.int32 and 0 <= int(table.min()) and int(table.max()) < experts
        assert all(len(set(row)) == len(row) for row in table.tolist())


# ---- pins on the plain implementation ---------------------------------------------------------------------
def test_plain_softmax_with_a_sink_is_a_softmax_with_one_more_score():
    g = torch.Generator().manual_seed(0)
    scores = torch.randn(4, 9, generator=g, dtype=torch.float64) * 3
    sink = torch.tensor(1.7, dtype=torch.float64)
    longer = torch.softmax(torch.cat([scores, sink.expand(4, 1)], dim=1), dim=1)
    assert torch.allclose(PP.softmax_with_sink(scores, sink), longer[:, :9])
    assert torch.allclose(PP.softmax_with_sink(scores, None), torch.softmax(scores, dim=1))
    assert float(PP.softmax_with_sink(torch.tensor([0.0], dtype=torch.float64), 0.0)) == 0.5  # the first token of a sequence


def test_plain_latent_attention_is_causal_and_needs_only_the_compressed_vector(tmp_path):
    folder = tiny_pinorax.write_model(tmp_path / "P", "P", loud=True)
    w = {k: v.double() if v.is_floating_point() else v for k, v in PP.load_weights(folder).items()}
    cfg = PP.read_config(folder)
    sizes = cfg["layers"][0]["mixer"]
    g = torch.Generator().manual_seed(1)
    h = torch.randn(12, cfg["width"], generator=g, dtype=torch.float64)
    full = PP.latent_attention(h, w, "l0.mix.", sizes, 1e-5)
    assert torch.allclose(PP.latent_attention(h[:7], w, "l0.mix.", sizes, 1e-5), full[:7])  # later tokens change nothing
    # the same through the compressed vector alone: queries mapped into its space, values mapped out of it
    H, D, V, R = sizes["heads"], sizes["dim"], sizes["vdim"], sizes["kv_rank"]
    c = PP.unit_rms(h @ w["l0.mix.dkv"].T, 1e-5) * w["l0.mix.dkv.norm"]
    q = (h @ w["l0.mix.q"].T).view(12, H, D)
    uk, uv = w["l0.mix.uk"].view(H, D, R), w["l0.mix.uv"].view(H, V, R)
    out = torch.zeros(12, H, V, dtype=torch.float64)
    for a in range(H):
        q_lat = q[:, a] @ uk[a]
        for i in range(12):
            p = PP.softmax_with_sink(sizes["scale"] * (c[: i + 1] @ q_lat[i]), w["l0.mix.sink"][a])
            out[i, a] = uv[a] @ (p @ c[: i + 1])
    again = (out.reshape(12, H * V) * torch.sigmoid(h @ w["l0.mix.g"].T)) @ w["l0.mix.o"].T
    assert torch.allclose(again, full, atol=1e-9)


def test_plain_experts_weigh_one_over_top_and_the_shared_one_counts_whole():
    g = torch.Generator().manual_seed(2)
    W, F = 10, 6
    w = {"table": torch.tensor([[0, 1, 2]] * 4, dtype=torch.int32)}
    for name in ("e0", "e1", "e2", "shared"):
        w[f"{name}.gate"], w[f"{name}.up"] = torch.randn(F, W, generator=g).double(), torch.randn(F, W, generator=g).double()
        w[f"{name}.down"] = torch.randn(W, F, generator=g).double()
    h = torch.randn(2, W, generator=g).double()
    mlp = {"router": {"top": 3}, "expert": {"limit": 0.7}, "shared": {"limit": 2.0}}
    mean = sum(PP.expert(h, w, f"e{e}.", 0.7) for e in range(3)) / 3
    assert torch.allclose(PP.routed_ff(h, [1, 3], w, "", mlp), mean + PP.expert(h, w, "shared.", 2.0))
    big = torch.full((1, W), 50.0).double()
    gate = (big @ w["e0.gate"].T)
    assert gate.abs().max() > 0.7 and PP.expert(big, w, "e0.", 0.7).abs().max() <= (0.7 * 1.7 * w["e0.down"].abs().sum(1)).max()


def test_plain_depth_average_and_layers_without_a_feed_forward(tmp_path):
    folder = tiny_pinorax.write_model(tmp_path / "P", "P")
    weights, cfg = PP.load_weights(folder), PP.read_config(folder)
    streams = []
    logits = PP.forward(weights, cfg, [5, 6, 7, 8], streams_out=streams)
    assert logits.shape == (4, 211) and len(streams) == 4 and float(logits.abs().max()) <= 12.0
    # with all the weight on the newest stream every layer hands on its own result
    plain = {k: v.clone() for k, v in weights.items()}
    for i in range(4):
        plain[f"l{i}.dwa"] = torch.tensor([0.0] * (i + 1) + [1.0])
    other = []
    PP.forward(plain, cfg, [5, 6, 7, 8], streams_out=other)
    assert not torch.allclose(other[1], streams[1])
    assert torch.allclose(PP.depth_average([torch.ones(2), 3 * torch.ones(2)], torch.tensor([0.5, 0.25])), torch.full((2,), 1.25))
    # prefixes give the same logits: the model is causal
    assert torch.allclose(PP.forward(weights, cfg, [5, 6, 7]), logits[:3])


def test_the_command_line_takes_the_design_from_a_folder_or_a_configuration(tmp_path, capsys):
    from rvllm_amd import cli

    (tmp_path / "config.json").write_text(json.dumps(tiny_pinorax.CONFIG_Q))
    assert cli.main(["--model", str(tmp_path), "--dry-run", "--prompt-ids", "1 2 96"], {}) == 0
    assert json.loads(capsys.readouterr().out)["architecture"] == "Pinorax"
    assert cli.main(["--model", str(tmp_path), "--dry-run", "--prompt-ids", "1 97"], {}) == 2  # outside the vocabulary
    capsys.readouterr()
    assert cli.main(["--random-weights", str(tmp_path / "config.json"), "--dry-run", "--prompt-len", "8"], {}) == 0
    assert json.loads(capsys.readouterr().out)["architecture"] == "Pinorax"
