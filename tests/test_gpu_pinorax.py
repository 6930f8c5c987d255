"""The Pinorax design on the GPU against the plain implementation (``plain_pinorax``): each mechanism alone at
the level of its kernels, then whole models through the step function under every way of cutting the work,
through ``bin/trace_run`` and through the engine's scheduler."""

import numpy as np
import pytest
import torch

import plain_pinorax as PP
import tiny_pinorax
import trace_tools as tt
from test_gpu_kernels import Case, dev, to_cache, from_cache, paged_setup
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.runner import ModelRunner
from rvllm_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def close(got, want, dtype, what=""):
    """Against the values' own size: 32-bit to a few roundings, bf16 to a few of its."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    scale = float(want.abs().max()) or 1.0
    worst = float((got - want).abs().max())
    assert worst <= (2e-5 if dtype == torch.float32 else 2e-2) * scale, f"{what}: {worst:.3e} against {scale:.3e}"


# --------------------------------------------------------------------------
# mechanisms alone
# --------------------------------------------------------------------------
@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("width", [7, 64, 100, 1000, 4100])
def test_norm_with_one_gain_reads_a_32_bit_stream(out_dtype, width):
    g = torch.Generator().manual_seed(width)
    x = torch.randn(9, width, generator=g) * 3.0
    gain = torch.tensor([1.37])
    want = PP.scalar_norm(x.double(), gain.double(), 1e-5)
    got = ops.scalar_rmsnorm(dev(x), dev(gain.to(torch.bfloat16)), 1e-5, out_dtype)
    assert got.dtype == out_dtype
    close(got, PP.scalar_norm(x.double(), gain.to(torch.bfloat16).double(), 1e-5), out_dtype, "all rows")
    rows = torch.tensor([8, 0, 3], dtype=torch.int32)
    close(ops.scalar_rmsnorm(dev(x), dev(gain), 1e-5, out_dtype, rows=dev(rows)), want[rows.long()], out_dtype, "picked rows")
    # eps sits under the root: rows of zeros stay zeros, tiny rows are not blown up to size one
    tiny = torch.full((1, width), 1e-4)
    close(ops.scalar_rmsnorm(dev(tiny), dev(gain), 1e-2, torch.float32), PP.scalar_norm(tiny.double(), gain.double(), 1e-2),
          torch.float32, "eps")


@pytest.mark.parametrize("out_dtype", DTYPES)
def test_embedding_adds_the_vector_of_the_position(out_dtype):
    g = torch.Generator().manual_seed(1)
    table = torch.randn(50, 72, generator=g).to(torch.bfloat16)
    pos = torch.randn(33, 72, generator=g).to(torch.bfloat16)
    ids = torch.tensor([4, 49, 0, 4], dtype=torch.int32)
    where = torch.tensor([0, 32, 7, 8], dtype=torch.int32)
    out = torch.empty(4, 72, dtype=out_dtype, device=DEV)
    ops.embed_positions(dev(table), dev(pos), dev(ids), dev(where), 1.0, out)
    close(out, table.double()[ids.long()] + pos.double()[where.long()], out_dtype)
    assert torch.equal(PP.embed([4, 49], table.double(), pos.double(), 31)[1], table.double()[49] + pos.double()[32])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,layers", [(40, 4), (256, 11), (1030, 4), (2048, 19)])
def test_residual_mix_keeps_every_layers_result_and_averages_over_depth(dtype, width, layers):
    g = torch.Generator().manual_seed(3)
    rows, mult = 5, 0.6
    x0 = torch.randn(rows, width, generator=g)
    x = dev(x0.clone())
    history = torch.full((layers + 1, rows, width), float("nan"), device=DEV)
    streams = [x0.double()]
    cur = x0.double()
    for i in range(layers):
        a = torch.randn(rows, width, generator=g).to(dtype)
        f = torch.randn(rows, width, generator=g).to(dtype) if i != 2 else None  # a layer without a feed-forward
        w = (torch.randn(i + 2, generator=g) * 0.5).to(torch.float32)
        gain = torch.tensor([0.8 + 0.1 * i])
        nxt = ops.residual_mix(x, dev(a), None if f is None else dev(f), mult, history, i + 2, dev(w), i == 0,
                               dev(gain), 1e-6, dtype)
        streams.append(cur + mult * (a.double() + (0 if f is None else f.double())))
        cur = PP.depth_average(streams, w.double())
        close(x, cur, torch.float32, f"layer {i} stream")
        close(history[i + 1], streams[-1], torch.float32, f"layer {i} kept result")
        close(nxt, PP.scalar_norm(cur, gain.double(), 1e-6), dtype, f"layer {i} next norm")
    close(history[0], x0, torch.float32, "the first stream is the first layer's input")


def test_residual_mix_without_depth_weights_and_from_partial_sums():
    g = torch.Generator().manual_seed(4)
    x0 = torch.randn(3, 96, generator=g)
    parts = torch.randn(5, 3, 96, generator=g)
    f = torch.randn(3, 96, generator=g).to(torch.bfloat16)
    x = dev(x0.clone())
    assert ops.residual_mix(x, ops.SlicedSums(dev(parts), torch.bfloat16), dev(f), 0.25) is None
    close(x, x0.double() + 0.25 * (parts.double().sum(0) + f.double()), torch.float32)


def sink_reference(case, scale, sinks):
    outs, t = [], 0
    group = case.nq // case.nkv
    for b, (s, n) in enumerate(case.portions):
        k, v = case.k_all[b].double(), case.v_all[b].double()
        for i in range(n):
            row = []
            for h in range(case.nq):
                scores = scale * (k[: s + i + 1, h // group] @ case.q[t + i, h].double())
                row.append(PP.softmax_with_sink(scores, None if sinks is None else sinks[h].double()) @ v[: s + i + 1, h // group])
            outs.append(torch.stack(row))
        t += n
    return torch.stack(outs)


def run_attention(case, kernel, scale, sinks, **kw):
    kp, vp = to_cache(case.k_log, case.v_log)
    T = case.q.shape[0]
    out = torch.full((T, case.nq * case.hd), float("nan"), dtype=case.dtype, device=DEV)
    q = dev(case.q.view(T, -1))
    s = None if sinks is None else dev(sinks.float())
    if kernel == "generic":
        ops.paged_attention_generic(q, kp, vp, dev(case.table), case.step.positions, case.step.token_req, out,
                                    case.nq, scale, None, s)
    else:
        ops.paged_attention_mfma(q, kp, vp, dev(case.table), case.step, out, case.nq, scale, None, sinks=s, **kw)
    return out.cpu().view(T, case.nq, case.hd)


PORTIONS = [(150, 53), (180, 1), (0, 40), (202, 1), (31, 2), (0, 1), (15, 1), (16, 1)]
MFMA_PATHS = {
    "as the engine picks": {},
    "keys split over waves": {"prefill_kernel": False},
    "three splits merged by the second kernel": {"prefill_kernel": False, "splits": (3, 96), "in_block": False},
    "splits merged inside the block": {"prefill_kernel": False, "in_block": True},
    "tiles shared through LDS": {"prefill_kernel": True},
    "tiles in pieces": {"prefill_kernel": True, "prefill_pieces": (1, 4)},
}


@pytest.mark.parametrize("heads,rank", [(6, 48), (16, 32), (4, 96), (3, 128), (1, 16), (32, 64), (17, 32), (24, 48),
                                        (40, 256)])  # beyond 16 heads: equal groups that share the cache's one head
@pytest.mark.parametrize("path", list(MFMA_PATHS))
def test_a_sink_counts_once_in_every_matrix_core_attention_kernel(heads, rank, path):
    """One key/value head shared by all query heads, as latent attention uses the kernels; each head's sink is
    large enough to take a fifth to nine tenths of the weight, so leaving it out, or counting it once a split,
    shows."""
    case = Case(PORTIONS, heads, 1, rank, 16, torch.bfloat16, 31)
    sinks = torch.linspace(4.0, 8.0, heads)
    scale = rank ** -0.5
    want = sink_reference(case, scale, sinks)
    assert (want - sink_reference(case, scale, None)).abs().max() > 0.1  # the sink matters
    if path == "splits merged inside the block" and ops.plan_attention_in_block(2, 203, min(heads, 16), None, rank) is None:
        with pytest.raises(ops.KernelError):  # a tile's columns do not fit the block's LDS: refused, never wrong
            run_attention(case, "mfma", scale, sinks, **MFMA_PATHS[path])
        return
    close(run_attention(case, "mfma", scale, sinks, **MFMA_PATHS[path]), want, torch.bfloat16, path)
    close(run_attention(case, "mfma", scale, None, **MFMA_PATHS[path]), sink_reference(case, scale, None),
          torch.bfloat16, path + ", no sink")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,rank", [(6, 48), (17, 40), (2, 272), (5, 7)])
def test_a_sink_in_the_attention_kernel_for_any_size(dtype, heads, rank):
    case = Case(PORTIONS, heads, 1, rank, 32, dtype, 32)
    sinks = torch.linspace(-2.0, 8.0, heads)
    close(run_attention(case, "generic", 0.21, sinks), sink_reference(case, 0.21, sinks), dtype)


@pytest.mark.parametrize("far", [0, 15, 16, 17, 255, 256, 700])
def test_one_far_key_carries_the_weight_against_the_sink(far):
    """A key 900 positions back at most, at a page's first and last slot, with a score far above all others and
    above the sink: every kernel's output is that key's value."""
    heads, rank = 4, 64
    for portions, kw in (([(905, 1)], {}), ([(880, 26)], {"prefill_kernel": True}), ([(905, 1)], {"prefill_kernel": False, "splits": (8, 128), "in_block": False})):
        case = Case(portions, heads, 1, rank, 16, torch.bfloat16, 33)
        k = case.k_all[0]
        k[far, 0] = 0
        k[far, 0, 5] = 40.0
        case.k_log[int(case.table[0, far // 16]), far % 16, 0] = k[far, 0]
        case.q[:, :, 5] = 6.0
        sinks = torch.full((heads,), 9.0)
        got = run_attention(case, "mfma", 0.125, sinks, **kw)
        close(got, sink_reference(case, 0.125, sinks), torch.bfloat16, str(portions))
        assert torch.allclose(got[0, 0].float(), case.v_all[0][far, 0].float(), atol=3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rank,page_size", [(32, 16), (40, 32), (272, 64), (512, 16)])
def test_the_compressed_vector_is_normed_and_written_for_both_products(dtype, rank, page_size):
    T, col0, ld = 37, 24, 24 + rank + 9
    g, k_pages, v_pages, table = paged_setup(T + 20, 1, rank, page_size, dtype, rank)
    raw = (torch.randn(T, ld, generator=g) * 2.0).to(dtype)
    weight = (1.0 + 0.2 * torch.randn(rank, generator=g)).to(torch.bfloat16)
    positions = torch.arange(20, 20 + T, dtype=torch.int32)  # the portion starts inside a page
    kp, vp = to_cache(k_pages, v_pages)
    ops.latent_norm_write(dev(raw), col0, rank, dev(weight), 1e-5, 0.0, dev(positions),
                          dev(torch.zeros(T, dtype=torch.int32)), dev(table), kp, vp)
    want = PP.unit_rms(raw[:, col0:col0 + rank].double(), 1e-5) * weight.double()
    k_back, v_back = from_cache(kp, vp)
    for t in range(T):
        p = int(positions[t])
        page, slot = int(table[0, p // page_size]), p % page_size
        close(k_back[page, slot, 0], want[t], dtype, f"key row of token {t}")
        assert torch.equal(k_back[page, slot, 0], v_back[page, slot, 0])
    assert float(k_back.abs().sum(dim=(1, 2, 3)).ne(0).sum()) <= -(-(20 + T) // page_size)  # no other page touched


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,heads,n,k", [(1, 6, 96, 64), (70, 3, 24, 40), (130, 17, 10, 7), (9, 1, 128, 128),
                                            (16, 2, 17, 72), (300, 5, 250, 16), (33, 8, 66, 200)])
def test_products_by_head_with_and_without_a_gate(dtype, rows, heads, n, k):
    g = torch.Generator().manual_seed(rows)
    lead = 16
    a = torch.randn(rows, lead + heads * k + 5, generator=g).to(dtype)
    w = (torch.randn(heads, n, k, generator=g) / k ** 0.5).to(dtype)
    gate = torch.randn(rows, 3 + heads * n, generator=g).to(dtype)
    want = torch.einsum("rhk,hnk->rhn", a[:, lead:lead + heads * k].double().view(rows, heads, k), w.double()).reshape(rows, -1)
    close(ops.gemm_heads(dev(a), lead, dev(w)), want, dtype, "plain")
    close(ops.gemm_heads(dev(a), lead, dev(w), gate=dev(gate), gate_col0=3),
          want * torch.sigmoid(gate[:, 3:].double()), dtype, "gated")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,experts,top,width,inner", [(1, 8, 1, 64, 24), (7, 5, 2, 40, 20), (300, 70, 3, 96, 36),
                                                           (65, 3, 3, 100, 50), (130, 2, 1, 72, 8), (33, 4, 2, 256, 200),
                                                           (16, 1, 1, 32, 72), (17, 9, 4, 128, 64), (400, 6, 2, 64, 40),
                                                           (300, 4, 2, 72, 200), (500, 16, 3, 256, 136), (129, 2, 2, 512, 264)])
def test_experts_chosen_by_the_tokens_id(dtype, tokens, experts, top, width, inner):
    g = torch.Generator().manual_seed(tokens + experts)
    vocab, limit = 53, 0.8
    table = torch.rand(vocab, experts, generator=g).argsort(dim=1)[:, :top].to(torch.int32)
    ids = torch.randint(0, vocab, (tokens,), generator=g, dtype=torch.int32)
    h = torch.randn(tokens, width, generator=g).to(dtype)
    w = {"table": table}
    for e in range(experts):
        w[f"e{e}.gate"] = (torch.randn(inner, width, generator=g) * 2 / width ** 0.5).to(dtype)
        w[f"e{e}.up"] = (torch.randn(inner, width, generator=g) * 2 / width ** 0.5).to(dtype)
        w[f"e{e}.down"] = (torch.randn(width, inner, generator=g) / inner ** 0.5).to(dtype)
    mlp = {"router": {"top": top}, "expert": {"limit": limit}, "shared": None}
    want = PP.routed_ff(h.double(), ids.tolist(), {k: (v.double() if v.is_floating_point() else v) for k, v in w.items()}, "", mlp)
    w_gu = dev(torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(experts)]))
    w_down = dev(torch.stack([w[f"e{e}.down"] for e in range(experts)]))
    tile, mfma = ops.moe_plan(dtype, tokens * top, width, inner)
    # bf16 sizes in eights run on the matrix cores, in tiles of 16 rows while the rows are few; all else in 64s
    assert mfma == (dtype == torch.bfloat16 and width % 8 == 0 and inner % 8 == 0)
    assert tile == (16 if mfma and tokens * top <= 256 else 64)
    slot_of, row_token, tile_group = ops.moe_route(dev(ids), tokens, dev(table), experts, tile)
    # the sorted order: every choice has a row of its own in a tile of its expert, rows know their tokens
    so, rt, tg = slot_of.cpu().view(tokens, top), row_token.cpu(), tile_group.cpu()
    assert so.min() >= 0 and so.flatten().unique().numel() == tokens * top
    for t in range(tokens):
        for c in range(top):
            assert rt[so[t, c]] == t and tg[so[t, c] // tile] == table[ids[t], c]
    assert int((rt >= 0).sum()) == tokens * top
    if mfma:  # the activation inside the product
        act = ops.gemm_experts(dev(h), w_gu, tile_group, row_index=row_token, tile=tile, mfma=True, glu=(limit, 1.702))
    else:
        act = ops.clamped_glu(ops.gemm_experts(dev(h), w_gu, tile_group, row_index=row_token, tile=tile), limit, 1.702)
    got = ops.moe_combine(ops.gemm_experts(act, w_down, tile_group, tile=tile, mfma=mfma), slot_of, top, 1.0 / top, tokens)
    close(got, want, dtype)
    if mfma:  # the same through the kernels that take any size
        s64, r64, t64 = ops.moe_route(dev(ids), tokens, dev(table), experts, 64)
        act = ops.clamped_glu(ops.gemm_experts(dev(h), w_gu, t64, row_index=r64), limit, 1.702)
        close(ops.moe_combine(ops.gemm_experts(act, w_down, t64), s64, top, 1.0 / top, tokens), want, dtype, "32-bit kernel")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_clamped_activation_at_and_beyond_its_limits(dtype):
    limit = 1.25
    gate = torch.tensor([[-9.0, -limit, -0.3, 0.0, 0.4, limit, 1.2501, 30.0]]).to(dtype)
    up = torch.tensor([[40.0, 1.3, limit, -limit, -1.26, -50.0, 0.2, -0.9]]).to(dtype)
    got = ops.clamped_glu(dev(torch.cat([gate, up], dim=1)), limit, 1.702)
    g, u = gate.double().clamp(max=limit), up.double().clamp(-limit, limit)
    close(got, g * torch.sigmoid(1.702 * g) * (u + 1.0), dtype)
    # a gate far below zero is not clamped; a gate far above counts as the limit, an up far below as minus the limit
    assert float(got[0, 0]) < 0
    assert abs(float(got[0, 7]) - limit / (1 + 2.718281828 ** (-1.702 * limit)) * 0.1) < 2e-2
    assert float(got[0, 5]) < 0


# --------------------------------------------------------------------------
# whole models through the step function
# --------------------------------------------------------------------------
LENGTHS = {"P": [1, 2, 17, 33, 64, 150], "Q": [3, 16, 65, 47, 130, 90], "P-loud": [5, 31, 32, 100, 129, 70]}
MODES = {"whole": tt.trace_whole, "tail": tt.trace_tail, "portions": tt.trace_portions, "mixed": tt.trace_mixed}


@pytest.fixture(scope="module")
def pinorax_dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("pinorax")
    return {"P": tiny_pinorax.write_model(root / "P", "P"), "Q": tiny_pinorax.write_model(root / "Q", "Q"),
            "P-loud": tiny_pinorax.write_model(root / "P-loud", "P", seed=5, loud=True)}


@pytest.fixture(scope="module")
def references(pinorax_dirs):
    out = {}
    for name, folder in pinorax_dirs.items():
        weights, cfg = PP.load_weights(folder), PP.read_config(folder)
        seqs = tt.make_sequences(cfg["vocab"], LENGTHS[name], seed=len(name) + ord(name[0]))
        out[name] = (seqs, {rid: PP.forward(weights, cfg, ids) for rid, ids in seqs.items()}, cfg["vocab"])
    return out


def make_runner(model_dir, dtype, max_tokens, page_size=16, **more):
    cfg = EngineConfig(dtype=dtype, page_size=page_size, max_model_len=max_tokens, max_num_seqs=4,
                       max_num_batched_tokens=max_tokens, max_prefill_chunk=max_tokens, max_cache_tokens=max_tokens,
                       **more)
    return ModelRunner.from_model_dir(model_dir, cfg)


def check(steps, outputs, refs, vocab, dtype, what):
    got = tt.collect(steps, outputs, vocab)
    prefix = steps[0]["entries"][0]["id"].split("-")[0]
    assert len(got) == len(refs)
    for name, ref in refs.items():
        tt.compare(got[f"{prefix}-{name}"], ref, dtype, f"{what} {name}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "P-loud"])
@pytest.mark.parametrize("mode", list(MODES))
def test_cuttings(pinorax_dirs, references, name, dtype, mode):
    """Whole prompts; prefill and then token-by-token decoding; portions down to two tokens and single tokens;
    unequal requests mixed in a batch, with a pool so small that pages and slots are used again."""
    seqs, refs, vocab = references[name]
    steps = MODES[mode](seqs)
    runner = make_runner(pinorax_dirs[name], dtype, tt.required_tokens(steps))
    check(steps, tt.run_in_process(runner, steps), refs, vocab, dtype, f"{name} {dtype} {mode}")
    assert all(g.pool.free_count == g.pool.num_pages for g in runner.cache.groups.values())
    assert runner.cache.slots.free_count == 4


@pytest.mark.parametrize("name", ["P", "Q"])
def test_cuttings_agree_bit_for_bit_in_32_bit(pinorax_dirs, references, name):
    """No logit depends on how the prompt was cut, on what else is in the batch or on the pages used."""
    seqs, refs, vocab = references[name]
    runner = make_runner(pinorax_dirs[name], "float32", 4 * 192)
    results = {}
    for mode, make in MODES.items():
        steps = make(seqs)
        got = tt.collect(steps, tt.run_in_process(runner, steps), vocab)
        results[mode] = {rid.split("-", 1)[1]: arr for rid, arr in got.items()}
    for mode in ("tail", "portions", "mixed"):
        for rid in seqs:
            assert np.array_equal(results[mode][rid], results["whole"][rid]), f"{name} {mode} {rid}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["tail", "mixed"])
def test_what_a_page_held_before_reaches_no_logit(pinorax_dirs, references, dtype, mode):
    seqs, refs, vocab = references["P-loud"]
    steps = MODES[mode](seqs)
    runner = make_runner(pinorax_dirs["P-loud"], dtype, tt.required_tokens(steps))
    for view in runner.storage.views:
        view.k_pages.fill_(float("nan"))
        view.v_pages.fill_(float("nan"))
    check(steps, tt.run_in_process(runner, steps), refs, vocab, dtype, f"NaN pages {dtype} {mode}")


@pytest.mark.parametrize("page_size", [32, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_page_sizes(pinorax_dirs, references, page_size, dtype):
    seqs, refs, vocab = references["P"]
    steps = tt.trace_mixed(seqs, seed=3)
    runner = make_runner(pinorax_dirs["P"], dtype, tt.required_tokens(steps), page_size=page_size)
    check(steps, tt.run_in_process(runner, steps), refs, vocab, dtype, f"page {page_size}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(pinorax_dirs, references, tmp_path, dtype):
    seqs, refs, vocab = references["Q"]
    steps, n = [], 0
    for make in MODES.values():
        part = make(seqs, first_step=n)
        steps += part
        n += len(part)
    outputs = tt.run_trace_program(pinorax_dirs["Q"], dtype, steps, tmp_path / "out", max_tokens=tt.required_tokens(steps))
    got = tt.collect(steps, outputs, vocab)
    for prefix in ("w", "t", "p", "m"):
        for name, ref in refs.items():
            tt.compare(got[f"{prefix}-{name}"], ref, dtype, f"trace_run {dtype} {prefix}-{name}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_sequences_far_keys_and_long_decoding(tmp_path_factory, dtype):
    """Wide layers with loud keys over a thousand tokens: a prompt in one step, one in portions that end inside
    pages, and the last 150 tokens decoded one by one (in bf16 from recorded graphs, across a bucket's edge at
    1 024 keys)."""
    folder = tiny_pinorax.write_model(tmp_path_factory.mktemp("R") / "R", "R", loud=True)
    weights, cfg = PP.load_weights(folder), PP.read_config(folder)
    ids = tt.make_sequences(cfg["vocab"], [1100], seed=77)["r0"]
    want = PP.forward(weights, cfg, ids)
    runner = make_runner(folder, dtype, 2304)
    runner.add_request("whole")
    got = runner.step([("whole", ids, list(range(len(ids))))]).float().cpu().numpy()
    runner.release("whole")
    tt.compare(got, want, dtype, "whole")
    runner.add_request("cut")
    rows, at = [], 0
    for size in (63, 2, 130, 255, 500):
        rows.append(runner.step([("cut", ids[at:at + size], list(range(size)))]).float().cpu().numpy())
        at += size
    while at < len(ids):
        rows.append(runner.step([("cut", ids[at:at + 1], [0])]).float().cpu().numpy().copy())
        at += 1
    runner.release("cut")
    tt.compare(np.concatenate(rows), want, dtype, "portions, then token by token")
    if dtype == "bfloat16":
        assert runner.graph_replays > 100


# --------------------------------------------------------------------------
# through the engine: scheduler, batching, sampling
# --------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_entry_point(pinorax_dirs, name, dtype):
    """Five prompts for two places, prompts in portions of five tokens, a pool of two requests' worth: requests
    wait, pages and slots change hands.  Every token is the plain model's choice (in bf16: within the
    tolerance of its largest logit)."""
    import rvllm_amd

    folder = pinorax_dirs[name]
    weights, cfg = PP.load_weights(folder), PP.read_config(folder)
    prompts = [[3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5], [27, 18, 28], [7], [11, 12, 13, 14, 15, 16, 17], [90, 2]]
    outs = rvllm_amd.generate(str(folder), prompts, max_tokens=12, dtype=dtype, max_model_len=64, max_num_seqs=2,
                              max_num_batched_tokens=16, max_prefill_chunk=5, max_cache_tokens=128)
    for prompt, out in zip(prompts, outs):
        assert len(out) == 12
        if dtype == "float32":
            assert out == PP.greedy(weights, cfg, prompt, 12)
        else:
            logits = PP.forward(weights, cfg, prompt + out)
            scale = float(logits.abs().max())
            for j, token in enumerate(out):
                row = logits[len(prompt) - 1 + j]
                assert row[token] >= row.max() - 2 * tt.TOLERANCE[dtype] * scale, f"token {j} of {prompt}"


def test_sampled_generation_runs_and_is_repeatable(pinorax_dirs):
    import rvllm_amd

    kw = dict(max_tokens=10, temperature=0.8, top_k=20, top_p=0.9, seed=4, dtype="bfloat16", max_model_len=64,
              max_num_seqs=3)
    prompts = [[1, 2, 3], [50, 60], [9, 9, 9, 9]]
    first = rvllm_amd.generate(str(pinorax_dirs["P"]), prompts, **kw)
    assert first == rvllm_amd.generate(str(pinorax_dirs["P"]), prompts, **kw)
    assert all(len(out) == 10 and all(0 <= t < 211 for t in out) for out in first)
