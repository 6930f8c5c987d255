"""The Rufedra design on the GPU against the plain implementation (``plain_rufedra``): each mechanism alone at the
level of its kernels, then whole models through the step function under every way of cutting the work, through
``bin/trace_run`` and through the engine's scheduler."""

import numpy as np
import pytest
import torch

import plain_rufedra as PR
import tiny_rufedra
import trace_tools as tt
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.batch import BatchBuilder, Portion
from rvllm_amd.engine.runner import ModelRunner
from rvllm_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def dev(t):
    return t.to(DEV).contiguous()


def close(got, want, dtype, what="", f32=2e-5, bf16=2e-2):
    """Against the values' own size: 32-bit to a few roundings, bf16 to a few of its."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, f"{what}: {tuple(got.shape)} against {tuple(want.shape)}"
    scale = float(want.abs().max()) or 1.0
    worst = float((got - want).abs().max())
    assert worst <= (f32 if dtype == torch.float32 else bf16) * scale, f"{what}: {worst:.3e} against {scale:.3e}"


def make_step(portions, slots):
    """A step of ``portions`` = [(first position, tokens)], request b in state slot ``slots[b]``; no page groups."""
    total = sum(n for _, n in portions)
    builder = BatchBuilder(torch.device(DEV), max(total, 1), max(len(portions), 1), {})
    return builder.build([Portion(b, [0] * n, start) for b, (start, n) in enumerate(portions)], {}, slots)


def cuts_of(total, sizes):
    """(first, count) pieces of ``total`` tokens, sizes taken in turn."""
    out, at, i = [], 0, 0
    while at < total:
        n = min(sizes[i % len(sizes)], total - at)
        out.append((at, n))
        at += n
        i += 1
    return out


# --------------------------------------------------------------------------
# mechanisms alone
# --------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps,channels,group", [(4, 96, 32), (1, 40, 40), (2, 70, 7), (5, 300, 100), (3, 64, 64)])
@pytest.mark.parametrize("aligned", [False, True])
def test_convolution_with_its_state_under_any_cutting(dtype, taps, channels, group, aligned):
    """Two requests in two slots out of five; portions of 1, 2, 3 and more tokens, shorter than the taps too; the
    state row that a portion leaves is what the next one starts from; with and without unit length and bias.
    ``aligned``: channels, rows and state on 16-byte boundaries, or at odd places."""
    g = torch.Generator().manual_seed(taps * 1000 + channels)
    lengths = [23, 9]
    c_in, c_out, s_off, pad = (8, 8, 16, 16) if aligned else (3, 1, 11, 6)
    xs = [(torch.randn(n, channels + pad, generator=g) * 2).to(dtype) for n in lengths]  # the channels lie inside wider rows
    w = torch.randn(channels, taps, generator=g) * 0.7
    bias = torch.randn(channels, generator=g)
    for unit_eps, b, moves in ((None, bias, False), (1e-6, None, False), (None, bias, True), (1e-6, None, True)):
        want = []
        for x in xs:
            y = PR.silu(PR.causal_conv(x[:, c_in:c_in + channels].double(), w.double(), None if b is None else b.double()))
            y = y.to(dtype).double()  # the activated output is rounded to the activations' type once
            if unit_eps is not None:
                y = PR.unit(y.view(-1, channels // group, group), unit_eps)
                y[:, :2] *= 0.25
                y = y.reshape(-1, channels)
            want.append(y)
        slots = torch.zeros(5, s_off + (taps - 1) * channels, device=DEV)
        slots[:, :s_off] = 7.0  # what lies before the state is someone else's
        got = [[], []]
        cuts = [cuts_of(lengths[0], [1, 2, 3, 1, 5, 2, 9]), cuts_of(lengths[1], [2, 1, 1, 5])]
        if moves:  # single tokens only: the convolution moves its state on itself
            cuts = [cuts_of(n, [1]) for n in lengths]
        for i in range(max(len(c) for c in cuts)):
            live = [r for r in range(2) if i < len(cuts[r])]
            step = make_step([cuts[r][i] for r in live], [3 if r == 0 else 1 for r in live])
            rows = torch.cat([xs[r][cuts[r][i][0]:cuts[r][i][0] + cuts[r][i][1]] for r in live])
            out = torch.full((rows.shape[0], channels + 2 * c_out), -5.0, dtype=torch.float32 if unit_eps else dtype,
                             device=DEV)
            ops.causal_conv(dev(rows), c_in, channels, dev(w), None if b is None else dev(b), slots, s_off, step, out,
                            c_out, group=group, unit_eps=unit_eps, scaled_groups=2, group_scale=0.25, move_state=moves)
            if not moves:
                ops.conv_state_update(dev(rows), c_in, channels, taps, slots, s_off, step)
            assert float(out[:, :c_out].max()) == -5.0 and float(out[:, -c_out:].max()) == -5.0
            at = 0
            for r in live:
                n = cuts[r][i][1]
                got[r].append(out[at:at + n, c_out:c_out + channels].float().cpu())
                at += n
        for r in range(2):
            close(torch.cat(got[r]), want[r], dtype, f"request {r} unit={unit_eps} moves={moves}", bf16=1e-2)
        assert float(slots[:, :s_off].min()) == 7.0
        if taps > 1:  # the other slots are untouched; the state holds the last inputs, oldest first
            assert float(slots[[0, 2, 4], s_off:].abs().max()) == 0.0
            close(slots[3, s_off:].view(taps - 1, channels), xs[0][-(taps - 1):, c_in:c_in + channels].float(),
                  torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dk,dv", [(4, 2, 16, 24), (1, 1, 40, 12), (6, 6, 7, 70), (2, 1, 128, 64),
                                                  (3, 1, 300, 5)])
def test_delta_rule_whole_and_cut_give_the_same_bits(dtype, heads, kv_heads, dk, dv):
    g = torch.Generator().manual_seed(heads * 100 + dk)
    T = 37
    width = 2 * kv_heads * dk + heads * dv
    qkv = torch.randn(T, width, generator=g)
    q = PR.unit(qkv[:, :kv_heads * dk].view(T, kv_heads, dk).double(), 1e-6) * dk ** -0.5
    k = PR.unit(qkv[:, kv_heads * dk:2 * kv_heads * dk].view(T, kv_heads, dk).double(), 1e-6)
    qkv[:, :kv_heads * dk] = q.reshape(T, -1).float()
    qkv[:, kv_heads * dk:2 * kv_heads * dk] = k.reshape(T, -1).float()
    ab = (torch.randn(T, 3 + 2 * heads, generator=g) * 2).to(dtype)
    A_log, dt_bias = torch.randn(heads, generator=g) * 0.5, torch.randn(heads, generator=g)
    a, b = ab[:, 1:1 + heads].double(), ab[:, 3 + heads:].double()
    decay = torch.exp(-torch.exp(A_log.double()) * PR.softplus(a + dt_bias.double()))
    beta = torch.sigmoid(b)
    want, last = [], []
    for h in range(heads):
        kv = h // (heads // kv_heads)
        o, S = PR.delta_recurrence(qkv[:, kv * dk:(kv + 1) * dk].double(),
                                   qkv[:, (kv_heads + kv) * dk:(kv_heads + kv + 1) * dk].double(),
                                   qkv[:, 2 * kv_heads * dk + h * dv:2 * kv_heads * dk + (h + 1) * dv].double(),
                                   decay[:, h], beta[:, h])
        want.append(o)
        last.append(S)
    want = torch.cat(want, 1)
    results = []
    for sizes in ([T], [1], [2, 3, 1, 7, 16]):
        slots = torch.zeros(3, 5 + heads * dk * dv, device=DEV)
        rows = []
        for first, n in cuts_of(T, sizes):
            step = make_step([(first, n)], [2])
            rows.append(ops.delta_rule(dev(qkv[first:first + n]), 0, kv_heads * dk, 2 * kv_heads * dk,
                                       dev(ab[first:first + n]), 1, 3 + heads, dev(A_log), dev(dt_bias), slots, 5, step,
                                       heads, kv_heads, dk, dv).cpu())
        results.append(torch.cat(rows))
        close(results[-1], want, torch.float32, f"cut {sizes}", f32=1e-4)
        close(slots[2, 5:].view(heads, dv, dk).transpose(1, 2), torch.stack(last), torch.float32, "the state", f32=1e-4)
        assert float(slots[:2].abs().max()) == 0.0 and float(slots[2, :5].abs().max()) == 0.0
    assert torch.equal(results[0], results[1]) and torch.equal(results[0], results[2])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels,n_state", [(48, 6), (100, 33), (7, 1), (328, 16), (65, 200)])
def test_selective_scan_whole_and_cut_and_two_requests(dtype, channels, n_state):
    g = torch.Generator().manual_seed(channels + n_state)
    T = [29, 6]
    data = []
    for n in T:
        x = (torch.randn(n, channels, generator=g)).to(dtype)
        z = (torch.randn(n, channels + 4, generator=g)).to(dtype)
        dt = (torch.randn(n, channels, generator=g)).to(dtype)
        bc = (torch.randn(n, 3 + 2 * n_state, generator=g)).to(dtype)
        data.append((x, z, dt, bc))
    dt_bias, D = torch.randn(channels, generator=g), torch.randn(channels, generator=g)
    A_log = torch.randn(channels, n_state, generator=g) * 0.5
    want = []
    for x, z, dt, bc in data:
        y, _ = PR.scan_recurrence(x.double(), PR.softplus(dt.double() + dt_bias.double()), -torch.exp(A_log.double()),
                                  bc[:, 1:1 + n_state].double(), bc[:, 3 + n_state:].double(), D.double())
        want.append(y * PR.silu(z[:, 4:].double()))
    outs = []
    for sizes in ([64], [1], [3, 2, 1, 11]):
        slots = torch.zeros(4, 2 + channels * n_state, device=DEV)
        cuts = [cuts_of(n, sizes) for n in T]
        got = [[], []]
        for i in range(max(len(c) for c in cuts)):
            live = [r for r in range(2) if i < len(cuts[r])]
            step = make_step([cuts[r][i] for r in live], [1 if r == 0 else 3 for r in live])
            piece = [torch.cat([data[r][j][cuts[r][i][0]:cuts[r][i][0] + cuts[r][i][1]] for r in live]) for j in range(4)]
            y = ops.selective_scan(dev(piece[0]), dev(piece[1]), 4, dev(piece[2]), dev(dt_bias), dev(piece[3]), 1,
                                   3 + n_state, dev(A_log), dev(D), slots, 2, step).float().cpu()
            at = 0
            for r in live:
                got[r].append(y[at:at + cuts[r][i][1]])
                at += cuts[r][i][1]
        outs.append([torch.cat(x) for x in got])
        for r in range(2):
            close(outs[-1][r], want[r], dtype, f"cut {sizes} request {r}", f32=1e-4)
    for r in range(2):
        assert torch.equal(outs[0][r], outs[1][r]) and torch.equal(outs[0][r], outs[2][r])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dv", [(4, 24), (1, 200), (7, 5), (2, 64)])
def test_output_norm_a_head_with_a_shared_weight_and_a_silu_gate(dtype, heads, dv):
    g = torch.Generator().manual_seed(dv)
    o = torch.randn(11, heads * dv, generator=g) * 4
    gate = torch.randn(11, heads * dv + 9, generator=g).to(dtype)
    w = torch.randn(dv, generator=g)
    want = PR.rms_norm(o.double().view(11, heads, dv), 1e-3, w.double()).reshape(11, -1) * PR.silu(gate[:, 9:].double())
    close(ops.head_norm_gate(dev(o), dev(gate), 9, dev(w), 1e-3, heads, dv, dtype), want, dtype)
    tiny = torch.full((1, heads * dv), 1e-3)  # eps sits under the root
    want = PR.rms_norm(tiny.double().view(1, heads, dv), 1e-2, w.double()).reshape(1, -1) * PR.silu(gate[:1, 9:].double())
    close(ops.head_norm_gate(dev(tiny), dev(gate[:1]), 9, dev(w), 1e-2, heads, dv, dtype), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,hd,rot,page_size", [(4, 2, 32, 16, 16), (3, 3, 20, 20, 32), (5, 1, 12, 6, 16),
                                                     (2, 1, 80, 80, 64), (2, 2, 272, 0, 16), (1, 1, 512, 130, 16)])
@pytest.mark.parametrize("mode", [ops.NORM_AFTER_ROTATION, ops.NORM_BEFORE_ROTATION, ops.NORM_NONE])
def test_rotation_in_halves_norm_and_keys_written_as_values(dtype, nq, nkv, hd, rot, page_size, mode):
    g = torch.Generator().manual_seed(hd + rot)
    positions = [0, 1, 15, 16, 17, 40, 77]
    T = len(positions)
    cols = (nq + nkv) * hd + 5
    proj = (torch.randn(T, cols, generator=g) * 3).to(dtype)
    bias = torch.randn(cols, generator=g) if mode == ops.NORM_AFTER_ROTATION else None
    raw = proj if bias is None else (proj.double() + bias.double()).to(dtype)  # a projection with its bias, as stored
    q_in = raw[:, 2:2 + nq * hd].double().view(T, nq, hd)
    k_in = raw[:, 2 + nq * hd:2 + (nq + nkv) * hd].double().view(T, nkv, hd)
    pos = torch.tensor(positions)
    weighted = mode == ops.NORM_BEFORE_ROTATION
    qw, kw = torch.randn(hd, generator=g), torch.randn(hd, generator=g)

    def plain(x, w):
        if mode == ops.NORM_BEFORE_ROTATION:
            return PR.rotate_halves(PR.rms_norm(x, 1e-5, w.double()), pos, rot, 100.0)
        r = PR.rotate_halves(x, pos, rot, 100.0)
        return PR.rms_norm(r, 1e-5) if mode == ops.NORM_AFTER_ROTATION else r

    half = rot // 2
    rope = None
    if rot:
        freq = torch.tensor([100.0 ** (-2.0 * i / rot) for i in range(half)], dtype=torch.float64)
        ang = pos.double()[:, None] * freq
        rope = (dev(torch.cos(ang).float()), dev(torch.sin(ang).float()))
    num_pages = 9
    table = torch.full((1, 8), -1, dtype=torch.int32)
    pages = {p // page_size for p in positions}
    for n, page in enumerate(sorted(pages)):
        table[0, page] = (n * 4 + 1) % num_pages
    k_pages = torch.zeros(num_pages, nkv, page_size, hd, dtype=dtype, device=DEV)
    v_pages = torch.zeros(num_pages, nkv, page_size // 16, hd, 16, dtype=dtype, device=DEV)
    q_out = torch.empty(T, nq * hd, dtype=dtype, device=DEV)
    ops.rotate_norm_write(dev(proj), 2, 2 + nq * hd, None, q_out, dev(qw) if weighted else None,
                          dev(kw) if weighted else None, 1e-5, 0.0, mode, rope, rot, dev(pos.int()),
                          dev(torch.zeros(T, dtype=torch.int32)), dev(table), k_pages, v_pages, nq, nkv, hd,
                          bias=None if bias is None else dev(bias))
    close(q_out.view(T, nq, hd), plain(q_in, qw), dtype, "queries")
    want_k = plain(k_in, kw)
    for t, p in enumerate(positions):
        page, slot = int(table[0, p // page_size]), p % page_size
        close(k_pages[page, :, slot], want_k[t], dtype, f"key at {p}")
        got_v = v_pages[page, :, slot // 16, :, slot % 16]
        assert torch.equal(got_v.cpu(), raw[t, 2 + nq * hd:2 + (nq + nkv) * hd].view(nkv, hd)), f"value at {p}"
    untouched = [p for p in range(num_pages) if p not in {int(table[0, page]) for page in pages}]
    assert float(k_pages[untouched].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [7, 64, 100, 1000, 4100])
def test_sandwich_on_a_32_bit_stream_with_a_scale_a_channel(dtype, width):
    g = torch.Generator().manual_seed(width)
    rows = 6
    x0 = torch.randn(rows, width, generator=g) * 3
    branch = (torch.randn(rows, width, generator=g) * 5).to(dtype)
    w_post, w_next, scale = (torch.randn(width, generator=g) for _ in range(3))
    added = x0.double() + PR.rms_norm(branch.double(), 1e-5, w_post.double()) * scale.double()
    x = dev(x0.clone())
    nxt = ops.add_rmsnorm_scaled(dev(branch), dev(w_post.to(dtype)), 1e-5, 0.0, dev(scale), x, dev(w_next), 1e-5, 0.0)
    ref = x0.double() + PR.rms_norm(branch.double(), 1e-5, w_post.to(dtype).double()) * scale.double()
    close(x, ref, torch.float32, "the stream stays 32-bit")
    assert nxt.dtype == dtype
    close(nxt, PR.rms_norm(ref, 1e-5, w_next.double()), dtype, "the next norm")
    # without a scale and without a next norm; the branch as unreduced partial sums
    x = dev(x0.clone())
    parts = torch.randn(3, rows, width, generator=g)
    assert ops.add_rmsnorm_scaled(ops.SlicedSums(dev(parts), dtype), dev(w_post), 1e-5, 0.0, None, x) is None
    close(x, x0.double() + PR.rms_norm(parts.double().sum(0), 1e-5, w_post.double()), torch.float32, "partial sums")
    # two branches with their weights, one stored and one as partial sums, normed as their sum
    x = dev(x0.clone())
    both = ops.BranchSum(dev(branch), ops.SlicedSums(dev(parts), dtype), -0.8, 1.3)
    nxt = ops.add_rmsnorm_scaled(both, dev(w_post), 1e-5, 0.0, dev(scale), x, dev(w_next), 1e-5, 0.0)
    mixed = -0.8 * branch.double() + 1.3 * parts.double().sum(0)
    ref = x0.double() + PR.rms_norm(mixed, 1e-5, w_post.double()) * scale.double()
    close(x, ref, torch.float32, "two branches")
    close(nxt, PR.rms_norm(ref, 1e-5, w_next.double()), dtype, "the next norm after two branches")
    close(ops.as_tensor(both), mixed, dtype, "two branches added up")
    # the norm that reads the stream and writes activations, whole and by rows
    close(ops.rmsnorm_cast(dev(x0), dev(w_next), 1e-5, 0.0, dtype), PR.rms_norm(x0.double(), 1e-5, w_next.double()), dtype)
    pick = torch.tensor([5, 0, 2], dtype=torch.int32)
    close(ops.rmsnorm_cast(dev(x0), dev(w_next), 1e-5, 0.0, dtype, rows=dev(pick)),
          PR.rms_norm(x0.double(), 1e-5, w_next.double())[pick.long()], dtype, "picked rows")
    assert float(added.abs().max()) > 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_weighted_sum_gate_and_logit_scale(dtype):
    g = torch.Generator().manual_seed(9)
    a = torch.randn(5, 70, generator=g).to(dtype)
    parts = torch.randn(2, 5, 70, generator=g)
    total = ops.weighted_sum(dev(a), ops.SlicedSums(dev(parts), dtype), -0.8, 1.3)
    assert total.data.dtype == torch.float32 and total.slices == 1
    close(total.data[0], -0.8 * a.double() + 1.3 * parts.double().sum(0), torch.float32)
    gate = torch.randn(5, 100, generator=g).to(dtype)
    for act, f in (("sigmoid", torch.sigmoid), ("silu", PR.silu)):
        got = ops.gate_mul_(dev(a.clone()), dev(gate), 30, act)
        close(got, a.double() * f(gate[:, 30:].double()), dtype, act)
    logits = torch.randn(3, 50, generator=g)
    close(ops.scale_(dev(logits.clone()), -2.5), logits.double() * -2.5, torch.float32)


# --------------------------------------------------------------------------
# whole models through the step function
# --------------------------------------------------------------------------
LENGTHS = {"A": [70, 1, 33, 2, 45, 17], "B": [40, 3, 25, 1, 18], "A-loud": [70, 29, 48, 5]}
MODES = {"whole": tt.trace_whole, "tail": tt.trace_tail, "portions": tt.trace_portions, "mixed": tt.trace_mixed}


@pytest.fixture(scope="module")
def rufedra_dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("rufedra")
    return {"A": tiny_rufedra.write_model(root / "A", "A"), "B": tiny_rufedra.write_model(root / "B", "B"),
            "A-loud": tiny_rufedra.write_model(root / "A-loud", "A", seed=5, loud=True)}


@pytest.fixture(scope="module")
def references(rufedra_dirs):
    out = {}
    for name, folder in rufedra_dirs.items():
        weights, cfg = PR.load_weights(folder), PR.read_config(folder)
        seqs = tt.make_sequences(cfg["vocab"], LENGTHS[name], seed=len(name) + ord(name[0]))
        refs = {rid: PR.forward(weights, cfg, ids) for rid, ids in seqs.items()}
        out[name] = (seqs, refs, cfg["vocab"])
        ROUNDING[name] = {rid: PR.rounding_error(weights, cfg, ids, refs[rid]) for rid, ids in seqs.items()}
    return out


# By model and request, the error at every position that rounding to bfloat16 alone causes in the plain
# implementation, where the design allows 16 bits.  This design norms every branch to size one before it adds it, so
# a branch's rounding enters the stream undiminished, and small models have positions where one head's read-out all
# but cancels; there the bf16 engine is held to three times that error instead of the flat share of the largest logit.
ROUNDING: dict = {}


def compare(got, ref, dtype, what, model=None, rid=None):
    if dtype == "bfloat16" and model in ROUNDING:
        got64 = np.asarray(got, dtype=np.float64)
        err = np.abs(got64 - ref.numpy()).max(-1)
        scale = float(ref.abs().max())
        allowed = np.maximum(tt.TOLERANCE[dtype] * scale, 3.0 * ROUNDING[model][rid].numpy())
        assert np.isfinite(got64).all() and got64.shape == tuple(ref.shape), what
        worst = int((err / allowed).argmax())
        assert err[worst] <= allowed[worst], (f"{what}: position {worst}: |diff| {err[worst]:.3e}, allowed "
                                              f"{allowed[worst]:.3e} (scale {scale:.3e})")
        return
    tt.compare(got, ref, dtype, what)


def make_runner(model_dir, dtype, max_tokens, page_size=16, **more):
    cfg = EngineConfig(dtype=dtype, page_size=page_size, max_model_len=max_tokens, max_num_seqs=4,
                       max_num_batched_tokens=max_tokens, max_prefill_chunk=max_tokens, max_cache_tokens=max_tokens,
                       **more)
    return ModelRunner.from_model_dir(model_dir, cfg)


def check(steps, outputs, refs, vocab, dtype, what, model=None):
    got = tt.collect(steps, outputs, vocab)
    prefix = steps[0]["entries"][0]["id"].split("-")[0]
    assert len(got) == len(refs)
    for name, ref in refs.items():
        compare(got[f"{prefix}-{name}"], ref, dtype, f"{what} {name}", model, name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_stream_after_every_layer(rufedra_dirs, dtype):
    """Layer by layer: the first layer that differs names the mechanism."""
    folder = rufedra_dirs["A"]
    weights, cfg = PR.load_weights(folder), PR.read_config(folder)
    ids = tt.make_sequences(cfg["vocab"], [50], seed=2)["r0"]
    want = []
    PR.forward(weights, cfg, ids, want)
    runner = make_runner(folder, dtype, 64)
    got = []
    for block in runner.model.blocks:
        inner = block.forward

        def spy(x, step, cache, entered=None, then=None, inner=inner):
            out = inner(x, step, cache, entered=entered, then=then)
            got.append(x.detach().float().cpu())
            return out

        block.forward = spy
    runner.add_request("a")
    runner.step([("a", ids, [len(ids) - 1])])
    assert len(got) == len(want)
    for i, (g_, w_) in enumerate(zip(got, want)):
        close(g_, w_, torch.float32 if dtype == "float32" else torch.bfloat16, f"after layer {i}", bf16=3e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "A-loud"])
@pytest.mark.parametrize("mode", list(MODES))
def test_cuttings(rufedra_dirs, references, name, dtype, mode):
    """Whole prompts; prefill and then token-by-token decoding; portions down to two tokens and single tokens;
    unequal requests mixed in a batch, with a pool so small that pages and slots are used again."""
    seqs, refs, vocab = references[name]
    steps = MODES[mode](seqs)
    runner = make_runner(rufedra_dirs[name], dtype, tt.required_tokens(steps))
    check(steps, tt.run_in_process(runner, steps), refs, vocab, dtype, f"{name} {dtype} {mode}", name)
    assert all(g.pool.free_count == g.pool.num_pages for g in runner.cache.groups.values())
    assert runner.cache.slots.free_count == 4


@pytest.mark.parametrize("name", ["A", "B"])
def test_cuttings_agree_bit_for_bit_in_32_bit(rufedra_dirs, references, name):
    """No logit depends on how the prompt was cut, on what else is in the batch or on the pages and slots used."""
    seqs, refs, vocab = references[name]
    runner = make_runner(rufedra_dirs[name], "float32", 4 * 192)
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
def test_what_a_page_or_slot_held_before_reaches_no_logit(rufedra_dirs, references, dtype, mode):
    """Pages full of NaN and state slots full of large numbers before the first request: pages are never read
    past a request's own tokens, and a slot is cleared when it is handed out."""
    seqs, refs, vocab = references["A-loud"]
    steps = MODES[mode](seqs)
    runner = make_runner(rufedra_dirs["A-loud"], dtype, tt.required_tokens(steps))

    def spoil(view):
        if isinstance(view, tuple):
            for member in view:
                spoil(member)
        elif hasattr(view, "k_pages"):
            view.k_pages.fill_(float("nan"))
            view.v_pages.fill_(float("nan"))
        elif view is not None:
            view.slots.fill_(1e4)

    for view in runner.storage.views:
        spoil(view)
    check(steps, tt.run_in_process(runner, steps), refs, vocab, dtype, f"spoiled {dtype} {mode}", "A-loud")


@pytest.mark.parametrize("page_size", [32, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_page_sizes(rufedra_dirs, references, page_size, dtype):
    seqs, refs, vocab = references["A"]
    steps = tt.trace_mixed(seqs, seed=3)
    runner = make_runner(rufedra_dirs["A"], dtype, tt.required_tokens(steps), page_size=page_size)
    check(steps, tt.run_in_process(runner, steps), refs, vocab, dtype, f"page {page_size}", "A")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(rufedra_dirs, references, tmp_path, dtype):
    seqs, refs, vocab = references["B"]
    steps, n = [], 0
    for make in MODES.values():
        part = make(seqs, first_step=n)
        steps += part
        n += len(part)
    outputs = tt.run_trace_program(rufedra_dirs["B"], dtype, steps, tmp_path / "out", max_tokens=tt.required_tokens(steps))
    got = tt.collect(steps, outputs, vocab)
    for prefix in ("w", "t", "p", "m"):
        for name, ref in refs.items():
            compare(got[f"{prefix}-{name}"], ref, dtype, f"trace_run {dtype} {prefix}-{name}", "B", name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_sequences_window_edges_and_long_decoding(tmp_path_factory, dtype):
    """Wide layers with loud keys over 700 tokens, windows of 100 and 64 that end inside pages: a prompt in one
    step, one in portions that end inside pages and windows, and the last 200 tokens decoded one by one (in bf16
    from recorded graphs), so that both windows pass wholly over decoded tokens."""
    folder = tiny_rufedra.write_model(tmp_path_factory.mktemp("C") / "C", "C", loud=True)
    weights, cfg = PR.load_weights(folder), PR.read_config(folder)
    ids = tt.make_sequences(cfg["vocab"], [700], seed=77)["r0"]
    want = PR.forward(weights, cfg, ids)
    runner = make_runner(folder, dtype, 1024)
    runner.add_request("whole")
    got = runner.step([("whole", ids, list(range(len(ids))))]).float().cpu().numpy()
    runner.release("whole")
    tt.compare(got, want, dtype, "whole")
    runner.add_request("cut")
    rows, at = [], 0
    for size in (63, 2, 36, 99, 1, 100, 130, 69):
        rows.append(runner.step([("cut", ids[at:at + size], list(range(size)))]).float().cpu().numpy())
        at += size
    while at < len(ids):
        rows.append(runner.step([("cut", ids[at:at + 1], [0])]).float().cpu().numpy().copy())
        at += 1
    runner.release("cut")
    tt.compare(np.concatenate(rows), want, dtype, "portions, then token by token")
    if dtype == "bfloat16":
        assert runner.graph_replays > 100


def test_a_key_just_inside_and_just_outside_the_window_shows(rufedra_dirs):
    """The loud model's logits move when the token at the window's far edge changes, and do not when the token
    one further back does, once no state carries it: checked on the plain implementation's attention and on the
    engine's, which must agree on which of the two matters."""
    folder = rufedra_dirs["A-loud"]
    weights, cfg = PR.load_weights(folder), PR.read_config(folder)
    m = cfg["layers"][0]["mixer"]["left"]
    window = m["mask"]["size"]
    g = torch.Generator().manual_seed(4)
    T = window + 6
    h = torch.randn(T, cfg["width"], generator=g, dtype=PR.F)
    base = PR.window_attention_mixer(h, weights, "l0.mix.left.", m, cfg["norm"]["eps"])
    for back, moves in ((window - 1, True), (window, False)):
        changed = h.clone()
        changed[T - 1 - back] += 3.0
        out = PR.window_attention_mixer(changed, weights, "l0.mix.left.", m, cfg["norm"]["eps"])
        assert bool((out[-1] - base[-1]).abs().max() > 1e-9) == moves


# --------------------------------------------------------------------------
# through the engine: scheduler, batching, sampling
# --------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(rufedra_dirs, name, dtype):
    """Five prompts for two places, prompts in portions of five tokens, a pool of two requests' worth: requests
    wait, pages and slots change hands.  Every token is the plain model's choice (in bf16: within the
    tolerance of its largest logit)."""
    import rvllm_amd

    folder = rufedra_dirs[name]
    weights, cfg = PR.load_weights(folder), PR.read_config(folder)
    prompts = [[3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5], [27, 18, 28], [7], [11, 12, 13, 14, 15, 16, 17], [90, 2]]
    outs = rvllm_amd.generate(str(folder), prompts, max_tokens=12, dtype=dtype, max_model_len=64, max_num_seqs=2,
                              max_num_batched_tokens=16, max_prefill_chunk=5, max_cache_tokens=128)
    for prompt, out in zip(prompts, outs):
        assert len(out) == 12
        if dtype == "float32":
            assert out == PR.greedy(weights, cfg, prompt, 12)
        else:
            logits = PR.forward(weights, cfg, prompt + out)
            scale = float(logits.abs().max())
            for j, token in enumerate(out):
                row = logits[len(prompt) - 1 + j]
                assert row[token] >= row.max() - 2 * tt.TOLERANCE[dtype] * scale, f"token {j} of {prompt}"


def test_sampled_generation_runs_and_is_repeatable(rufedra_dirs):
    import rvllm_amd

    kw = dict(max_tokens=10, temperature=0.8, top_k=20, top_p=0.9, seed=4, dtype="bfloat16", max_model_len=64,
              max_num_seqs=3)
    prompts = [[1, 2, 3], [50, 60], [9, 9, 9, 9]]
    first = rvllm_amd.generate(str(rufedra_dirs["A"]), prompts, **kw)
    assert first == rvllm_amd.generate(str(rufedra_dirs["A"]), prompts, **kw)
    assert all(len(out) == 10 and all(0 <= t < 211 for t in out) for out in first)
