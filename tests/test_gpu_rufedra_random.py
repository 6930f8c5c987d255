"""Rufedra configurations drawn at random against the plain implementation: 1-6 layers of either kind in any order,
with a feed-forward or none; delta rule with 1-8 heads over 1-8 key heads, key sizes 4-160, value sizes 4-96, 1-5 taps;
attention with 1-16 query heads a key/value head, head sizes 8-272 (multiples of 16 or not), windows of 1-150,
rotations of none, a part or all of a head, any base; scans of 8-200 channels with 1-70 states, ranks 1-24, 1-5 taps;
any multipliers, scales and eps; sequences of 1-260 tokens under the four cuttings, pages of 16 / 32 / 64, both dtypes.
Either dtype is held to the larger of its flat share of the largest logit and three times the error that rounding
alone causes at the position (``plain_rufedra.rounding_error``, measured with bf16's roundings; a 32-bit engine rounds
65 536 times finer but at every operation, counted as twice as often): a model drawn at random has positions, early
in a sequence above all, where a delta head's read-out all but cancels and the norm behind it blows the remainder up.  A few seeds are committed; ``draw`` serves a longer run
by hand."""

import json
import random

import numpy as np
import pytest
import torch

import plain_rufedra as PR
import tiny_rufedra
import trace_tools as tt
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu


def draw(seed: int) -> dict:
    rng = random.Random(seed)
    eights = rng.random() < 0.6  # sizes the matrix-core kernels take, or any

    def size(lo, hi):
        return rng.randrange(lo, hi + 1, 8) if eights else rng.randint(lo, hi)

    def mlp():
        return rng.choice([None, {"kind": "dense", "ff": size(8, 200)}])

    layers = []
    for _ in range(rng.randint(1, 6)):
        if rng.random() < 0.5:
            kv_heads = rng.choice([1, 1, 2, 3, 4, 8])
            heads = kv_heads * rng.choice([1, 1, 2, 4]) if kv_heads < 8 else 8
            layers.append({"type": "delta", "mlp": mlp(), "mixer": {
                "heads": heads, "kv_heads": kv_heads, "dim": size(8, 160) if eights else rng.randint(4, 160),
                "vdim": size(8, 96) if eights else rng.randint(4, 96), "conv": rng.randint(1, 5)}})
        else:
            kv_heads = rng.choice([1, 1, 2, 3, 4])
            heads = kv_heads * rng.choice([1, 2, 4, 8, 16, 17] if kv_heads == 1 else [1, 2, 4])
            dim = rng.choice([16, 32, 48, 64, 96, 128, 256]) if rng.random() < 0.6 else 2 * rng.randint(4, 136)
            dims = rng.choice([0, dim, 2 * rng.randint(1, dim // 2)])
            left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": rng.uniform(0.02, 0.4),
                    "mask": {"size": rng.choice([1, 2, 15, 16, 17, 33, rng.randint(3, 150)])},
                    "rot": {"dims": dims, "base": rng.choice([37.5, 10000.0, 1000000.0])}}
            right = {"inner": size(8, 200), "state": rng.choice([1, 4, 16, 16, 24, 33, 64, 70]),
                     "dt_rank": rng.choice([1, 3, 8, 16, 24]), "conv": rng.randint(1, 5)}
            layers.append({"type": "parallel", "mlp": mlp(), "mixer": {
                "left": left, "right": right, "left_scale": rng.choice([1.0, rng.uniform(-1.5, 1.5)]),
                "right_scale": rng.choice([1.0, rng.uniform(0.2, 1.5)])}})
    return {"architecture": "Rufedra", "vocab": rng.randint(5, 700), "width": size(16, 160),
            "embedding": {"scale": rng.choice([1.0, rng.uniform(0.5, 12.0)])},
            "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "logit_scale": rng.choice([1.0, rng.uniform(0.3, 3.0)]),
            "layers": layers}


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8])
def test_a_configuration_drawn_at_random(tmp_path, seed):
    doc = draw(seed)
    tiny_rufedra.CONFIGS["random"] = (doc, seed)
    try:
        folder = tiny_rufedra.write_model(tmp_path / "m", "random", loud=seed % 2 == 0)
    finally:
        del tiny_rufedra.CONFIGS["random"]
    weights, cfg = PR.load_weights(folder), PR.read_config(folder)
    rng = random.Random(seed + 1000)
    lengths = [rng.choice([1, 2, 15, 16, 17, 33]), rng.randint(3, 120), rng.randint(100, 260)]
    seqs = tt.make_sequences(cfg["vocab"], lengths, seed=seed)
    refs = {rid: PR.forward(weights, cfg, ids) for rid, ids in seqs.items()}
    rounding = {rid: PR.rounding_error(weights, cfg, ids, refs[rid]).numpy() for rid, ids in seqs.items()}
    page_size = rng.choice([16, 32, 64])
    for dtype in ("float32", "bfloat16"):
        for mode, make in (("whole", tt.trace_whole), ("tail", tt.trace_tail), ("portions", tt.trace_portions),
                           ("mixed", tt.trace_mixed)):
            steps = make(seqs, seed=seed) if mode in ("portions", "mixed") else make(seqs)
            most = max(tt.required_tokens(steps), page_size)
            runner = ModelRunner.from_model_dir(folder, EngineConfig(
                dtype=dtype, page_size=page_size, max_model_len=most, max_num_seqs=4, max_num_batched_tokens=most,
                max_prefill_chunk=most, max_cache_tokens=most))
            got = tt.collect(steps, tt.run_in_process(runner, steps), cfg["vocab"])
            prefix = steps[0]["entries"][0]["id"].split("-")[0]
            for name, ref in refs.items():
                what = f"seed {seed} {dtype} {mode} {name}: {json.dumps(doc)}"
                arr = np.asarray(got[f"{prefix}-{name}"], dtype=np.float64)
                assert arr.shape == tuple(ref.shape) and np.isfinite(arr).all(), what
                err = np.abs(arr - ref.numpy()).max(-1)
                finer = 1.0 if dtype == "bfloat16" else 2.0 ** -15
                allowed = np.maximum(tt.TOLERANCE[dtype] * float(ref.abs().max()), 3.0 * finer * rounding[name])
                worst = int((err / allowed).argmax())
                assert err[worst] <= allowed[worst], f"position {worst}: {err[worst]:.3e} > {allowed[worst]:.3e}; {what}"
