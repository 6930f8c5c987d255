"""Pinorax configurations drawn at random against the plain implementation: 1-5 layers in any order of
feed-forwards (none, dense, experts with or without a shared one), 1-40 heads, head sizes 1-72, ranks 8-288 (multiples
of 16 or not), widths and inner sizes that are multiples of 8 or not, 1-9 experts with 1-3 choices, any multiplier,
scale, eps, limits, soft-cap or none; sequences of 1-300 tokens under the four cuttings, pages of 16 / 32 / 64, both
dtypes.  A few seeds are committed; ``draw`` serves a longer run by hand."""

import json
import random

import numpy as np
import pytest
import torch

import plain_pinorax as PP
import tiny_pinorax
import trace_tools as tt
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu


def draw(seed: int) -> dict:
    rng = random.Random(seed)
    eights = rng.random() < 0.6  # sizes the matrix-core kernels take, or any

    def size(lo, hi):
        return rng.randrange(lo, hi + 1, 8) if eights else rng.randint(lo, hi)

    width = size(16, 160)
    layers = []
    for _ in range(rng.randint(1, 5)):
        heads = rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 17, 20, 32, 40])
        rank = rng.choice([16, 32, 48, 64, 96, 128]) if rng.random() < 0.7 else rng.randint(8, 288)
        mixer = {"heads": heads, "dim": size(8, 72) if eights else rng.randint(1, 72), "vdim": size(8, 48) if eights else
                 rng.randint(1, 48), "kv_rank": rank, "scale": rng.uniform(0.05, 0.5)}
        kind = rng.choice(["none", "dense", "moe", "moe", "moe-noshared"])
        if kind == "none":
            mlp = None
        elif kind == "dense":
            mlp = {"kind": "dense", "ff": size(8, 200)}
        else:
            experts = rng.randint(1, 9)
            mlp = {"kind": "moe", "expert": {"ff": size(8, 96), "limit": rng.uniform(0.3, 4.0)},
                   "router": {"experts": experts, "top": rng.randint(1, min(3, experts))},
                   "shared": None if kind == "moe-noshared" else {"ff": size(8, 96), "limit": rng.uniform(0.3, 4.0)}}
        layers.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
    return {"architecture": "Pinorax", "vocab": rng.randint(5, 700), "width": width, "max_positions": 320,
            "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "residual_mult": rng.uniform(0.2, 1.5),
            "logit_softcap": rng.choice([None, rng.uniform(3.0, 40.0)]), "layers": layers}


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8])
def test_a_configuration_drawn_at_random(tmp_path, seed):
    doc = draw(seed)
    tiny_pinorax.CONFIGS["random"] = (doc, seed)
    try:
        folder = tiny_pinorax.write_model(tmp_path / "m", "random", loud=seed % 2 == 0)
    finally:
        del tiny_pinorax.CONFIGS["random"]
    weights, cfg = PP.load_weights(folder), PP.read_config(folder)
    rng = random.Random(seed + 1000)
    lengths = [rng.choice([1, 2, 15, 16, 17, 33]), rng.randint(3, 120), rng.randint(100, 300)]
    seqs = tt.make_sequences(cfg["vocab"], lengths, seed=seed)
    refs = {rid: PP.forward(weights, cfg, ids) for rid, ids in seqs.items()}
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
                tt.compare(got[f"{prefix}-{name}"], ref, dtype, f"seed {seed} {dtype} {mode} {name}: {json.dumps(doc)}")
