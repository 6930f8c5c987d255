"""Small Rufedra configurations for the tests.  They differ from one another in every size and constant, and use
what a given checkpoint may happen to make equal or 1.

A  five layers, parallel first: delta layers with and without a feed-forward, 3 and 2 taps; attention heads of 32
   (the matrix-core kernels in bf16) with a window of 21, a rotation of 16 of 32 dimensions; 6 states
B  widths that are no multiple of 8, attention heads of 20 with the whole head rotated, one key/value head a query
   head, a window of 1 (a token sees itself only) and one of 7, delta with kv_heads = heads and dim != vdim,
   a convolution of one tap (no state) and one of five, a dt_rank of 3, 33 states, scales that are negative or 1
C  layers wide enough for long sequences: windows of 100 and 64 that end inside pages, no rotation in one layer
"""

from __future__ import annotations

import json
from pathlib import Path

import torch


def _delta(heads, kv_heads, dim, vdim, conv, mlp=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": mlp}


def _parallel(left, right, left_scale, right_scale, mlp=None):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def _left(heads, kv_heads, dim, scale, window, dims, base):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "mask": {"size": window},
            "rot": {"dims": dims, "base": base}}


def _right(inner, state, dt_rank, conv):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


CONFIG_A = {
    "architecture": "Rufedra", "vocab": 211, "width": 64, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5},
    "logit_scale": 0.5,
    "layers": [
        _parallel(_left(4, 2, 32, 0.2, 21, 16, 10000.0), _right(48, 6, 4, 3), 0.7, 1.3, _dense(96)),
        _delta(4, 2, 16, 24, 3),
        _delta(2, 1, 24, 8, 2, _dense(40)),
        _parallel(_left(6, 1, 16, 0.3, 5, 16, 500.0), _right(80, 16, 8, 4), 1.1, 0.6),
        _delta(3, 3, 8, 16, 4),
    ],
}

CONFIG_B = {
    "architecture": "Rufedra", "vocab": 97, "width": 100, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
    "logit_scale": 1.0,
    "layers": [
        _delta(5, 5, 12, 20, 1, _dense(50)),
        _parallel(_left(3, 3, 20, 0.25, 1, 20, 100.0), _right(36, 33, 3, 5), -0.8, 1.0, _dense(44)),
        _parallel(_left(5, 1, 12, 0.4, 7, 6, 37.5), _right(50, 1, 5, 1), 1.0, 0.45),
        _delta(1, 1, 40, 36, 5),
    ],
}

CONFIG_C = {
    "architecture": "Rufedra", "vocab": 1500, "width": 256, "embedding": {"scale": 16.0}, "norm": {"eps": 1e-6},
    "logit_scale": 1.5,
    "layers": [
        _delta(4, 2, 64, 64, 4),
        _parallel(_left(8, 2, 64, 0.125, 100, 32, 1000000.0), _right(384, 16, 16, 4), 1.2, 0.9, _dense(320)),
        _parallel(_left(4, 4, 48, 0.15, 64, 0, 10000.0), _right(256, 8, 8, 2), 0.8, 1.0),
        _delta(8, 1, 32, 48, 3, _dense(256)),
    ],
}

CONFIGS = {"A": (CONFIG_A, 21), "B": (CONFIG_B, 22), "C": (CONFIG_C, 23)}


def write_model(folder, name: str, seed=None, loud: bool = False) -> Path:
    """Writes configuration ``name`` with random weights through the framework's random-weights mode, then rescales
    them so that every part matters: a matrix keeps its input's size (rows of variance 1 / inputs), the embedding
    is of order one, norm weights and layer scales lie about one.
    ``loud``: queries and keys of the attention are scaled up so that a softmax hangs on single keys, so that a
    key just inside or just outside a window shows in the logits."""
    from safetensors.torch import load_file

    from rvllm_amd.models.registry import architecture_of
    from rvllm_amd.weights.random_init import write_random_model
    from rvllm_amd.weights.safetensors_io import write_safetensors

    doc, default_seed = CONFIGS[name]
    config = architecture_of(doc).read_config(doc, f"tiny config {name}")
    out = write_random_model(Path(folder), config, default_seed if seed is None else seed, torch.bfloat16)
    (out / "config.json").write_text(json.dumps(doc, indent=2))
    tensors = load_file(str(out / "model.safetensors"))
    for key, t in list(tensors.items()):
        x = t.float()
        last = key.split(".")[-1]
        if key == "embed":
            x = x * 50.0
        elif ".norm" in key and x.dim() == 1 and not key.endswith("mix.norm"):
            x = 1.0 + x * 2.0  # written with a deviation of 0.1
        elif key.endswith((".q.b", ".k.b")):
            x = x * 25.0
        elif x.dim() == 2 and last not in ("conv", "A_log"):
            x = x * (50.0 / x.shape[1] ** 0.5)
            if loud and key.endswith((".left.q", ".left.k")):
                x = x * 3.0
        elif key.endswith(".mix.dt_bias"):
            # decays between a half and one, as trained models of this kind have them: a head whose decay wipes its
            # matrix reads out little but its own token's write, which can all but cancel, and the norm that follows
            # would blow that remainder up to size one, in any arithmetic
            x = x - 2.0
        tensors[key] = x.to(torch.bfloat16)
    write_safetensors(out / "model.safetensors", tensors, metadata={"format": "pt"})
    return out
