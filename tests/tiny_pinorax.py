"""Small Pinorax configurations for the tests.  They differ from one another in every size and constant, and use
what a given checkpoint may happen to make equal or 1: several experts a token, a score scale that is not
dim^-1/2, a multiplier of 1, layers without a feed-forward or without a shared expert, no soft-cap.

P  four layers, every layer its own head sizes: experts (2 of 5, shared), dense, none, experts (3 of 3, no shared);
   ranks that are multiples of 16, so bf16 attention runs on the matrix cores
Q  widths that are no multiple of 8, a rank of 40 and 17 heads: bf16 takes the kernels for any size
R  layers wide enough for long sequences: far keys, page borders; 20 heads in a layer (two groups over one cached head)
"""

from __future__ import annotations

import json
from pathlib import Path

import torch


def _mixer(heads, dim, vdim, kv_rank, scale):
    return {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale}


def _moe(experts, top, ff, limit, shared=None):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top},
            "shared": shared}


def _layer(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


CONFIG_P = {
    "architecture": "Pinorax", "vocab": 211, "width": 64, "max_positions": 640, "norm": {"eps": 1e-5},
    "residual_mult": 0.7, "logit_softcap": 12.0,
    "layers": [
        _layer(_mixer(4, 16, 24, 32, 0.3), _moe(5, 2, 24, 0.9, {"ff": 40, "limit": 1.3})),
        _layer(_mixer(3, 8, 8, 48, 0.2), {"kind": "dense", "ff": 72}),
        _layer(_mixer(2, 32, 16, 16, 0.11), None),
        _layer(_mixer(8, 8, 16, 64, 0.5), _moe(3, 3, 16, 2.0, None)),
    ],
}

CONFIG_Q = {
    "architecture": "Pinorax", "vocab": 97, "width": 100, "max_positions": 300, "norm": {"eps": 1e-6},
    "residual_mult": 1.0, "logit_softcap": None,
    "layers": [
        _layer(_mixer(17, 6, 10, 40, 0.4), {"kind": "dense", "ff": 50}),
        _layer(_mixer(1, 20, 12, 24, 0.25), _moe(7, 1, 30, 1.1, {"ff": 18, "limit": 0.5})),
        _layer(_mixer(5, 12, 4, 272, 0.3), _moe(2, 2, 44, 3.0, None)),
    ],
}

CONFIG_R = {
    "architecture": "Pinorax", "vocab": 1500, "width": 256, "max_positions": 2304, "norm": {"eps": 1e-6},
    "residual_mult": 0.4, "logit_softcap": 20.0,
    "layers": [
        _layer(_mixer(8, 32, 32, 128, 0.2), _moe(16, 2, 64, 1.5, {"ff": 64, "limit": 1.0})),
        _layer(_mixer(20, 16, 24, 64, 0.15), {"kind": "dense", "ff": 320}),
    ],
}

CONFIGS = {"P": (CONFIG_P, 11), "Q": (CONFIG_Q, 12), "R": (CONFIG_R, 13)}


def write_model(folder, name: str, seed=None, loud: bool = False) -> Path:
    """Writes configuration ``name`` with random weights through the framework's random-weights mode, then
    rescales them so that every part matters: a matrix keeps its input's size (rows of variance 1 / inputs),
    embeddings and biases are of order one, so that the residual stream, both branches and the logits are all
    of order one and a part that is wrong shows in the logits.  ``loud``: the key projections are scaled up so
    that scores spread over tens of units (a softmax then hangs on single keys, far ones included, and on its
    sink), and the sinks are moved to where they take a visible share."""
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
        if not t.is_floating_point():
            continue
        x = t.float()
        if key in ("embed", "pos"):
            x = x * 40.0
        elif key.endswith(".b"):
            x = x * 20.0
        elif x.dim() == 2 and not key.endswith((".mix.uk", ".mix.uv")):
            x = x * (50.0 / x.shape[1] ** 0.5)
        elif key.endswith((".mix.uk", ".mix.uv")):  # written with a deviation of 0.1
            x = x * (10.0 / x.shape[1] ** 0.5) * (6.0 if loud and key.endswith("uk") else 1.0)
        elif key.endswith(".mix.sink") and loud:
            x = x * 2.0 + 3.0
        tensors[key] = x.to(torch.bfloat16)
    write_safetensors(out / "model.safetensors", tensors, metadata={"format": "pt"})
    return out
