"""A plain, slow implementation of the Pinorax decoder: whole sequences, no cache, one function per mechanism,
plain PyTorch operations on the CPU.  It shares no code with the engine and does not follow its order of work:
keys and values are made for every head from the compressed vector, scores are taken key by key, and experts run
one token at a time.  The tests compare the engine with it.

Notation: T tokens, W the model's width, H heads, D a head's query/key size, V its value size, R the rank of the
compressed vector, E experts, F an expert's inner size.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def read_config(model_dir) -> dict:
    return json.loads((Path(model_dir) / "config.json").read_text())


def load_weights(model_dir) -> dict:
    """All tensors of model.safetensors, by name, through the safetensors package (not the engine's reader)."""
    from safetensors.torch import load_file

    return load_file(str(Path(model_dir) / "model.safetensors"))


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last dimension, eps under the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """One gain for all coordinates."""
    return unit_rms(x, eps) * gain.reshape(())


def embed(tokens, table: torch.Tensor, positions: torch.Tensor, first_position: int = 0) -> torch.Tensor:
    """The token's vector plus the vector of its position; positions count from 0."""
    ids = torch.as_tensor(tokens, dtype=torch.long)
    where = torch.arange(first_position, first_position + len(ids))
    return table[ids] + positions[where]


def softmax_with_sink(scores: torch.Tensor, sink) -> torch.Tensor:
    """Weights of the visible keys (last dimension) when the denominator holds one more term exp(sink); masked keys
    are -inf.  ``sink`` None: the ordinary softmax."""
    top = scores.max(dim=-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, torch.as_tensor(sink, dtype=scores.dtype).expand_as(top))
    e = torch.exp(scores - top)
    total = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(torch.as_tensor(sink, dtype=scores.dtype) - top)
    return e / total


def latent_attention(h: torch.Tensor, w: dict, p: str, sizes: dict, eps: float) -> torch.Tensor:
    """h [T, W] -> [T, W].  c_j = norm(W_dkv h_j) * g is all that later tokens need of token j; head a's key and
    value of token j are rows a D .. a D + D of W_uk c_j and rows a V .. a V + V of W_uv c_j."""
    T = h.shape[0]
    H, D, V = sizes["heads"], sizes["dim"], sizes["vdim"]
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    c = unit_rms(h @ w[p + "dkv"].T, eps) * w[p + "dkv.norm"]
    k = (c @ w[p + "uk"].T).reshape(T, H, D)
    v = (c @ w[p + "uv"].T).reshape(T, H, V)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for a in range(H):
        for i in range(T):  # token i sees j <= i
            s = (k[: i + 1, a] @ q[i, a]) * sizes["scale"]
            out[i, a] = softmax_with_sink(s, w[p + "sink"][a]) @ v[: i + 1, a]
    gate = torch.sigmoid(h @ w[p + "g"].T)
    return (out.reshape(T, H * V) * gate) @ w[p + "o"].T


def dense_ff(h: torch.Tensor, w: dict, p: str) -> torch.Tensor:
    gate = h @ w[p + "gate"].T + w[p + "gate.b"]
    up = h @ w[p + "up"].T + w[p + "up.b"]
    return (gate * torch.sigmoid(gate) * up) @ w[p + "down"].T + w[p + "down.b"]


def expert(h: torch.Tensor, w: dict, p: str, limit: float) -> torch.Tensor:
    """Gate capped from above, up clamped on both sides; no biases."""
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def routed_ff(h: torch.Tensor, tokens, w: dict, p: str, mlp: dict) -> torch.Tensor:
    """The experts of a token are the entries of its id's row of the table, each weighing 1 / top."""
    top = mlp["router"]["top"]
    table = w[p + "table"]
    out = torch.zeros_like(h)
    for t, token in enumerate(tokens):
        for e in table[int(token)].tolist():
            out[t] += expert(h[t], w, f"{p}e{int(e)}.", mlp["expert"]["limit"]) / top
    if mlp.get("shared") is not None:
        out = out + expert(h, w, p + "shared.", mlp["shared"]["limit"])
    return out


def depth_average(streams: list, weights: torch.Tensor) -> torch.Tensor:
    assert len(streams) == weights.numel()
    return sum(weights[j] * streams[j] for j in range(len(streams)))


def softcap(logits: torch.Tensor, cap) -> torch.Tensor:
    return logits if cap is None else cap * torch.tanh(logits / cap)


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
def forward(weights: dict, cfg: dict, tokens, dtype=torch.float64, streams_out=None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence.  ``streams_out``: a list that receives what leaves every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = embed(tokens, w["embed"], w["pos"])
    results = [x]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = scalar_norm(x, w[p + "norm1"], eps)
        assert layer["type"] == "latent_attention"
        both = latent_attention(h, w, p + "mix.", layer["mixer"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            both = both + (dense_ff(h, w, p + "mlp.") if mlp["kind"] == "dense"
                           else routed_ff(h, tokens, w, p + "mlp.", mlp))
        results.append(x + mult * both)
        x = depth_average(results, w[p + "dwa"])
        if streams_out is not None:
            streams_out.append(x)
    return softcap(scalar_norm(x, w["final.norm"], eps) @ w["head"].T, cfg.get("logit_softcap"))


def pick_greedy(row: torch.Tensor) -> int:
    """The lowest id among the largest logits."""
    return int((row == row.max()).nonzero()[0])


def greedy(weights: dict, cfg: dict, prompt, steps: int, dtype=torch.float64) -> list[int]:
    ids, out = list(prompt), []
    for _ in range(steps):
        out.append(pick_greedy(forward(weights, cfg, ids, dtype)[-1]))
        ids.append(out[-1])
    return out
