"""The Rufedra design written plainly: whole sequences, no cache, no state carried between calls, 64-bit, a loop
over tokens wherever the design has a recurrence.  One function a mechanism; the GPU tests hold the engine's
kernels, parts and whole models against these.  Nothing here is shared with the product path.

Notation: T tokens, h the normed input of a sublayer, W a matrix stored [out, in] and applied as h @ W.T.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

F = torch.float64

# What the design allows in 16 bits (the inputs and outputs of matrix products, the short convolutions with their
# activations, gated outputs) passes through ``r``; with ``rounded()`` it is rounded to bfloat16 there and nowhere
# else, so that the difference to the unrounded run is the error that rounding alone causes in this model at every
# position: the yardstick that the bf16 engine is held against.
_ROUND = False


def r(t):
    return t.to(torch.bfloat16).to(F) if _ROUND else t


class rounded:
    def __enter__(self):
        global _ROUND
        _ROUND = True

    def __exit__(self, *exc):
        global _ROUND
        _ROUND = False


def read_config(folder) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def load_weights(folder) -> dict:
    from safetensors.torch import load_file

    return {k: (v.to(F) if v.is_floating_point() else v) for k, v in load_file(str(Path(folder) / "model.safetensors")).items()}


# ---- pieces ------------------------------------------------------------------
def rms_norm(x, eps, weight=None):
    """x / sqrt(mean(x^2) + eps), times the weight if there is one."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(x):
    return x * torch.sigmoid(x)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(x):
    return torch.clamp(x, min=0) + torch.log1p(torch.exp(-x.abs()))


def causal_conv(x, taps_w, bias=None, before=None):
    """y[t, c] = bias[c] + sum_j taps_w[c, j] * x[t - (K - 1) + j, c]; rows before the first are ``before``
    ([K - 1, C], the inputs that came earlier) or zeros."""
    T, C = x.shape
    K = taps_w.shape[1]
    pad = torch.zeros(K - 1, C, dtype=x.dtype) if before is None else before
    xp = torch.cat([pad, x], 0)
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(K):
            y[t] += taps_w[:, j] * xp[t + j]
    return y if bias is None else y + bias


def unit(x, eps):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def delta_recurrence(q, k, v, decay, beta, S=None):
    """One head.  q, k [T, dk], v [T, dv], decay, beta [T].  Returns (o [T, dv], the last S [dk, dv])."""
    T, dk = k.shape
    dv = v.shape[1]
    S = torch.zeros(dk, dv, dtype=F) if S is None else S.clone()
    o = torch.zeros(T, dv, dtype=F)
    for t in range(T):
        S = decay[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o, S


def delta_mixer(h, W, p, m, eps, unit_eps=1e-6):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = r(silu(causal_conv(r(h @ W[p + "q"].T), W[p + "q.conv"]))).view(T, G, dk)
    k = r(silu(causal_conv(r(h @ W[p + "k"].T), W[p + "k.conv"]))).view(T, G, dk)
    v = r(silu(causal_conv(r(h @ W[p + "v"].T), W[p + "v.conv"]))).view(T, H, dv)
    q = unit(q, unit_eps) * dk ** -0.5
    k = unit(k, unit_eps)
    beta = torch.sigmoid(r(h @ W[p + "b"].T))
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * softplus(r(h @ W[p + "a"].T) + W[p + "dt_bias"]))
    o = torch.stack([delta_recurrence(q[:, i // (H // G)], k[:, i // (H // G)], v[:, i], decay[:, i], beta[:, i])[0]
                     for i in range(H)], 1)
    o = r(rms_norm(o, eps, W[p + "norm"]).reshape(T, H * dv) * silu(r(h @ W[p + "g"].T)))
    return o @ W[p + "o"].T


def rotate_halves(x, positions, dims, base):
    """x [T, heads, d]: the first ``dims`` dimensions turn, i with i + dims/2, by position * base^(-2i/dims)."""
    if dims == 0:
        return x
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = positions.to(F)[:, None] * freq
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def window_softmax_attention(q, k, v, scale, window):
    """q [T, H, d], k, v [T, G, d]: position i sees j with 0 <= i - j < window."""
    T, H, _ = q.shape
    G = k.shape[1]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (i - j >= 0) & (i - j < window)
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        out[:, h] = torch.softmax(s, -1) @ v[:, g]
    return out


def window_attention_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = r(h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = r(h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    v = k  # the values are the keys as projected
    pos = torch.arange(T)
    q = r(rms_norm(rotate_halves(q, pos, m["rot"]["dims"], m["rot"]["base"]), eps))
    k = r(rms_norm(rotate_halves(k, pos, m["rot"]["dims"], m["rot"]["base"]), eps))
    out = r(window_softmax_attention(q, k, v, m["scale"], m["mask"]["size"]).reshape(T, H * d))
    return r(out * torch.sigmoid(r(h @ W[p + "g"].T))) @ W[p + "o"].T


def scan_recurrence(x, step, A, B, C, D, S=None):
    """x, step [T, I]; A [I, N]; B, C [T, N]; D [I].  Returns (y [T, I], the last S [I, N])."""
    T, I = x.shape
    S = torch.zeros(I, A.shape[1], dtype=F) if S is None else S.clone()
    y = torch.zeros(T, I, dtype=F)
    for t in range(T):
        S = torch.exp(step[t][:, None] * A) * S + (step[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + D * x[t]
    return y, S


def scan_mixer(h, W, p, m):
    I, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = r(h @ W[p + "in"].T)
    x, z = xz[:, :I], xz[:, I:]
    x = r(silu(causal_conv(x, W[p + "conv"], W[p + "conv.b"])))
    low = r(x @ W[p + "x"].T)
    step = softplus(r(low[:, :R] @ W[p + "dt"].T) + W[p + "dt.b"])
    y, _ = scan_recurrence(x, step, -torch.exp(W[p + "A_log"]), low[:, R:R + N], low[:, R + N:], W[p + "D"])
    return r(y * silu(z)) @ W[p + "o"].T


def feed_forward(h, W, p):
    return r(gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def mixer(h, W, p, layer, eps):
    if layer["type"] == "delta":
        return delta_mixer(h, W, p + "mix.", layer["mixer"], eps)
    m = layer["mixer"]
    return (m["left_scale"] * window_attention_mixer(h, W, p + "mix.left.", m["left"], eps)
            + m["right_scale"] * scan_mixer(h, W, p + "mix.right.", m["right"]))


# ---- the model -----------------------------------------------------------------
def forward(W, cfg, ids, streams=None):
    """Logits [T, vocab] of one sequence; ``streams`` collects the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(ids, dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + rms_norm(mixer(r(rms_norm(x, eps, W[p + "norm1"])), W, p, layer, eps), eps, W[p + "norm1b"]) * W[p + "ls1"]
        if layer["mlp"] is not None:
            f = feed_forward(r(rms_norm(x, eps, W[p + "norm2"])), W, p + "mlp.")
            x = x + rms_norm(f, eps, W[p + "norm2b"]) * W[p + "ls2"]
        if streams is not None:
            streams.append(x.clone())
    return (r(rms_norm(x, eps, W["final.norm"])) @ W["head"].T) * cfg["logit_scale"]


def rounding_error(W, cfg, ids, exact=None):
    """For every position, the largest difference that rounding alone (``rounded``) makes to a logit."""
    exact = forward(W, cfg, ids) if exact is None else exact
    with rounded():
        coarse = forward(W, cfg, ids)
    return (coarse - exact).abs().max(-1).values


def greedy(W, cfg, prompt, count):
    ids = list(prompt)
    for _ in range(count):
        ids.append(int(forward(W, cfg, ids)[-1].argmax()))
    return ids[len(prompt):]
