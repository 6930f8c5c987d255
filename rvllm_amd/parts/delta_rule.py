"""The gated delta rule: a mixer that keeps a matrix a head instead of keys and values.

For the tokens of a request in their order, head h with key head g = h // (heads / kv_heads):

    S <- decay * S;   u = beta * (v - S^T k);   S <- S + k u^T;   o = S^T q

with S [dim, vdim] starting at zero, so the read-out sees the token's own write.  q, k (``kv_heads`` heads of
``dim``) and v (``heads`` heads of ``vdim``) are projections of the layer's input that pass a short causal
convolution over time for every channel (``conv`` taps, no bias) and silu; q and k are then scaled to unit length
per head, x / sqrt(sum x^2 + unit_eps), and q also by dim^(-1/2).  beta = sigmoid(W_b h) and
decay = exp(-exp(A_log) * softplus(W_a h + dt_bias)), one each a head.  Every head's o is RMS-normed over vdim
with a weight that the heads share, multiplied by silu(W_g h) and projected by W_o.

What a request keeps between steps is one float32 slot: the last ``conv - 1`` inputs of the convolutions' channels
and S of every head.  S, decay, beta, the unit norms and the output norm are 32-bit whatever the activations' type.

Parameters: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv``, ``eps`` (the output norm's), ``unit_eps``, and
``names``: role (``q``, ``k``, ``v``, ``q_conv``, ``k_conv``, ``v_conv``, ``b``, ``a``, ``A_log``, ``dt_bias``,
``norm``, ``g``, ``o``) -> the tensor's whole name under the layer's prefix.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, ParamSpec, StateNeed, StateView
from .linear import decode_weight, linear, linear_unrounded, tensor_names
from .registry import MIXERS
from .spec import PartSpec


class GatedDeltaRule(Mixer):
    NAMES = {"q": "mix.q", "k": "mix.k", "v": "mix.v", "q_conv": "mix.q.conv", "k_conv": "mix.k.conv",
             "v_conv": "mix.v.conv", "b": "mix.b", "a": "mix.a", "A_log": "mix.A_log", "dt_bias": "mix.dt_bias",
             "norm": "mix.norm", "g": "mix.g", "o": "mix.o"}

    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.heads = int(spec["heads"])
        self.kv_heads = int(spec["kv_heads"])
        self.dim = int(spec["dim"])
        self.vdim = int(spec["vdim"])
        self.taps = int(spec["conv"])
        self.eps = float(spec["eps"])
        self.unit_eps = float(spec.get("unit_eps", 1e-6))
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads cannot share {self.kv_heads} query/key heads")
        if self.taps < 1:
            raise ValueError("a convolution needs at least one tap")
        self.names = tensor_names(self.NAMES, spec.get("names"))
        self.qk_size = self.kv_heads * self.dim
        self.v_size = self.heads * self.vdim
        # columns of the fused projection: q | k | v | g | b | a
        self.conv_channels = 2 * self.qk_size + self.v_size
        self.g_col = self.conv_channels
        self.b_col = self.g_col + self.v_size
        self.a_col = self.b_col + self.heads
        # the slot: the convolutions' last inputs [conv - 1, channels], then S [heads, dim, vdim]
        self.s_off = (self.taps - 1) * self.conv_channels
        self.state_size = self.s_off + self.heads * self.dim * self.vdim
        self.w_in = self.w_o = self.conv_qk = self.conv_v = self.A_log = self.dt_bias = self.norm_w = None

    # ---- weights -----------------------------------------------------
    def param_specs(self, prefix: str) -> list[ParamSpec]:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        H = self.hidden_size
        return [
            ParamSpec(at["q"], (self.qk_size, H)), ParamSpec(at["k"], (self.qk_size, H)),
            ParamSpec(at["v"], (self.v_size, H)),
            ParamSpec(at["q_conv"], (self.qk_size, self.taps), init=("normal", 0.5)),
            ParamSpec(at["k_conv"], (self.qk_size, self.taps), init=("normal", 0.5)),
            ParamSpec(at["v_conv"], (self.v_size, self.taps), init=("normal", 0.5)),
            ParamSpec(at["b"], (self.heads, H)), ParamSpec(at["a"], (self.heads, H)),
            ParamSpec(at["A_log"], (self.heads,), init=("normal", 0.5)),
            ParamSpec(at["dt_bias"], (self.heads,), init=("normal", 0.5)),
            ParamSpec(at["norm"], (self.vdim,), init=("normal_about", 1.0, 0.1)),
            ParamSpec(at["g"], (self.v_size, H)), ParamSpec(at["o"], (H, self.v_size)),
        ]

    def bind(self, tensors, prefix, device, dtype) -> None:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}

        def get(role, to=dtype):
            return tensors[at[role]].to(device=device, dtype=to)

        rows = [get(role) for role in ("q", "k", "v", "g", "b", "a")]
        self.w_in = decode_weight(torch.cat(rows, dim=0).contiguous(), self.tiled_weights)
        self.w_o = decode_weight(get("o").contiguous(), self.tiled_weights)
        f32 = torch.float32  # what enters the recurrence and the convolutions' sums is 32-bit
        self.conv_qk = torch.cat([get("q_conv", f32), get("k_conv", f32)], dim=0).contiguous()
        self.conv_v = get("v_conv", f32).contiguous()
        self.A_log = get("A_log", f32).contiguous()
        self.dt_bias = get("dt_bias", f32).contiguous()
        self.norm_w = get("norm", f32).contiguous()

    # ---- state -------------------------------------------------------
    def cache_need(self) -> StateNeed:
        return StateNeed((self.state_size,), torch.float32)

    # ---- run ---------------------------------------------------------
    def forward(self, x: torch.Tensor, step, cache: StateView) -> torch.Tensor:
        if not cache.writes:
            raise ValueError("a delta-rule layer moves its state on with every token and cannot read another's")
        n = x.shape[0]
        slots = cache.slots
        proj = linear(x, self.w_in)  # [n, q | k | v | g | b | a]
        qk = 2 * self.qk_size
        qkv = torch.empty((n, self.conv_channels), dtype=torch.float32, device=x.device)
        moves = ops.conv_moves_state(step)  # single tokens: the convolutions move their state on themselves
        ops.causal_conv(proj, 0, qk, self.conv_qk, None, slots, 0, step, qkv, 0, group=self.dim,
                        unit_eps=self.unit_eps, scaled_groups=self.kv_heads, group_scale=self.dim ** -0.5,
                        state_ld=self.conv_channels, move_state=moves)
        ops.causal_conv(proj, qk, self.v_size, self.conv_v, None, slots, qk, step, qkv, qk,
                        state_ld=self.conv_channels, move_state=moves)
        if not moves:
            ops.conv_state_update(proj, 0, self.conv_channels, self.taps, slots, 0, step)
        o = ops.delta_rule(qkv, 0, self.qk_size, qk, proj, self.a_col, self.b_col, self.A_log, self.dt_bias, slots,
                           self.s_off, step, self.heads, self.kv_heads, self.dim, self.vdim)
        y = ops.head_norm_gate(o, proj, self.g_col, self.norm_w, self.eps, self.heads, self.vdim, x.dtype)
        return linear_unrounded(y, self.w_o)


MIXERS.register("gated_delta_rule", GatedDeltaRule)
