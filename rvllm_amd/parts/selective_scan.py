"""The selective scan (a diagonal state-space mixer with input-dependent steps).

W_in h = [x | z], ``inner`` channels each.  x passes a short causal convolution over time for every channel
(``conv`` taps, with a bias) and silu.  W_x x = [dt | B | C] with ``dt_rank``, ``state`` and ``state`` numbers;
step = softplus(W_dt dt + dt_bias), one a channel; A = -exp(A_log) [inner, state].  For the tokens of a request in
their order, channel c and state n:

    S[c, n] <- exp(step_c A[c, n]) S[c, n] + step_c x_c B_n;    y_c = sum_n S[c, n] C_n + D_c x_c

then y * silu(z) and W_o.  S starts at zero.  What a request keeps between steps is one float32 slot: the last
``conv - 1`` inputs of the convolution and S.  S, the steps, the decays and their exponentials are 32-bit whatever
the activations' type.

Parameters: ``inner``, ``state``, ``dt_rank``, ``conv``, and ``names``: role (``in``, ``conv``, ``conv_bias``,
``x``, ``dt``, ``dt_bias``, ``A_log``, ``D``, ``o``) -> the tensor's whole name under the layer's prefix.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, ParamSpec, StateNeed, StateView
from .linear import decode_weight, linear, linear_unrounded, tensor_names
from .registry import MIXERS
from .spec import PartSpec


class SelectiveScan(Mixer):
    NAMES = {"in": "mix.in", "conv": "mix.conv", "conv_bias": "mix.conv.b", "x": "mix.x", "dt": "mix.dt",
             "dt_bias": "mix.dt.b", "A_log": "mix.A_log", "D": "mix.D", "o": "mix.o"}

    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.inner = int(spec["inner"])
        self.n_state = int(spec["state"])
        self.dt_rank = int(spec["dt_rank"])
        self.taps = int(spec["conv"])
        if min(self.inner, self.n_state, self.dt_rank, self.taps) < 1:
            raise ValueError("a selective scan needs positive sizes")
        self.names = tensor_names(self.NAMES, spec.get("names"))
        self.s_off = (self.taps - 1) * self.inner
        self.state_size = self.s_off + self.inner * self.n_state
        self.w_in = self.w_x = self.w_dt = self.w_o = None
        self.conv_w = self.conv_b = self.dt_b = self.A_log = self.D = None

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        H, I, N, R = self.hidden_size, self.inner, self.n_state, self.dt_rank
        return [
            ParamSpec(at["in"], (2 * I, H)),
            ParamSpec(at["conv"], (I, self.taps), init=("normal", 0.5)),
            ParamSpec(at["conv_bias"], (I,), init=("normal", 0.1)),
            ParamSpec(at["x"], (R + 2 * N, I)),
            ParamSpec(at["dt"], (I, R), init=("normal", 0.1)),
            ParamSpec(at["dt_bias"], (I,), init=("normal", 0.5)),
            ParamSpec(at["A_log"], (I, N), init=("normal", 0.5)),
            ParamSpec(at["D"], (I,), init=("normal_about", 1.0, 0.1)),
            ParamSpec(at["o"], (H, I)),
        ]

    def bind(self, tensors, prefix, device, dtype) -> None:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}

        def get(role, to=dtype):
            return tensors[at[role]].to(device=device, dtype=to).contiguous()

        self.w_in = decode_weight(get("in"), self.tiled_weights)
        self.w_x = decode_weight(get("x"), self.tiled_weights)
        self.w_dt = decode_weight(get("dt"), self.tiled_weights)
        self.w_o = decode_weight(get("o"), self.tiled_weights)
        f32 = torch.float32
        self.conv_w, self.conv_b = get("conv", f32), get("conv_bias", f32)
        self.dt_b, self.A_log, self.D = get("dt_bias", f32), get("A_log", f32), get("D", f32)

    def cache_need(self) -> StateNeed:
        return StateNeed((self.state_size,), torch.float32)

    def forward(self, x: torch.Tensor, step, cache: StateView) -> torch.Tensor:
        if not cache.writes:
            raise ValueError("a selective-scan layer moves its state on with every token and cannot read another's")
        n = x.shape[0]
        slots = cache.slots
        I, N, R = self.inner, self.n_state, self.dt_rank
        proj = linear(x, self.w_in)  # [n, x | z]
        xc = torch.empty((n, I), dtype=x.dtype, device=x.device)
        moves = ops.conv_moves_state(step)  # single tokens: the convolution moves its state on itself
        ops.causal_conv(proj, 0, I, self.conv_w, self.conv_b, slots, 0, step, xc, move_state=moves)
        if not moves:
            ops.conv_state_update(proj, 0, I, self.taps, slots, 0, step)
        dbc = linear(xc, self.w_x)  # [n, dt | B | C]
        dt = linear(dbc[:, :R], self.w_dt)
        y = ops.selective_scan(xc, proj, I, dt, self.dt_b, dbc, R, R + N, self.A_log, self.D, slots, self.s_off, step)
        return linear_unrounded(y, self.w_o)


MIXERS.register("selective_scan", SelectiveScan)
