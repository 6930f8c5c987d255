"""Attention over a compressed key/value vector (latent attention), without positions.

Every token keeps one vector c of ``kv_rank`` numbers, the RMS-normed output
of a down projection; a head's keys and values are up projections of it,
k_h = U_h c and v_h = V_h c.  Only c is cached, as one key/value head of
``kv_rank`` dimensions in the paged cache, and the up projections move to the
query's side of the products:

    score_h(i, j) = scale * q_h(i) . (U_h c_j) = scale * (U_h^T q_h(i)) . c_j
    out_h(i)      = sum_j p_h(i, j) V_h c_j    = V_h (sum_j p_h(i, j) c_j)

so the attention kernels see ``heads`` query heads of ``kv_rank`` dimensions
that share one key/value head whose keys and values are both c.  Order of work
for a step's tokens: one fused projection to q | c_raw | gate, norm of c_raw
and its write into the pages, U_h^T q_h for every head, attention (causal,
with an optional sink in every head's softmax), V_h on the result times
sigmoid(gate), output projection.

Parameters: ``heads``, ``dim`` (a head's query/key size), ``vdim`` (its value
size), ``kv_rank``, ``scale``, ``eps`` of the norm of c, ``sink`` (whether the
heads have one), ``gate`` (whether the output is gated), ``window`` (None:
every earlier token is visible), and ``names``: role (``q``, ``dkv``,
``dkv_norm``, ``uk``, ``uv``, ``sink``, ``g``, ``o``) -> the tensor's whole name
under the layer's prefix.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import KVCacheView, KVNeed, Mixer, ParamSpec
from .linear import decode_weight, linear, tensor_names
from .registry import MIXERS
from .spec import PartSpec


class LatentAttention(Mixer):
    NAMES = {"q": "mix.q", "dkv": "mix.dkv", "dkv_norm": "mix.dkv.norm", "uk": "mix.uk", "uv": "mix.uv",
             "sink": "mix.sink", "g": "mix.g", "o": "mix.o"}

    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.heads = int(spec["heads"])
        self.dim = int(spec["dim"])
        self.vdim = int(spec["vdim"])
        self.kv_rank = int(spec["kv_rank"])
        self.scale = float(spec["scale"])
        self.eps = float(spec["eps"])
        self.has_sink = bool(spec.get("sink", False))
        self.has_gate = bool(spec.get("gate", False))
        window = spec.get("window")
        self.window: Optional[int] = None if window is None else int(window)
        self.names = tensor_names(self.NAMES, spec.get("names"))
        self.q_size = self.heads * self.dim
        self.v_size = self.heads * self.vdim
        self.w_in = self.w_o = self.w_uk_t = self.w_uv = self.c_norm_w = self.sinks = None

    # ---- weights -----------------------------------------------------
    def param_specs(self, prefix: str) -> list[ParamSpec]:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        specs = [
            ParamSpec(at["q"], (self.q_size, self.hidden_size)),
            ParamSpec(at["dkv"], (self.kv_rank, self.hidden_size)),
            ParamSpec(at["dkv_norm"], (self.kv_rank,), init=("normal_about", 1.0, 0.1)),
            ParamSpec(at["uk"], (self.q_size, self.kv_rank), init=("normal", 0.1)),
            ParamSpec(at["uv"], (self.v_size, self.kv_rank), init=("normal", 0.1)),
            ParamSpec(at["o"], (self.hidden_size, self.v_size)),
        ]
        if self.has_sink:
            specs.append(ParamSpec(at["sink"], (self.heads,), init=("normal", 1.0)))
        if self.has_gate:
            specs.append(ParamSpec(at["g"], (self.v_size, self.hidden_size)))
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}

        def get(role):
            return tensors[at[role]].to(device=device, dtype=dtype)

        # queries, the compressed vector and the gate come from one product against their joined rows
        rows = [get("q"), get("dkv")] + ([get("g")] if self.has_gate else [])
        self.w_in = decode_weight(torch.cat(rows, dim=0).contiguous(), self.tiled_weights)
        self.w_o = decode_weight(get("o").contiguous(), self.tiled_weights)
        # U_h^T q_h as a product against rows: head h's matrix [kv_rank, dim] is U_h transposed
        self.w_uk_t = get("uk").reshape(self.heads, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = get("uv").reshape(self.heads, self.vdim, self.kv_rank).contiguous()
        self.c_norm_w = tensors[at["dkv_norm"]].to(device).contiguous()
        if self.has_sink:  # the softmax is 32-bit, and so is what enters it
            self.sinks = tensors[at["sink"]].to(device=device, dtype=torch.float32).contiguous()

    # ---- cache -------------------------------------------------------
    def cache_need(self) -> KVNeed:
        return KVNeed(1, self.kv_rank, self.window)

    # ---- run ---------------------------------------------------------
    def forward(self, x: torch.Tensor, step, cache: KVCacheView) -> torch.Tensor:
        n = x.shape[0]
        proj = linear(x, self.w_in)  # [n, q | c_raw | gate]
        table = step.block_tables[cache.group]
        if cache.writes:
            ops.latent_norm_write(proj, self.q_size, self.kv_rank, self.c_norm_w, self.eps, 0.0, step.positions,
                                  step.token_req, table, cache.k_pages, cache.v_pages)
        q_lat = ops.gemm_heads(proj, 0, self.w_uk_t)  # [n, heads * kv_rank]
        o_lat = torch.empty_like(q_lat)
        ops.paged_attention(q_lat, cache.k_pages, cache.v_pages, table, step, o_lat, self.heads, self.scale,
                            self.window, sinks=self.sinks)
        gate_at = self.q_size + self.kv_rank
        out = ops.gemm_heads(o_lat, 0, self.w_uv, gate=proj if self.has_gate else None, gate_col0=gate_at)
        return linear(out, self.w_o, sliced_ok=True)


MIXERS.register("latent_attention", LatentAttention)
