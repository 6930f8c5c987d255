"""Several mixers side by side in one layer: all read the layer's input, and the layer's mixer output is the
weighted sum of theirs, sum_i scale_i * mixer_i(h).

Parameters: ``members``: a list of {"mixer": PartSpec, "scale": number}.  Each member is built from the mixers'
registry and names its own tensors (its ``names``).  What the members keep between steps is declared as the
tuple of their needs, and ``forward`` hands each member its own view.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, ParamSpec
from .registry import MIXERS
from .spec import PartSpec


class SideBySide(Mixer):
    def __init__(self, spec: PartSpec, *, hidden_size: int):
        members = list(spec["members"])
        if len(members) < 2:
            raise ValueError("mixers side by side are two at least")
        self.members = [MIXERS.build(m["mixer"], hidden_size=hidden_size) for m in members]
        self.scales = [float(m.get("scale", 1.0)) for m in members]

    @property
    def capturable(self) -> bool:
        return all(m.capturable for m in self.members)

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        return [s for m in self.members for s in m.param_specs(prefix)]

    def bind(self, tensors, prefix, device, dtype) -> None:
        for m in self.members:
            m.tiled_weights = self.tiled_weights
            m.bind(tensors, prefix, device, dtype)

    def cache_need(self) -> tuple:
        return tuple(m.cache_need() for m in self.members)

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        outs = [m.forward(x, step, view) for m, view in zip(self.members, cache)]
        if len(outs) == 2:  # left to the kernel that norms the sum and adds it to the stream
            return ops.BranchSum(outs[0], outs[1], self.scales[0], self.scales[1])
        total = ops.weighted_sum(outs[0], outs[1], self.scales[0], self.scales[1])
        for out, scale in zip(outs[2:-1], self.scales[2:-1]):
            total = ops.weighted_sum(total, out, 1.0, scale)
        return ops.BranchSum(total, outs[-1], 1.0, self.scales[-1])


MIXERS.register("side_by_side", SideBySide)
