"""Arrangements of norm, mixer, feed-forward and residual sum in a layer.

``sandwich``: a norm before and after each branch; the normed branch output
is added to the residual stream
(v3/crates/rvllm-loader/src/metal_host.rs:501,606-628; the order of launches:
v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:1-28):

    x = x + post_attention_layernorm(mixer(input_layernorm(x)))
    x = x + post_feedforward_layernorm(ff(pre_feedforward_layernorm(x)))

A block may hand the next block its entry norm already applied (``then``),
which lets the kernel that adds the feed-forward branch also write the next
layer's normed input.  Parameters of ``sandwich``: ``norm_names`` (the four
norms' names under the layer's prefix, the Gemma names if absent) and
``layer_scale`` = (name, name) or None: one learned number a channel that the
normed mixer branch, and one that the normed feed-forward branch, is multiplied
by before it is added (x = x + ls1 * norm(mixer(..))).  A layer whose
feed-forward is ``none`` has the first sublayer only and asks for the first two
norms only.  The residual stream may be 32-bit under bf16 activations
(``ModelSpec.residual_float32``); the norms then read the one and write the other.

``parallel``: one norm, both branches read its output, and their sum is added
with a multiplier; the residual stream is 32-bit whatever the activations' type:

    h = norm(x);  X = x + residual_mult * (mixer(h) + ff(h))

With ``depth_average`` = {"name", "terms", "slots"} what goes on to the next
layer is a learned average over depth, x = sum_j w[j] * X_j over the first
``terms`` of: the first layer's input and every layer's X so far (``slots`` in
all; the tensor ``<layer>.<name>`` holds the ``terms`` weights).  The X_j of a
step live in ``step.shared`` and end with it.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import Block, Norm, ParamSpec, tensor_path
from .norm import ScalarRMSNorm
from .registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS
from .spec import LayerSpec, PartSpec


class SandwichBlock(Block):
    NORM_NAMES = ("input_layernorm", "post_attention_layernorm", "pre_feedforward_layernorm",
                  "post_feedforward_layernorm")

    def __init__(self, spec: PartSpec, *, layer: LayerSpec, hidden_size: int):
        self.hidden_size = hidden_size
        self.mixer = MIXERS.build(layer.mixer, hidden_size=hidden_size)
        self.feed_forward = FEED_FORWARDS.build(layer.feed_forward, hidden_size=hidden_size)
        self.has_feed_forward = layer.feed_forward.kind != "none"
        names = tuple(spec.get("norm_names") or self.NORM_NAMES)
        if len(names) != 4:
            raise ValueError("a sandwich has four norms: before and after the mixer, before and after the feed-forward")
        if not self.has_feed_forward:
            names = names[:2]
        self.norms = [NORMS.build(layer.norm, width=hidden_size, name=name) for name in names]
        self.norm_in, self.norm_post_mixer = self.norms[:2]
        self.norm_pre_ff, self.norm_post_ff = self.norms[2:] if self.has_feed_forward else (None, None)
        scale_names = spec.get("layer_scale")
        self.scale_names = None if scale_names is None else tuple(str(n) for n in scale_names)
        if self.scale_names is not None and len(self.scale_names) != 2:
            raise ValueError("layer_scale names two tensors: the mixer branch's and the feed-forward branch's")
        self.scale_mixer: Optional[torch.Tensor] = None
        self.scale_ff: Optional[torch.Tensor] = None

    def parts(self):
        return (self.mixer, self.feed_forward, *self.norms)

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        specs = [s for part in self.parts() for s in part.param_specs(prefix)]
        if self.scale_names is not None:
            used = self.scale_names if self.has_feed_forward else self.scale_names[:1]
            specs += [ParamSpec(tensor_path(prefix, name), (self.hidden_size,), init=("normal_about", 1.0, 0.1))
                      for name in used]
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        for part in self.parts():
            part.bind(tensors, prefix, device, dtype)
        if self.scale_names is not None:  # applied in 32-bit with the norm
            self.scale_mixer = tensors[tensor_path(prefix, self.scale_names[0])].to(
                device=device, dtype=torch.float32).contiguous()
            if self.has_feed_forward:
                self.scale_ff = tensors[tensor_path(prefix, self.scale_names[1])].to(
                    device=device, dtype=torch.float32).contiguous()

    def entry_norm(self) -> Optional[Norm]:
        return self.norm_in

    @staticmethod
    def _add(norm: Norm, branch, x, then, scale):
        if scale is None:
            return norm.add_into(branch, x, then=then)
        return norm.add_into(branch, x, then=then, scale=scale)

    def forward(self, x: torch.Tensor, step, cache, entered: Optional[torch.Tensor] = None,
                then: Optional[Norm] = None) -> Optional[torch.Tensor]:
        h = entered if entered is not None else self.norm_in.forward(x)
        a = self.mixer.forward(h, step, cache)
        if not self.has_feed_forward:
            return self._add(self.norm_post_mixer, a, x, then, self.scale_mixer)
        h = self._add(self.norm_post_mixer, a, x, self.norm_pre_ff, self.scale_mixer)
        f = self.feed_forward.forward(h, step)
        return self._add(self.norm_post_ff, f, x, then, self.scale_ff)


class ParallelBlock(Block):
    HISTORY = "parallel_block.depth_history"  # key in step.shared: (the X_j, how many are written)

    def __init__(self, spec: PartSpec, *, layer: LayerSpec, hidden_size: int):
        self.hidden_size = hidden_size
        self.residual_mult = float(spec.get("residual_mult", 1.0))
        self.norm_name = str(spec.get("norm_name", "norm"))
        depth = spec.get("depth_average")
        self.depth = None if depth is None else {"name": str(depth["name"]), "terms": int(depth["terms"]),
                                                 "slots": int(depth["slots"])}
        if self.depth is not None and not 2 <= self.depth["terms"] <= self.depth["slots"]:
            raise ValueError(f"a depth average over {self.depth['terms']} of {self.depth['slots']} streams")
        self.mixer = MIXERS.build(layer.mixer, hidden_size=hidden_size)
        self.feed_forward = FEED_FORWARDS.build(layer.feed_forward, hidden_size=hidden_size)
        self.norm = NORMS.build(layer.norm, width=hidden_size, name=self.norm_name)
        self.depth_weights: Optional[torch.Tensor] = None

    def parts(self):
        return (self.mixer, self.feed_forward, self.norm)

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        specs = [s for part in self.parts() for s in part.param_specs(prefix)]
        if self.depth is not None:
            specs.append(ParamSpec(tensor_path(prefix, self.depth["name"]), (self.depth["terms"],),
                                   init=("normal_about", 1.0 / self.depth["terms"], 0.05)))
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        for part in self.parts():
            part.bind(tensors, prefix, device, dtype)
        if self.depth is not None:  # averaged in 32-bit
            self.depth_weights = tensors[tensor_path(prefix, self.depth["name"])].to(
                device=device, dtype=torch.float32).contiguous()

    def entry_norm(self) -> Optional[Norm]:
        return self.norm

    def forward(self, x: torch.Tensor, step, cache, entered: Optional[torch.Tensor] = None,
                then: Optional[Norm] = None) -> Optional[torch.Tensor]:
        h = entered if entered is not None else self.norm.forward(x)
        a = self.mixer.forward(h, step, cache)
        f = self.feed_forward.forward(h, step)
        history, terms, seed = None, 0, False
        if self.depth is not None:
            terms = self.depth["terms"]
            kept = step.shared.get(self.HISTORY)
            if kept is None:  # the first layer of the step: its input is the first of the streams
                kept = [torch.empty((self.depth["slots"], *x.shape), dtype=torch.float32, device=x.device), 1]
                step.shared[self.HISTORY] = kept
                seed = True
            history = kept[0]
            if kept[1] != terms - 1:
                raise ValueError(f"a depth average over {terms} streams, but the step has written {kept[1]}")
            kept[1] = terms
        fused = isinstance(then, ScalarRMSNorm)
        nxt = ops.residual_mix(x, a, f, self.residual_mult, history, terms, self.depth_weights, seed,
                               then.gain if fused else None, then.eps if fused else 0.0,
                               then.out_dtype if fused else None)
        if then is not None and not fused:
            return then.forward(x)
        return nxt


BLOCKS.register("sandwich", SandwichBlock)
BLOCKS.register("parallel", ParallelBlock)
