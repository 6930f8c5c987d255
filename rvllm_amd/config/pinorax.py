"""Typed configuration of the Pinorax decoder, read from config.json.

The file gives every size and every constant that differs between models of
the design:

    architecture     "Pinorax"
    vocab, width, max_positions
    norm.eps         of every RMS norm
    residual_mult    the multiplier of a layer's two branches
    logit_softcap    cap * tanh(logits / cap); absent or null: none
    layers[i]        type (the mixer's kind), mixer (its sizes), mlp (null: none;
                     kind "dense": ff; kind "moe": expert {ff, limit},
                     router {experts, top}, shared {ff, limit} or null)

What the design fixes is stated in ``models/pinorax.py``.  As with the other
readers, every problem of a file is reported in one ``ConfigError``.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Optional

from .errors import ConfigError
from .fields import FieldReader

ARCHITECTURE = "Pinorax"
MAX_LAYERS = 1024
MAX_WIDTH = 1 << 20
MAX_VOCAB = 1 << 22
MAX_CONTEXT = 1 << 20
MIXER_TYPES = ("latent_attention",)
MLP_KINDS = ("dense", "moe")


@dataclasses.dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float


@dataclasses.dataclass(frozen=True)
class ExpertSizes:
    ff: int
    limit: float


@dataclasses.dataclass(frozen=True)
class MlpConfig:
    kind: str  # "dense" or "moe"
    ff: int = 0  # dense
    expert: Optional[ExpertSizes] = None
    experts: int = 0
    top: int = 0
    shared: Optional[ExpertSizes] = None


@dataclasses.dataclass(frozen=True)
class PinoraxLayer:
    type: str
    mixer: LatentAttentionSizes
    mlp: Optional[MlpConfig]


@dataclasses.dataclass(frozen=True)
class PinoraxConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    residual_mult: float
    layers: tuple[PinoraxLayer, ...]
    logit_softcap: Optional[float] = None
    architecture: str = ARCHITECTURE

    # ---- reading -----------------------------------------------------
    @classmethod
    def from_dict(cls, doc: dict, source: str = "config.json") -> "PinoraxConfig":
        r = FieldReader(doc)
        problems = r.problems
        vocab = r.integer("vocab", lo=1, hi=MAX_VOCAB)
        width = r.integer("width", lo=1, hi=MAX_WIDTH)
        max_positions = r.integer("max_positions", lo=1, hi=MAX_CONTEXT)
        residual_mult = r.real("residual_mult")
        cap = r.real("logit_softcap", default=None, positive=True)
        norm = r.raw("norm")
        eps = 0.0
        if not isinstance(norm, dict):
            problems.append("missing or invalid required object norm")
        else:
            nr = FieldReader(norm)
            eps = nr.real("eps", positive=True)
            problems += [f"norm: {p}" for p in nr.problems]
        raw_layers = r.raw("layers")
        layers = []
        if not isinstance(raw_layers, list) or not raw_layers:
            problems.append("missing or invalid required list layers")
        elif len(raw_layers) > MAX_LAYERS:
            problems.append(f"{len(raw_layers)} layers, at most {MAX_LAYERS}")
        else:
            for i, entry in enumerate(raw_layers):
                layer, found = _read_layer(entry)
                problems += [f"layers[{i}]: {p}" for p in found]
                layers.append(layer)
        if problems:
            raise ConfigError(source, problems)
        return cls(vocab, width, max_positions, eps, residual_mult, tuple(layers), cap)

    def to_dict(self) -> dict:
        def sizes(e: ExpertSizes) -> dict:
            return {"ff": e.ff, "limit": e.limit}

        layers = []
        for layer in self.layers:
            mlp: Any = None
            if layer.mlp is not None and layer.mlp.kind == "dense":
                mlp = {"kind": "dense", "ff": layer.mlp.ff}
            elif layer.mlp is not None:
                mlp = {"kind": "moe", "expert": sizes(layer.mlp.expert),
                       "router": {"experts": layer.mlp.experts, "top": layer.mlp.top},
                       "shared": None if layer.mlp.shared is None else sizes(layer.mlp.shared)}
            layers.append({"type": layer.type, "mixer": dataclasses.asdict(layer.mixer), "mlp": mlp})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "max_positions": self.max_positions, "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "logit_softcap": self.logit_softcap, "layers": layers}


def _read_expert(obj: Any, what: str, problems: list) -> Optional[ExpertSizes]:
    if not isinstance(obj, dict):
        problems.append(f"missing or invalid required object {what}")
        return None
    r = FieldReader(obj)
    out = ExpertSizes(r.integer("ff", lo=1, hi=MAX_WIDTH), r.real("limit", positive=True))
    problems += [f"{what}: {p}" for p in r.problems]
    return out


def _read_layer(entry: Any) -> tuple[Optional[PinoraxLayer], list]:
    problems: list = []
    if not isinstance(entry, dict):
        return None, ["must be an object"]
    r = FieldReader(entry)
    kind = r.string("type")
    if kind and kind not in MIXER_TYPES:
        r.problem(f"unknown mixer type {kind!r}; known: {', '.join(MIXER_TYPES)}")
    mixer = None
    raw_mixer = r.raw("mixer")
    if not isinstance(raw_mixer, dict):
        r.problem("missing or invalid required object mixer")
    else:
        m = FieldReader(raw_mixer)
        mixer = LatentAttentionSizes(m.integer("heads", lo=1, hi=4096), m.integer("dim", lo=1, hi=4096),
                                     m.integer("vdim", lo=1, hi=4096), m.integer("kv_rank", lo=1, hi=4096),
                                     m.real("scale", positive=True))
        problems += [f"mixer: {p}" for p in m.problems]
    mlp = None
    raw_mlp = entry.get("mlp")
    if raw_mlp is not None:
        if not isinstance(raw_mlp, dict):
            r.problem("mlp must be an object or null")
        else:
            f = FieldReader(raw_mlp)
            mlp_kind = f.string("kind")
            if mlp_kind == "dense":
                mlp = MlpConfig("dense", ff=f.integer("ff", lo=1, hi=MAX_WIDTH))
            elif mlp_kind == "moe":
                found: list = []
                expert = _read_expert(raw_mlp.get("expert"), "expert", found)
                shared = None if raw_mlp.get("shared") is None else _read_expert(raw_mlp.get("shared"), "shared", found)
                experts = top = 0
                router = raw_mlp.get("router")
                if not isinstance(router, dict):
                    found.append("missing or invalid required object router")
                else:
                    q = FieldReader(router)
                    experts = q.integer("experts", lo=1, hi=1024)
                    top = q.integer("top", lo=1, hi=1024)
                    if not q.problems and top > experts:
                        q.problem(f"top={top} of experts={experts}")
                    found += [f"router: {p}" for p in q.problems]
                for p in found:
                    f.problem(p)
                mlp = MlpConfig("moe", expert=expert, experts=experts, top=top, shared=shared)
            elif mlp_kind:
                f.problem(f"unknown kind {mlp_kind!r}; known: {', '.join(MLP_KINDS)}")
            problems += [f"mlp: {p}" for p in f.problems]
    problems = r.problems + problems
    if problems:
        return None, problems
    return PinoraxLayer(kind, mixer, mlp), []
