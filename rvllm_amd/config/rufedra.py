"""Typed configuration of the Rufedra decoder, read from config.json.

The file gives every size and every constant that differs between models of
the design:

    architecture       "Rufedra"
    vocab, width
    embedding.scale    what a token's vector is multiplied by
    norm.eps           of every RMS norm
    logit_scale        what the logits are multiplied by
    layers[i]          type ("delta" or "parallel"), mixer (its sizes), mlp (null: none; kind "dense": ff)
      delta            heads, kv_heads, dim, vdim, conv
      parallel         left {heads, kv_heads, dim, vdim, scale, mask.size, rot.dims, rot.base}, left_scale,
                       right {inner, state, dt_rank, conv}, right_scale

What the design fixes is stated in ``models/rufedra.py``.  As with the other
readers, every problem of a file is reported in one ``ConfigError``.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Optional, Union

from .errors import ConfigError
from .fields import FieldReader

ARCHITECTURE = "Rufedra"
MAX_LAYERS = 1024
MAX_WIDTH = 1 << 20
MAX_VOCAB = 1 << 22
MAX_CONTEXT = 1 << 20  # the design has no table of positions; a request is held to this many tokens
MAX_TAPS = 16
MIXER_TYPES = ("delta", "parallel")
MLP_KINDS = ("dense",)


@dataclasses.dataclass(frozen=True)
class DeltaSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclasses.dataclass(frozen=True)
class WindowAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int      # mask.size: a token sees itself and the window - 1 before it
    rot_dims: int    # rot.dims
    rot_base: float  # rot.base


@dataclasses.dataclass(frozen=True)
class ScanSizes:
    inner: int
    state: int
    dt_rank: int
    conv: int


@dataclasses.dataclass(frozen=True)
class ParallelSizes:
    left: WindowAttentionSizes
    right: ScanSizes
    left_scale: float
    right_scale: float


@dataclasses.dataclass(frozen=True)
class DenseMlp:
    ff: int
    kind: str = "dense"


@dataclasses.dataclass(frozen=True)
class RufedraLayer:
    type: str
    mixer: Union[DeltaSizes, ParallelSizes]
    mlp: Optional[DenseMlp]


@dataclasses.dataclass(frozen=True)
class RufedraConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    logit_scale: float
    layers: tuple[RufedraLayer, ...]
    architecture: str = ARCHITECTURE

    @classmethod
    def from_dict(cls, doc: dict, source: str = "config.json") -> "RufedraConfig":
        r = FieldReader(doc)
        problems = r.problems
        vocab = r.integer("vocab", lo=1, hi=MAX_VOCAB)
        width = r.integer("width", lo=1, hi=MAX_WIDTH)
        logit_scale = r.real("logit_scale")
        embedding_scale = _sub(doc, "embedding", problems, lambda f: f.real("scale"), 1.0)
        eps = _sub(doc, "norm", problems, lambda f: f.real("eps", positive=True), 1.0)
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
        return cls(vocab, width, embedding_scale, eps, logit_scale, tuple(layers))

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "delta":
                mixer: Any = dataclasses.asdict(m)
            else:
                a, s = m.left, m.right
                mixer = {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim,
                                  "scale": a.scale, "mask": {"size": a.window},
                                  "rot": {"dims": a.rot_dims, "base": a.rot_base}},
                         "left_scale": m.left_scale, "right": dataclasses.asdict(s), "right_scale": m.right_scale}
            mlp = None if layer.mlp is None else {"kind": layer.mlp.kind, "ff": layer.mlp.ff}
            layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "logit_scale": self.logit_scale, "layers": layers}


def _sub(doc: dict, key: str, problems: list, read, fallback):
    """``read(FieldReader(doc[key]))``, with the sub-object's problems filed under its key."""
    obj = doc.get(key)
    if not isinstance(obj, dict):
        problems.append(f"missing or invalid required object {key}")
        return fallback
    f = FieldReader(obj)
    value = read(f)
    problems += [f"{key}: {p}" for p in f.problems]
    return value


def _read_delta(obj: dict, problems: list) -> DeltaSizes:
    m = FieldReader(obj)
    sizes = DeltaSizes(m.integer("heads", lo=1, hi=4096), m.integer("kv_heads", lo=1, hi=4096),
                       m.integer("dim", lo=1, hi=1024), m.integer("vdim", lo=1, hi=4096),
                       m.integer("conv", lo=1, hi=MAX_TAPS))
    if not m.problems and sizes.heads % sizes.kv_heads:
        m.problem(f"heads={sizes.heads} must be a multiple of kv_heads={sizes.kv_heads}")
    problems += [f"mixer: {p}" for p in m.problems]
    return sizes


def _read_parallel(obj: dict, problems: list) -> Optional[ParallelSizes]:
    found: list = []
    m = FieldReader(obj)
    left_scale, right_scale = m.real("left_scale"), m.real("right_scale")
    found += m.problems
    left = right = None
    raw_left = obj.get("left")
    if not isinstance(raw_left, dict):
        found.append("missing or invalid required object left")
    else:
        a = FieldReader(raw_left)
        heads, kv_heads = a.integer("heads", lo=1, hi=4096), a.integer("kv_heads", lo=1, hi=4096)
        dim, vdim = a.integer("dim", lo=1, hi=512), a.integer("vdim", lo=1, hi=512)
        scale = a.real("scale", positive=True)
        sub: list = []
        window = _sub(raw_left, "mask", sub, lambda f: f.integer("size", lo=1, hi=MAX_CONTEXT), 1)
        dims = _sub(raw_left, "rot", sub, lambda f: f.integer("dims", lo=0, hi=512), 0)
        base = _sub(raw_left, "rot", [], lambda f: f.real("base", positive=True), 1.0)
        if isinstance(raw_left.get("rot"), dict):
            f = FieldReader(raw_left["rot"])
            f.real("base", positive=True)
            sub += [f"rot: {p}" for p in f.problems]
        for p in sub:
            a.problem(p)
        if not a.problems:
            if heads % kv_heads:
                a.problem(f"heads={heads} must be a multiple of kv_heads={kv_heads}")
            if vdim != dim:
                a.problem(f"vdim={vdim} must equal dim={dim}: the values are the keys")
            if dims % 2 or dims > dim:
                a.problem(f"rot.dims={dims} must be even and at most dim={dim}")
        found += [f"left: {p}" for p in a.problems]
        left = WindowAttentionSizes(heads, kv_heads, dim, vdim, scale, window, dims, base)
    raw_right = obj.get("right")
    if not isinstance(raw_right, dict):
        found.append("missing or invalid required object right")
    else:
        s = FieldReader(raw_right)
        right = ScanSizes(s.integer("inner", lo=1, hi=MAX_WIDTH), s.integer("state", lo=1, hi=256),
                          s.integer("dt_rank", lo=1, hi=MAX_WIDTH), s.integer("conv", lo=1, hi=MAX_TAPS))
        found += [f"right: {p}" for p in s.problems]
    problems += [f"mixer: {p}" for p in found]
    if found:
        return None
    return ParallelSizes(left, right, left_scale, right_scale)


def _read_layer(entry: Any) -> tuple[Optional[RufedraLayer], list]:
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
    elif kind == "delta":
        mixer = _read_delta(raw_mixer, problems)
    elif kind == "parallel":
        mixer = _read_parallel(raw_mixer, problems)
    mlp = None
    raw_mlp = entry.get("mlp")
    if raw_mlp is not None:
        if not isinstance(raw_mlp, dict):
            r.problem("mlp must be an object or null")
        else:
            f = FieldReader(raw_mlp)
            mlp_kind = f.string("kind")
            if mlp_kind == "dense":
                mlp = DenseMlp(f.integer("ff", lo=1, hi=MAX_WIDTH))
            elif mlp_kind:
                f.problem(f"unknown kind {mlp_kind!r}; known: {', '.join(MLP_KINDS)}")
            problems += [f"mlp: {p}" for p in f.problems]
    problems = r.problems + problems
    if problems:
        return None, problems
    return RufedraLayer(kind, mixer, mlp), []
