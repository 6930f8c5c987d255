"""The Rufedra decoder as a ``ModelSpec``.

What the design fixes (not read from config.json):
  * the embedding is the token's vector times ``embedding.scale``; the residual stream is 32-bit;
  * a layer is a sandwich: x += ls1 * norm1b(mixer(norm1(x))), then x += ls2 * norm2b(ff(norm2(x))), every norm an
    RMS norm with a plain weight, ls1 / ls2 one learned number a channel; a layer without a feed-forward has the
    first sublayer only;
  * mixer ``delta``: the gated delta rule with short convolutions and silu on q, k and v, unit q and k
    (x / sqrt(sum x^2 + 1e-6), q also times dim^(-1/2)), an output norm per head with a shared weight, a silu gate;
  * mixer ``parallel``: two mixers on the same input, weighted by ``left_scale`` and ``right_scale``.  Left:
    grouped-query attention over a sliding window whose values are the keys as projected (no value projection),
    biases on q and k, a rotation of the first ``rot.dims`` dimensions of a head in halves with frequencies
    base^(-2i/dims), then an RMS norm without a weight per head, ordinary softmax, a sigmoid gate on the
    concatenated heads.  Right: a selective scan with a biased short convolution;
  * the feed-forward is dense and gated with the tanh form of gelu, without biases;
  * the model's norm, an untied head, the logits times ``logit_scale``.
Tensor names: ``embed``, ``l<i>.norm1`` / ``norm1b`` / ``norm2`` / ``norm2b``, ``l<i>.ls1`` / ``ls2``, ``l<i>.mix.*``
(``mix.left.*`` and ``mix.right.*`` in a parallel layer), ``l<i>.mlp.*``, ``final.norm``, ``head``; weights have no
suffix, biases end in ``.b``.
"""

from __future__ import annotations

from ..config.rufedra import ARCHITECTURE, MAX_CONTEXT, RufedraConfig
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .registry import Architecture, register_architecture

UNIT_EPS = 1e-6  # inside the root of the delta rule's unit q and k


def _delta(m, eps: float) -> PartSpec:
    return PartSpec("gated_delta_rule", {
        "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv, "eps": eps,
        "unit_eps": UNIT_EPS,
    })


def _window_attention(a, eps: float) -> PartSpec:
    return PartSpec("attention", {
        "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim, "scale": a.scale, "window": a.window,
        "values": "keys", "gate": "sigmoid", "bias": ["q", "k"],
        "qk_norm": {"eps": eps, "weight": False, "after_rotation": True},
        "position": PartSpec("rope", {"theta": a.rot_base, "rotary_dim": a.rot_dims, "exponent_over": "rotary_dim",
                                      "pairing": "rotary_half"}) if a.rot_dims else PartSpec("none"),
        "names": {"q": "mix.left.q", "k": "mix.left.k", "g": "mix.left.g", "o": "mix.left.o"},
        "weight_suffix": "", "bias_suffix": ".b",
    })


def _scan(s) -> PartSpec:
    names = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "x": "x", "dt": "dt", "dt_bias": "dt.b",
             "A_log": "A_log", "D": "D", "o": "o"}
    return PartSpec("selective_scan", {
        "inner": s.inner, "state": s.state, "dt_rank": s.dt_rank, "conv": s.conv,
        "names": {role: f"mix.right.{name}" for role, name in names.items()},
    })


def build_spec(cfg: RufedraConfig) -> ModelSpec:
    eps = cfg.norm_eps
    norm = PartSpec("rmsnorm", {"eps": eps, "suffix": ""})
    layers = []
    for i, layer in enumerate(cfg.layers):
        if layer.type == "delta":
            mixer = _delta(layer.mixer, eps)
        else:
            m = layer.mixer
            mixer = PartSpec("side_by_side", {"members": [
                {"mixer": _window_attention(m.left, eps), "scale": m.left_scale},
                {"mixer": _scan(m.right), "scale": m.right_scale},
            ]})
        if layer.mlp is None:
            ff = PartSpec("none")
        else:
            ff = PartSpec("gated_mlp", {
                "intermediate_size": layer.mlp.ff, "activation": "gelu_tanh",
                "names": {"gate": "mlp.gate", "up": "mlp.up", "down": "mlp.down"}, "weight_suffix": "",
                "unrounded_output": True,
            })
        block = PartSpec("sandwich", {"norm_names": ("norm1", "norm1b", "norm2", "norm2b"),
                                      "layer_scale": ("ls1", "ls2")})
        layers.append(LayerSpec(prefix=f"l{i}", block=block, mixer=mixer, feed_forward=ff, norm=norm))
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=MAX_CONTEXT,
        embedding=PartSpec("scaled_embedding", {"scale": cfg.embedding_scale, "name": "embed", "suffix": ""}),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(i) for i in range(len(layers))),
        final_norm=norm,
        head=PartSpec("lm_head", {"tied": False, "scale": cfg.logit_scale, "weight_name": "head"}),
        prefix="",
        final_norm_name="final.norm",
        residual_float32=True,
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    read_config=RufedraConfig.from_dict,
    build_spec=build_spec,
    write_config=RufedraConfig.to_dict,
))
