"""The Pinorax decoder as a ``ModelSpec``.

What the design fixes (not read from config.json):
  * the embedding is the token's vector plus a learned vector of its position, unscaled;
  * every layer has one RMS norm with a single number as gain; the mixer and the feed-forward both read its
    output and their sum, times ``residual_mult``, is added to the residual stream, which is 32-bit;
  * after every layer the stream that goes on is a learned average of the embedding's output and the results
    of all layers so far (``l<i>.dwa``: i + 2 weights);
  * the mixer is latent attention without positions: causal, a sink in every head's softmax, the output gated
    by sigmoid of a projection of the layer's input, the compressed vector RMS-normed with a plain weight;
  * a dense feed-forward is silu-gated with biases on its three projections; an expert is gated with clamped
    inputs, g * sigmoid(1.702 g) * (u + 1), without biases; experts are chosen by the token's id from a stored
    table, each with weight 1 / top; a shared expert of the same form may run for every token;
  * the model's norm, an untied head, and the logits' soft-cap.
Tensor names: ``embed``, ``pos``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.dwa``, ``final.norm``,
``head``; weights have no suffix, biases end in ``.b``.
"""

from __future__ import annotations

from ..config.pinorax import ARCHITECTURE, PinoraxConfig
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .registry import Architecture, register_architecture

EXPERT_SIGMOID_SLOPE = 1.702


def build_spec(cfg: PinoraxConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm_scalar", {"eps": cfg.norm_eps, "suffix": ""})
    count = len(cfg.layers)
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        mixer = PartSpec(layer.type, {
            "heads": m.heads, "dim": m.dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
            "eps": cfg.norm_eps, "sink": True, "gate": True, "window": None,
        })
        if layer.mlp is None:
            ff = PartSpec("none")
        elif layer.mlp.kind == "dense":
            ff = PartSpec("gated_mlp", {
                "intermediate_size": layer.mlp.ff, "activation": "silu", "bias": True,
                "names": {"gate": "mlp.gate", "up": "mlp.up", "down": "mlp.down"},
                "weight_suffix": "", "bias_suffix": ".b",
            })
        else:
            shared = layer.mlp.shared
            ff = PartSpec("routed_experts", {
                "router": "token_table", "experts": layer.mlp.experts, "top": layer.mlp.top,
                "vocab_size": cfg.vocab, "intermediate_size": layer.mlp.expert.ff,
                "activation": "clamped_glu", "limit": layer.mlp.expert.limit, "alpha": EXPERT_SIGMOID_SLOPE,
                "shared": None if shared is None else {"intermediate_size": shared.ff, "limit": shared.limit,
                                                        "alpha": EXPERT_SIGMOID_SLOPE},
            })
        block = PartSpec("parallel", {
            "residual_mult": cfg.residual_mult, "norm_name": "norm1",
            "depth_average": {"name": "dwa", "terms": i + 2, "slots": count + 1},
        })
        layers.append(LayerSpec(prefix=f"l{i}", block=block, mixer=mixer, feed_forward=ff, norm=norm))
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=cfg.max_positions,
        embedding=PartSpec("positional_embedding", {"scale": 1.0, "max_position": cfg.max_positions,
                                                    "name": "embed", "position_name": "pos", "suffix": ""}),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(i) for i in range(count)),
        final_norm=norm,
        head=PartSpec("lm_head", {"tied": False, "softcap": cfg.logit_softcap, "weight_name": "head"}),
        prefix="",
        final_norm_name="final.norm",
        residual_float32=True,
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    read_config=PinoraxConfig.from_dict,
    build_spec=build_spec,
    write_config=PinoraxConfig.to_dict,
))
