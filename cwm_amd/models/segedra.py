"""The Segedra decoder as a plan of parts.

A scaled embedding that starts every residual stream; pre-norm layers of attention (grouped heads, a norm over
the whole query and key projections, partial rotation, a sliding window, a sink in the softmax) and a
feed-forward that is dense (squared relu) or a mixture of experts (scores over all experts, a correction for the
choice only, clamped gated experts), each sublayer joined to the streams by a hyper-connection; a range of layers
may run several times with the same weights, every pass with a cache of its own; the final norm reads the sum of
the streams and the head is the embedding table.  Norm weights are stored around zero and applied as 1 + w.
Tensor names: `embed`, `l<i>.norm1`, `l<i>.hc1.{in,out,mix}`, `l<i>.mix.{q,k,v,o,q.norm,k.norm,sink}`, `l<i>.norm2`,
`l<i>.hc2.*`, `l<i>.mlp.{up,down}` or `l<i>.mlp.{router,correction,e<j>.gate,e<j>.up,e<j>.down}`, `final.norm`.
"""

from __future__ import annotations

from ..config.registry import register_architecture
from ..config.segedra import AttentionConfig, SegedraConfig
from ..parts.base import LayerCall, LayerPlan, ModelPlan, PartChoice, PartSlot

ARCHITECTURE_NAME = "Segedra"

EXPERT_SIGMOID_SLOPE = 1.702  # the design's constant in an expert's g * sigmoid(1.702 g) * (u + 1)


def build_plan(config: SegedraConfig) -> ModelPlan:
    width = config.width
    streams = config.streams or 1
    norm = PartChoice("stream_rmsnorm", {"dim": width, "eps": config.norm.eps, "streams": streams, "offset": 1.0, "tensor": ""})
    if config.streams is None:
        connection = PartChoice("residual_sum", {})
    else:
        connection = PartChoice("hyper_connection", {"streams": streams})
    layers = []
    for i, layer in enumerate(config.layers):
        sizes = layer.mixer_config()
        if not isinstance(sizes, AttentionConfig):  # pragma: no cover  (LayerConfig has refused it)
            raise TypeError(f"layer {i}: no part for {type(sizes).__name__}")
        rotation = None
        if sizes.rot is not None and sizes.rot.dims > 0:
            rotation = PartChoice("rotary", {"head_dim": sizes.rot.dims, "theta": sizes.rot.base})
        mixer = PartChoice(
            "sink_attention",
            {
                "dim": width, "n_heads": sizes.heads, "n_kv_heads": sizes.kv_heads, "qk_dim": sizes.dim, "v_dim": sizes.vdim,
                "scale": sizes.scale, "window": sizes.mask.size if sizes.mask is not None else None, "qk_norm": True,
                "eps": config.norm.eps, "sink": True, "position_encoding": rotation,
            },
        )
        parts = {
            "norm1": PartSlot("norm", norm, "norm1"),
            "connection1": PartSlot("connection", connection, "hc1."),
            "mixer": PartSlot("mixer", mixer, "mix."),
        }
        if layer.mlp is not None:
            if layer.mlp.kind == "dense":
                feed_forward = PartChoice("activated_mlp", {"dim": width, "hidden_dim": layer.mlp.ff, "activation": "relu2"})
            else:
                feed_forward = PartChoice(
                    "routed_experts",
                    {
                        "dim": width, "hidden_dim": layer.mlp.expert.ff, "n_experts": layer.mlp.router.experts, "top": layer.mlp.router.top,
                        "scores": "softmax_all", "correction": True, "weight_scale": layer.mlp.router.scale, "renormalize": False,
                        "activation": "clamped_swish", "act_alpha": EXPERT_SIGMOID_SLOPE, "act_limit": layer.mlp.expert.limit,
                    },
                )
            parts["norm2"] = PartSlot("norm", norm, "norm2")
            parts["connection2"] = PartSlot("connection", connection, "hc2.")
            parts["feed_forward"] = PartSlot("feed_forward", feed_forward, "mlp.")
        layers.append(LayerPlan(prefix=f"l{i}.", block="connected_pre_norm", parts=parts))
    sizes = {"vocab_size": config.vocab, "dim": width, "tensor": ""}
    return ModelPlan(
        vocab_size=config.vocab,
        dim=width,
        layers=layers,
        run_order=[LayerCall(layer=i) for i in config.layer_order()],
        embedding=PartSlot("embedding", PartChoice("token_embedding", {**sizes, "scale": config.embedding.scale, "streams": streams}), "embed"),
        final_norm=PartSlot("norm", norm, "final.norm"),
        head=PartSlot("head", PartChoice("linear_head", sizes), "embed"),
        max_positions=config.max_positions,
    )


register_architecture(ARCHITECTURE_NAME, SegedraConfig, build_plan)
