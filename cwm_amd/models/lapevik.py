"""The Lapevik decoder as a plan of parts.

Embedding followed by the model's group norm; layers of a token shift, a mixer (selective state space or
attention through a latent) and, where the layer has one, routed experts, each sublayer's output normalised
before it joins the residual; the model's norm once more and a head on the embedding table.  Tensor names:
`embed`, `embed.norm`, `l<i>.shift`, `l<i>.mix.*`, `l<i>.norm1`, `l<i>.mlp.*`, `l<i>.norm2`, `final.norm`.
"""

from __future__ import annotations

from ..config.lapevik import LapevikConfig, LatentAttentionConfig, StateSpaceConfig
from ..config.registry import register_architecture
from ..parts.base import LayerCall, LayerPlan, ModelPlan, PartChoice, PartSlot

ARCHITECTURE_NAME = "Lapevik"


def build_plan(config: LapevikConfig) -> ModelPlan:
    width = config.width
    norm = PartChoice("group_rmsnorm", {"dim": width, "eps": config.norm.eps, "groups": config.norm.groups, "tensor": ""})
    layers = []
    for i, layer in enumerate(config.layers):
        sizes = layer.mixer_config()
        if isinstance(sizes, StateSpaceConfig):
            mixer = PartChoice(
                "selective_state_space",
                {
                    "dim": width, "heads": sizes.heads, "head_dim": sizes.vdim, "state": sizes.state, "groups": sizes.groups,
                    "norm_groups": sizes.norm_groups, "taps": sizes.conv, "eps": config.norm.eps,
                },
            )
        elif isinstance(sizes, LatentAttentionConfig):
            mixer = PartChoice(
                "latent_attention",
                {
                    "dim": width, "n_heads": sizes.heads, "head_dim": sizes.dim, "rot_dim": sizes.rot_dim, "v_dim": sizes.vdim,
                    "kv_rank": sizes.kv_rank, "q_rank": sizes.q_rank, "scale": sizes.scale, "eps": config.norm.eps,
                    "position_encoding": PartChoice("rotary", {"head_dim": sizes.rot.dims, "theta": sizes.rot.base}) if sizes.rot.dims else None,
                },
            )
        else:  # pragma: no cover  (LayerConfig has refused it)
            raise TypeError(f"layer {i}: no part for {type(sizes).__name__}")
        parts = {
            "shift": PartSlot("mixer", PartChoice("token_shift", {"dim": width, "tensor": ""}), "shift"),
            "mixer": PartSlot("mixer", mixer, "mix."),
            "norm1": PartSlot("norm", norm, "norm1"),
        }
        if layer.mlp is not None:
            experts = PartChoice(
                "routed_experts",
                {"dim": width, "hidden_dim": layer.mlp.expert.ff, "n_experts": layer.mlp.router.experts, "top": layer.mlp.router.top},
            )
            parts["feed_forward"] = PartSlot("feed_forward", experts, "mlp.")
            parts["norm2"] = PartSlot("norm", norm, "norm2")
        layers.append(LayerPlan(prefix=f"l{i}.", block="post_norm", parts=parts))
    sizes = {"vocab_size": config.vocab, "dim": width}
    return ModelPlan(
        vocab_size=config.vocab,
        dim=width,
        layers=layers,
        run_order=[LayerCall(layer=i) for i in range(len(layers))],
        embedding=PartSlot("embedding", PartChoice("normed_embedding", {**sizes, "tensor": "", "norm": norm, "norm_prefix": ".norm"}), "embed"),
        final_norm=PartSlot("norm", norm, "final.norm"),
        head=PartSlot("head", PartChoice("linear_head", {**sizes, "tensor": ""}), "embed"),
        max_positions=config.max_positions,
    )


register_architecture(ARCHITECTURE_NAME, LapevikConfig, build_plan)
