"""Fomunex decoder: configuration -> model description, and its registry entry.

Layer ``i``'s tensors are ``l<i>.norm1``, ``l<i>.norm2`` (one number each), ``l<i>.mix.*`` and
``l<i>.mlp.*`` (dense: ``up``, ``down``, ``act``; experts ``e<n>.gate`` / ``e<n>.up`` / ``e<n>.down`` and
``router``); the two ends are ``embed``, ``pos`` (learned position vectors), ``final.norm`` and
``head``.  A layer that uses another layer's tensors is one more place in the run order for that
layer, with a cache or state of its own.
"""

from __future__ import annotations

from ..config.fomunex import (
    CappedAttentionConfig,
    ExpertsFeedForwardConfig,
    FomunexConfig,
    StateSpaceConfig,
    WkvConfig,
)
from ..config.registry import register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec

# what the design fixes
DISTANCE_SLOPE_EXPONENT = 8.0  # head h of H takes 2^(-8 (h + 1) / H) off a score per position of distance
EXPERT_ALPHA = 1.702  # the sigmoid's slope in the experts' activation


def build_fomunex_spec(cfg: FomunexConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "checkpoint_name": name,
                                    "single_weight": True})

    owners = [i for i, layer in enumerate(cfg.layers) if layer.weights_of is None]
    place_of = {i: n for n, i in enumerate(owners)}
    layers = []
    for i in owners:
        layer = cfg.layers[i]
        prefix = f"l{i}."
        m = layer.mixer
        if isinstance(m, CappedAttentionConfig):
            mixer = PartSpec(
                "gqa_attention",
                {
                    "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                    "value_dim": m.vdim, "window": m.window, "softmax_scale": m.scale, "qk_norm_eps": cfg.norm_eps,
                    "qk_norm_weights": False, "score_cap": m.softcap,
                    "distance_slope_exponent": DISTANCE_SLOPE_EXPONENT, "sink_name": "sink",
                    "checkpoint_prefix": prefix + "mix.", "q_name": "q", "k_name": "k", "v_name": "v", "o_name": "o",
                },
            )
        elif isinstance(m, WkvConfig):
            mixer = PartSpec(
                "wkv",
                {
                    "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "decay_rank": m.rank,
                    "norm_eps": cfg.norm_eps, "checkpoint_prefix": prefix + "mix.",
                },
            )
        elif isinstance(m, StateSpaceConfig):
            mixer = PartSpec(
                "state_space",
                {
                    "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.vdim, "state_size": m.state,
                    "groups": m.groups, "conv_taps": m.conv, "norm_groups": m.norm_groups, "norm_eps": cfg.norm_eps,
                    "checkpoint_prefix": prefix + "mix.",
                },
            )
        else:  # pragma: no cover  (the configuration class admits no other)
            raise ValueError(f"layer {i}: no mixer for {type(m).__name__}")
        ff = ff_norm = None
        if layer.mlp is not None:
            if isinstance(layer.mlp, ExpertsFeedForwardConfig):
                ff = PartSpec(
                    "routed_experts",
                    {
                        "hidden_size": cfg.width, "num_experts": layer.mlp.experts, "top": layer.mlp.top,
                        "expert_size": layer.mlp.expert_ff, "activation": "silu", "gated": True,
                        "limit": layer.mlp.limit, "alpha": EXPERT_ALPHA, "scores": "sigmoid",
                        "weights_scale": "input", "checkpoint_prefix": prefix + "mlp.",
                    },
                )
            else:
                ff = PartSpec(
                    "two_layer",
                    {
                        "hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "activation": "polynorm",
                        "activation_eps": cfg.norm_eps, "activation_name": "act",
                        "checkpoint_prefix": prefix + "mlp.",
                    },
                )
            ff_norm = norm(prefix + "norm2")
        layers.append(
            LayerSpec(mixer=mixer, feed_forward=ff, mixer_norm=norm(prefix + "norm1"), feed_forward_norm=ff_norm,
                      checkpoint_prefix=prefix)
        )
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        layers=tuple(layers),
        final_norm=norm("final.norm"),
        embedding=PartSpec(
            "token_embedding",
            {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "checkpoint_name": "embed",
             "position_table_name": "pos", "positions": cfg.max_positions},
        ),
        output=PartSpec(
            "linear_output",
            {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "checkpoint_name": "head", "tied_to": None,
             "scale": cfg.logit_scale, "softcap": cfg.logit_softcap},
        ),
        run_order=tuple(place_of[i] for i in cfg.run_order()),
        max_position=cfg.max_positions,
    )


register_architecture("Fomunex", FomunexConfig, build_fomunex_spec, aliases=("fomunex",), replace=True)
