"""Miborax decoder: configuration -> model description, and its registry entry.

Layer ``i``'s tensors are ``l<i>.norm1`` / ``l<i>.norm1.b`` and ``l<i>.norm2`` / ``l<i>.norm2.b``
(the two layer norms), ``l<i>.mix.*`` (``q`` or ``dq`` / ``dq.norm`` / ``uq``; ``dkv`` /
``dkv.norm`` unless the layer reads another's rows; ``uk``, ``uv``, ``sink``, ``o``; ``g`` where
heads are gated) and ``l<i>.mlp.*`` (experts ``e<n>.gate`` / ``e<n>.up`` / ``e<n>.down``,
``router``, ``router.b``); the two ends are ``embed`` (also the output projection) and
``final.norm`` / ``final.norm.b``.
"""

from __future__ import annotations

from ..config.miborax import MiboraxConfig
from ..config.registry import register_architecture
from .spec import IgnoreRule, LayerSpec, ModelSpec, PartSpec, linear_output, token_embedding_scaled


def build_miborax_spec(cfg: MiboraxConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("layernorm", {"size": cfg.width, "eps": cfg.norm_eps, "checkpoint_name": name,
                                      "bias_checkpoint_name": name + ".b"})

    layers = []
    unread = []
    for i, layer in enumerate(cfg.layers):
        prefix = f"l{i}."
        m = layer.mixer
        owner = i if m.kv_from is None else m.kv_from
        mixer = PartSpec(
            "latent_attention",
            {
                "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim,
                "value_dim": m.vdim, "kv_rank": m.kv_rank, "q_rank": m.q_rank, "window": m.window,
                "cache_window": cfg.cache_window(owner), "softmax_scale": m.scale, "norm_eps": cfg.norm_eps,
                "sink": True, "gate": layer.type == "latent_attention", "owns_latent": m.kv_from is None,
                "checkpoint_prefix": prefix + "mix.",
            },
        )
        position = PartSpec(
            "rope", {"head_dim": m.rot_dim, "theta": m.rotary_base, "rotary_dim": m.rotary_dims, "pairing": "interleaved"}
        )
        ff = ff_norm = None
        if layer.mlp is not None:
            ff = PartSpec(
                "routed_experts",
                {
                    "hidden_size": cfg.width, "num_experts": layer.mlp.experts, "top": layer.mlp.top,
                    "expert_size": layer.mlp.expert_ff, "activation": "silu", "gated": True,
                    "router_bias_name": "router.b", "checkpoint_prefix": prefix + "mlp.",
                },
            )
            ff_norm = norm(prefix + "norm2")
        else:
            # a checkpoint may still carry the second norm of a layer without a feed-forward:
            # nothing reads its output
            unread.append(IgnoreRule(rf"l{i}\.norm2(\.b)?"))
        layers.append(
            LayerSpec(
                mixer=mixer, feed_forward=ff, mixer_norm=norm(prefix + "norm1"), feed_forward_norm=ff_norm,
                block=PartSpec("parallel"), position=position, checkpoint_prefix=prefix,
                share_cache_with=m.kv_from,
            )
        )
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        layers=tuple(layers),
        final_norm=norm("final.norm"),
        embedding=token_embedding_scaled(cfg.vocab, cfg.width, "embed", cfg.embedding_scale),
        # the output projection is the embedding's table: the checkpoint ships no tensor of its own
        output=linear_output(cfg.vocab, cfg.width, "head", tied=True),
        ignore_tensors=tuple(unread),
    )


register_architecture("Miborax", MiboraxConfig, build_miborax_spec, aliases=("miborax",), replace=True)
