"""The Miborax decoder's typed configuration: the keys of its ``config.json``.

A Miborax model is a list of layers whose two sub-layers read the same stream through a layer
norm each (weight and bias).  A layer's mixer is attention through a latent: the cache holds,
per token, one RMS-normed row and one rotated key part shared by all heads, and each head turns
the row into its keys and values with matrices of its own.  Two mixer types exist.
``latent_attention``: queries through an RMS-normed latent of ``q_rank`` channels, every earlier
position visible, a sigmoid gate per head.  ``latent_attention_2``: queries from one projection, a
sliding window (``mask.size``), and optionally ``kv_from``: the layer has no latent projection
and reads the rows another layer cached.  Both add ``exp`` of a learned number per head to the
softmax's denominator.  The feed-forward is a mixture of gated experts with a router bias, or
absent.  The embedding is scaled; the output projection is the embedding table.  Every size and
every constant that differs between models of the design is a key here.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, normalise_dtype_name, require

MIXER_TYPES = ("latent_attention", "latent_attention_2")
FEED_FORWARD_KINDS = ("moe",)


def _positive(where: str, data: Mapping[str, Any], key: str) -> int:
    if not isinstance(data, Mapping):
        raise ConfigError(f"{where} must be an object")
    value = require(data, key, int)
    if value < 1:
        raise ConfigError(f"{where}: {key!r} must be a positive integer, got {value!r}")
    return value


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int  # channels of a query / key head that do not rotate
    rot_dim: int  # channels of the shared key part (and of a query head's second part)
    vdim: int  # channels of a value head
    kv_rank: int  # channels of the cached latent row
    q_rank: int  # channels of the query latent; 0: queries come from one projection
    scale: float  # factor of the scores
    rotary_base: float
    rotary_dims: int  # leading channels of the shared part that rotate
    window: int  # positions a query sees, its own included; 0: all before it
    kv_from: int | None  # the layer whose cached rows this one reads; None: its own

    @classmethod
    def from_dict(cls, where: str, kind: str, data: Mapping[str, Any]) -> "LatentMixerConfig":
        heads, dim = _positive(where, data, "heads"), _positive(where, data, "dim")
        rot_dim, vdim = _positive(where, data, "rot_dim"), _positive(where, data, "vdim")
        kv_rank = _positive(where, data, "kv_rank")
        rot = data.get("rot")
        if not isinstance(rot, Mapping):
            raise ConfigError(f"{where}: 'rot' must give the rotation's base and dims")
        dims = _positive(where + ".rot", rot, "dims")
        base = require(rot, "base", float)
        if rot_dim % 2 or dims % 2 or dims > rot_dim or not base > 0:
            raise ConfigError(
                f"{where}: a rotation of {dims} of {rot_dim} shared channels with base {base!r} (even counts, "
                "at most the shared part, a positive base)"
            )
        q_rank = window = 0
        kv_from = None
        if kind == "latent_attention":
            q_rank = _positive(where, data, "q_rank")
            if data.get("kv_from") is not None:
                raise ConfigError(f"{where}: a {kind} layer has a latent projection of its own")
        else:
            if data.get("q_rank") is not None:
                raise ConfigError(f"{where}: a {kind} layer's queries come from one projection")
            if data.get("kv_from") is not None:
                kv_from = require(data, "kv_from", int)
        mask = data.get("mask")
        if mask is not None:
            window = _positive(where + ".mask", mask, "size")
        elif kind == "latent_attention_2":
            raise ConfigError(f"{where}: a {kind} layer needs 'mask' with its window's size")
        return cls(heads, dim, rot_dim, vdim, kv_rank, q_rank, require(data, "scale", float), float(base), dims,
                   window, kv_from)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
            "kv_rank": self.kv_rank, "scale": self.scale,
            "rot": {"base": self.rotary_base, "dims": self.rotary_dims},
        }
        if self.q_rank:
            out["q_rank"] = self.q_rank
        if self.window:
            out["mask"] = {"size": self.window}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class GatedExpertsConfig:
    experts: int
    top: int
    expert_ff: int
    kind: str = "moe"

    def to_dict(self) -> dict[str, Any]:
        return {"kind": "moe", "expert": {"ff": self.expert_ff}, "router": {"experts": self.experts, "top": self.top}}


def _feed_forward(where: str, data: Mapping[str, Any]) -> GatedExpertsConfig:
    if not isinstance(data, Mapping):
        raise ConfigError(f"{where} must be an object or null")
    kind = data.get("kind", "moe")
    if kind not in FEED_FORWARD_KINDS:
        raise ConfigError(f"{where}: feed-forward kind {kind!r} is not one of {', '.join(FEED_FORWARD_KINDS)}")
    router = data.get("router")
    experts = _positive(where + ".router", router, "experts")
    top = _positive(where + ".router", router, "top")
    if top > experts:
        raise ConfigError(f"{where}.router: a token cannot use {top} of {experts} experts")
    return GatedExpertsConfig(experts, top, _positive(where + ".expert", data.get("expert"), "ff"))


@dataclass(frozen=True)
class MiboraxLayerConfig:
    type: str  # one of MIXER_TYPES
    mixer: LatentMixerConfig
    mlp: GatedExpertsConfig | None

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


@dataclass(frozen=True)
class MiboraxConfig:
    architecture: str
    width: int
    vocab: int
    embedding_scale: float
    norm_eps: float
    layers: tuple[MiboraxLayerConfig, ...]
    torch_dtype: str
    eos_token_ids: tuple[int, ...] = ()

    # the names the rest of the engine asks any configuration for
    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], overrides: Mapping[str, Any] | None = None) -> "MiboraxConfig":
        data = dict(data)
        if overrides:
            data.update(overrides)
        listed = data.get("layers")
        if not isinstance(listed, (list, tuple)) or not listed:
            raise ConfigError("config.json key 'layers' must list at least one layer")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            kind = require(entry, "type", str)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}: mixer type {kind!r} is not one of {', '.join(MIXER_TYPES)}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, Mapping):
                raise ConfigError(f"{where}: 'mixer' must give the mixer's sizes")
            mlp = entry.get("mlp")
            layers.append(MiboraxLayerConfig(
                kind, LatentMixerConfig.from_dict(where + ".mixer", kind, mixer),
                _feed_forward(where + ".mlp", mlp) if mlp is not None else None,
            ))
        for i, layer in enumerate(layers):
            src = layer.mixer.kv_from
            if src is None:
                continue
            where = f"layers[{i}].mixer"
            if not 0 <= src < i:
                raise ConfigError(f"{where}: kv_from {src} must name an earlier layer")
            theirs, mine = layers[src].mixer, layer.mixer
            if theirs.kv_from is not None:
                raise ConfigError(f"{where}: layer {src} has no latent projection of its own to read from")
            same = ("kv_rank", "rot_dim", "rotary_base", "rotary_dims")
            if any(getattr(theirs, k) != getattr(mine, k) for k in same):
                raise ConfigError(f"{where}: layer {src}'s cached rows differ in {', '.join(same)}")
        embedding = data.get("embedding") or {}
        norm = data.get("norm") or {}
        eps = require(norm, "eps", float)
        if not eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {eps!r}")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos))
        return cls(
            architecture=require(data, "architecture", str),
            width=_positive("config.json", data, "width"),
            vocab=_positive("config.json", data, "vocab"),
            embedding_scale=float(embedding.get("scale", 1.0)),
            norm_eps=eps,
            layers=tuple(layers),
            torch_dtype=normalise_dtype_name(data.get("torch_dtype") or data.get("dtype") or "bfloat16"),
            eos_token_ids=eos_ids,
        )

    def cache_window(self, owner: int) -> int:
        """Positions the cache of layer ``owner`` must keep: the longest view among the layer
        itself and the layers that read its rows (0, everything, if any of them sees it all)."""
        views = [self.layers[owner].mixer.window]
        views += [layer.mixer.window for layer in self.layers if layer.mixer.kv_from == owner]
        return 0 if 0 in views else max(views)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": self.architecture,
            "width": self.width,
            "vocab": self.vocab,
            "embedding": {"scale": self.embedding_scale},
            "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
            "torch_dtype": self.torch_dtype,
        }
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
