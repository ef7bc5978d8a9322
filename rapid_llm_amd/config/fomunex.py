"""The Fomunex decoder's typed configuration: the keys of its ``config.json``.

A Fomunex model is a list of pre-norm layers whose norms have one learned number each.  A
layer's mixer is one of three: softmax attention without rotation (queries and keys divided by
their root mean square per head, capped scores, a distance penalty per head, a sliding window,
one learned term per head in the softmax's denominator), an RWKV-style recurrence with
token-shift mixes and a decay per key channel (``wkv``), or a state-space recurrence with a
short causal convolution in front of it (``mamba2``).  Its feed-forward is dense with a
polynomial activation over normalised powers, a mixture of clamped gated experts behind a
sigmoid router, or absent.  A layer may use another layer's tensors (``weights_of``) with a
cache or state of its own.  Learned position vectors are added to the embedding; the logits
are scaled and capped.  Every size and every constant that differs between models of the
design is a key here; nothing of them appears anywhere else in the package.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, normalise_dtype_name, require

MIXER_TYPES = ("attention", "wkv", "mamba2")
FEED_FORWARD_KINDS = ("dense", "moe")


def _positive(where: str, data: Mapping[str, Any], key: str) -> int:
    if not isinstance(data, Mapping):
        raise ConfigError(f"{where} must be an object")
    value = require(data, key, int)
    if value < 1:
        raise ConfigError(f"{where}: {key!r} must be a positive integer, got {value!r}")
    return value


def _number(where: str, data: Mapping[str, Any], key: str) -> float:
    if not isinstance(data, Mapping):
        raise ConfigError(f"{where} must be an object")
    return float(require(data, key, float))


@dataclass(frozen=True)
class CappedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int  # size of a query or key head
    vdim: int  # size of a value head
    scale: float  # factor of the scores
    softcap: float  # scores become softcap * tanh(score / softcap); 0: no cap
    window: int  # positions a query sees, its own included; 0: all before it

    @classmethod
    def from_dict(cls, where: str, data: Mapping[str, Any]) -> "CappedAttentionConfig":
        heads = _positive(where, data, "heads")
        kv_heads = _positive(where, data, "kv_heads") if data.get("kv_heads") is not None else heads
        dim = _positive(where, data, "dim")
        vdim = _positive(where, data, "vdim") if data.get("vdim") is not None else dim
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} heads are not divisible by {kv_heads} kv_heads")
        if dim % 2 or dim > 256 or vdim > 256:
            raise ConfigError(
                f"{where}: the attention kernels take even key sizes and value sizes up to 256, got {dim} and {vdim}"
            )
        cap = float(data.get("softcap") or 0.0)
        if cap < 0:
            raise ConfigError(f"{where}: softcap must not be negative, got {cap}")
        window = 0
        if data.get("mask") is not None:
            window = _positive(where + ".mask", data["mask"], "size")
        return cls(heads, kv_heads, dim, vdim, _number(where, data, "scale"), cap, window)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
        }
        if self.softcap:
            out["softcap"] = self.softcap
        if self.window:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class WkvConfig:
    heads: int
    dim: int  # key and value channels of a head
    # inner size of the decay's two small matrices; 0: whatever the checkpoint's tensors have
    rank: int = 0

    @classmethod
    def from_dict(cls, where: str, data: Mapping[str, Any]) -> "WkvConfig":
        rank = data.get("rank") or 0
        if not isinstance(rank, int) or isinstance(rank, bool) or rank < 0:
            raise ConfigError(f"{where}: rank must be a size, got {rank!r}")
        return cls(_positive(where, data, "heads"), _positive(where, data, "dim"), rank)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"heads": self.heads, "dim": self.dim}
        if self.rank:
            out["rank"] = self.rank
        return out


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int  # channels of a head
    state: int  # state size N
    groups: int  # groups that share B and C
    conv: int  # taps of the causal convolution
    norm_groups: int  # equal parts the gated output is normed in

    @classmethod
    def from_dict(cls, where: str, data: Mapping[str, Any]) -> "StateSpaceConfig":
        heads, vdim = _positive(where, data, "heads"), _positive(where, data, "vdim")
        state, groups = _positive(where, data, "state"), _positive(where, data, "groups")
        conv, parts = _positive(where, data, "conv"), _positive(where, data, "norm_groups")
        if heads % groups:
            raise ConfigError(f"{where}: {heads} heads are not divisible by {groups} groups")
        if (heads * vdim) % parts:
            raise ConfigError(f"{where}: {heads * vdim} channels are not divisible into {parts} normed parts")
        return cls(heads, vdim, state, groups, conv, parts)

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups,
                "conv": self.conv, "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class DenseFeedForwardConfig:
    ff: int
    kind: str = "dense"

    def to_dict(self) -> dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class ExpertsFeedForwardConfig:
    experts: int
    top: int
    expert_ff: int
    limit: float  # clamp of the experts' gate and up values
    kind: str = "moe"

    def to_dict(self) -> dict[str, Any]:
        return {
            "kind": "moe",
            "expert": {"ff": self.expert_ff, "limit": self.limit},
            "router": {"experts": self.experts, "top": self.top},
        }


def _feed_forward(where: str, data: Mapping[str, Any]):
    if not isinstance(data, Mapping):
        raise ConfigError(f"{where} must be an object or null")
    kind = data.get("kind", "dense")
    if kind == "dense":
        return DenseFeedForwardConfig(_positive(where, data, "ff"))
    if kind == "moe":
        router, expert = data.get("router"), data.get("expert")
        experts = _positive(where + ".router", router, "experts")
        top = _positive(where + ".router", router, "top")
        if top > experts:
            raise ConfigError(f"{where}.router: a token cannot use {top} of {experts} experts")
        limit = _number(where + ".expert", expert, "limit")
        if not limit > 0:
            raise ConfigError(f"{where}.expert: limit must be positive, got {limit}")
        return ExpertsFeedForwardConfig(experts, top, _positive(where + ".expert", expert, "ff"), limit)
    raise ConfigError(f"{where}: feed-forward kind {kind!r} is not one of {', '.join(FEED_FORWARD_KINDS)}")


_MIXER_CONFIGS = {"attention": CappedAttentionConfig, "wkv": WkvConfig, "mamba2": StateSpaceConfig}


@dataclass(frozen=True)
class FomunexLayerConfig:
    type: str  # one of MIXER_TYPES
    mixer: CappedAttentionConfig | WkvConfig | StateSpaceConfig
    mlp: DenseFeedForwardConfig | ExpertsFeedForwardConfig | None
    weights_of: int | None = None  # the layer whose tensors this one uses

    def to_dict(self) -> dict[str, Any]:
        out = {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out


@dataclass(frozen=True)
class FomunexConfig:
    architecture: str
    width: int
    vocab: int
    max_positions: int  # rows of the learned position table
    norm_eps: float
    logit_scale: float
    logit_softcap: float  # 0: no cap
    layers: tuple[FomunexLayerConfig, ...]
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
    def from_dict(cls, data: Mapping[str, Any], overrides: Mapping[str, Any] | None = None) -> "FomunexConfig":
        data = dict(data)
        if overrides:
            data.update(overrides)
        listed = data.get("layers")
        if not isinstance(listed, (list, tuple)) or not listed:
            raise ConfigError("config.json key 'layers' must list at least one layer")
        layers: list[FomunexLayerConfig] = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            kind = require(entry, "type", str)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}: mixer type {kind!r} is not one of {', '.join(MIXER_TYPES)}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, Mapping):
                raise ConfigError(f"{where}: 'mixer' must give the mixer's sizes")
            mlp = entry.get("mlp")
            layer = FomunexLayerConfig(
                kind, _MIXER_CONFIGS[kind].from_dict(where + ".mixer", mixer),
                _feed_forward(where + ".mlp", mlp) if mlp is not None else None,
                entry.get("weights_of"),
            )
            src = layer.weights_of
            if src is not None:
                if not isinstance(src, int) or isinstance(src, bool) or not 0 <= src < len(listed) or src == i:
                    raise ConfigError(f"{where}: weights_of must name another layer, got {src!r}")
            layers.append(layer)
        for i, layer in enumerate(layers):
            if layer.weights_of is None:
                continue
            owner = layers[cls._owner(layers, i)]
            if (owner.type, owner.mixer, owner.mlp) != (layer.type, layer.mixer, layer.mlp):
                raise ConfigError(f"layers[{i}] uses the tensors of layer {layer.weights_of} but differs from it")
        norm = data.get("norm") or {}
        eps = require(norm, "eps", float)
        if not eps > 0:
            raise ConfigError(f"norm.eps must be positive, got {eps!r}")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos))
        cap = float(data.get("logit_softcap") or 0.0)
        if cap < 0:
            raise ConfigError(f"logit_softcap must not be negative, got {cap}")
        return cls(
            architecture=require(data, "architecture", str),
            width=_positive("config.json", data, "width"),
            vocab=_positive("config.json", data, "vocab"),
            max_positions=_positive("config.json", data, "max_positions"),
            norm_eps=eps,
            logit_scale=float(data["logit_scale"]) if data.get("logit_scale") is not None else 1.0,
            logit_softcap=cap,
            layers=tuple(layers),
            torch_dtype=normalise_dtype_name(data.get("torch_dtype") or data.get("dtype") or "bfloat16"),
            eos_token_ids=eos_ids,
        )

    @staticmethod
    def _owner(layers, i: int) -> int:
        """The layer whose tensors layer ``i`` runs: ``weights_of`` followed until a layer that has its own."""
        seen = set()
        while layers[i].weights_of is not None:
            if i in seen:
                raise ConfigError(f"layers[{i}]: weights_of leads back to the layer itself")
            seen.add(i)
            i = layers[i].weights_of
        return i

    def run_order(self) -> tuple[int, ...]:
        """For every place in the run order, the layer whose tensors run there."""
        return tuple(self._owner(self.layers, i) for i in range(len(self.layers)))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": self.architecture,
            "width": self.width,
            "vocab": self.vocab,
            "max_positions": self.max_positions,
            "norm": {"eps": self.norm_eps},
            "logit_scale": self.logit_scale,
            "layers": [layer.to_dict() for layer in self.layers],
            "torch_dtype": self.torch_dtype,
        }
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
