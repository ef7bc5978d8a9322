"""Small Fomunex configurations that differ in every size and option, and random weights for
them, made here tensor by tensor (names and shapes written out once more, independent of the
package's own list of parameters)."""

from __future__ import annotations

import json
import random
from pathlib import Path

import torch


def _attn(heads, kv_heads, dim, vdim, scale, window=None, softcap=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if softcap:
        m["softcap"] = softcap
    return m


def _wkv(heads, dim, rank):
    return {"heads": heads, "dim": dim, "rank": rank}


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def _layer(kind, mixer, mlp, weights_of=None):
    out = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


# A: grouped heads with value heads wider than the keys, a window of 19 and capped scores; a time
# mixing of three heads; a state-space layer of two groups, three taps and four normed parts
# without a feed-forward; then each of the first two once more with the same tensors and a cache
# or state of its own; a state-space layer of one group and four taps; two of six experts; pages of 8
FOMU_A = {
    "architecture": "Fomunex", "width": 96, "vocab": 211, "max_positions": 512, "norm": {"eps": 3e-6},
    "logit_scale": 0.7, "logit_softcap": 12.0,
    "layers": [
        _layer("attention", _attn(4, 2, 16, 32, 0.3, window=19, softcap=8.0), _dense(80)),
        _layer("wkv", _wkv(3, 16, 8), _moe(6, 2, 24, 2.0)),
        _layer("mamba2", _ssm(4, 16, 24, 2, 3, 4), None),
        _layer("attention", _attn(4, 2, 16, 32, 0.3, window=19, softcap=8.0), _dense(80), weights_of=0),
        _layer("wkv", _wkv(3, 16, 8), _moe(6, 2, 24, 2.0), weights_of=1),
        _layer("mamba2", _ssm(2, 32, 16, 1, 4, 1), _dense(48)),
    ],
}
PAGE_A = 8

# B: the smallest of everything: one head, attention that sees every key and has no cap, a window
# of the own key alone, one expert, a convolution of a single tap, a state of one number, logits
# neither scaled nor capped, pages of 4
FOMU_B = {
    "architecture": "Fomunex", "width": 64, "vocab": 130, "max_positions": 200, "norm": {"eps": 1e-6},
    "logit_scale": 1.0,
    "layers": [
        _layer("attention", _attn(1, 1, 16, 16, 0.25), _moe(1, 1, 16, 1.0)),
        _layer("mamba2", _ssm(1, 16, 1, 1, 1, 1), _dense(16)),
        _layer("wkv", _wkv(1, 32, 1), None),
        _layer("attention", _attn(2, 2, 16, 16, 0.2, window=1, softcap=50.0), _moe(3, 1, 32, 0.5)),
    ],
}
PAGE_B = 4

# C: sizes that no vector access divides and that lie between the matrix cores' steps: heads of
# 24 with values of 10, a time mixing of 20 channels a head and a decay of rank 3, states of 12
# with heads of 10 in three groups and five normed parts that cut through heads, experts of 27
# hidden units of which three of five are used, width 100, vocabulary 97, pages of 8
FOMU_C = {
    "architecture": "Fomunex", "width": 100, "vocab": 97, "max_positions": 300, "norm": {"eps": 1e-5},
    "logit_scale": 1.3, "logit_softcap": 20.0,
    "layers": [
        _layer("mamba2", _ssm(6, 10, 12, 3, 2, 5), _moe(5, 3, 27, 1.5)),
        _layer("attention", _attn(6, 3, 24, 10, 0.2, window=33, softcap=15.0), _dense(50)),
        _layer("wkv", _wkv(5, 20, 3), _dense(36)),
        _layer("attention", _attn(3, 1, 12, 22, 0.3, window=9), None),
    ],
}
PAGE_C = 8

# D: heads of the sizes real models have: keys of 64 with values of 32 behind a window of 70, a
# time mixing with heads of 64, states of 64 with heads of 64 and eight taps, eight experts;
# the recurrent layers come first and the attention reads one kv head; pages of 16
FOMU_D = {
    "architecture": "Fomunex", "width": 128, "vocab": 300, "max_positions": 1024, "norm": {"eps": 2e-5},
    "logit_scale": 0.4, "logit_softcap": 25.0,
    "layers": [
        _layer("wkv", _wkv(2, 64, 16), _dense(160)),
        _layer("mamba2", _ssm(2, 64, 64, 1, 8, 2), _moe(8, 2, 32, 3.0)),
        _layer("attention", _attn(4, 1, 64, 32, 0.11, window=70, softcap=40.0), _dense(96)),
        _layer("wkv", _wkv(2, 64, 16), _dense(160), weights_of=0),
    ],
}
PAGE_D = 16

FOMU = {"A": (FOMU_A, PAGE_A, 601), "B": (FOMU_B, PAGE_B, 602), "C": (FOMU_C, PAGE_C, 603), "D": (FOMU_D, PAGE_D, 604)}


def tensor_shapes(cfg) -> dict[str, tuple[int, ...]]:
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "pos": (cfg["max_positions"], w), "final.norm": (), "head": (cfg["vocab"], w)}
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = ()
        if layer["type"] == "attention":
            out[p + "mix.q"] = (m["heads"] * m["dim"], w)
            out[p + "mix.k"] = (m["kv_heads"] * m["dim"], w)
            out[p + "mix.v"] = (m["kv_heads"] * m["vdim"], w)
            out[p + "mix.sink"] = (m["heads"],)
            out[p + "mix.o"] = (w, m["heads"] * m["vdim"])
        elif layer["type"] == "wkv":
            inner = m["heads"] * m["dim"]
            for s in "rkvgw":
                out[p + "mix.mu." + s] = (w,)
            for s in "rkvg":
                out[p + "mix." + s] = (inner, w)
            out[p + "mix.w1"] = (m["rank"], w)
            out[p + "mix.w2"] = (inner, m["rank"])
            out[p + "mix.w0"] = (inner,)
            out[p + "mix.u"] = (m["heads"], m["dim"])
            out[p + "mix.norm"] = (inner,)
            out[p + "mix.o"] = (w, inner)
        else:
            inner = m["heads"] * m["vdim"]
            channels = inner + 2 * m["groups"] * m["state"]
            out[p + "mix.in"] = (inner + channels + m["heads"], w)
            out[p + "mix.conv"] = (channels, m["conv"])
            out[p + "mix.conv.b"] = (channels,)
            for s in ("dt_bias", "A_log", "D"):
                out[p + "mix." + s] = (m["heads"],)
            out[p + "mix.norm"] = (inner,)
            out[p + "mix.o"] = (w, inner)
        mlp = layer["mlp"]
        if mlp is None:
            continue
        out[p + "norm2"] = ()
        if mlp["kind"] == "dense":
            out[p + "mlp.up"] = (mlp["ff"], w)
            out[p + "mlp.down"] = (w, mlp["ff"])
            out[p + "mlp.act"] = (4,)
        else:
            out[p + "mlp.router"] = (mlp["router"]["experts"], w)
            for e in range(mlp["router"]["experts"]):
                out[p + f"mlp.e{e}.gate"] = (mlp["expert"]["ff"], w)
                out[p + f"mlp.e{e}.up"] = (mlp["expert"]["ff"], w)
                out[p + f"mlp.e{e}.down"] = (w, mlp["expert"]["ff"])
    return out


def make_weights(cfg, seed: int, sharp: float = 1.0) -> dict[str, torch.Tensor]:
    """Weights as a bfloat16 checkpoint stores them.  Projections are drawn at the scale that keeps
    activations of order one.  The query projections are multiplied by ``sharp``, so that few keys
    carry a query's weight and a key lost at a window's edge moves the output; the sinks are of the
    size of the larger scores, so that a sink left out or scaled shows.  The router's rows are
    large, so that the experts' scores lie apart.  Decays are spread from fast to very slow (a
    token far back still counts in some channels); step sizes and the state-space decays likewise.
    Position vectors and the activation's four numbers are of order one."""
    gen = torch.Generator().manual_seed(seed)

    def normal(shape, std=1.0, mean=0.0):
        return mean + std * torch.randn(shape, generator=gen)

    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        fan = shape[-1] if len(shape) == 2 else 1
        if name in ("embed", "pos"):
            t = normal(shape, 0.5)
        elif last in ("norm1", "norm2", "norm") or name == "final.norm":
            t = normal(shape, 0.1, 1.0)
        elif ".mu." in name:
            t = torch.rand(shape, generator=gen)
        elif last == "sink":
            t = normal(shape, 1.5, 2.0)
        elif last == "router":
            t = normal(shape, 6.0 / fan**0.5)
        elif last == "q":
            t = normal(shape, 1.5 * sharp / fan**0.5)
        elif last == "w0":
            t = normal(shape, 1.5, -2.5)
        elif last == "w1":
            t = normal(shape, 1.0 / fan**0.5)
        elif last == "w2":
            t = normal(shape, 1.0 / fan**0.5)
        elif last == "u":
            t = normal(shape, 0.5)
        elif last == "conv":
            t = normal(shape, 0.6)
        elif name.endswith("conv.b"):
            t = normal(shape, 0.2)
        elif last == "dt_bias":
            t = normal(shape, 1.0, -1.0)
        elif last == "A_log":
            t = normal(shape, 1.0, -1.0)
        elif last == "D":
            t = normal(shape, 0.3, 1.0)
        elif last == "act":
            t = normal(shape, 0.4, 0.6)
        else:
            t = normal(shape, 1.5 / fan**0.5)
        out[name] = t
    return {name: t.to(torch.bfloat16) for name, t in out.items()}


def make_model_dir(tmp_path: Path, which: str, sharp: float = 1.0, cfg=None, seed: int | None = None) -> Path:
    from safetensors.torch import save_file

    base, _page, base_seed = FOMU[which]
    cfg = cfg or base
    out = Path(tmp_path) / f"fomu_{which}_{sharp}_{seed}"
    out.mkdir(parents=True, exist_ok=True)
    (out / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in make_weights(cfg, base_seed if seed is None else seed, sharp).items()},
              str(out / "model.safetensors"))
    return out


def load_plain(model_dir: Path):
    from safetensors.torch import load_file

    return json.loads((Path(model_dir) / "config.json").read_text()), load_file(str(Path(model_dir) / "model.safetensors"))


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


# --------------------------------------------------------------------------- #
# how a bfloat16 engine is compared
# --------------------------------------------------------------------------- #
# Where two experts' scores lie closer than rounding moves them, the rounded stream picks the other
# expert, in an engine as in the plain implementation with rounded activations, and that token's
# row moves by its whole feed-forward output (and, through the recurrent states, some later rows
# with it).  So the engine's typical rows are compared with the typical rows of the plain
# implementation with rounded activations, and a tenth of the rows may lie far out.
BF16_TIMES_ROUNDING = 3.0
BF16_ROWS_BEYOND = 0.1


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row the root mean square of ``got - want`` over the spread of ``want``."""
    return (got.double() - want.double()).square().mean(dim=1).sqrt() / float(want.double().std())


def rounding_figure(rounded: torch.Tensor, want: torch.Tensor) -> float:
    return float(row_errors(rounded, want).quantile(0.9))
