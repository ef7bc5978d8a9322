"""Small Miborax configurations that differ in every size and option, and random weights for
them, made here tensor by tensor (names and shapes written out once more, independent of the
package's own list of parameters)."""

from __future__ import annotations

import json
import random
from pathlib import Path

import torch


def _mix(heads, dim, rot_dim, vdim, kv_rank, scale, base, window=None, q_rank=None, kv_from=None, rot_dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}}
    if window:
        m["mask"] = {"size": window}
    if q_rank:
        m["q_rank"] = q_rank
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _windowed(mixer, mlp):
    return {"type": "latent_attention_2", "mixer": mixer, "mlp": mlp}


def _causal(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


# A: value heads wider and narrower than the unrotated key part, a rotated part wider and narrower
# than it, a latent narrower than a head's keys and wider than all of them; a window of 19; a reader
# of layer 0's rows with a longer window (41: the cache keeps the longer view) and other head
# counts, without a feed-forward; a layer with a window of 7 and a reader with the same window;
# a query latent narrower than the width; all experts chosen, one of three, two of six; pages of 8
MIBO_A = {
    "architecture": "Miborax", "width": 96, "vocab": 211, "embedding": {"scale": 7.5}, "norm": {"eps": 3e-6},
    "layers": [
        _windowed(_mix(4, 16, 32, 48, 32, 0.2, 10000.0, window=19), _moe(6, 2, 40)),
        _causal(_mix(3, 32, 16, 16, 80, 0.17, 500.0, q_rank=48), _moe(4, 4, 24)),
        _windowed(_mix(2, 48, 32, 16, 32, 0.15, 10000.0, window=41, kv_from=0), None),
        _windowed(_mix(5, 16, 16, 32, 16, 0.3, 77.0, window=7), _moe(3, 1, 32)),
        _windowed(_mix(3, 32, 16, 16, 16, 0.25, 77.0, window=7, kv_from=3), _moe(6, 2, 40)),
    ],
}
PAGE_A = 8

# B: the smallest of everything: one head, one expert, a window of the own key alone, a window of
# five read from that layer's rows, a query latent as wide as the model, no scaling of the
# embedding, pages of 4
MIBO_B = {
    "architecture": "Miborax", "width": 64, "vocab": 130, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
    "layers": [
        _causal(_mix(1, 16, 16, 16, 16, 0.25, 10000.0, q_rank=64), _moe(1, 1, 16)),
        _windowed(_mix(2, 16, 16, 32, 32, 0.2, 100.0, window=1), _moe(3, 1, 32)),
        _windowed(_mix(1, 32, 16, 16, 32, 0.2, 100.0, window=5, kv_from=1), _moe(2, 2, 16)),
    ],
}
PAGE_B = 4

# C: rows of 128 and 160 channels, eight heads, windows of 64 and 130 (longer than most requests),
# a windowed layer that reads the rows of a layer that sees everything (the cache keeps all), the
# layer that sees everything comes first, no feed-forward in the last layer, pages of 16
MIBO_C = {
    "architecture": "Miborax", "width": 128, "vocab": 300, "embedding": {"scale": 11.0}, "norm": {"eps": 2e-5},
    "layers": [
        _causal(_mix(8, 32, 32, 16, 96, 0.11, 50000.0, q_rank=32), _moe(8, 3, 48)),
        _windowed(_mix(4, 64, 32, 64, 96, 0.09, 50000.0, window=64, kv_from=0), _moe(5, 2, 32)),
        _windowed(_mix(2, 16, 16, 128, 144, 0.12, 1000.0, window=130), None),
    ],
}
PAGE_C = 16

# D: sizes that no vector access divides and that lie between the matrix cores' steps (a latent of
# 18 channels with a rotated part of 6 of which 4 rotate, heads of 10 + 6 with values of 22, width
# 100, vocabulary 97, experts of 27 and 9 hidden units): every kernel takes its element-by-element
# path and the bfloat16 products go to the library
MIBO_D = {
    "architecture": "Miborax", "width": 100, "vocab": 97, "embedding": {"scale": 10.0}, "norm": {"eps": 1e-5},
    "layers": [
        _windowed(_mix(5, 10, 6, 22, 18, 0.3, 300.0, window=33, rot_dims=4), _moe(5, 2, 27)),
        _causal(_mix(3, 12, 10, 6, 26, 0.2, 10000.0, q_rank=14), _moe(2, 1, 9)),
        _windowed(_mix(2, 6, 6, 10, 18, 0.35, 300.0, window=9, kv_from=0, rot_dims=4), _moe(5, 2, 27)),
    ],
}
PAGE_D = 8

MIBO = {"A": (MIBO_A, PAGE_A, 501), "B": (MIBO_B, PAGE_B, 502), "C": (MIBO_C, PAGE_C, 503), "D": (MIBO_D, PAGE_D, 504)}


def tensor_shapes(cfg) -> dict[str, tuple[int, ...]]:
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "final.norm": (w,), "final.norm.b": (w,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        heads, per_head = m["heads"], m["dim"] + m["rot_dim"]
        out[p + "norm1"] = (w,)
        out[p + "norm1.b"] = (w,)
        if layer["type"] == "latent_attention":
            out[p + "mix.dq"] = (m["q_rank"], w)
            out[p + "mix.dq.norm"] = (m["q_rank"],)
            out[p + "mix.uq"] = (heads * per_head, m["q_rank"])
            out[p + "mix.g"] = (heads, w)
        else:
            out[p + "mix.q"] = (heads * per_head, w)
        if "kv_from" not in m:
            out[p + "mix.dkv"] = (m["kv_rank"] + m["rot_dim"], w)
            out[p + "mix.dkv.norm"] = (m["kv_rank"],)
        out[p + "mix.uk"] = (heads * m["dim"], m["kv_rank"])
        out[p + "mix.uv"] = (heads * m["vdim"], m["kv_rank"])
        out[p + "mix.sink"] = (heads,)
        out[p + "mix.o"] = (w, heads * m["vdim"])
        mlp = layer["mlp"]
        if mlp is None:
            continue
        out[p + "norm2"] = (w,)
        out[p + "norm2.b"] = (w,)
        out[p + "mlp.router"] = (mlp["router"]["experts"], w)
        out[p + "mlp.router.b"] = (mlp["router"]["experts"],)
        for e in range(mlp["router"]["experts"]):
            out[p + f"mlp.e{e}.gate"] = (mlp["expert"]["ff"], w)
            out[p + f"mlp.e{e}.up"] = (mlp["expert"]["ff"], w)
            out[p + f"mlp.e{e}.down"] = (w, mlp["expert"]["ff"])
    return out


def make_weights(cfg, seed: int, sharp: float = 1.0) -> dict[str, torch.Tensor]:
    """Weights as a bfloat16 checkpoint stores them.  Projections are drawn at the scale that
    keeps activations of order one; the router's rows are large and its biases of order one, so
    that the experts' logits lie far apart and both terms decide choices; the query
    projections are multiplied by ``sharp``: few keys then carry each query's weight, and a key
    lost at a window's edge moves the output; the sinks are of the size of the larger scores, so that
    a sink left out or scaled shows; norm biases and head gates are of order one."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            t = torch.randn(shape, generator=gen) * 0.5
        elif last == "b" and "norm" in name:
            t = 0.3 * torch.randn(shape, generator=gen)
        elif last == "b":  # the router's bias
            t = torch.randn(shape, generator=gen)
        elif last == "norm" or last in ("norm1", "norm2"):
            t = 1.0 + 0.1 * torch.randn(shape, generator=gen)
        elif last == "sink":
            t = 2.0 + 1.5 * torch.randn(shape, generator=gen)
        elif last == "router":
            t = torch.randn(shape, generator=gen) * (6.0 / shape[-1] ** 0.5)
        elif last in ("q", "uq"):
            t = torch.randn(shape, generator=gen) * (1.5 * sharp / shape[-1] ** 0.5)
        elif last == "g":
            t = torch.randn(shape, generator=gen) * (2.0 / shape[-1] ** 0.5)
        else:
            t = torch.randn(shape, generator=gen) * (1.5 / shape[-1] ** 0.5)
        out[name] = t
    return {name: t.to(torch.bfloat16) for name, t in out.items()}


def make_model_dir(tmp_path: Path, which: str, sharp: float = 1.0, cfg=None, seed: int | None = None) -> Path:
    from safetensors.torch import save_file

    base, _page, base_seed = MIBO[which]
    cfg = cfg or base
    out = Path(tmp_path) / f"mibo_{which}_{sharp}_{seed}"
    out.mkdir(parents=True, exist_ok=True)
    (out / "config.json").write_text(json.dumps(cfg))
    save_file(make_weights(cfg, base_seed if seed is None else seed, sharp), str(out / "model.safetensors"))
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
# Where two experts' router logits lie closer than rounding moves them, the rounded stream picks
# the other expert, in an engine as in the plain implementation with rounded activations, and that
# token's row moves by its whole feed-forward output.  With random weights this happens to about
# one token in a hundred and cannot be designed away (logits and their rounding scale together).
# So rows are compared with what rounding does to nine rows in ten, and a few rows may lie beyond
# (one in fifty, or twice as many as in the plain implementation with rounded activations):
# a fault in a mechanism moves many rows (the CPU tests show how many), and one wrong row among
# many is what the float32 comparison and the kernel tests with keys made to stand out are for.
BF16_TIMES_ROUNDING = 3.0
BF16_ROWS_BEYOND = 0.02


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row the root mean square of ``got - want`` over the spread of ``want``."""
    return (got.double() - want.double()).square().mean(dim=1).sqrt() / float(want.double().std())


def rounding_figure(rounded: torch.Tensor, want: torch.Tensor) -> float:
    return float(row_errors(rounded, want).quantile(0.9))


def share_beyond(got: torch.Tensor, want: torch.Tensor, figure: float) -> float:
    """The share of rows that are off by more than the bound allows."""
    return float((row_errors(got, want) > BF16_TIMES_ROUNDING * figure).double().mean())
