"""Call wrappers around the HIP kernels: host-side checks, then one launch on the current stream.

Nothing here computes: every function validates its operands (device, type, contiguity,
shape) and hands raw pointers to the compiled library.  There is no fallback; without a
GPU or without the compiled library these raise.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from . import build
from .upload import upload_ints

F32, BF16 = 0, 1
_TAG = {torch.float32: F32, torch.bfloat16: BF16}

_core: ctypes.CDLL | None = None
_attn: dict[int, ctypes.CDLL] = {}
_mlstm: ctypes.CDLL | None = None


class KernelError(RuntimeError):
    pass


class Chip:
    """What the launch rules know about the device: its number of compute units, read once on
    the host (the kernels that decide by it are handed the same number), and what follows
    from it.  Without a device the rules are asked about the chip they were measured on."""

    def __init__(self, units: int) -> None:
        if units < 1:
            raise KernelError(f"a chip has at least one compute unit, got {units}")
        self.units = units
        self.first_round = units  # workgroups that start first, one on each compute unit
        self.decode_resident = 3 * units  # decode-attention workgroups the chip holds at a time
        self.prefill_slots = 2 * units  # wave groups of four the prefill kernel keeps at a time


MEASURED_CHIP = Chip(256)  # MI355X
_chips: dict[int, Chip] = {}


def chip() -> Chip:
    """The current device's geometry (the measured chip's where no device is visible)."""
    if not torch.cuda.is_available():
        return MEASURED_CHIP
    dev = torch.cuda.current_device()
    found = _chips.get(dev)
    if found is None:
        found = _chips[dev] = Chip(torch.cuda.get_device_properties(dev).multi_processor_count)
    return found


def require_gpu() -> None:
    if not torch.cuda.is_available():
        raise KernelError(
            "rapid_llm_amd runs its model on a HIP device only (no CPU implementation exists) "
            "and no GPU is visible to this process"
        )


def core() -> ctypes.CDLL:
    global _core
    if _core is None:
        _core = build.load(build.core_library())
    return _core


def attention_lib(head_dim: int) -> ctypes.CDLL:
    lib = _attn.get(head_dim)
    if lib is None:
        lib = build.load(build.attention_library(head_dim))
        if lib.rl_attn_head_dim() != head_dim:
            raise KernelError(f"attention library for head size {head_dim} reports {lib.rl_attn_head_dim()}")
        _attn[head_dim] = lib
    return lib


_attn_tile: dict[tuple[int, int], ctypes.CDLL] = {}


def attention_tile_lib(head_dim: int, value_dim: int) -> ctypes.CDLL:
    lib = _attn_tile.get((head_dim, value_dim))
    if lib is None:
        lib = build.load(build.attention_tile_library(head_dim, value_dim))
        if (lib.rl_attn_tile_head_dim(), lib.rl_attn_tile_value_dim()) != (head_dim, value_dim):
            raise KernelError(f"tile attention library for head sizes {head_dim} / {value_dim} reports others")
        _attn_tile[(head_dim, value_dim)] = lib
    return lib


def mlstm_lib() -> ctypes.CDLL:
    global _mlstm
    if _mlstm is None:
        _mlstm = build.load(build.mlstm_library())
        if _mlstm.rl_mlstm_max_key_dim() != MLSTM_MAX_KEY_DIM:
            raise KernelError(
                f"the recurrence library takes key sizes up to {_mlstm.rl_mlstm_max_key_dim()}, "
                f"the launch rules expect {MLSTM_MAX_KEY_DIM}"
            )
    return _mlstm


_recurrent: ctypes.CDLL | None = None


def recurrent_lib() -> ctypes.CDLL:
    global _recurrent
    if _recurrent is None:
        _recurrent = build.load(build.recurrent_library())
        if _recurrent.rl_recurrent_max_head_dim() != WKV_MAX_HEAD_DIM or _recurrent.rl_conv_max_taps() != CONV_MAX_TAPS:
            raise KernelError("the recurrence library's limits are not the launch rules'")
    return _recurrent


def _stream() -> ctypes.c_void_p:
    # the raw handle of the current stream of the current device, without the stream object
    # that ``torch.cuda.current_stream()`` builds (2.8 against 0.2 us a call, on every launch)
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _tag(dtype: torch.dtype) -> int:
    try:
        return _TAG[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, got {dtype}") from None


def _need(t: torch.Tensor, name: str, dtype: torch.dtype | None = None, shape=None) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name} must live on the GPU, is on {t.device}")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous (shape {tuple(t.shape)}, strides {t.stride()})")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, is {t.dtype}")
    if shape is not None:
        have = t.shape
        if len(shape) != len(have):
            raise KernelError(f"{name} must have shape {tuple(shape)}, has {tuple(have)}")
        for want, size in zip(shape, have):
            if want is not None and want != size:
                raise KernelError(f"{name} must have shape {tuple(shape)}, has {tuple(have)}")


def _ok(code: int, what: str) -> None:
    if code != 0:
        reason = {1: "an argument the kernel refuses", 2: "the launch failed"}.get(code, "unknown")
        raise KernelError(f"{what}: error {code} ({reason})")


# --------------------------------------------------------------------------- #


def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, fed: Optional[torch.Tensor] = None,
          scale: float = 1.0, positions: Optional[torch.Tensor] = None,
          inv_freq: Optional[torch.Tensor] = None, pos_table: Optional[torch.Tensor] = None) -> None:
    """``out[t] = table[ids[t]] * scale``; an id ``-(r + 1)`` takes ``fed[r]``, the token a
    sampling kernel chose in row ``r`` of the previous step.  With ``inv_freq`` (float32, one
    frequency per pair of channels) the sinusoidal vector of ``positions[t]`` is added: channel
    ``2i`` gets the sine, ``2i + 1`` the cosine of the float32 product ``positions[t] * inv_freq[i]``.
    With ``pos_table`` (rows of the table's type) row ``positions[t]`` is added, unscaled; the
    caller checks that every position has a row."""
    tokens = ids.numel()
    vocab, hidden = table.shape
    _need(ids, "ids", torch.int32)
    _need(table, "embedding table")
    _need(out, "out", torch.float32, (tokens, hidden))
    if fed is not None:
        _need(fed, "fed", torch.int32)
    if inv_freq is not None:
        _need(inv_freq, "inv_freq", torch.float32, ((hidden + 1) // 2,))
        if positions is None:
            raise KernelError("a sinusoidal position vector needs the tokens' positions")
        _need(positions, "positions", torch.int32, (tokens,))
    if pos_table is not None:
        _need(pos_table, "position table", table.dtype, (None, hidden))
        if positions is None:
            raise KernelError("learned position vectors need the tokens' positions")
        _need(positions, "positions", torch.int32, (tokens,))
    with_positions = inv_freq is not None or pos_table is not None
    _ok(
        core().rl_embed(
            _p(ids), _p(fed), 0 if fed is None else fed.numel(), _p(table), _tag(table.dtype), _p(out),
            tokens, hidden, vocab, ctypes.c_float(scale), _p(positions if with_positions else None),
            _p(inv_freq), _p(pos_table), 0 if pos_table is None else pos_table.shape[0], _stream(),
        ),
        "rl_embed",
    )


def read_buffer(buf: torch.Tensor, blocks: int = 4096) -> None:
    """Stream a buffer through the compute units once (a measurement of read bandwidth)."""
    if not buf.is_cuda or not buf.is_contiguous():
        raise KernelError("read_buffer takes a contiguous GPU tensor")
    sink = torch.zeros(1, dtype=torch.int32, device=buf.device)
    _ok(
        core().rl_read_buffer(_p(buf), ctypes.c_size_t(buf.numel() * buf.element_size()), _p(sink), blocks, _stream()),
        "rl_read_buffer",
    )


def add_rmsnorm(
    residual: torch.Tensor,
    delta: Optional[torch.Tensor],
    weight: torch.Tensor,
    out: torch.Tensor,
    eps: float,
    rows: Optional[torch.Tensor] = None,
) -> None:
    tokens, hidden = residual.shape
    _need(residual, "residual", torch.float32)
    _need(weight, "norm weight", torch.float32, (hidden,))
    out_rows = tokens if rows is None else rows.numel()
    _need(out, "out", None, (out_rows, hidden))
    if delta is not None:
        _need(delta, "delta", out.dtype, (tokens, hidden))
    if rows is not None:
        _need(rows, "rows", torch.int32)
    _ok(
        core().rl_add_rmsnorm(
            _p(residual), _p(delta), _p(weight), _p(out), _p(rows), out_rows, hidden,
            ctypes.c_float(eps), _tag(out.dtype), _stream(),
        ),
        "rl_add_rmsnorm",
    )


def normed_add_rmsnorm(
    residual: torch.Tensor,
    y: torch.Tensor,
    y_weight: torch.Tensor,
    y_eps: float,
    weight: Optional[torch.Tensor],
    out: Optional[torch.Tensor],
    eps: float,
    rows: Optional[torch.Tensor] = None,
) -> None:
    """``residual += rmsnorm(y) * y_weight`` (float32, in place), then, unless ``out`` is ``None``,
    ``out = rmsnorm(residual) * weight``: a sub-layer's output that passes a norm of its own on
    its way into the stream, and the next sub-layer's norm, in one kernel.  ``rows`` as in
    :func:`add_rmsnorm`."""
    tokens, hidden = residual.shape
    _need(residual, "residual", torch.float32)
    _need(y, "y", None, (tokens, hidden))
    _need(y_weight, "norm weight of y", torch.float32, (hidden,))
    out_rows = tokens if rows is None else rows.numel()
    if out is not None:
        _need(out, "out", y.dtype, (out_rows, hidden))
        _need(weight, "norm weight", torch.float32, (hidden,))
    if rows is not None:
        _need(rows, "rows", torch.int32)
    _ok(
        core().rl_normed_add_rmsnorm(
            _p(residual), _p(y), _p(y_weight), ctypes.c_float(y_eps), _p(weight if out is not None else None),
            _p(out), _p(rows), out_rows, hidden, ctypes.c_float(eps), _tag(y.dtype), _stream(),
        ),
        "rl_normed_add_rmsnorm",
    )


def pair_rows(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> None:
    """``out[t] = [a[t] | b[t]]``: two float32 streams side by side in ``out``'s type."""
    tokens, hidden = a.shape
    _need(a, "a", torch.float32)
    _need(b, "b", torch.float32, (tokens, hidden))
    _need(out, "out", None, (tokens, 2 * hidden))
    _ok(core().rl_pair_rows(_p(a), _p(b), _p(out), tokens, hidden, _tag(out.dtype), _stream()), "rl_pair_rows")


UNARY_ACTIVATIONS = {"gelu_tanh": 0, "relu_squared": 1, "tanh": 2}


def unary_act(x: torch.Tensor, out: torch.Tensor, kind: str, route: Optional[torch.Tensor] = None,
              expert_ff: int = 0) -> None:
    """``out = act(x)`` for a one-operand activation (:data:`UNARY_ACTIVATIONS`).  With ``route``
    (float32 ``[tokens, experts]``) the first ``experts * expert_ff`` columns are the hidden units
    of the experts side by side and expert ``e``'s are multiplied by ``route[t, e]``."""
    if kind not in UNARY_ACTIVATIONS:
        raise KernelError(f"activation {kind!r} is not one of {sorted(UNARY_ACTIVATIONS)}")
    tokens, cols = x.shape
    _need(x, "x")
    _need(out, "out", x.dtype, (tokens, cols))
    experts = 0
    if route is not None:
        experts = route.shape[1]
        _need(route, "route", torch.float32, (tokens, experts))
        if expert_ff < 1 or experts * expert_ff > cols:
            raise KernelError(f"{experts} experts of {expert_ff} hidden units do not fit rows of {cols}")
    _ok(
        core().rl_unary_act(_p(x), _p(out), tokens, cols, UNARY_ACTIVATIONS[kind], _p(route), experts, expert_ff,
                            _tag(x.dtype), _stream()),
        "rl_unary_act",
    )


ROUTE_MAX_EXPERTS = 1024


def route(logits: torch.Tensor, top: int, scale: float) -> None:
    """In place: router logits ``[tokens, experts]`` (float32) become the experts' weights: the
    softmax scores of the ``top`` largest, divided by their sum (+ 1e-20), times ``scale``; 0
    for every other expert."""
    tokens, experts = logits.shape
    _need(logits, "router logits", torch.float32)
    if not 1 <= top <= experts <= ROUTE_MAX_EXPERTS:
        raise KernelError(f"the router kernel chooses 1 to {experts} of at most {ROUTE_MAX_EXPERTS} experts, not {top}")
    _ok(core().rl_route(_p(logits), tokens, experts, top, ctypes.c_float(scale), _stream()), "rl_route")


ROUTER_SCORES = {"softmax": 0, "sigmoid": 1}


def router(x: torch.Tensor, w: torch.Tensor, top: int, scale: float, bias: Optional[torch.Tensor] = None,
           scores: str = "softmax") -> torch.Tensor:
    """The experts' weights ``[tokens, experts]`` (float32) of rows ``x`` under the float32 router
    matrix ``w [experts, k]``: the product in float32 (plus ``bias``, one number an expert),
    softmax over all experts, the ``top`` largest scores over their sum (+ 1e-20) times ``scale``
    (which is the softmax over the chosen logits alone), 0 elsewhere.  With ``scores="sigmoid"`` an
    expert's score is the sigmoid of its logit and a chosen expert's weight is its score times
    ``scale``, not divided by anything.  One kernel; a token's result does not depend on the rest
    of the step."""
    if scores not in ROUTER_SCORES:
        raise KernelError(f"router scores are one of {sorted(ROUTER_SCORES)}, not {scores!r}")
    tokens, k = x.shape
    experts = w.shape[0]
    _need(x, "x")
    _need(w, "router matrix", torch.float32, (experts, k))
    if not 1 <= top <= experts <= ROUTE_MAX_EXPERTS:
        raise KernelError(f"the router kernel chooses 1 to {experts} of at most {ROUTE_MAX_EXPERTS} experts, not {top}")
    if bias is not None:
        _need(bias, "router bias", torch.float32, (experts,))
    out = torch.empty((tokens, experts), dtype=torch.float32, device=x.device)
    _ok(core().rl_router(_p(x), _p(w), _p(out), tokens, k, experts, top, ctypes.c_float(scale), _p(bias),
                         ROUTER_SCORES[scores], _tag(x.dtype), _stream()),
        "rl_router")
    return out


GLU_ALPHA = 1.702  # the sigmoid's slope in the clamped gated activation


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, limit: float = 0.0, alpha: float = GLU_ALPHA,
           route: Optional[torch.Tensor] = None, expert_ff: int = 0, route_input: bool = False) -> None:
    """The gated activation of a packed ``[gate | up]`` row.  ``limit`` 0: ``silu(g) * u``.
    ``limit > 0``: ``g' * sigmoid(alpha g') * (u' + 1)`` with ``g' = min(g, limit)`` and
    ``u' = clamp(u, -limit, limit)``.  With ``route`` (float32 ``[tokens, experts]``) the first
    ``experts * expert_ff`` hidden units are those of the experts side by side and expert ``e``'s
    are multiplied by ``route[t, e]``; with ``route_input`` its gate and up values are, before the
    activation (the expert read a scaled input)."""
    if route_input and route is None:
        raise KernelError("scaling the experts' inputs needs their weights")
    tokens, two_i = gate_up.shape
    if limit < 0:
        raise KernelError(f"the gated activation's limit must not be negative, got {limit}")
    if two_i % 2:
        raise KernelError(f"the packed [gate | up] row must have even width, has {two_i}")
    _need(gate_up, "gate_up")
    _need(out, "out", gate_up.dtype, (tokens, two_i // 2))
    experts = 0
    if route is not None:
        experts = route.shape[1]
        _need(route, "route", torch.float32, (tokens, experts))
        if expert_ff < 1 or experts * expert_ff > two_i // 2:
            raise KernelError(f"{experts} experts of {expert_ff} hidden units do not fit rows of {two_i // 2}")
    _ok(
        core().rl_swiglu(
            _p(gate_up), _p(out), tokens, two_i // 2, _tag(out.dtype), ctypes.c_float(limit),
            ctypes.c_float(alpha), _p(route), experts, int(expert_ff), int(bool(route_input)), _stream(),
        ),
        "rl_swiglu",
    )


def polynorm(x: torch.Tensor, out: torch.Tensor, coefficients: torch.Tensor, eps: float) -> None:
    """``out = a N(x) + b N(x^2) + c N(x^3) + e`` row by row, with element-wise powers, ``N``
    dividing a row by its root mean square (``eps`` inside the root) and ``coefficients`` =
    ``(a, b, c, e)`` float32; sums and statistics float32.  ``out`` may be ``x``."""
    tokens, cols = x.shape
    _need(x, "x")
    _need(out, "out", x.dtype, (tokens, cols))
    _need(coefficients, "coefficients", torch.float32, (4,))
    _ok(core().rl_polynorm(_p(x), _p(out), tokens, cols, _p(coefficients), ctypes.c_float(eps), _tag(x.dtype),
                           _stream()),
        "rl_polynorm")


def scale_cap(values: torch.Tensor, scale: float, cap: float) -> None:
    """In place on a float32 tensor: ``v * scale`` and then, with ``cap`` > 0, ``cap * tanh(v / cap)``."""
    _need(values, "values", torch.float32)
    if cap < 0:
        raise KernelError(f"a cap must not be negative, got {cap}")
    _ok(core().rl_scale_cap(_p(values), ctypes.c_size_t(values.numel()), ctypes.c_float(scale),
                            ctypes.c_float(cap), _stream()),
        "rl_scale_cap")


def cast(src: torch.Tensor, dst: torch.Tensor) -> None:
    _need(src, "src")
    _need(dst, "dst")
    if src.numel() != dst.numel():
        raise KernelError(f"cast of {src.numel()} elements into {dst.numel()}")
    _ok(
        core().rl_cast(
            _p(src), _tag(src.dtype), _p(dst), _tag(dst.dtype), ctypes.c_size_t(src.numel()), _stream()
        ),
        "rl_cast",
    )


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> None:
    """``y[r, :] += bias`` in place (``bias`` float32)."""
    rows, cols = y.shape
    _need(y, "y")
    _need(bias, "bias", torch.float32, (cols,))
    _ok(core().rl_add_bias(_p(y), _p(bias), rows, cols, _tag(y.dtype), _stream()), "rl_add_bias")


def head_gate(y: torch.Tensor, packed: torch.Tensor, gate_col: int, heads: int, d: int) -> None:
    """``y[t, h, :] *= sigmoid(packed[t, gate_col + h])`` in place: one gate a head, read from
    the columns ``gate_col .. gate_col + heads`` of the mixer's packed projection."""
    tokens = y.shape[0]
    _need(y, "y", None, (tokens, heads * d))
    _need(packed, "packed", y.dtype, (tokens, None))
    if not 0 <= gate_col <= packed.shape[1] - heads:
        raise KernelError(f"gate columns {gate_col}..{gate_col + heads} lie outside rows of {packed.shape[1]}")
    _ok(
        core().rl_head_gate(_p(y), _p(packed), packed.shape[1], gate_col, tokens, heads, d, _tag(y.dtype), _stream()),
        "rl_head_gate",
    )


def rope_table(inv_freq: torch.Tensor, positions: int) -> tuple[torch.Tensor, torch.Tensor]:
    _need(inv_freq, "inv_freq", torch.float32)
    half = inv_freq.numel()
    cos = torch.empty((positions, half), dtype=torch.float32, device=inv_freq.device)
    sin = torch.empty_like(cos)
    _ok(core().rl_rope_table(_p(inv_freq), _p(cos), _p(sin), positions, half, _stream()), "rl_rope_table")
    return cos, sin


# which channels of a head form a rotated pair, as the kernels number them: channel i with
# i + (rotated channels) / 2, or channel 2i with 2i + 1
ROTARY_PAIRINGS = {"half_split": 0, "interleaved": 1}


def qknorm_rope_kvwrite(
    qkv: torch.Tensor,
    q_out: Optional[torch.Tensor],
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    q_norm_w: Optional[torch.Tensor],
    k_norm_w: Optional[torch.Tensor],
    cos: Optional[torch.Tensor],
    sin: Optional[torch.Tensor],
    positions: torch.Tensor,
    token_slot: torch.Tensor,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    eps: float,
    max_position: int,
    pairing: str = "half_split",
    value_head0: Optional[int] = None,
    bias: Optional[torch.Tensor] = None,
    value_dim: Optional[int] = None,
) -> None:
    """Norm + rotate q and k, write k and v to the cache pages (skipped when the caches
    are ``None``: a layer that reads another layer's cache).  ``q_out`` ``None``: the query
    heads are left as they are (the attention kernels finish them themselves, see
    :func:`attention_prepares_queries`).  ``max_position`` is the
    largest position in the batch, checked against the rotation table and block table.
    The tables' width says how many channels rotate (``2 * cos.shape[1]``, the first of a
    head), ``pairing`` which of them form a pair (:data:`ROTARY_PAIRINGS`).

    A packed row holds the query heads, then the key heads, and the value heads from head
    ``value_head0`` on (default ``nq + nkv``, right behind the keys; ``nq``: the values are the
    keys as projected, before the rotation); it may be wider than that (columns of the same
    product that another kernel reads).  ``value_dim``: the size of a value head where it is not
    ``d`` (the values then lie behind the keys).  ``bias`` (float32, one entry a column of the packed
    row): the projection's bias, added to the heads as they are read, before norm and rotation,
    instead of by a kernel of its own after the product."""
    if pairing not in ROTARY_PAIRINGS:
        raise KernelError(f"rotation pairing {pairing!r} is not one of {sorted(ROTARY_PAIRINGS)}")
    tokens = qkv.shape[0]
    if value_head0 is None:
        value_head0 = nq + nkv
    dv = d if value_dim is None else int(value_dim)
    if dv != d and value_head0 != nq + nkv:
        raise KernelError("value heads of a size of their own lie behind the keys")
    value_col0 = value_head0 * d
    _need(qkv, "qkv", None, (tokens, None))
    row_width = qkv.shape[1]
    if (value_head0 < 0 or not 1 <= dv <= 256 or row_width < max(value_col0 + nkv * dv, (nq + nkv) * d)
            or (d % 8 == 0 and row_width % 8)):
        # (heads in steps of 8 channels are read 8 or 16 bytes at a time, so rows must start aligned)
        raise KernelError(
            f"packed rows of {row_width} columns do not hold {nq} query and {nkv} key heads of {d} and {nkv} "
            f"value heads of {dv} (values from column {value_col0}) in whole groups of 8 columns"
        )
    if q_out is not None:
        _need(q_out, "q_out", qkv.dtype, (tokens, nq * d))
    _need(positions, "positions", torch.int32, (tokens,))
    _need(token_slot, "token_slot", torch.int32, (tokens,))
    _need(block_table, "block_table", torch.int32)
    write = k_cache is not None
    if write:
        pages = k_cache.shape[0]
        _need(k_cache, "k_cache", qkv.dtype, (pages, nkv, page_size, d))
        _need(v_cache, "v_cache", qkv.dtype, (pages, nkv, dv, page_size))
        if max_position // page_size >= block_table.shape[1]:
            raise KernelError(
                f"position {max_position} needs page {max_position // page_size} of a block "
                f"table with {block_table.shape[1]} columns"
            )
    for w, name in ((q_norm_w, "q_norm weight"), (k_norm_w, "k_norm weight")):
        if w is not None:
            _need(w, name, torch.float32, (d,))
    half = 0
    if cos is not None:
        half = cos.shape[1]
        _need(cos, "cos table", torch.float32, (None, half))
        _need(sin, "sin table", torch.float32, tuple(cos.shape))
        if not 1 <= half <= d // 2:
            raise KernelError(f"rotation tables of {half} pairs do not fit a head of {d} channels")
        if max_position >= cos.shape[0]:
            raise KernelError(
                f"position {max_position} is beyond the rotation table of {cos.shape[0]} positions"
            )
    if bias is not None:
        _need(bias, "bias of the packed projection", torch.float32, (row_width,))
    _ok(
        core().rl_qknorm_rope_kvwrite(
            _p(qkv), _p(q_out), _p(k_cache), _p(v_cache), _p(q_norm_w), _p(k_norm_w), _p(cos),
            _p(sin), _p(positions), _p(token_slot), _p(block_table), block_table.stride(0),
            page_size, tokens, nq, nkv, d, half, ROTARY_PAIRINGS[pairing], ctypes.c_float(eps), int(write),
            row_width, value_col0, dv, _p(bias), _tag(qkv.dtype), _stream(),
        ),
        "rl_qknorm_rope_kvwrite",
    )


def attention_generic(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    out: torch.Tensor,
    positions: torch.Tensor,
    token_slot: torch.Tensor,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    window: int,
    scale: float,
    max_position: int,
    value_dim: Optional[int] = None,
    keep_first: int = 0,
    sink: bool = False,
    sink_values: Optional[torch.Tensor] = None,
    score_cap: float = 0.0,
    slopes: Optional[torch.Tensor] = None,
) -> None:
    tokens = q.shape[0]
    pages = k_cache.shape[0]
    dv = d if value_dim is None else int(value_dim)
    if sink_values is not None:
        _need(sink_values, "sink values", torch.float32, (nq,))
    if slopes is not None:
        _need(slopes, "distance slopes", torch.float32, (nq,))
    if score_cap < 0:
        raise KernelError(f"the cap of the scores must not be negative, got {score_cap}")
    _need(q, "q", None, (tokens, nq * d))
    _need(out, "out", q.dtype, (tokens, nq * dv))
    _need(k_cache, "k_cache", q.dtype, (pages, nkv, page_size, d))
    _need(v_cache, "v_cache", q.dtype, (pages, nkv, dv, page_size))
    _need(positions, "positions", torch.int32, (tokens,))
    _need(token_slot, "token_slot", torch.int32, (tokens,))
    _need(block_table, "block_table", torch.int32)
    if max_position // page_size >= block_table.shape[1]:
        raise KernelError(
            f"position {max_position} needs page {max_position // page_size} of a block table "
            f"with {block_table.shape[1]} columns"
        )
    _ok(
        core().rl_attention_generic(
            _p(q), _p(k_cache), _p(v_cache), _p(out), _p(positions), _p(token_slot),
            _p(block_table), block_table.stride(0), page_size, tokens, nq, nkv, d, window,
            ctypes.c_float(scale), dv, int(keep_first), int(bool(sink) or sink_values is not None),
            _p(sink_values), ctypes.c_float(score_cap), _p(slopes), _tag(q.dtype), _stream(),
        ),
        "rl_attention_generic",
    )


def add_layernorm(
    residual: torch.Tensor,
    delta1: Optional[torch.Tensor],
    delta2: Optional[torch.Tensor],
    weight1: Optional[torch.Tensor],
    bias1: Optional[torch.Tensor],
    out1: Optional[torch.Tensor],
    weight2: Optional[torch.Tensor] = None,
    bias2: Optional[torch.Tensor] = None,
    out2: Optional[torch.Tensor] = None,
    eps: float = 1e-5,
    rows: Optional[torch.Tensor] = None,
) -> None:
    """``residual += delta1 + delta2`` (float32, in place; either may be ``None``), then
    ``out1 = layernorm(residual) * weight1 + bias1`` and, with ``out2``, a second layer norm of
    the same rows under ``weight2`` and ``bias2``: the statistics (mean, and the mean of the
    squared deviations from it) are computed once.  ``out1`` ``None``: only the add.  ``rows`` as
    in :func:`add_rmsnorm`."""
    tokens, hidden = residual.shape
    _need(residual, "residual", torch.float32)
    out_rows = tokens if rows is None else rows.numel()
    dtype = None
    for out, w, b, name in ((out1, weight1, bias1, "first"), (out2, weight2, bias2, "second")):
        if out is None:
            continue
        _need(out, f"{name} output", dtype, (out_rows, hidden))
        dtype = out.dtype
        _need(w, f"{name} norm weight", torch.float32, (hidden,))
        _need(b, f"{name} norm bias", torch.float32, (hidden,))
    if out2 is not None and out1 is None:
        raise KernelError("a second layer norm comes with a first")
    for d in (delta1, delta2):
        if d is not None:
            _need(d, "delta", dtype, (tokens, hidden))
            dtype = d.dtype
    if dtype is None:
        return  # nothing to add and nothing to produce
    if rows is not None:
        _need(rows, "rows", torch.int32)
    _ok(
        core().rl_add_layernorm(
            _p(residual), _p(delta1), _p(delta2), _p(weight1), _p(bias1), _p(out1), _p(weight2), _p(bias2),
            _p(out2), _p(rows), out_rows, hidden, ctypes.c_float(eps), _tag(dtype), _stream(),
        ),
        "rl_add_layernorm",
    )


def latent_rows(
    packed: torch.Tensor,
    q_rank: int,
    q_norm_w: Optional[torch.Tensor],
    q_latent_out: Optional[torch.Tensor],
    kv_col: int,
    kv_rank: int,
    rot_dim: int,
    kv_norm_w: Optional[torch.Tensor],
    cos: Optional[torch.Tensor],
    sin: Optional[torch.Tensor],
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    positions: torch.Tensor,
    token_slot: torch.Tensor,
    block_table: torch.Tensor,
    page_size: int,
    eps: float,
    max_position: int,
) -> None:
    """From the packed rows of a latent mixer's first product: with ``q_rank`` the query latent
    (columns ``[0, q_rank)``) RMS-normed under ``q_norm_w`` into ``q_latent_out``; with caches the
    key/value latent (``kv_rank`` columns from ``kv_col``) RMS-normed under ``kv_norm_w`` and the
    ``rot_dim`` columns behind it, whose first ``2 * cos.shape[1]`` channels rotate as interleaved
    pairs, written to the token's place: ``k_cache [pages, 1, page, kv_rank + rot_dim]`` holds
    ``[latent | rotated part]``, ``v_cache [pages, 1, kv_rank, page]`` the latent transposed."""
    tokens, row_width = packed.shape
    _need(packed, "packed rows")
    _need(positions, "positions", torch.int32, (tokens,))
    _need(token_slot, "token_slot", torch.int32, (tokens,))
    _need(block_table, "block_table", torch.int32)
    if q_rank:
        _need(q_norm_w, "query latent norm weight", torch.float32, (q_rank,))
        _need(q_latent_out, "query latent", packed.dtype, (tokens, q_rank))
        if q_rank > row_width:
            raise KernelError(f"a query latent of {q_rank} columns in rows of {row_width}")
    half = 0
    if k_cache is not None:
        pages = k_cache.shape[0]
        _need(k_cache, "k_cache", packed.dtype, (pages, 1, page_size, kv_rank + rot_dim))
        _need(v_cache, "v_cache", packed.dtype, (pages, 1, kv_rank, page_size))
        _need(kv_norm_w, "latent norm weight", torch.float32, (kv_rank,))
        if kv_col < 0 or kv_col + kv_rank + rot_dim > row_width or rot_dim % 2:
            raise KernelError(
                f"a latent of {kv_rank} + {rot_dim} columns from column {kv_col} in rows of {row_width}"
            )
        if max_position // page_size >= block_table.shape[1]:
            raise KernelError(
                f"position {max_position} needs page {max_position // page_size} of a block table "
                f"with {block_table.shape[1]} columns"
            )
        if cos is not None:
            half = cos.shape[1]
            _need(cos, "cos table", torch.float32, (None, half))
            _need(sin, "sin table", torch.float32, tuple(cos.shape))
            if 2 * half > rot_dim or max_position >= cos.shape[0]:
                raise KernelError(
                    f"rotation tables of {half} pairs and {cos.shape[0]} positions for a part of {rot_dim} "
                    f"channels at position {max_position}"
                )
    _ok(
        core().rl_latent_rows(
            _p(packed), row_width, tokens, int(q_rank), _p(q_norm_w), _p(q_latent_out), int(kv_col), int(kv_rank),
            int(rot_dim), _p(kv_norm_w), _p(cos), _p(sin), half, _p(k_cache), _p(v_cache), _p(positions),
            _p(token_slot), _p(block_table), block_table.stride(0), page_size, ctypes.c_float(eps),
            _tag(packed.dtype), _stream(),
        ),
        "rl_latent_rows",
    )


def rotate_tail(
    q: torch.Tensor, out: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
    positions: torch.Tensor, heads: int, d: int, rot_dim: int, out_width: int, offset: int, max_position: int,
) -> None:
    """``out[t, h, offset : offset + rot_dim]`` = the last ``rot_dim`` channels of head ``h`` of
    ``q`` (rows that begin with ``heads * (d + rot_dim)`` channels and may be wider), the first
    ``2 * cos.shape[1]`` of them rotated as interleaved pairs by the token's position; ``out`` has
    ``out_width`` channels a head."""
    tokens = q.shape[0]
    _need(q, "q", None, (tokens, None))
    if q.shape[1] < heads * (d + rot_dim):
        raise KernelError(f"rows of {q.shape[1]} channels do not hold {heads} heads of {d} + {rot_dim}")
    _need(out, "out", q.dtype, (tokens, heads * out_width))
    _need(positions, "positions", torch.int32, (tokens,))
    half = 0
    if cos is not None:
        half = cos.shape[1]
        _need(cos, "cos table", torch.float32, (None, half))
        _need(sin, "sin table", torch.float32, tuple(cos.shape))
        if max_position >= cos.shape[0]:
            raise KernelError(f"position {max_position} is beyond the rotation table of {cos.shape[0]} positions")
    if rot_dim % 2 or 2 * half > rot_dim or offset < 0 or offset + rot_dim > out_width:
        raise KernelError(f"{rot_dim} channels ({half} pairs rotate) at {offset} of heads of {out_width}")
    _ok(
        core().rl_rotate_tail(
            _p(q), _p(out), _p(cos), _p(sin), _p(positions), tokens, heads, d, rot_dim, half, out_width, offset,
            q.shape[1], _tag(q.dtype), _stream(),
        ),
        "rl_rotate_tail",
    )


def head_product(
    x: torch.Tensor, w: torch.Tensor, y: torch.Tensor, heads: int, x_head: int, x_off: int, y_head: int, y_off: int,
    gate: Optional[torch.Tensor] = None, gate_col: int = 0,
) -> None:
    """``y[t, y_off + h * y_head + o] = sum_i w[h, o, i] * x[t, x_off + h * x_head + i]``: one small
    matrix a head (``w [heads, O, I]``), applied to a slice of every head of ``x`` and written into
    a slice of every head of ``y``.  ``gate``: the result is multiplied by
    ``sigmoid(gate[t, gate_col + h])``.  Sizes in steps of 16 (and offsets in steps of 4) run on
    the matrix cores, in the type of the operands (float32: the true 32-bit instruction)."""
    tokens = x.shape[0]
    _need(x, "x", None, (tokens, None))
    _need(y, "y", x.dtype, (tokens, None))
    _need(w, "head matrices", x.dtype, (heads, None, None))
    O, I = w.shape[1], w.shape[2]
    if x_off < 0 or x_off + (heads - 1) * x_head + I > x.shape[1]:
        raise KernelError(f"{heads} heads of {I} inputs every {x_head} from {x_off} lie outside rows of {x.shape[1]}")
    if y_off < 0 or y_off + (heads - 1) * y_head + O > y.shape[1]:
        raise KernelError(f"{heads} heads of {O} outputs every {y_head} from {y_off} lie outside rows of {y.shape[1]}")
    gate_row = 0
    if gate is not None:
        _need(gate, "gate", x.dtype, (tokens, None))
        gate_row = gate.shape[1]
        if not 0 <= gate_col <= gate_row - heads:
            raise KernelError(f"gate columns {gate_col}..{gate_col + heads} lie outside rows of {gate_row}")
    _ok(
        core().rl_head_product(
            _p(x), _p(w), _p(y), tokens, heads, I, O, x.shape[1], x_head, x_off, y.shape[1], y_head, y_off,
            _p(gate), gate_row, gate_col, _tag(x.dtype), _stream(),
        ),
        "rl_head_product",
    )


def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """``out[M,N] = a[M,K] @ w[N,K]^T`` in true float32.  Rows may be strided (views of wider
    matrices); the inner dimension must be contiguous."""
    for t, name in ((a, "a"), (w, "w"), (out, "out")):
        if not t.is_cuda or t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1:
            raise KernelError(f"gemm_f32 operand {name} must be a float32 GPU matrix with unit inner stride")
    m, k = a.shape
    n, k2 = w.shape
    if k != k2 or out.shape != (m, n):
        raise KernelError(f"gemm_f32 shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    _ok(
        core().rl_gemm_f32(_p(a), _p(w), _p(out), m, n, k, a.stride(0), w.stride(0), out.stride(0), _stream()),
        "rl_gemm_f32",
    )


def _row_index(row_index: Optional[torch.Tensor]) -> None:
    if row_index is not None:
        _need(row_index, "row_index", torch.int32)
        if row_index.dim() != 1:
            raise KernelError(f"row_index must have one dimension, got {tuple(row_index.shape)}")


def argmax(logits: torch.Tensor, out: torch.Tensor, row_index: Optional[torch.Tensor] = None) -> None:
    """``out[b]`` = arg-max of row ``row_index[b]`` of ``logits`` (row ``b`` without an index)."""
    vocab = logits.shape[1]
    rows = out.shape[0]
    _need(logits, "logits", torch.float32)
    _need(out, "out", torch.int32, (rows,))
    _row_index(row_index)
    if row_index is not None and row_index.shape[0] != rows:
        raise KernelError(f"{row_index.shape[0]} row indices for {rows} outputs")
    if row_index is None and logits.shape[0] != rows:
        raise KernelError(f"{logits.shape[0]} rows of logits for {rows} outputs")
    lib = core()
    slices = lib.rl_argmax_slices(vocab)
    part_v = part_i = None
    if slices > 1 and rows * 4 < slices * 16:  # few wide rows: two stages fill the chip
        part_v = torch.empty((rows, slices), dtype=torch.float32, device=logits.device)
        part_i = torch.empty((rows, slices), dtype=torch.int32, device=logits.device)
    _ok(
        lib.rl_argmax(_p(logits), _p(row_index), _p(out), _p(part_v), _p(part_i), rows, vocab, _stream()),
        "rl_argmax",
    )


_PENALTY_MAX_VOCAB = 40 * 1024 * 8  # one bit per token id in 40 KB of LDS


def _penalty_fits(vocab: int) -> None:
    if vocab > _PENALTY_MAX_VOCAB:
        raise KernelError(
            f"the repetition penalty keeps one bit per token id in 40 KB of LDS: vocabulary "
            f"{vocab} is beyond {_PENALTY_MAX_VOCAB}"
        )


def _fed_tokens(fed: Optional[torch.Tensor], out: Optional[torch.Tensor]) -> None:
    if fed is None:
        return
    _need(fed, "fed", torch.int32)
    if fed.dim() != 1:
        raise KernelError(f"fed tokens must be one-dimensional, are {tuple(fed.shape)}")
    if out is not None and _overlap(fed, out):
        raise KernelError("the fed tokens share memory with the tokens this call chooses")


def _overlap(a: torch.Tensor, b: torch.Tensor) -> bool:
    a0, b0 = a.data_ptr(), b.data_ptr()
    return a0 < b0 + b.numel() * b.element_size() and b0 < a0 + a.numel() * a.element_size()


def sample(
    logits: torch.Tensor,
    row_params: torch.Tensor,
    history: Optional[torch.Tensor],
    out: torch.Tensor,
    out_logprob: Optional[torch.Tensor],
    any_penalty: bool,
    row_index: Optional[torch.Tensor] = None,
    fed: Optional[torch.Tensor] = None,
) -> None:
    """General token selection (penalty, temperature, nucleus, seeded draw), one row per
    workgroup.  ``row_params [rows * 8]`` int32 as the kernel documents them; output row
    ``b`` reads row ``row_index[b]`` of ``logits`` (row ``b`` without an index).  A negative
    entry ``-(r + 1)`` of ``history`` is read as ``fed[r]``; ``fed`` must not share memory
    with ``out``."""
    vocab = logits.shape[1]
    rows = out.shape[0]
    _need(logits, "logits", torch.float32)
    _need(row_params, "row_params", torch.int32, (rows * 8,))
    _need(out, "out", torch.int32, (rows,))
    _row_index(row_index)
    if (row_index.shape[0] if row_index is not None else logits.shape[0]) != rows:
        raise KernelError(f"{rows} outputs do not match the rows to read")
    if out_logprob is not None:
        _need(out_logprob, "out_logprob", torch.float32, (rows,))
    if history is not None:
        _need(history, "history", torch.int32)
    if any_penalty:
        _penalty_fits(vocab)
    _fed_tokens(fed, out)
    _ok(
        core().rl_sample(
            _p(logits), _p(row_index), _p(row_params), _p(history), _p(fed),
            0 if fed is None else fed.shape[0], _p(out), _p(out_logprob), rows, vocab,
            int(bool(any_penalty)), _stream(),
        ),
        "rl_sample",
    )


def logprobs(
    logits: torch.Tensor,
    targets: torch.Tensor,
    k: int,
    row_params: Optional[torch.Tensor] = None,
    history: Optional[torch.Tensor] = None,
    any_penalty: bool = False,
    row_index: Optional[torch.Tensor] = None,
    fed: Optional[torch.Tensor] = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Log-probability of ``targets[b]`` and the ``k`` most likely tokens of every row:
    ``(target [rows] float32, top ids [rows, k] int32, top log-probabilities [rows, k]
    float32)``, descending, equal values by ascending id.  With ``row_params`` the
    distribution is the one ``sample`` draws from (penalty, temperature; greedy rows count
    as temperature 1); without, log_softmax of the raw logits.  ``fed`` as for ``sample``."""
    vocab = logits.shape[1]
    rows = targets.shape[0]
    _need(logits, "logits", torch.float32)
    _need(targets, "targets", torch.int32, (rows,))
    _row_index(row_index)
    if (row_index.shape[0] if row_index is not None else logits.shape[0]) != rows:
        raise KernelError(f"{rows} targets do not match the rows to read")
    if not 0 <= k <= vocab:
        raise KernelError(f"top-k width {k} is outside [0, vocabulary {vocab}]")
    if row_params is not None:
        _need(row_params, "row_params", torch.int32, (rows * 8,))
    if history is not None:
        _need(history, "history", torch.int32)
    if any_penalty:
        _penalty_fits(vocab)
        if row_params is None or history is None:
            raise KernelError("a penalty needs row_params and history")
    _fed_tokens(fed, None)
    target_lp = torch.empty(rows, dtype=torch.float32, device=logits.device)
    top_ids = torch.empty((rows, k), dtype=torch.int32, device=logits.device)
    top_lp = torch.empty((rows, k), dtype=torch.float32, device=logits.device)
    _ok(
        core().rl_logprobs(
            _p(logits), _p(row_index), _p(row_params), _p(history), _p(fed),
            0 if fed is None else fed.shape[0], _p(targets), _p(target_lp),
            _p(top_ids if k else None), _p(top_lp if k else None), rows, vocab, k,
            int(bool(any_penalty)), _stream(),
        ),
        "rl_logprobs",
    )
    return target_lp, top_ids, top_lp


def sample_uniform(seed: int, counter: int) -> float:
    """The kernel's own uniform draw, computed by the library on the host."""
    fn = core().rl_sample_uniform
    fn.restype = ctypes.c_float
    return float(fn(ctypes.c_uint(seed & 0xFFFFFFFF), ctypes.c_uint((seed >> 32) & 0xFFFFFFFF), ctypes.c_uint(counter)))


SKINNY_MAX_ROWS = 16  # rows up to which the hand-written bandwidth-bound product is used
def _skinny_tiles(rows: int, out_features: int, plain: bool = False, units: int | None = None) -> int:
    """Weight rows per workgroup of the skinny product, as the kernel's code for them: 1 (16 rows,
    one tile, which leaves the most workgroups), 2 (32 rows) or, for a product that only stores
    its result (``plain``), 3 (24 rows: one tile and a half).

    A compute unit streams at most so fast, so what counts is the most rows a unit gets: the
    rounds of workgroups times their rows.  A matrix of 257 to 1,023 tiles takes 24 rows where
    that gives the fewest (6,144 outputs = 384 tiles: 256 workgroups, one a unit; microseconds at
    1 / 8 / 16 rows of X with 16, 32 and 24 weight rows a workgroup: 11.6 12.3 11.0 / 13.9 12.8
    11.1 / 16.6 14.1 12.0; 5,120 outputs 11.4 11.2 9.8 / 13.1 12.1 10.3 / 16.2 13.7 11.6; but
    7,168 outputs = 448 tiles, where 24 rows make 299 workgroups and a second round, 14.9 15.0
    18.6 / 17.8 15.6 20.4).  Otherwise one tile, except where two were measured faster: from 8
    rows of X on when one tile would leave some units with two workgroups and some with one; and
    with more than 12 rows on matrices of a thousand tiles and more (151,936 outputs: 275 / 244
    at 16 rows, but 216 / 233 at 8)."""
    units = chip().units if units is None else units
    blocks = -(-out_features // 16)
    if plain and units < blocks < 4 * units:
        def most_rows(rows_per_group: int) -> int:
            groups = -(-out_features // rows_per_group)
            return -(-groups // units) * rows_per_group
        if most_rows(24) < min(most_rows(16), most_rows(32)):
            return 3
    if rows >= 8 and units < blocks < 2 * units:
        return 2
    if rows > 12 and blocks >= 4 * units:
        return 2
    return 1


def _scaled_args(scaled, rows: int, k: int) -> tuple:
    """The kernels' arguments for an X whose norm factor is still to be applied."""
    if scaled is None:
        return (None, 0, 0, ctypes.c_float(0.0))
    _need(scaled.partial, "partial sums of squares", torch.float32)
    if scaled.partial.dim() != 2 or scaled.partial.shape[1] != 16 or scaled.size != k or rows > 16:
        raise KernelError(
            f"scaled rows of width {scaled.size} with partials {tuple(scaled.partial.shape)} do not fit "
            f"a product of {rows} rows over {k}"
        )
    return (_p(scaled.partial), scaled.partial.shape[0], scaled.size, ctypes.c_float(scaled.eps))


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, scaled=None) -> torch.Tensor:
    """``x[M,K] @ w[N,K]^T`` with bfloat16 operands and float32 accumulation.  ``scaled``
    (few rows only): the rows of ``x`` still lack their norm's factor, which is applied to
    the result (see ``gemm_bf16_residual``).

    Up to 16 rows (decode) run the hand-written bandwidth-bound kernel, which can write
    float32 directly; so does the kernel for 17 to 64 rows over wide matrices.  Small matrices
    run the one-launch tile product up to 512 rows.  Everything else goes to the library
    product, as the reference's dense products do (``F.linear``); a bfloat16 result is returned
    as is and widened by the caller."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    if k != w.shape[1]:
        raise KernelError(f"gemm_bf16 shapes do not agree: x {tuple(x.shape)}, w {tuple(w.shape)}")
    if m <= SKINNY_MAX_ROWS and k % 8 == 0:
        if out_dtype not in (torch.bfloat16, torch.float32):
            raise KernelError(f"gemm_bf16 writes bfloat16 or float32, not {out_dtype}")
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        nt = _skinny_tiles(m, n, plain=True)
        _ok(
            core().rl_gemm_skinny(
                _p(x), _p(w), _p(out), m, n, k, k, k, n, _tag(out_dtype), nt, *_scaled_args(scaled, m, k), _stream()
            ),
            "rl_gemm_skinny",
        )
        return out
    if scaled is not None:
        raise KernelError(f"scaled rows need the few-row product: {m} rows over {k}")
    if _tile_applies(m, n, k, n):
        out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
        _ok(
            core().rl_gemm_tile(_p(x), _p(w), _p(out), m, n, k, k, k, n, 0, ctypes.c_float(0.0), ctypes.c_float(0.0),
                                _stream()),
            "rl_gemm_tile",
        )
        return out
    plan = rows_plan(m, n, k, swiglu=False)
    if plan is not None:
        wide = torch.float32 if out_dtype == torch.float32 else torch.bfloat16
        out = torch.empty((m, n), dtype=wide, device=x.device)
        _ok(
            core().rl_gemm_rows(_p(x), _p(w), _p(out), m, n, k, k, k, n, 0, _tag(wide), *plan, ctypes.c_float(0.0),
                                ctypes.c_float(0.0), _stream()),
            "rl_gemm_rows",
        )
        return out
    return library_product(x, w)


# How many products went to the library since the process started.  A step that is recorded into
# a graph is meant to hold this package's kernels only where they exist; whoever records one
# reads the counter before and after.
library_products = 0


def library_product(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x w^T`` by the library (hipBLASLt behind ``torch.matmul``), as the reference's dense
    products are ``F.linear``: the many-row products of prompt steps, and what no kernel of
    this package takes."""
    global library_products
    library_products += 1
    return torch.matmul(x, w.t())


ROWS_MAX_ROWS = 64  # rows up to which wide matrices run the kernel that keeps X in registers


def rows_plan(m: int, n: int, k: int, swiglu: bool, units: int | None = None) -> tuple[int, int] | None:
    """(result tiles a workgroup holds, workgroups) for the product of 17 to 64 rows over a wide
    matrix with ``n`` result columns (with SwiGLU a tile is a gate and an up tile), ``None`` where
    that kernel does not apply.  A compute unit gets one workgroup with an even share of the
    tiles where a workgroup can hold such a share (the packed gate and up matrices of Qwen3-8B:
    768 pairs, three a unit); a matrix with more tiles than that (the vocabulary) is cut into
    workgroups of the most tiles one holds, which the chip takes in turn."""
    if not (SKINNY_MAX_ROWS < m <= ROWS_MAX_ROWS) or n % 16 or k % 128 or k < 128:
        return None
    if os.environ.get("RAPID_LLM_ROWS_PRODUCT") == "0":  # the library instead, for comparing the two
        return None
    units = chip().units if units is None else units
    tiles = n // 16
    if 2 * tiles < units:  # too few workgroups to stream from
        return None
    holds = ((2, 3, 5) if m <= 48 else (2, 3)) if swiglu else (1, 2, 3, 6)
    share = -(-tiles // min(units, tiles))
    for per in holds:
        if per >= share:
            return per, min(units, tiles)
    if (swiglu and share > 5) or (not swiglu and share < 24):
        # More tiles a compute unit than a workgroup holds (beyond 48 rows a workgroup holds
        # three pairs, and a matrix of up to five pairs a unit is cut into groups of three).  For the packed gate and up matrices
        # of the 32B shape (524 MB, 12.5 tiles a unit) the library's kernel streams at 5.4 TB/s
        # at every row count: 97 to 106 us at 17 to 64 rows against 99 to 136 here in any cut with
        # SwiGLU, 91 against 116 at 32 rows without.  Only for the vocabulary (37 tiles a unit)
        # are its kernels the slower ones (348 us against 294 at 32 rows of the 32B shape).
        return None
    per = holds[-1]
    return per, -(-tiles // per)


def gemm_bf16_residual(
    x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor
) -> tuple[torch.Tensor, torch.Tensor]:
    """The few-row product with the residual epilogue: ``residual += x w^T`` (the product
    rounded to bfloat16 first, as a stored result would be) in place; returns
    ``(residual * norm_weight`` as bfloat16, ``partial [workgroups, 16]`` float32``)`` with the
    sums of squares of each workgroup's columns of every row.  A consumer that takes the rows
    as ``scaled`` input finishes the norm."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    if k != w.shape[1] or m > SKINNY_MAX_ROWS or k % 8:
        raise KernelError(
            f"gemm_bf16_residual takes up to {SKINNY_MAX_ROWS} rows over a multiple of 8: "
            f"x {tuple(x.shape)}, w {tuple(w.shape)}"
        )
    _need(residual, "residual", torch.float32, (m, n))
    _need(norm_weight, "norm weight", torch.float32, (n,))
    lib = core()
    nt = _skinny_tiles(m, n)
    rows = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    partial = torch.empty((lib.rl_gemm_skinny_parts(n, nt), 16), dtype=torch.float32, device=x.device)
    _ok(
        lib.rl_gemm_skinny_residual(
            _p(x), _p(w), m, n, k, k, k, nt, _p(residual), _p(norm_weight), _p(rows), _p(partial), _stream()
        ),
        "rl_gemm_skinny_residual",
    )
    return rows, partial


TILE_MAX_ROWS = 512  # rows up to which small matrices run the one-launch tile product
_TILE_MAX_WEIGHTS = 7 << 20  # elements of a matrix (14 MB) up to which it is used
_TILE_MIN_COLS = 2048  # fewer columns leave too few workgroups


def _tile_applies(m: int, weight_rows: int, k: int, cols: int) -> bool:
    """Whether the one-launch tile product takes ``m`` rows over a ``[weight_rows, k]`` matrix
    with ``cols`` result columns.  It is for steps of tens to hundreds of rows over matrices of
    a few megabytes, where a kernel's time is its start and its chain of dependent steps, not
    its bytes.  Measured against the library, microseconds at 17 / 64 / 256 rows (the library
    first): 4,096 x 1,024 8.2 / 5.9, 8.7 / 7.8, 9.0 / 8.3; the packed gate and up matrices of
    6,144 x 1,024 with SwiGLU in the epilogue against the library and the activation kernel
    13.4 / 8.2, 13.5 / 10.9, 17.9 / 14.8 (inside a Qwen3-0.6B decode step the library's two
    take 11.5 and 13.8 + 4.6).  From 4,096 x 2,048 on the library is as fast or faster (11.1 /
    11.3, 11.6 / 14.4, 13.1 / 13.8), and matrices of 1,024 rows leave too few workgroups
    (1,024 x 2,048: 8.2 / 9.0, 8.2 / 12.1, 8.6 / 12.3).  Beyond 256 rows the library's kernels
    are the faster ones on the device (512 rows: 10.6 / 12.2, with the activation 20.1 / 19.1;
    1,024 rows: 13.5 / 21.3 and 25.7 / 32.6), but a step of a few hundred tokens of so small a
    model is bound by the host, where a call of the library costs 18 us and one of this kernel
    6: a 512-token prompt of the Qwen3-0.6B shape 5.4 -> 4.2 ms.  Hence up to 512 rows."""
    return (
        SKINNY_MAX_ROWS < m <= TILE_MAX_ROWS
        and k % 128 == 0
        and cols % 4 == 0
        and cols * (weight_rows // cols) >= _TILE_MIN_COLS
        and weight_rows * k <= _TILE_MAX_WEIGHTS
    )


# Rows up to which a product's runs of K may be left to the norm that follows.  Beyond 64 rows the
# kernel runs blocks of 64 rows.  Against the library's product and the plain norm, microseconds
# (the library first): Qwen3-8B output projection 18.7 / 15.2 at 64 rows, 28.1 / 19.9 at 128,
# 36.5 / 24.4 at 192, 27.1 / 30.1 at 256; down projection 40.6 / 30.6, 68.8 / 42.4, 92.6 / 56.4,
# 57.4 / 72.6; the 32B shape's down projection 160 / 65, 184 / 100, 214 / 137, 265 / 180.  The
# library's time jumps between neighbouring row counts (the 8B down projection: 51.8 at 144 rows,
# 78.8 at 160, 55.4 at 176), this kernel's grows with the blocks of 64; from about 200 rows on
# the library's best kernels are the faster ones.  Small matrices (the 0.6B and 1.7B shapes) are
# within a microsecond either way from 144 rows on.
MID_MAX_ROWS = 192
_MID_BLOCK_ROWS = 64  # weight rows per workgroup of the mid-size product
_MID_MAX_BLOCKS = 128  # wider matrices than this many workgroups stay with the library


def mid_runs(n: int, k: int, units: int | None = None) -> int:
    """Runs of K for the mid-size product of an ``[n, k]`` matrix, 0 where it does not apply:
    enough to put a workgroup on every compute unit, at least four chunks of 128 each."""
    units = chip().units if units is None else units
    blocks = -(-n // _MID_BLOCK_ROWS)
    if k % 128 or n % 4 or blocks > _MID_MAX_BLOCKS:
        return 0
    chunks = k // 128
    ks = max(1, min(units // blocks, chunks // 4, 8))
    while ks > 1 and -(-chunks // ks) * (ks - 1) >= chunks:  # every run holds a chunk
        ks -= 1
    return ks


def gemm_bf16_parts(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x[M,K] @ w[N,K]^T`` for 17 to 192 rows as float32 runs of K, ``[runs, M, N]``: their sum
    is the product.  For products whose result goes into the residual: the norm that follows
    adds the runs (``add_rmsnorm_parts``)."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    ks = mid_runs(n, k)
    if k != w.shape[1] or m > MID_MAX_ROWS or ks < 1:
        raise KernelError(f"gemm_bf16_parts does not take x {tuple(x.shape)}, w {tuple(w.shape)}")
    parts = torch.empty((ks, m, n), dtype=torch.float32, device=x.device)
    _ok(core().rl_gemm_mid_parts(_p(x), _p(w), _p(parts), m, n, k, k, k, ks, _stream()), "rl_gemm_mid_parts")
    return parts


def add_rmsnorm_parts(
    residual: torch.Tensor, parts: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, eps: float
) -> None:
    """``residual += bfloat16(sum of parts)`` in place, ``out = norm(residual) * weight``."""
    runs, tokens, hidden = parts.shape
    _need(residual, "residual", torch.float32, (tokens, hidden))
    _need(parts, "parts", torch.float32)
    _need(weight, "norm weight", torch.float32, (hidden,))
    _need(out, "out", torch.bfloat16, (tokens, hidden))
    _ok(
        core().rl_add_rmsnorm_parts(
            _p(residual), _p(parts), runs, _p(weight), _p(out), tokens, hidden, ctypes.c_float(eps), _stream()
        ),
        "rl_add_rmsnorm_parts",
    )


def gemm_bf16_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor, scaled=None, limit: float = 0.0,
                     alpha: float = GLU_ALPHA) -> torch.Tensor | None:
    """``act(x Wg^T, x Wu^T)`` for the packed ``[gate | up]`` matrix in one kernel: for few rows,
    and for up to 512 rows over a small matrix; ``None`` when the shape is not one a fused kernel
    takes.  ``act`` is ``silu(g) * u``, or with a ``limit`` the clamped variant of :func:`swiglu`.
    ``scaled``: as in ``gemm_bf16``."""
    m, k = x.shape
    glu = (ctypes.c_float(limit), ctypes.c_float(alpha))
    two_i = w_gate_up.shape[0]
    if k % 8 or two_i % 2 or x.dtype != torch.bfloat16 or w_gate_up.dtype != torch.bfloat16:
        return None
    if m > SKINNY_MAX_ROWS:
        inter = two_i // 2
        if scaled is not None:
            return None
        _need(x, "x", torch.bfloat16)
        _need(w_gate_up, "w_gate_up", torch.bfloat16, (two_i, k))
        if _tile_applies(m, two_i, k, inter):
            out = torch.empty((m, inter), dtype=torch.bfloat16, device=x.device)
            _ok(core().rl_gemm_tile(_p(x), _p(w_gate_up), _p(out), m, inter, k, k, k, inter, 1, *glu, _stream()), "rl_gemm_tile")
            return out
        plan = rows_plan(m, inter, k, swiglu=True)
        if plan is None:
            return None
        out = torch.empty((m, inter), dtype=torch.bfloat16, device=x.device)
        _ok(
            core().rl_gemm_rows(_p(x), _p(w_gate_up), _p(out), m, inter, k, k, k, inter, 1, BF16, *plan, *glu, _stream()),
            "rl_gemm_rows",
        )
        return out
    _need(x, "x", torch.bfloat16)
    _need(w_gate_up, "w_gate_up", torch.bfloat16, (two_i, k))
    inter = two_i // 2
    out = torch.empty((m, inter), dtype=torch.bfloat16, device=x.device)
    nt = 2  # one (gate, up) pair of tiles per workgroup
    _ok(
        core().rl_gemm_skinny_swiglu(
            _p(x), _p(w_gate_up), _p(out), m, inter, k, k, k, inter, nt, chip().units,
            *_scaled_args(scaled, m, k), *glu, _stream()
        ),
        "rl_gemm_skinny_swiglu",
    )
    return out


class AttentionPlan:
    """Per-step launch data of the matrix-core attention kernels for one group size G
    (query heads per kv head): which requests are single tokens (decode kernel) and how the
    portions of the others are cut into row tiles (prefill kernel)."""

    __slots__ = ("num_decode", "seq_token", "max_decode_ctx", "num_tiles", "tile_info", "tile_keys", "orders",
                 "_prefill_tokens", "_prefill_list", "_decode_order")

    def __init__(self, ctx, group: int, tile_rows: int) -> None:
        self._decode_order = None
        fixed = _static(ctx).get("decode_only_tokens")
        if fixed is not None:
            # a step of single tokens whose index list is already on the device (graphs)
            self.num_decode = fixed.numel()
            self.seq_token = None  # request i is token i: the kernels skip the lookup
            self.max_decode_ctx = max(ctx.h_seq_starts) + 1
            self.num_tiles = 0
            self.tile_info = None
            self.tile_keys = []
            self.orders = {}
            self._prefill_list, self._prefill_tokens = [], None
            return
        dec_tokens: list[int] = []
        self._prefill_list, self._prefill_tokens = [], None
        tile_list: list[tuple[int, int, int, int]] = []
        self.max_decode_ctx = 0
        at = 0
        for start, n in zip(ctx.h_seq_starts, ctx.h_seq_lens):
            if n == 1:
                dec_tokens.append(at)
                self.max_decode_ctx = max(self.max_decode_ctx, start + 1)
            else:
                for row0 in range(0, n * group, tile_rows):
                    tile_list.append((at, start, n, row0))
                self._prefill_list.extend(range(at, at + n))
            at += n
        tiles = [v for t in tile_list for v in t]
        # keys each tile reads: what its workgroups cost
        self.tile_keys = [t[1] + min(t[2], (t[3] + tile_rows) // group) for t in tile_list]
        self.orders = {}
        self.num_decode = len(dec_tokens)
        self.num_tiles = len(tiles) // 4
        device = ctx.token_ids.device
        packed = upload_ints(dec_tokens + tiles, device)
        self.seq_token = packed[: self.num_decode]
        self.tile_info = packed[self.num_decode :]

    def prefill_tokens(self, device) -> torch.Tensor:
        """Indices in the step of the tokens that belong to portions (not single tokens)."""
        if self._prefill_tokens is None:
            self._prefill_tokens = upload_ints(self._prefill_list, device)
        return self._prefill_tokens

    def decode_order(self, ctx) -> torch.Tensor:
        """The step's single-token requests, longest context first, sorted on the device from the
        step's positions (a replayed step has nothing else); made once a step, for every layer."""
        if self._decode_order is None:
            order = torch.empty(self.num_decode, dtype=torch.int32, device=ctx.positions.device)
            _ok(
                core().rl_order_by_length(_p(ctx.positions), _p(self.seq_token), self.num_decode, _p(order), _stream()),
                "rl_order_by_length",
            )
            self._decode_order = order
        return self._decode_order

    def work_order(self, nkv: int, device, resident: int = 1) -> torch.Tensor:
        """Order in which the (tile, kv head) pairs of the prefill kernel are handed out:
        longest first, so that the short ones fill the gaps at the end.  Where a compute unit
        holds two workgroups at a time (``resident == 2``), the first round, one workgroup on
        every unit, takes the longest, and the second round, which joins them on the same
        units, the shortest in ascending order, so that a unit's two workgroups add up alike."""
        order = self.orders.get((nkv, resident))
        if order is None:
            items = sorted(range(self.num_tiles * nkv), key=lambda i: (-self.tile_keys[i // nkv], i))
            if resident == 2:
                round_one = chip().first_round
                first = items[:round_one]
                rest = items[round_one:]
                second = rest[::-1][:round_one]
                middle = rest[: max(0, len(rest) - round_one)]
                items = first + second + middle
            order = upload_ints(items, device)
            self.orders[(nkv, resident)] = order
        return order


# A decode launch splits the keys until it has a workgroup for every compute unit; the fewest
# keys a split is worth (measured at 2,048 keys, 8 kv heads on 256 units: 1 request 128 keys a
# split, 8 requests 512, 64 requests no split; at 512 keys 128 a split for 1 and 8 requests;
# finer splits only add merge work).  A launch of more workgroups than the chip holds at a
# time (``Chip.decode_resident``) hands them out longest request first.
_MIN_SPLIT_KEYS = 128
_MAX_SPLIT_PAGES = 1024  # page ids of one split are staged in LDS
# The prefill kernel cuts its tiles' keys into runs when a launch has fewer workgroups than the
# chip has slots for (``Chip.prefill_slots``) and tiles of at least twice this many keys (a
# portion of one long prompt).
_PREFILL_SPLIT_KEYS = 512
_PREFILL_MAX_SPLITS = 8


def tile_rows_of(lib) -> int:
    return lib.rl_attn_prefill_rows()


_PREFILL_STEP_KEYS = 64  # keys per step of the prefill kernel
# what a step costs more when the two wave groups of a compute unit walk one tile in lockstep
# than when they belong to two tiles and drift apart (measured: 3.17 against 2.83 us)
_PREFILL_PAIRED_COST = 1.12
# a tile that outlasts the others ends alone on its compute unit and steps faster there than
# beside a second workgroup (2,048 tokens behind 2,048: 139 us with one wave group a tile,
# 157 us with two, where whole steps at the shared rate would say 181 against 152)
_PREFILL_ALONE = 0.8
# what cutting the tiles' keys into runs costs, in steps: the runs' partial results are
# written, and read and folded by a second kernel (1,024 tokens from their start: 33 us whole,
# 47 us in two runs)
_PREFILL_MERGE_STEPS = 5


def _prefill_shape(plan: "AttentionPlan", nkv: int, window: int, tile_rows: int,
                   units: int | None = None) -> tuple[int, int]:
    """(wave groups per workgroup, runs the keys of every tile are cut into) for a launch of
    the prefill kernel, from an estimate of the launch's length in steps: the longest tile's
    steps (halved where two wave groups share it, divided where its keys are cut into runs) or
    the steps there are for every slot of the chip, whichever is more.  Few, long tiles (a
    portion of one long prompt) come out with their keys cut into runs, folded by the merge
    kernel; a prompt from its start, whose last rows alone see many keys, with two wave groups
    a tile; a launch with work for every slot with neither."""
    slots = (chip() if units is None else Chip(units)).prefill_slots
    keys = plan.tile_keys
    if window > 0:
        keys = [min(k, window + tile_rows) for k in keys]
    items = plan.num_tiles * nkv
    steps = [-(-k // _PREFILL_STEP_KEYS) for k in keys]
    longest = max(steps)
    share = nkv * sum(steps) / slots  # steps per slot if the work were spread evenly
    best = (max(longest * _PREFILL_ALONE, share), 1, 1)
    paired = max(-(-longest // 2), share) * _PREFILL_PAIRED_COST
    if paired < best[0]:
        best = (paired, 2, 1)
    if items < slots:
        most = min(_PREFILL_MAX_SPLITS, -(-slots // items), max(keys) // _PREFILL_SPLIT_KEYS)
        for nsplit in range(2, most + 1):
            cost = max(-(-longest // nsplit), share) + _PREFILL_MERGE_STEPS
            if cost < best[0]:
                best = (cost, 1, nsplit)
    return best[1], best[2]


def _static(ctx) -> dict:
    """Where launch data that depends on the step's shape alone is kept (``StepContext.static``:
    it survives from the eager run before a recording into the recording)."""
    static = getattr(ctx, "static", None)
    return ctx.extra if static is None else static


def _f32_tiles(ctx, group: int, tile_rows: int = 16) -> tuple[torch.Tensor, int]:
    """Tiles of ``tile_rows`` (token, head of the group) rows, request by request: ``[tiles, 3]``
    int32 (first token of the request in the step, its tokens, first row of the tile).  A function
    of the requests' token counts alone."""
    key = ("f32_tiles", group) if tile_rows == 16 else ("row_tiles", group, tile_rows)
    store = _static(ctx)
    made = store.get(key)
    if made is None:
        tiles: list[int] = []
        at = 0
        for n in ctx.h_seq_lens:
            for row0 in range(0, n * group, tile_rows):
                tiles += [at, n, row0]
            at += n
        made = (upload_ints(tiles, ctx.token_ids.device), len(tiles) // 3)
        store[key] = made
    return made


def attention_f32(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    out: torch.Tensor,
    ctx,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    window: int,
    scale: float,
) -> None:
    """float32 attention of every token of the step on the float32 matrix instruction; a
    row's result is the same bit for bit however the step was cut."""
    tokens = q.shape[0]
    pages = k_cache.shape[0]
    _need(q, "q", torch.float32, (tokens, nq * d))
    _need(out, "out", torch.float32, (tokens, nq * d))
    _need(k_cache, "k_cache", torch.float32, (pages, nkv, page_size, d))
    _need(v_cache, "v_cache", torch.float32, (pages, nkv, d, page_size))
    _need(ctx.positions, "positions", torch.int32, (tokens,))
    _need(ctx.token_slot, "token_slot", torch.int32, (tokens,))
    _need(block_table, "block_table", torch.int32)
    if page_size % 4:
        raise KernelError(f"the float32 attention reads four keys of a page at once: page size {page_size}")
    if ctx.max_position // page_size >= block_table.shape[1]:
        raise KernelError(
            f"position {ctx.max_position} needs page {ctx.max_position // page_size} of a block table "
            f"with {block_table.shape[1]} columns"
        )
    if nkv > 65535:
        raise KernelError(f"{nkv} kv heads exceed the launch grid")
    tiles, num_tiles = _f32_tiles(ctx, nq // nkv)
    _ok(
        attention_lib(d).rl_attn_f32(
            _p(q), _p(k_cache), _p(v_cache), _p(out), _p(tiles), num_tiles, _p(ctx.positions),
            _p(ctx.token_slot), _p(block_table), block_table.stride(0), page_size, nq, nkv, window,
            ctypes.c_float(scale), _stream(),
        ),
        "rl_attn_f32",
    )


def attention_tile(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    out: torch.Tensor,
    ctx,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    dv: int,
    window: int,
    keep_first: int,
    sink: bool,
    scale: float,
    sink_values: Optional[torch.Tensor] = None,
    score_cap: float = 0.0,
    slopes: Optional[torch.Tensor] = None,
) -> None:
    """Attention of every token of the step, in tiles of 16 rows on the matrix cores, for value
    heads of a size of their own, a window that keeps a request's first ``keep_first`` positions
    visible, and (``sink``) a softmax with 1 added to its denominator, or with ``sink_values``
    (float32, one number a query head) ``exp`` of the head's number.  ``score_cap`` c > 0 turns a
    scaled score s into ``c * tanh(s / c)``; ``slopes`` (float32, one number a query head) then take
    ``slope * (distance between query and key)`` off it.  float32 (bit for bit the same however
    the step was cut) or bfloat16."""
    tokens = q.shape[0]
    if sink_values is not None:
        _need(sink_values, "sink values", torch.float32, (nq,))
        sink = True
    if slopes is not None:
        _need(slopes, "distance slopes", torch.float32, (nq,))
    if score_cap < 0:
        raise KernelError(f"the cap of the scores must not be negative, got {score_cap}")
    pages = k_cache.shape[0]
    _need(q, "q", None, (tokens, nq * d))
    _need(out, "out", q.dtype, (tokens, nq * dv))
    _need(k_cache, "k_cache", q.dtype, (pages, nkv, page_size, d))
    _need(v_cache, "v_cache", q.dtype, (pages, nkv, dv, page_size))
    _need(ctx.positions, "positions", torch.int32, (tokens,))
    _need(ctx.token_slot, "token_slot", torch.int32, (tokens,))
    _need(block_table, "block_table", torch.int32)
    if page_size % 4:
        raise KernelError(f"the tile attention reads four keys of a page at once: page size {page_size}")
    if ctx.max_position // page_size >= block_table.shape[1]:
        raise KernelError(
            f"position {ctx.max_position} needs page {ctx.max_position // page_size} of a block table "
            f"with {block_table.shape[1]} columns"
        )
    if nkv > 65535 or window < 0 or keep_first < 0:
        raise KernelError(f"{nkv} kv heads, window {window}, {keep_first} kept positions")
    lib = attention_tile_lib(d, dv)
    group = nq // nkv
    # a bfloat16 step with portions: tiles of several blocks of 16 rows, so that the keys a
    # workgroup reads serve more rows (float32 keeps one order of summation, whatever the step)
    tile_rows = 16
    longest = max(ctx.h_seq_lens)
    if q.dtype == torch.bfloat16 and longest * group > 16:
        tile_rows = lib.rl_attn_tile_wide_rows()
        if longest == 1 and tile_rows > 16:
            # single tokens whose heads fill several blocks of rows: where the keys are many,
            # dealing them to several workgroups is worth more than sharing a key tile between
            # the blocks of one
            blocks = len(ctx.h_seq_lens) * -(-group // 16) * nkv
            bound = _static(ctx).get("context_bound", ctx.max_position + 1)
            if tile_splits(blocks, bound, window, keep_first) > 1:
                tile_rows = 16
    tiles, num_tiles = _f32_tiles(ctx, group, tile_rows)
    # few tiles over many keys (a step of single tokens, mostly): a tile's keys are dealt to
    # several workgroups, on compute units of their own, and their shares merged
    nsplit, part = 1, None
    if q.dtype == torch.bfloat16 and tile_rows == 16:
        nsplit = tile_splits(num_tiles * nkv, _static(ctx).get("context_bound", ctx.max_position + 1), window, keep_first)
        if nsplit > 1:
            part = torch.empty((tokens, nq, nsplit, dv + 2), dtype=torch.float32, device=q.device)
    _ok(
        lib.rl_attn_tile(
            _p(q), _p(k_cache), _p(v_cache), _p(out), _p(tiles), num_tiles, _p(ctx.positions),
            _p(ctx.token_slot), _p(block_table), block_table.stride(0), page_size, nq, nkv, window,
            int(keep_first), int(bool(sink)), ctypes.c_float(scale), nsplit, _p(part), tokens, tile_rows,
            _tag(q.dtype), _p(sink_values), ctypes.c_float(score_cap), _p(slopes), _stream(),
        ),
        "rl_attn_tile",
    )


_TILE_SPLIT_KEYS = 128  # fewest keys a workgroup's share of a tile is worth
_TILE_MAX_SPLITS = 16


def tile_splits(workgroups: int, span: int, window: int, keep_first: int, units: int | None = None) -> int:
    """Workgroups a tile's keys are dealt to in a bfloat16 launch of ``workgroups`` (tile, kv head)
    pairs over at most ``span`` keys: as many as give every compute unit one, each with a share
    that is worth a workgroup."""
    units = chip().units if units is None else units
    keys = span if window <= 0 else min(span, window + keep_first + 16)
    return max(1, min(_TILE_MAX_SPLITS, units // max(workgroups, 1), keys // _TILE_SPLIT_KEYS))


def paged_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    out: torch.Tensor,
    ctx,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    window: int,
    scale: float,
    prepare: Optional[tuple] = None,
    value_dim: Optional[int] = None,
    keep_first: int = 0,
    sink: bool = False,
    sink_values: Optional[torch.Tensor] = None,
    score_cap: float = 0.0,
    slopes: Optional[torch.Tensor] = None,
) -> None:
    """Attention of every token of the step over its request's cached keys.

    Head sizes in steps of 16 run on the matrix cores: float32 on the float32 kernel,
    bfloat16 on the bfloat16 kernels (single tokens go to the split-key decode kernel, portions
    to the tiled prefill kernel).  Other head sizes run the FMA kernel in either type.

    ``prepare`` = ``(q_norm_w, cos, sin, eps)``: ``q`` is the packed [q | k | v] row of every token,
    and the kernels norm and rotate the query heads as they read them (only where
    :func:`attention_prepares_queries` says so).

    ``value_dim`` (the size of a value head, where it is not ``d``), ``keep_first`` (with a window:
    the request's first positions stay visible behind it) and ``sink`` (1 added to the softmax's
    denominator: a key of score 0 without a value; with ``sink_values`` its score is a number of
    the query head, not scaled), ``score_cap`` (a scaled score s becomes ``cap * tanh(s / cap)``) and
    ``slopes`` (one number a query head, times the distance between query and key, taken off the
    score) send the step to the kernels that take them:
    tiles of 16 rows on the matrix cores for head sizes in steps of 16, the FMA kernel otherwise."""
    if prepare is not None and not attention_prepares_queries(q.dtype, d, 0 if prepare[1] is None else prepare[1].shape[1]):
        raise KernelError("the attention kernels do not finish the queries of this head size, type or rotation")
    dv = d if value_dim is None else int(value_dim)
    keep_first = int(keep_first) if window > 0 else 0  # without a window every key is seen anyway
    if dv != d or keep_first or sink or sink_values is not None or score_cap or slopes is not None:
        # value heads of their own size, kept first positions, one more term in the denominator
        if prepare is not None:
            raise KernelError("queries are finished before an attention with these options")
        if d % 16 == 0 and dv % 16 == 0 and page_size % 4 == 0:
            attention_tile(q, k_cache, v_cache, out, ctx, block_table, page_size, nq, nkv, d, dv,
                           window, keep_first, sink, scale, sink_values, score_cap, slopes)
        else:
            attention_generic(
                q, k_cache, v_cache, out, ctx.positions, ctx.token_slot, block_table, page_size,
                nq, nkv, d, window, scale, ctx.max_position, dv, keep_first, sink, sink_values, score_cap, slopes,
            )
        return
    if q.dtype == torch.float32 and d % 16 == 0:
        attention_f32(q, k_cache, v_cache, out, ctx, block_table, page_size, nq, nkv, d, window, scale)
        return
    if q.dtype != torch.bfloat16 or d % 16:
        attention_generic(
            q, k_cache, v_cache, out, ctx.positions, ctx.token_slot, block_table, page_size,
            nq, nkv, d, window, scale, ctx.max_position,
        )
        return
    tokens = q.shape[0]
    pages = k_cache.shape[0]
    _need(q, "q", torch.bfloat16, (tokens, (nq * d) if prepare is None else (nq + 2 * nkv) * d))
    _need(out, "out", torch.bfloat16, (tokens, nq * d))
    _need(k_cache, "k_cache", torch.bfloat16, (pages, nkv, page_size, d))
    _need(v_cache, "v_cache", torch.bfloat16, (pages, nkv, d, page_size))
    _need(block_table, "block_table", torch.int32)
    if page_size % 4:
        raise KernelError(f"the matrix-core attention kernels need a page size that is a multiple of 4, got {page_size}")
    if ctx.max_position // page_size >= block_table.shape[1]:
        raise KernelError(
            f"position {ctx.max_position} needs page {ctx.max_position // page_size} of a block "
            f"table with {block_table.shape[1]} columns"
        )
    q_norm_w = cos = sin = None
    eps = 0.0
    if prepare is not None:
        q_norm_w, cos, sin, eps = prepare
        if q_norm_w is not None:
            _need(q_norm_w, "q_norm weight", torch.float32, (d,))
        if cos is not None:
            _need(cos, "cos table", torch.float32, (None, d // 2))
            _need(sin, "sin table", torch.float32, tuple(cos.shape))
            if ctx.max_position >= cos.shape[0]:
                raise KernelError(
                    f"position {ctx.max_position} is beyond the rotation table of {cos.shape[0]} positions"
                )
    if ctx.max_position >= (1 << 32) // page_size:
        # the prefill kernel divides positions by the page size with one multiplication
        raise KernelError(f"position {ctx.max_position} is too large for pages of {page_size} tokens")
    lib = attention_lib(d)
    group = nq // nkv
    plan = attention_plan(ctx, group, d)
    if plan.num_tiles:
        groups, nsplit = _prefill_shape(plan, nkv, window, tile_rows_of(lib))
        part_o = part_ml = tokens_list = None
        if nsplit > 1:
            part_o = torch.empty((tokens, nq, nsplit, d), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((tokens, nq, nsplit, 2), dtype=torch.float32, device=q.device)
            tokens_list = plan.prefill_tokens(q.device)
        _ok(
            lib.rl_attn_prefill(
                _p(q), _p(k_cache), _p(v_cache), _p(out), _p(plan.tile_info),
                _p(plan.work_order(nkv, q.device, 2 // groups)), plan.num_tiles,
                _p(ctx.token_slot), _p(block_table), block_table.stride(0), page_size, nq, nkv,
                window, ctypes.c_float(scale), groups, nsplit, _p(part_o), _p(part_ml), _p(tokens_list),
                0 if tokens_list is None else tokens_list.numel(),
                int(prepare is not None), _p(q_norm_w), _p(cos), _p(sin), ctypes.c_float(eps), _stream(),
            ),
            "rl_attn_prefill",
        )
    if plan.num_decode:
        # single tokens beside portions: their keys and values are in the cache already
        fused = None if prepare is None else (q_norm_w, None, cos, sin, None, None, eps)
        _decode_launch(lib, plan, ctx, q, k_cache, v_cache, out, block_table, page_size, nq, nkv, d,
                       window, scale, fused)


def attention_prepares_queries(x_dtype: torch.dtype, d: int, rotary_half: int, pairing: str = "half_split") -> bool:
    """Whether the bfloat16 attention kernels can norm and rotate the query heads themselves, from
    the packed rows: a head size whose rotation pairs stay within a lane, the half-split rotation
    of the whole head or none."""
    if x_dtype != torch.bfloat16 or d % 64 or rotary_half not in (0, d // 2):
        return False
    return not (rotary_half and pairing != "half_split")


def attention_plan(ctx, group: int, d: int) -> AttentionPlan:
    """The step's launch data for one group size, made once and kept with the step."""
    key = ("attention_plan", group)
    plan = ctx.extra.get(key)
    if plan is None:
        plan = AttentionPlan(ctx, group, attention_lib(d).rl_attn_prefill_rows())
        ctx.extra[key] = plan
    return plan


def _decode_launch(lib, plan, ctx, q, k_cache, v_cache, out, block_table, page_size, nq, nkv, d,
                   window, scale, fused) -> None:
    """Split-key decode attention of the step's single tokens.  ``fused`` is ``None`` (``q``
    holds finished queries) or ``(q_norm_w, k_norm_w, cos, sin, k_write, v_write, eps)`` with
    ``q`` the packed [q | k | v] rows."""
    # under a graph the split is laid out for the longest context of the graph's bucket
    span = _static(ctx).get("context_bound", plan.max_decode_ctx)
    pairs, chunk, nsplit = _decode_split(plan.num_decode, nq, nkv, span, page_size, window)
    if plan.num_decode > 65535:
        raise KernelError(f"{plan.num_decode} single-token requests exceed the decode kernel's launch grid")
    # with more workgroups than start at once, the longest requests go first
    order = plan.decode_order(ctx) if pairs * nsplit > chip().decode_resident else None
    part_o = part_ml = None
    if nsplit > 1:
        part_o = torch.empty((plan.num_decode, nq, nsplit, d), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((plan.num_decode, nq, nsplit, 2), dtype=torch.float32, device=q.device)
    qn = kn = cos = sin = kw = vw = None
    eps = 0.0
    if fused is not None:
        qn, kn, cos, sin, kw, vw, eps = fused
    _ok(
        lib.rl_attn_decode(
            _p(q), _p(k_cache), _p(v_cache), _p(out), _p(part_o), _p(part_ml),
            _p(plan.seq_token), _p(order), _p(ctx.positions), _p(ctx.token_slot), _p(block_table),
            block_table.stride(0), page_size, plan.num_decode, nq, nkv, window,
            ctypes.c_float(scale), chunk, nsplit, int(fused is not None), _p(qn), _p(kn), _p(cos),
            _p(sin), _p(kw), _p(vw), ctypes.c_float(eps), _stream(),
        ),
        "rl_attn_decode",
    )


def _decode_split(num_decode: int, nq: int, nkv: int, span: int, page_size: int, window: int,
                  units: int | None = None) -> tuple[int, int, int]:
    """(workgroups before splitting, keys a split, splits) of a decode launch of ``num_decode``
    single tokens over at most ``span`` keys: splits of a multiple of 128 keys, as many as put a
    workgroup on every compute unit, each within what the kernel stages of page ids."""
    units = chip().units if units is None else units
    if window > 0:
        span = min(span, window + 31)
    chunks = (nq // nkv + 15) // 16
    pairs = num_decode * nkv * chunks
    want = max(1, units // pairs)
    chunk = max(_MIN_SPLIT_KEYS, -(-(-(-span // want)) // 128) * 128)
    chunk = min(chunk, max(32, ((_MAX_SPLIT_PAGES - 1) * page_size - 31) // 32 * 32))
    return pairs, chunk, -(-span // chunk)


def decode_scratch_bytes(rows: int, nq: int, nkv: int, d: int, span: int, page_size: int, window: int) -> int:
    """Bytes of split results (float32 outputs, maxima and sums) that a decode launch of
    ``rows`` single tokens over at most ``span`` keys keeps between its two kernels."""
    _, _, nsplit = _decode_split(rows, nq, nkv, span, page_size, window)
    return 0 if nsplit == 1 else rows * nq * nsplit * (d + 2) * 4


def decode_attention_fusable(ctx, x_dtype: torch.dtype, group: int, d: int, rotary_half: int,
                             pairing: str = "half_split") -> bool:
    """Whether the step is one the fused decode kernel takes: bfloat16, single tokens only,
    a head size whose rotation pairs stay within a lane, the half-split rotation of the whole
    head or none."""
    if not attention_prepares_queries(x_dtype, d, rotary_half, pairing):
        return False
    plan = attention_plan(ctx, group, d)
    return plan.num_tiles == 0 and plan.num_decode > 0


def decode_attention_fused(
    qkv: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    out: torch.Tensor,
    ctx,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    window: int,
    scale: float,
    q_norm_w: Optional[torch.Tensor],
    k_norm_w: Optional[torch.Tensor],
    cos: Optional[torch.Tensor],
    sin: Optional[torch.Tensor],
    eps: float,
    write_cache: bool,
) -> None:
    """Per-head norm, rotation, cache write and split-key attention of a step of single
    tokens in one kernel (plus the merge of the splits).  Same result as
    ``qknorm_rope_kvwrite`` followed by ``paged_attention`` up to rounding."""
    tokens = qkv.shape[0]
    pages = k_cache.shape[0]
    _need(qkv, "qkv", torch.bfloat16, (tokens, (nq + 2 * nkv) * d))
    _need(out, "out", torch.bfloat16, (tokens, nq * d))
    _need(k_cache, "k_cache", torch.bfloat16, (pages, nkv, page_size, d))
    _need(v_cache, "v_cache", torch.bfloat16, (pages, nkv, d, page_size))
    _need(block_table, "block_table", torch.int32)
    if page_size % 4:
        raise KernelError(f"the matrix-core attention kernels need a page size that is a multiple of 4, got {page_size}")
    if ctx.max_position // page_size >= block_table.shape[1]:
        raise KernelError(
            f"position {ctx.max_position} needs page {ctx.max_position // page_size} of a block "
            f"table with {block_table.shape[1]} columns"
        )
    for w, name in ((q_norm_w, "q_norm weight"), (k_norm_w, "k_norm weight")):
        if w is not None:
            _need(w, name, torch.float32, (d,))
    if cos is not None:
        _need(cos, "cos table", torch.float32, (None, d // 2))
        _need(sin, "sin table", torch.float32, tuple(cos.shape))
        if ctx.max_position >= cos.shape[0]:
            raise KernelError(
                f"position {ctx.max_position} is beyond the rotation table of {cos.shape[0]} positions"
            )
    lib = attention_lib(d)
    if not lib.rl_attn_decode_fusable():
        raise KernelError(f"the fused decode kernel needs a head size that is a multiple of 64, got {d}")
    plan = attention_plan(ctx, nq // nkv, d)
    if plan.num_tiles or plan.num_decode != tokens:
        raise KernelError("the fused decode kernel takes steps of single tokens only")
    fused = (q_norm_w, k_norm_w, cos, sin, k_cache if write_cache else None,
             v_cache if write_cache else None, eps)
    _decode_launch(lib, plan, ctx, qkv, k_cache, v_cache, out, block_table, page_size, nq, nkv, d,
                   window, scale, fused)


# --------------------------------------------------------------------------- #
# matrix-memory recurrence
# --------------------------------------------------------------------------- #
MLSTM_MAX_KEY_DIM = 256  # the scan stages a token's query and key of one head in LDS
MLSTM_CHUNK = 64  # tokens a chunk of the chunked form
MLSTM_CHUNKED_FROM = 16  # a step whose longest portion has so many tokens runs the chunked form


def _mlstm_chunks(ctx):
    """The step's chunk tables, made once a step and shared by its layers: per chunk
    (request, first token, tokens, 0), per request (first chunk, chunks)."""
    key = "mlstm_chunks"
    found = ctx.extra.get(key) if hasattr(ctx, "extra") else None
    if found is None:
        chunks, per_seq, at = [], [], 0
        for i, n in enumerate(ctx.h_seq_lens):
            per_seq += [len(chunks) // 4, -(-n // MLSTM_CHUNK)]
            for lo in range(0, n, MLSTM_CHUNK):
                chunks += [i, at + lo, min(MLSTM_CHUNK, n - lo), 0]
            at += n
        dev = ctx.seq_slots.device
        found = (upload_ints(chunks, dev), len(chunks) // 4, upload_ints(per_seq, dev))
        if hasattr(ctx, "extra"):
            ctx.extra[key] = found
    return found


def gate_product(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x w^T`` in float32 for a float32 matrix ``w`` of few rows (the gates of a recurrence,
    two a head) and rows ``x`` of either type: one launch, no widened copy of ``x``."""
    tokens, k = x.shape
    n = w.shape[0]
    _need(x, "x")
    _need(w, "gate weights", torch.float32, (n, k))
    out = torch.empty((tokens, n), dtype=torch.float32, device=x.device)
    _ok(mlstm_lib().rl_gate_product(_p(x), _p(w), _p(out), tokens, k, n, _tag(x.dtype), _stream()), "rl_gate_product")
    return out


def mlstm(
    packed: torch.Tensor,
    columns: tuple[int, int, int, int],
    gate_pre: torch.Tensor,
    gate_bias: Optional[torch.Tensor],
    norm_weight: torch.Tensor,
    out: torch.Tensor,
    ctx,
    S: torch.Tensor,
    n: torch.Tensor,
    m: torch.Tensor,
    heads: int,
    dk: int,
    dv: int,
    cap: float,
    eps: float,
    chunked: Optional[bool] = None,
) -> None:
    """The matrix-memory mixer between its projections and its output projection.

    ``packed [T, width]`` holds, from the columns ``columns = (q, k, v, g)`` on, every token's
    query and key heads (``heads * dk`` each), value heads and output gates (``heads * dv``
    each); ``gate_pre [T, 2 * heads]`` float32 the pre-activations of the input gates, then of
    the forget gates (``gate_bias`` is added to them).  The per-request state ``S [slots, heads,
    dk, dv]``, ``n [slots, heads, dk]``, ``m [slots, heads]`` (float32) is read at the rows
    ``ctx.seq_slots`` and left as it is after each request's last token of the step.
    ``out [T, heads * dv]``: every head's output divided by its root mean square, times
    ``norm_weight``, times the sigmoid of the output gate.

    Three forms of the recurrence, which differ by rounding: a step of single tokens streams
    every state through once; short portions run token by token with the state in registers;
    and ``chunked`` (by default a step whose longest portion has 16 tokens or more) runs chunks
    of 64 tokens on the matrix cores."""
    tokens, width = packed.shape
    q_col, k_col, v_col, g_col = (int(c) for c in columns)
    _need(packed, "packed projections")
    _need(gate_pre, "gate pre-activations", torch.float32, (tokens, 2 * heads))
    if gate_bias is not None:
        _need(gate_bias, "gate bias", torch.float32, (2 * heads,))
    _need(norm_weight, "head norm weight", torch.float32, (heads * dv,))
    _need(out, "out", packed.dtype, (tokens, heads * dv))
    slots = S.shape[0]
    _need(S, "state S", torch.float32, (slots, heads, dk, dv))
    _need(n, "state n", torch.float32, (slots, heads, dk))
    _need(m, "state m", torch.float32, (slots, heads))
    _need(ctx.cu_seqlens, "cu_seqlens", torch.int32, (ctx.num_seqs + 1,))
    _need(ctx.seq_slots, "seq_slots", torch.int32, (ctx.num_seqs,))
    if not 1 <= dk <= MLSTM_MAX_KEY_DIM:
        raise KernelError(f"the recurrence takes key sizes up to {MLSTM_MAX_KEY_DIM}, got {dk}")
    for name, col, size in (("q", q_col, heads * dk), ("k", k_col, heads * dk), ("v", v_col, heads * dv),
                            ("g", g_col, heads * dv)):
        if col < 0 or col + size > width:
            raise KernelError(f"columns {col}..{col + size} of {name} lie outside packed rows of {width}")
    if ctx.h_seq_slots and max(ctx.h_seq_slots) >= slots:
        raise KernelError(f"slot {max(ctx.h_seq_slots)} is outside a state of {slots} slots")
    if sum(ctx.h_seq_lens) != tokens:
        raise KernelError(f"the step's requests bring {sum(ctx.h_seq_lens)} tokens, the rows are {tokens}")
    lib = mlstm_lib()
    dev = packed.device
    log_keep = torch.empty((tokens, heads), dtype=torch.float32, device=dev)
    log_take = torch.empty_like(log_keep)
    m_tok = torch.empty_like(log_keep)
    # rows of the unfinished outputs: dv numerators, then n . q, padded to a multiple of 16 bytes
    raw = torch.empty((tokens, heads, (dv + 4) & ~3), dtype=torch.float32, device=dev)
    _ok(
        lib.rl_mlstm_gates(
            _p(gate_pre), _p(gate_bias), _p(ctx.cu_seqlens), _p(ctx.seq_slots), _p(m), _p(log_keep),
            _p(log_take), _p(m_tok), ctx.num_seqs, heads, ctypes.c_float(cap), max(ctx.h_seq_lens, default=1),
            _stream(),
        ),
        "rl_mlstm_gates",
    )
    chunked = max(ctx.h_seq_lens, default=0) >= MLSTM_CHUNKED_FROM if chunked is None else chunked
    if chunked:
        # portions of prompts: every chunk of 64 tokens at once on the matrix cores
        chunks, nchunks, seq_chunks = _mlstm_chunks(ctx)
        U = torch.empty((nchunks, heads, dk, dv), dtype=torch.float32, device=dev)
        Un = torch.empty((nchunks, heads, dk), dtype=torch.float32, device=dev)
        decay = torch.empty((nchunks, heads), dtype=torch.float32, device=dev)
        _ok(
            lib.rl_mlstm_chunked(
                _p(packed), width, q_col, k_col, v_col, _p(log_keep), _p(log_take), _p(chunks), nchunks,
                _p(seq_chunks), _p(ctx.seq_slots), ctx.num_seqs, _p(U), _p(Un), _p(decay), _p(S), _p(n), _p(raw),
                heads, dk, dv, ctypes.c_float(float(dk) ** -0.5), _tag(packed.dtype), _stream(),
            ),
            "rl_mlstm_chunked",
        )
    elif tokens == ctx.num_seqs:
        # single tokens only: the state goes through once, as a stream
        _ok(
            lib.rl_mlstm_step(
                _p(packed), width, q_col, k_col, v_col, _p(log_keep), _p(log_take), _p(ctx.seq_slots), _p(S),
                _p(n), _p(raw), tokens, heads, dk, dv, ctypes.c_float(float(dk) ** -0.5), _tag(packed.dtype),
                _stream(),
            ),
            "rl_mlstm_step",
        )
    else:
        _ok(
            lib.rl_mlstm_scan(
                _p(packed), width, q_col, k_col, v_col, _p(log_keep), _p(log_take), _p(ctx.cu_seqlens),
                _p(ctx.seq_slots), _p(S), _p(n), _p(raw), ctx.num_seqs, heads, dk, dv,
                ctypes.c_float(float(dk) ** -0.5), _tag(packed.dtype), _stream(),
            ),
            "rl_mlstm_scan",
        )
    _ok(
        lib.rl_mlstm_finish(
            _p(raw), _p(m_tok), _p(packed), width, g_col, _p(norm_weight), _p(out), tokens, heads, dv,
            ctypes.c_float(eps), _tag(packed.dtype), _stream(),
        ),
        "rl_mlstm_finish",
    )


# --------------------------------------------------------------------------- #
# token-shift time mixing and the state-space mixer
# --------------------------------------------------------------------------- #
WKV_MAX_HEAD_DIM = 256  # a thread keeps one column of a head's state in registers
SSM_MAX_STATE = 256
SSM_MAX_HEAD_DIM = 256
CONV_MAX_TAPS = 16


def _step_requests(ctx, tokens: int, slots: int) -> None:
    """The per-request tables every recurrent kernel walks, checked against the rows and the state."""
    _need(ctx.cu_seqlens, "cu_seqlens", torch.int32, (ctx.num_seqs + 1,))
    _need(ctx.seq_slots, "seq_slots", torch.int32, (ctx.num_seqs,))
    if ctx.h_seq_slots and max(ctx.h_seq_slots) >= slots:
        raise KernelError(f"slot {max(ctx.h_seq_slots)} is outside a state of {slots} slots")
    if sum(ctx.h_seq_lens) != tokens or (ctx.h_seq_lens and min(ctx.h_seq_lens) < 1):
        raise KernelError(f"the step's requests bring {list(ctx.h_seq_lens)} tokens, the rows are {tokens}")


def token_shift(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, mixes: torch.Tensor, mix_last: torch.Tensor,
                ctx) -> None:
    """The five mixes of a token-shift mixer: with ``h'`` the row before a token's (the request's
    ``state`` row, float32 ``[slots, width]``, before its first token of the step), branch ``b``
    reads ``h + (h' - h) * mu[b]`` (``mu`` float32 ``[5 * width]``).  Branches 0 to 3 go to
    ``mixes [4, tokens, width]`` in the type of ``x``, branch 4 to ``mix_last [tokens, width]`` in
    float32.  Afterwards every request's state row holds its last row of the step."""
    tokens, width = x.shape
    _need(x, "x")
    _need(mu, "mix coefficients", torch.float32, (5 * width,))
    _need(state, "shift state", torch.float32, (None, width))
    _need(mixes, "mixes", x.dtype, (4, tokens, width))
    _need(mix_last, "float32 mix", torch.float32, (tokens, width))
    _step_requests(ctx, tokens, state.shape[0])
    _ok(
        recurrent_lib().rl_token_shift(_p(x), _p(mu), _p(state), _p(mixes), _p(mix_last), _p(ctx.cu_seqlens),
                                       _p(ctx.seq_slots), ctx.num_seqs, tokens, width, _tag(x.dtype), _stream()),
        "rl_token_shift",
    )


def wkv(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, decay_pre: torch.Tensor,
        decay_bias: torch.Tensor, bonus: torch.Tensor, norm_weight: torch.Tensor, out: torch.Tensor, ctx,
        S: torch.Tensor, heads: int, d: int, eps: float) -> None:
    """The time-mixing recurrence between its projections and its output projection.  ``r, k, v,
    g [T, heads * d]``; ``decay_pre`` float32: the decay of a key channel is ``exp(-exp(decay_pre +
    decay_bias))``; ``bonus [heads, d]`` weighs the current token's own key.  Per head, with the state ``S [slots, heads, d, d]`` (float32, kept
    value channel first: ``S[.., j, i]`` belongs to key channel ``i`` and value channel ``j``) read at
    the rows ``ctx.seq_slots`` and left as it is after each request's last token::

        o = (S + diag(bonus) k v^T)^T r        S <- diag(decay) S + k v^T

    ``out``: every head's ``o`` divided by its root mean square (``eps`` inside the root), times
    ``norm_weight``, times ``silu(g)``."""
    tokens, inner = r.shape
    if inner != heads * d or not 1 <= d <= WKV_MAX_HEAD_DIM:
        raise KernelError(f"rows of {inner} are not {heads} heads of {d} (at most {WKV_MAX_HEAD_DIM}) channels")
    for t, name in ((r, "r"), (k, "k"), (v, "v"), (g, "g"), (out, "out")):
        _need(t, name, r.dtype, (tokens, inner))
    _need(decay_pre, "decay pre-activations", torch.float32, (tokens, inner))
    _need(decay_bias, "decay bias", torch.float32, (inner,))
    _need(bonus, "bonus", torch.float32, (heads, d))
    _need(norm_weight, "head norm weight", torch.float32, (inner,))
    _need(S, "state", torch.float32, (None, heads, d, d))
    _step_requests(ctx, tokens, S.shape[0])
    raw = torch.empty((tokens, inner), dtype=torch.float32, device=r.device)  # the heads' outputs before their norm
    _ok(
        recurrent_lib().rl_wkv_scan(_p(r), _p(k), _p(v), _p(g), _p(decay_pre), _p(decay_bias), _p(bonus),
                                    _p(norm_weight), _p(out), _p(raw), _p(ctx.cu_seqlens), _p(ctx.seq_slots), _p(S),
                                    ctx.num_seqs, tokens, heads, d, ctypes.c_float(eps), _tag(r.dtype), _stream()),
        "rl_wkv_scan",
    )


def causal_conv(packed: torch.Tensor, col0: int, weight: torch.Tensor, bias: torch.Tensor, state: torch.Tensor,
                out: torch.Tensor, ctx) -> None:
    """A causal convolution per channel over the columns ``col0 ..`` of ``packed``, with bias and
    silu: ``weight [channels, taps]`` float32, whose last column meets the current token.  Inputs
    before a request's first token of the step are its ``state`` rows (float32 ``[slots, taps - 1,
    channels]``, oldest first; one row that is never read for a single tap), which afterwards hold
    the last ``taps - 1`` inputs the request has seen.  ``out [tokens, channels]`` float32."""
    tokens, width = packed.shape
    channels, taps = weight.shape
    _need(packed, "packed rows")
    _need(weight, "convolution taps", torch.float32)
    _need(bias, "convolution bias", torch.float32, (channels,))
    _need(state, "convolution state", torch.float32, (None, max(taps - 1, 1), channels))
    _need(out, "out", torch.float32, (tokens, channels))
    if not 1 <= taps <= CONV_MAX_TAPS or col0 < 0 or col0 + channels > width:
        raise KernelError(f"{taps} taps over columns {col0}..{col0 + channels} of rows of {width}")
    _step_requests(ctx, tokens, state.shape[0])
    _ok(
        recurrent_lib().rl_causal_conv(_p(packed), width, int(col0), _p(weight), _p(bias), _p(state), _p(out),
                                       _p(ctx.cu_seqlens), _p(ctx.seq_slots), ctx.num_seqs, tokens, channels, taps,
                                       _tag(packed.dtype), _stream()),
        "rl_causal_conv",
    )


def state_space_scan(mixed: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, decay_log: torch.Tensor,
                     skip: torch.Tensor, packed: torch.Tensor, out: torch.Tensor, ctx, S: torch.Tensor,
                     heads: int, p: int, n: int, groups: int) -> None:
    """The state-space recurrence.  ``mixed [T, heads * p + 2 * groups * n]`` float32: ``x``, ``B``
    and ``C`` behind their convolution; ``dt_raw [T, heads]`` float32.  Per head (which reads group
    ``head // (heads / groups)``), with ``dt = softplus(dt_raw + dt_bias)`` and the state ``S [slots,
    heads, p, n]`` (float32, the head's channel first) read at the rows ``ctx.seq_slots`` and left
    after each request's last token::

        S <- exp(-exp(decay_log) dt) S + dt B x^T        y = S^T C + skip x

    ``out [T, heads * p]`` float32: ``y * silu(z)``, ``z`` the first ``heads * p`` columns of ``packed``."""
    tokens = mixed.shape[0]
    inner = heads * p
    if groups < 1 or heads % groups or not 1 <= n <= SSM_MAX_STATE or not 1 <= p <= SSM_MAX_HEAD_DIM:
        raise KernelError(f"{heads} heads of {p} channels in {groups} groups with states of {n}")
    _need(mixed, "convolved rows", torch.float32, (tokens, inner + 2 * groups * n))
    _need(dt_raw, "step sizes", torch.float32, (tokens, heads))
    for t, name in ((dt_bias, "step bias"), (decay_log, "decay"), (skip, "skip")):
        _need(t, name, torch.float32, (heads,))
    _need(packed, "packed rows", None, (tokens, None))
    if packed.shape[1] < inner:
        raise KernelError(f"packed rows of {packed.shape[1]} hold no gate of {inner} channels")
    _need(out, "out", torch.float32, (tokens, inner))
    _need(S, "state", torch.float32, (None, heads, p, n))
    _step_requests(ctx, tokens, S.shape[0])
    _ok(
        recurrent_lib().rl_ssm_scan(_p(mixed), _p(dt_raw), _p(dt_bias), _p(decay_log), _p(skip), _p(packed),
                                    packed.shape[1], _p(out), _p(ctx.cu_seqlens), _p(ctx.seq_slots),
                                    _p(S), ctx.num_seqs, tokens, heads, p, n, groups, _tag(packed.dtype), _stream()),
        "rl_ssm_scan",
    )


def group_rmsnorm(y: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, parts: int, eps: float) -> None:
    """Every row of ``y`` (float32) in ``parts`` equal parts, each divided by its own root mean
    square (``eps`` inside the root), times ``weight``; ``out`` in either type."""
    tokens, width = y.shape
    _need(y, "y", torch.float32)
    _need(weight, "norm weight", torch.float32, (width,))
    _need(out, "out", None, (tokens, width))
    if parts < 1 or width % parts:
        raise KernelError(f"rows of {width} do not divide into {parts} parts")
    _ok(
        recurrent_lib().rl_group_rmsnorm(_p(y), _p(weight), _p(out), tokens, width, parts, ctypes.c_float(eps),
                                         _tag(out.dtype), _stream()),
        "rl_group_rmsnorm",
    )
