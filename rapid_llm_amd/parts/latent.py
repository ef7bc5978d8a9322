"""Attention through a latent: per token the cache holds one normed row ``c`` and one rotated
key part ``kr`` that all heads share, and every head has small matrices of its own that turn
``c`` into its keys (``Uk_h``) and values (``Uv_h``).

Head ``h`` scores key ``j`` with ``(qn_h . Uk_h c_j + qr_h . kr_j) * scale``; its output is
``Uv_h sum_j p_j c_j``.  Neither keys nor values are ever formed: the query takes the key matrix
in (``qa_h = Uk_h^T qn_h``, a vector as wide as ``c``), the softmax weights average the rows ``c``
themselves, and ``Uv_h`` is applied to that one average.  What is left is attention of ``heads``
query heads over one shared key row ``[c | kr]`` whose values are its first ``kv_rank`` channels:
the tile attention of this package with one kv head, key size ``kv_rank + rot_dim`` and value
size ``kv_rank`` (the FMA kernel for sizes off the matrix cores' grid).  The key row is paged as
it is read, and the latent a second time transposed, as that kernel's second product wants it.

Per step: one packed product of the mixer's input (query part, latent row, head gates), a row
kernel (RMS norms of the latents, rotation of ``kr``, cache write), the query latent's second
product where queries pass a latent of their own, the heads' key matrices and the rotation of
``qr`` into ``[qa | qr]``, attention, the heads' value matrices (with the gate) and the output
projection.

Options, each a parameter: ``q_rank`` (queries through an RMS-normed latent; 0: one projection),
``window`` (a query sees its own and the ``window - 1`` positions before it; 0: all), ``sink``
(a learned number per head whose ``exp`` joins the softmax's denominator, unscaled), ``gate``
(head ``h``'s output times the sigmoid of a projection of the mixer's input), ``owns_latent``
(``False``: the layer has no latent projection and reads the rows another layer cached, with key
and value matrices of its own) and ``cache_window`` (how much the cache must keep: the longest
view of any layer that reads it).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Mixer, ParamSpec, Source
from .linear import Linear


class LatentAttention(Mixer):
    replayable = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        head_dim: int,  # channels of a head's query and key that do not rotate
        rot_dim: int,  # channels of the key part that all heads share (and of a query head's second part)
        value_dim: int,
        kv_rank: int,
        softmax_scale: float,
        norm_eps: float,
        checkpoint_prefix: str,
        q_rank: int = 0,
        window: int = 0,
        cache_window: int | None = None,
        sink: bool = False,
        gate: bool = False,
        owns_latent: bool = True,
        position=None,
        name: str = "mixer",
        q_name: str = "q",
        q_down_name: str = "dq",
        q_up_name: str = "uq",
        q_norm_name: str = "dq.norm",
        kv_down_name: str = "dkv",
        kv_norm_name: str = "dkv.norm",
        k_up_name: str = "uk",
        v_up_name: str = "uv",
        sink_name: str = "sink",
        gate_name: str = "g",
        o_name: str = "o",
    ) -> None:
        for what, n in (("heads", num_heads), ("head_dim", head_dim), ("value_dim", value_dim), ("kv_rank", kv_rank)):
            if n < 1:
                raise ValueError(f"a latent attention needs a positive {what}, got {n}")
        if rot_dim < 0 or rot_dim % 2 or q_rank < 0 or window < 0:
            raise ValueError(f"rot_dim {rot_dim} (even), q_rank {q_rank} and window {window} must not be negative")
        self.hidden_size, self.nq, self.d, self.rd = hidden_size, num_heads, head_dim, rot_dim
        self.dv, self.r, self.q_rank = value_dim, kv_rank, q_rank
        self.key_dim = kv_rank + rot_dim  # the cached key row [c | kr], and a finished query head
        if self.key_dim % 2:
            raise ValueError(f"the cached row of {kv_rank} + {rot_dim} channels must have an even width")
        on_grid = self.key_dim % 16 == 0 and kv_rank % 16 == 0
        if not on_grid and self.key_dim > 256:
            raise ValueError(
                f"a cached row of {self.key_dim} channels off the matrix cores' grid of 16 is more than the "
                "kernel for any size takes (256)"
            )
        self.scale, self.eps = float(softmax_scale), float(norm_eps)
        self.window = int(window)
        self.cache_window = self.window if cache_window is None else int(cache_window)
        if self.cache_window and (not self.window or self.window > self.cache_window):
            raise ValueError(f"a view of {self.window or 'all'} positions over a cache that keeps {self.cache_window}")
        self.sink, self.gate, self.owns_latent = bool(sink), bool(gate), bool(owns_latent)
        self.position = position
        rotary_dim = int(getattr(position, "rotary_dim", 0) or 0)
        if rotary_dim and (getattr(position, "pairing", None) != "interleaved" or rotary_dim > rot_dim):
            raise ValueError(
                f"the latent attention rotates interleaved pairs of at most its {rot_dim} shared channels, "
                f"not {rotary_dim} as {getattr(position, 'pairing', None)!r}"
            )
        self.prefix, self.name = checkpoint_prefix, name
        self.names = dict(q=q_name, dq=q_down_name, uq=q_up_name, qn=q_norm_name, dkv=kv_down_name,
                          kvn=kv_norm_name, uk=k_up_name, uv=v_up_name, sink=sink_name, g=gate_name, o=o_name)
        # the packed first product: [query part | latent row | gates | padding]
        self.q_rows = q_rank if q_rank else num_heads * (head_dim + rot_dim)
        self.kv_rows = self.key_dim if self.owns_latent else 0
        self.gate_rows = num_heads if self.gate else 0
        rows = self.q_rows + self.kv_rows + self.gate_rows
        self.pad_rows = -rows % 8
        self.first = Linear(hidden_size, rows + self.pad_rows)
        self.q_up = Linear(q_rank, num_heads * (head_dim + rot_dim)) if q_rank else None
        self.o = Linear(num_heads * value_dim, hidden_size)

    # ---- tensors ---------------------------------------------------------------
    def param_specs(self) -> list[ParamSpec]:
        p, n, h = self.prefix, self.names, self.hidden_size
        packed = [Source(p + (n["dq"] if self.q_rank else n["q"]), self.q_rows)]
        if self.owns_latent:
            packed.append(Source(p + n["dkv"], self.kv_rows))
        if self.gate:
            packed.append(Source(p + n["g"], self.gate_rows))
        if self.pad_rows:
            packed.append(Source("", self.pad_rows))
        specs = [
            ParamSpec(self.name + ".first", (self.first.out_features, h), "matrix", tuple(packed)),
            ParamSpec(self.name + ".uk", (self.nq * self.d, self.r), "matrix", (Source(p + n["uk"], self.nq * self.d),)),
            ParamSpec(self.name + ".uv", (self.nq * self.dv, self.r), "matrix", (Source(p + n["uv"], self.nq * self.dv),)),
            ParamSpec(self.name + ".o", (h, self.nq * self.dv), "matrix", (Source(p + n["o"], h),)),
        ]
        if self.q_rank:
            specs += [
                ParamSpec(self.name + ".uq", (self.q_up.out_features, self.q_rank), "matrix",
                          (Source(p + n["uq"], self.q_up.out_features),)),
                ParamSpec(self.name + ".q_norm", (self.q_rank,), "vector", (Source(p + n["qn"], self.q_rank),),
                          init="norm"),
            ]
        if self.owns_latent:
            specs.append(ParamSpec(self.name + ".kv_norm", (self.r,), "vector", (Source(p + n["kvn"], self.r),),
                                   init="norm"))
        if self.sink:
            specs.append(ParamSpec(self.name + ".sink", (self.nq,), "vector", (Source(p + n["sink"], self.nq),)))
        return specs

    def bind(self, params, runtime) -> None:
        self.first.bind(params[self.name + ".first"])
        self.o.bind(params[self.name + ".o"])
        if self.q_up is not None:
            self.q_up.bind(params[self.name + ".uq"])
            self.q_norm_w = params[self.name + ".q_norm"]
        else:
            self.q_norm_w = None
        self.kv_norm_w = params[self.name + ".kv_norm"] if self.owns_latent else None
        self.sink_values = params[self.name + ".sink"] if self.sink else None
        # one small matrix a head, outputs by inputs: the key matrices are applied transposed
        # (from a head's query channels to the latent's), so their copy is laid out that way once
        uk = params[self.name + ".uk"].view(self.nq, self.d, self.r)
        self.uk_t = uk.transpose(1, 2).contiguous()
        self.uv = params[self.name + ".uv"].view(self.nq, self.dv, self.r)
        self.runtime = runtime

    # ---- cache -----------------------------------------------------------------
    def cache_need(self) -> CacheNeed:
        # one shared "kv head": keys [pages, 1, page, kv_rank + rot_dim], the latent once more
        # transposed as values [pages, 1, kv_rank, page]
        return CacheNeed.keys_and_values(1, self.key_dim, window=self.cache_window, value_dim=self.r)

    def recorded_step_bytes(self, rows: int, context_bound: int, page_size: int) -> int:
        splits = ops.tile_splits(rows, context_bound, self.window, 0)
        return 0 if splits == 1 else rows * self.nq * splits * (self.r + 2) * 4

    # ---- step ------------------------------------------------------------------
    def forward(self, x, ctx, cache):
        tokens = x.shape[0]
        packed = self.first(x)
        table = ctx.block_tables[cache.group_id]
        pos = self.position
        cos = pos.cos if pos is not None else None
        sin = pos.sin if pos is not None else None
        q_latent = None
        if self.q_rank:
            q_latent = torch.empty((tokens, self.q_rank), dtype=packed.dtype, device=x.device)
        writes = self.owns_latent and cache.owns_pages
        ops.latent_rows(
            packed, self.q_rank, self.q_norm_w, q_latent, self.q_rows, self.r, self.rd, self.kv_norm_w, cos, sin,
            cache.k if writes else None, cache.v if writes else None,
            ctx.positions, ctx.token_slot, table, cache.page_size, self.eps, ctx.max_position,
        )
        q = self.q_up(q_latent) if self.q_rank else packed
        # a finished query head: [Uk_h^T qn_h | rotated qr_h], as wide as a cached row
        full = torch.empty((tokens, self.nq * self.key_dim), dtype=packed.dtype, device=x.device)
        ops.head_product(q, self.uk_t, full, self.nq, self.d + self.rd, 0, self.key_dim, 0)
        if self.rd:
            ops.rotate_tail(q, full, cos, sin, ctx.positions, self.nq, self.d, self.rd, self.key_dim, self.r,
                            ctx.max_position)
        mean = torch.empty((tokens, self.nq * self.r), dtype=packed.dtype, device=x.device)
        ops.paged_attention(
            full, cache.k, cache.v, mean, ctx, table, cache.page_size, self.nq, 1, self.key_dim, self.window,
            self.scale, value_dim=self.r, sink_values=self.sink_values,
        )
        out = torch.empty((tokens, self.nq * self.dv), dtype=packed.dtype, device=x.device)
        ops.head_product(
            mean, self.uv, out, self.nq, self.r, 0, self.dv, 0,
            gate=packed if self.gate else None, gate_col=self.q_rows + self.kv_rows,
        )
        return self.o.deferred(out, ctx)


MIXERS.register("latent_attention", LatentAttention)
