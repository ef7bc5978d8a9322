"""Grouped-query attention over the paged cache.

Per step: fused QKV projection (rapid_llm/models/base.py:121-132), per-head RMSNorm of q
and k over head_dim before the rotation (:134-137), rotation (:139-140), write of this
step's keys and values into their pages (rapid_llm/modules/attention.py:126-138), attention
of every query over its request's cached keys up to its own position (:157-240), output
projection (base.py:164-165).  The norm, the rotation and the cache write are one kernel.
How the rotation is applied is the position part's to say (its tables' width: how many of a
head's channels rotate; its ``pairing``: which of them form a pair); the kernels here take
every such case, the fastest ones the half-split rotation of the whole head.

Keys and values are always read back from the pages, also for the tokens of the current
step, so that one code path serves whole prompts, portions and single decoded tokens
(the reference switches kernels by phase, attention.py:179-240).  ``window`` > 0 limits a
query at position p to keys ``[p - window + 1, p]`` (rapid_llm/engine/kv_cache_spec.py:203-222).

Two options change what the packed projection holds.  ``values="keys"``: there is no value
projection, a token's values are its keys as projected, before the rotation; the packed row is
``[q | k]`` and the cache write reads the values from the key columns.  ``head_gate_name``: a
projection of one number per query head rides in the same product (rows behind the keys and
values, padded to a multiple of 8), and every head's output is multiplied by the sigmoid of its
number before the output projection.

Three more options send a layer to the attention kernels that take them (tiles of 16 rows on the
matrix cores, in both types).  ``value_dim``: value heads of a size of their own (the packed row
is ``[q | k | v]`` with narrower or wider ``v`` heads, the value pages and the heads' outputs have
that size, the output projection reads ``num_heads * value_dim`` columns).  ``keep_first``: with
a window, a request's first positions stay visible to every later query, and their pages stay
mapped.  ``sink``: the softmax's denominator is ``1 + sum_j exp(s_j)``, as if one more key of
score 0 and without a value were always seen.
"""

from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Mixer, ParamSpec, Source
from .linear import Linear


class GQAAttention(Mixer):
    replayable = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        checkpoint_prefix: str,
        qk_norm_eps: float | None = None,
        window: int = 0,
        position=None,
        softmax_scale: float | None = None,
        name: str = "mixer",
        q_name: str = "q_proj.weight",
        k_name: str = "k_proj.weight",
        v_name: str = "v_proj.weight",
        o_name: str = "o_proj.weight",
        q_norm_name: str = "q_norm.weight",
        k_norm_name: str = "k_norm.weight",
        qkv_bias: bool = False,
        o_bias: bool = False,
        values: str = "own",
        head_gate_name: str | None = None,
        bias_names: dict[str, str] | None = None,
        value_dim: int | None = None,
        keep_first: int = 0,
        sink: bool = False,
        sink_name: str | None = None,
        qk_norm_weights: bool = True,
        score_cap: float = 0.0,
        distance_slope_exponent: float | None = None,
    ) -> None:
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not divisible by {num_kv_heads} kv heads")
        if head_dim % 2 or not 2 <= head_dim <= 256:
            # multiples of 16 run on the matrix cores, every other even size on the kernel that
            # takes any size (an architecture's configuration may be stricter)
            raise ValueError(f"attention kernels take even head sizes up to 256, got {head_dim}")
        self.hidden_size = hidden_size
        self.nq, self.nkv, self.d = num_heads, num_kv_heads, head_dim
        self.dv = head_dim if value_dim is None else int(value_dim)
        if not 1 <= self.dv <= 256:
            raise ValueError(f"attention kernels take value heads of up to 256 channels, got {self.dv}")
        if self.dv != head_dim and (values == "keys" or head_gate_name):
            raise ValueError("value heads of a size of their own come with a value projection and without head gates")
        if keep_first < 0:
            raise ValueError(f"a window keeps a number of first positions, not {keep_first}")
        self.keep_first = int(keep_first) if window else 0  # without a window every key is seen
        self.sink = bool(sink) or sink_name is not None
        self.sink_name = sink_name
        self.sink_values = None
        self.qk_norm_weights = bool(qk_norm_weights)
        if score_cap < 0:
            raise ValueError(f"the cap of the scores must not be negative, got {score_cap}")
        self.score_cap = float(score_cap)
        self.slope_exponent = None if distance_slope_exponent is None else float(distance_slope_exponent)
        self.slopes = None
        self.prefix = checkpoint_prefix
        self.qk_norm_eps = qk_norm_eps
        self.window = int(window)
        self.position = position
        # what the position part says about its rotation must be something the kernels can do
        rotary_dim = int(getattr(position, "rotary_dim", 0) or 0)
        pairing = getattr(position, "pairing", "half_split")
        if rotary_dim % 2 or rotary_dim > head_dim:
            raise ValueError(f"the position encoding rotates {rotary_dim} channels of heads of {head_dim}")
        if pairing not in ops.ROTARY_PAIRINGS:
            raise ValueError(
                f"the attention kernels rotate pairs as {sorted(ops.ROTARY_PAIRINGS)}, not as {pairing!r}"
            )
        if values not in ("own", "keys"):
            raise ValueError(f"the values are the mixer's 'own' projection or its 'keys', not {values!r}")
        self.scale = float(softmax_scale) if softmax_scale is not None else 1.0 / math.sqrt(head_dim)
        self.name = name
        self.names = dict(q=q_name, k=k_name, v=v_name, o=o_name, qn=q_norm_name, kn=k_norm_name,
                          g=head_gate_name)
        self.bias_names = dict(bias_names or {})
        self.values_are_keys = values == "keys"
        # the packed row: query heads, key heads, value heads unless they are the keys, then
        # one gate per query head, padded so that rows stay whole groups of 8 columns
        self.value_head0 = num_heads if self.values_are_keys else num_heads + num_kv_heads
        self.qkv_rows = (num_heads + num_kv_heads) * head_dim + (0 if self.values_are_keys else num_kv_heads * self.dv)
        self.gate_rows = num_heads if head_gate_name else 0
        self.gate_pad = -(self.qkv_rows + self.gate_rows) % 8 if self.gate_rows else 0
        # the options that only the tile kernels (or the kernel for any size) take
        self.extended = (self.dv != head_dim or self.keep_first > 0 or self.sink or self.score_cap > 0
                         or self.slope_exponent is not None)
        self.plain_row = not self.values_are_keys and not self.gate_rows and not self.extended
        self.row_pad = -self.qkv_rows % 8 if (self.extended and not self.gate_rows) else 0
        self.qkv = Linear(hidden_size, self.qkv_rows + self.gate_rows + self.gate_pad + self.row_pad)
        self.o = Linear(num_heads * self.dv, hidden_size)
        self.q_norm_w = self.k_norm_w = None
        # Qwen3 has neither (rapid_llm/models/qwen3.py:16-18: qkv_bias=False); architectures of the
        # same skeleton do (rapid_llm/models/base.py:121-132 passes bias=qkv_bias), under the
        # projections' names with ".bias" in place of ".weight"
        self.qkv_bias, self.o_bias = bool(qkv_bias), bool(o_bias)

    # ---- tensors ---------------------------------------------------------------
    def param_specs(self) -> list[ParamSpec]:
        p, n = self.prefix, self.names
        q_rows, kv_rows = self.nq * self.d, self.nkv * self.d
        v_rows = self.nkv * self.dv
        packed = [Source(p + n["q"], q_rows), Source(p + n["k"], kv_rows)]
        if not self.values_are_keys:
            packed.append(Source(p + n["v"], v_rows))
        if self.gate_rows:
            packed.append(Source(p + n["g"], self.gate_rows))
        if self.gate_pad + self.row_pad:
            packed.append(Source("", self.gate_pad + self.row_pad))  # rows of zeros
        specs = [
            ParamSpec(self.name + ".qkv", (self.qkv.out_features, self.hidden_size), "matrix", tuple(packed)),
            ParamSpec(self.name + ".o", (self.hidden_size, self.nq * self.dv), "matrix",
                      (Source(p + n["o"], self.hidden_size),)),
        ]
        if self.sink_name is not None:
            specs.append(ParamSpec(self.name + ".sink", (self.nq,), "vector", (Source(p + self.sink_name, self.nq),)))
        if self.qk_norm_eps is not None and self.qk_norm_weights:
            specs += [
                ParamSpec(self.name + ".q_norm", (self.d,), "vector", (Source(p + n["qn"], self.d),), init="norm"),
                ParamSpec(self.name + ".k_norm", (self.d,), "vector", (Source(p + n["kn"], self.d),), init="norm"),
            ]

        def bias_of(which: str) -> str:
            if which in self.bias_names:
                return self.bias_names[which]
            weight_name = n[which]
            return weight_name[: -len("weight")] + "bias" if weight_name.endswith("weight") else weight_name + ".bias"

        if self.qkv_bias:
            biases = [Source(p + bias_of("q"), q_rows), Source(p + bias_of("k"), kv_rows)]
            if not self.values_are_keys:
                biases.append(Source(p + bias_of("v"), v_rows))
            if self.gate_rows + self.gate_pad + self.row_pad:
                biases.append(Source("", self.gate_rows + self.gate_pad + self.row_pad))  # the gates have none
            specs.append(ParamSpec(self.name + ".qkv_bias", (self.qkv.out_features,), "vector", tuple(biases)))
        if self.o_bias:
            specs.append(ParamSpec(
                self.name + ".o_bias", (self.hidden_size,), "vector", (Source(p + bias_of("o"), self.hidden_size),)
            ))
        return specs

    def bind(self, params, runtime) -> None:
        bias = params[self.name + ".qkv_bias"] if self.qkv_bias else None
        # A plain [q | k | v] row may run through kernels that read the packed row themselves
        # (the fused decode step, queries finished inside the attention kernels): its bias is
        # added after the product.  Any other row always passes the kernel that norms, rotates
        # and writes the cache, which adds the bias as it reads the heads.
        self.bias_in_kernel = None if self.plain_row else bias
        self.qkv.bind(params[self.name + ".qkv"], bias if self.plain_row else None)
        self.o.bind(params[self.name + ".o"], params[self.name + ".o_bias"] if self.o_bias else None)
        if self.qk_norm_eps is not None and self.qk_norm_weights:
            self.q_norm_w = params[self.name + ".q_norm"]
            self.k_norm_w = params[self.name + ".k_norm"]
        elif self.qk_norm_eps is not None:
            # a norm without a learned weight: the kernels get a weight of ones
            self.q_norm_w = self.k_norm_w = torch.ones(self.d, dtype=torch.float32, device=runtime.device)
        if self.sink_name is not None:
            self.sink_values = params[self.name + ".sink"]
        if self.slope_exponent is not None:
            h = torch.arange(1, self.nq + 1, dtype=torch.float64)
            self.slopes = torch.exp2(-self.slope_exponent * h / self.nq).to(torch.float32).to(runtime.device)
        self.runtime = runtime

    # ---- cache -----------------------------------------------------------------
    def cache_need(self) -> CacheNeed:
        return CacheNeed.keys_and_values(
            self.nkv, self.d, window=self.window, value_dim=self.dv, keep_first=self.keep_first
        )

    def recorded_step_bytes(self, rows: int, context_bound: int, page_size: int) -> int:
        if self.extended:
            # the shares of a tile's keys that several workgroups leave for the merge kernel
            splits = ops.tile_splits(rows * self.nkv, context_bound, self.window, self.keep_first)
            return 0 if splits == 1 else rows * self.nq * splits * (self.dv + 2) * 4
        return ops.decode_scratch_bytes(rows, self.nq, self.nkv, self.d, context_bound, page_size, self.window)

    # ---- step ------------------------------------------------------------------
    @property
    def accepts_scaled_rows(self) -> bool:
        return self.qkv.takes_scaled_rows()

    def forward(self, x, ctx, cache):
        tokens = x.shape[0]
        qkv = self.qkv(x)
        table = ctx.block_tables[cache.group_id]
        pos_enc = self.position
        cos = pos_enc.cos if pos_enc is not None else None
        sin = pos_enc.sin if pos_enc is not None else None
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        out = torch.empty((tokens, self.nq * self.dv), dtype=qkv.dtype, device=x.device)
        rotary_half = cos.shape[1] if cos is not None else 0
        pairing = getattr(pos_enc, "pairing", "half_split") if cos is not None else "half_split"
        if self.plain_row and ops.decode_attention_fusable(
            ctx, qkv.dtype, self.nq // self.nkv, self.d, rotary_half, pairing
        ):
            # a step of single tokens: norm, rotation, cache write and attention in one kernel
            ops.decode_attention_fused(
                qkv, cache.k, cache.v, out, ctx, table, cache.page_size, self.nq, self.nkv, self.d,
                self.window, self.scale, self.q_norm_w, self.k_norm_w, cos, sin, eps, cache.owns_pages,
            )
            return self.o.deferred(out, ctx)
        # where the attention kernels can finish the query heads as they read them, only the keys
        # and values are prepared here, and the queries are never written out
        in_kernel = self.plain_row and ops.attention_prepares_queries(qkv.dtype, self.d, rotary_half, pairing)
        q = None if in_kernel else torch.empty((tokens, self.nq * self.d), dtype=qkv.dtype, device=x.device)
        ops.qknorm_rope_kvwrite(
            qkv, q,
            cache.k if cache.owns_pages else None,
            cache.v if cache.owns_pages else None,
            self.q_norm_w, self.k_norm_w, cos, sin,
            ctx.positions, ctx.token_slot, table, cache.page_size,
            self.nq, self.nkv, self.d, eps, ctx.max_position, pairing, self.value_head0, self.bias_in_kernel,
            self.dv,
        )
        ops.paged_attention(
            qkv if in_kernel else q, cache.k, cache.v, out, ctx, table, cache.page_size,
            self.nq, self.nkv, self.d, self.window, self.scale,
            prepare=(self.q_norm_w, cos, sin, eps) if in_kernel else None,
            value_dim=self.dv, keep_first=self.keep_first, sink=self.sink, sink_values=self.sink_values,
            score_cap=self.score_cap, slopes=self.slopes,
        )
        if self.gate_rows:
            ops.head_gate(out, qkv, self.qkv_rows, self.nq, self.d)
        return self.o.deferred(out, ctx)


MIXERS.register("gqa_attention", GQAAttention)
