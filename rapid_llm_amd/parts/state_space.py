"""A state-space recurrence (state-space duality form) behind a short causal convolution, as a
mixer with a fixed-size state per request.

One product lays a token out as ``[z: inner | x: inner | B: groups * N | C: groups * N | dt: heads]``
(``inner = heads * head_dim``).  ``x``, ``B`` and ``C`` together pass a causal convolution per
channel (``taps`` taps, the last one meeting the current token, zeros before a request's start)
with a bias, and silu.  ``dt = softplus(dt + dt_bias)``.  Per head (head h reads group
``h // (heads / groups)``), with the state ``S [N, head_dim]``::

    S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T          y_t = S_t^T C_t + D x_t

``y`` (heads side by side) is multiplied by ``silu(z)``, divided by its root mean square in
``norm_groups`` equal parts, multiplied by a weight, and the output projection follows.

The packed product runs in the compute type.  The step sizes come from a product of their own
with the same rows of the matrix held in float32; the convolution's sums, softplus, the decays,
the state, the gate and the norm are float32 (``csrc/recurrent.hip``).  The state and the
convolution's last ``taps - 1`` inputs live in the request's slot (``cache.states``).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Mixer, ParamSpec, Source, StateSpec
from .linear import Linear


class StateSpace(Mixer):
    replayable = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        head_dim: int,
        state_size: int,
        groups: int,
        conv_taps: int,
        norm_groups: int,
        norm_eps: float,
        checkpoint_prefix: str,
        position=None,  # the recurrence knows order by itself
        name: str = "mixer",
        in_name: str = "in",
        conv_name: str = "conv",
        conv_bias_name: str = "conv.b",
        dt_bias_name: str = "dt_bias",
        decay_name: str = "A_log",
        skip_name: str = "D",
        norm_name: str = "norm",
        o_name: str = "o",
    ) -> None:
        if num_heads % groups:
            raise ValueError(f"{num_heads} heads are not divisible by {groups} groups")
        if (num_heads * head_dim) % norm_groups:
            raise ValueError(f"{num_heads * head_dim} channels are not divisible into {norm_groups} normed parts")
        if not 1 <= state_size <= ops.SSM_MAX_STATE or not 1 <= head_dim <= ops.SSM_MAX_HEAD_DIM:
            raise ValueError(
                f"the recurrence's kernel takes states of up to {ops.SSM_MAX_STATE} and heads of up to "
                f"{ops.SSM_MAX_HEAD_DIM} channels, got {state_size} and {head_dim}"
            )
        if not 1 <= conv_taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"the convolution's kernel takes up to {ops.CONV_MAX_TAPS} taps, got {conv_taps}")
        self.hidden_size, self.heads, self.p, self.n = hidden_size, num_heads, head_dim, state_size
        self.groups, self.taps, self.parts, self.eps = groups, conv_taps, norm_groups, float(norm_eps)
        self.prefix, self.name = checkpoint_prefix, name
        self.names = dict(inp=in_name, conv=conv_name, conv_b=conv_bias_name, dt_bias=dt_bias_name, a=decay_name,
                          d=skip_name, norm=norm_name, o=o_name)
        self.inner = num_heads * head_dim
        self.channels = self.inner + 2 * groups * state_size  # what the convolution mixes: x, B, C
        self.packed_rows = self.inner + self.channels  # z in front of them
        self.in_proj = Linear(hidden_size, self.packed_rows)
        self.dt_proj = Linear(hidden_size, num_heads)
        self.o = Linear(self.inner, hidden_size)

    def param_specs(self) -> list[ParamSpec]:
        p, n, h = self.prefix, self.names, self.hidden_size
        rows = self.packed_rows + self.heads
        return [
            ParamSpec(self.name + ".in", (rows, h), "matrix", (Source(p + n["inp"], rows),)),
            ParamSpec(self.name + ".conv", (self.channels, self.taps), "vector", (Source(p + n["conv"], self.channels),)),
            ParamSpec(self.name + ".conv_bias", (self.channels,), "vector", (Source(p + n["conv_b"], self.channels),)),
            ParamSpec(self.name + ".dt_bias", (self.heads,), "vector", (Source(p + n["dt_bias"], self.heads),)),
            ParamSpec(self.name + ".decay", (self.heads,), "vector", (Source(p + n["a"], self.heads),)),
            ParamSpec(self.name + ".skip", (self.heads,), "vector", (Source(p + n["d"], self.heads),), init="norm"),
            ParamSpec(self.name + ".norm", (self.inner,), "vector", (Source(p + n["norm"], self.inner),), init="norm"),
            ParamSpec(self.name + ".o", (h, self.inner), "matrix", (Source(p + n["o"], h),)),
        ]

    def bind(self, params, runtime) -> None:
        w = params[self.name + ".in"]
        self.in_proj.bind(w[: self.packed_rows])  # the leading rows of a row-major matrix: no copy
        # the step sizes enter the recurrence: their rows once more, in float32
        self.dt_proj.bind(w[self.packed_rows :].to(torch.float32).contiguous())
        self.conv = params[self.name + ".conv"]
        self.conv_bias = params[self.name + ".conv_bias"]
        self.dt_bias = params[self.name + ".dt_bias"]
        self.decay = params[self.name + ".decay"]
        self.skip = params[self.name + ".skip"]
        self.norm_weight = params[self.name + ".norm"]
        self.o.bind(params[self.name + ".o"])

    def cache_need(self) -> CacheNeed:
        return CacheNeed(
            "state",
            states=(
                StateSpec("conv", (max(self.taps - 1, 1), self.channels), "float32"),
                StateSpec("S", (self.heads, self.p, self.n), "float32"),  # a channel's states side by side
            ),
        )

    def forward(self, x, ctx, cache):
        tokens = x.shape[0]
        packed = self.in_proj(x)
        dt = self.dt_proj(x, out_dtype=torch.float32)
        mixed = torch.empty((tokens, self.channels), dtype=torch.float32, device=x.device)
        ops.causal_conv(packed, self.inner, self.conv, self.conv_bias, cache.states["conv"], mixed, ctx)
        gated = torch.empty((tokens, self.inner), dtype=torch.float32, device=x.device)
        ops.state_space_scan(mixed, dt, self.dt_bias, self.decay, self.skip, packed, gated, ctx, cache.states["S"],
                             self.heads, self.p, self.n, self.groups)
        out = torch.empty((tokens, self.inner), dtype=x.dtype, device=x.device)
        ops.group_rmsnorm(gated, self.norm_weight, out, self.parts, self.eps)
        return self.o.deferred(out, ctx)


MIXERS.register("state_space", StateSpace)
