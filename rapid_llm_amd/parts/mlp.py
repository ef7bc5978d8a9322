"""Feed-forwards.  Dense gated feed-forward: ``down(act(gate(x), up(x)))`` with ``act(g, u) = silu(g) * u``
(SwiGLU), or, with a ``limit``, the clamped variant ``g' * sigmoid(alpha * g') * (u' + 1)`` where
``g' = min(g, limit)`` and ``u' = clamp(u, -limit, limit)``.

Gate and up are one packed matrix ``[2I, H]`` with rows ``[gate | up]``
(rapid_llm/models/base.py:401-404, rapid_llm/modules/linear.py:157-172), so one product
feeds the activation kernel (rapid_llm/modules/mlp.py:67-68).

Beside it a two-layer feed-forward without a gate, ``down(act(up(x)))``, and a mixture of such
experts behind a softmax router.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, ParamSpec, Source
from .lazy import ScaledRows
from .linear import Linear


class SwiGLU(FeedForward):
    replayable = True

    def __init__(
        self,
        hidden_size: int,
        intermediate_size: int,
        checkpoint_prefix: str,
        name: str = "ff",
        gate_name: str = "gate_proj.weight",
        up_name: str = "up_proj.weight",
        down_name: str = "down_proj.weight",
        limit: float = 0.0,
        alpha: float = ops.GLU_ALPHA,
    ) -> None:
        if limit < 0:
            raise ValueError(f"the gated activation's limit must not be negative, got {limit}")
        self.limit, self.alpha = float(limit), float(alpha)
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.prefix = checkpoint_prefix
        self.name = name
        self.names = (gate_name, up_name, down_name)
        self.gate_up = Linear(hidden_size, 2 * intermediate_size)
        self.down = Linear(intermediate_size, hidden_size)

    def param_specs(self) -> list[ParamSpec]:
        h, i = self.hidden_size, self.intermediate_size
        g, u, d = (self.prefix + n for n in self.names)
        return [
            ParamSpec(self.name + ".gate_up", (2 * i, h), "matrix", (Source(g, i), Source(u, i))),
            ParamSpec(self.name + ".down", (h, i), "matrix", (Source(d, h),)),
        ]

    def bind(self, params, runtime) -> None:
        self.gate_up.bind(params[self.name + ".gate_up"])
        self.down.bind(params[self.name + ".down"])

    @property
    def accepts_scaled_rows(self) -> bool:
        return self.gate_up.takes_scaled_rows()

    def forward(self, x, ctx):
        w = self.gate_up.weight
        if w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16:
            # few rows: product and activation in one kernel
            glu = dict(limit=self.limit, alpha=self.alpha)
            act = (ops.gemm_bf16_swiglu(x.rows, w, scaled=x, **glu) if isinstance(x, ScaledRows)
                   else ops.gemm_bf16_swiglu(x, w, **glu))
            if act is not None:
                return self.down.deferred(act, ctx)
        gu = self.gate_up(x)
        act = torch.empty((x.shape[0], self.intermediate_size), dtype=gu.dtype, device=x.device)
        ops.swiglu(gu, act, self.limit, self.alpha)
        return self.down.deferred(act, ctx)


class TwoLayer(FeedForward):
    """``down(act(up(x)))`` with a one-operand activation (``ops.UNARY_ACTIVATIONS``: the tanh form
    of gelu, or the square of relu); no gate, no biases.

    ``activation="polynorm"`` acts on a token's whole hidden vector ``z`` instead: ``a N(z) + b N(z^2)
    + c N(z^3) + e`` with element-wise powers, ``N`` dividing a vector by its root mean square
    (``activation_eps`` inside the root) and the four learned numbers ``a, b, c, e`` of the tensor
    ``activation_name``; statistics and sums are float32."""

    replayable = True

    def __init__(
        self,
        hidden_size: int,
        intermediate_size: int,
        checkpoint_prefix: str,
        activation: str,
        name: str = "ff",
        up_name: str = "up",
        down_name: str = "down",
        activation_name: str = "act",
        activation_eps: float = 0.0,
    ) -> None:
        self.polynorm = activation == "polynorm"
        if not self.polynorm and activation not in ops.UNARY_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not 'polynorm' or one of {sorted(ops.UNARY_ACTIVATIONS)}")
        if self.polynorm and not activation_eps > 0:
            raise ValueError(f"the normalised powers need a positive epsilon, got {activation_eps}")
        self.activation_name, self.activation_eps = activation_name, float(activation_eps)
        self.coefficients = None
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.prefix, self.activation, self.name = checkpoint_prefix, activation, name
        self.names = (up_name, down_name)
        self.up = Linear(hidden_size, intermediate_size)
        self.down = Linear(intermediate_size, hidden_size)

    def param_specs(self) -> list[ParamSpec]:
        h, i = self.hidden_size, self.intermediate_size
        u, d = (self.prefix + n for n in self.names)
        specs = [
            ParamSpec(self.name + ".up", (i, h), "matrix", (Source(u, i),)),
            ParamSpec(self.name + ".down", (h, i), "matrix", (Source(d, h),)),
        ]
        if self.polynorm:
            specs.append(ParamSpec(self.name + ".act", (4,), "vector", (Source(self.prefix + self.activation_name, 4),),
                                   init="norm"))
        return specs

    def bind(self, params, runtime) -> None:
        self.up.bind(params[self.name + ".up"])
        self.down.bind(params[self.name + ".down"])
        if self.polynorm:
            self.coefficients = params[self.name + ".act"]

    def forward(self, x, ctx):
        hidden = self.up(x)
        if self.polynorm:
            ops.polynorm(hidden, hidden, self.coefficients, self.activation_eps)
        else:
            ops.unary_act(hidden, hidden, self.activation)
        return self.down.deferred(hidden, ctx)


class RoutedExperts(FeedForward):
    """A mixture of two-layer experts: every token uses the ``top`` experts that a softmax router
    scores highest, weighted by their scores over the chosen ones' sum (which is the softmax over
    the chosen logits alone), times ``route_scale``; a shared expert (``shared_size`` > 0) runs for
    every token and is added.  ``gated``: the experts are gated ones, ``down(silu(gate(x)) * up(x))``;
    their gate and up projections form one packed matrix, all gates first; with ``limit`` > 0 their
    activation is the clamped one, ``g' * sigmoid(alpha g') * (u' + 1)``.  ``router_bias_name``:
    the router's logits get a bias, one number an expert.  ``scores="sigmoid"``: an expert's score
    is the sigmoid of its logit, and the chosen experts' weights are their scores as they are
    (times ``route_scale``), not divided by their sum.  ``weights_scale="input"`` (gated experts): the
    weight multiplies what the expert reads, not what it returns; its first products being linear,
    the gate and up values are multiplied by it before they are clamped.

    The router's product and scores are float32 in every engine (its matrix is held in
    float32).  The experts' up projections are one packed matrix ``[experts * expert_size +
    shared_size, hidden]`` and their down projections one matrix side by side over the same
    columns, so a step is two products whatever the tokens chose: the activation kernel
    multiplies every expert's hidden units by the token's weight for that expert, which is 0
    for an expert the token does not use.  Every expert's weights are read in every step; nothing
    is gathered, no shape depends on the routing, and a token's result does not depend on the
    rest of the batch."""

    replayable = True

    def __init__(
        self,
        hidden_size: int,
        num_experts: int,
        top: int,
        expert_size: int,
        checkpoint_prefix: str,
        activation: str,
        route_scale: float = 1.0,
        shared_size: int = 0,
        name: str = "ff",
        router_name: str = "router",
        expert_prefix: str = "e",
        shared_prefix: str = "shared.",
        up_name: str = "up",
        down_name: str = "down",
        gated: bool = False,
        gate_name: str = "gate",
        router_bias_name: str | None = None,
        limit: float = 0.0,
        alpha: float = ops.GLU_ALPHA,
        scores: str = "softmax",
        weights_scale: str = "output",
    ) -> None:
        self.gated = bool(gated)
        if scores not in ops.ROUTER_SCORES:
            raise ValueError(f"router scores are one of {sorted(ops.ROUTER_SCORES)}, not {scores!r}")
        if weights_scale not in ("output", "input") or (weights_scale == "input" and not gated):
            raise ValueError(f"an expert's weight scales its 'output', or the 'input' of a gated expert, not {weights_scale!r}")
        if limit < 0 or (limit and not gated):
            raise ValueError(f"a limit of {limit} needs gated experts and must not be negative")
        self.limit, self.alpha, self.scores = float(limit), float(alpha), scores
        self.scale_input = weights_scale == "input"
        if self.gated:
            if activation != "silu":
                raise ValueError(f"gated experts use the silu gate, not {activation!r}")
        elif activation not in ops.UNARY_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(ops.UNARY_ACTIVATIONS)}")
        self.gate_name, self.router_bias_name = gate_name, router_bias_name
        self.router_bias = None
        if not 1 <= top <= num_experts <= ops.ROUTE_MAX_EXPERTS:
            raise ValueError(f"a token uses 1 to {num_experts} of at most {ops.ROUTE_MAX_EXPERTS} experts, not {top}")
        self.hidden_size, self.num_experts, self.top = hidden_size, num_experts, top
        self.expert_size, self.shared_size = expert_size, shared_size
        self.route_scale = float(route_scale)
        self.prefix, self.activation, self.name = checkpoint_prefix, activation, name
        self.names = (router_name, expert_prefix, shared_prefix, up_name, down_name)
        self.inner = num_experts * expert_size + shared_size
        self.router = Linear(hidden_size, num_experts)
        self.up = Linear(hidden_size, (2 if self.gated else 1) * self.inner)
        self.down = Linear(self.inner, hidden_size)

    def _sources(self, which: str, rows_of_expert: int, rows_of_shared: int) -> tuple[Source, ...]:
        _, expert, shared, _, _ = self.names
        out = [Source(f"{self.prefix}{expert}{e}.{which}", rows_of_expert) for e in range(self.num_experts)]
        if self.shared_size:
            out.append(Source(f"{self.prefix}{shared}{which}", rows_of_shared))
        return tuple(out)

    def param_specs(self) -> list[ParamSpec]:
        h = self.hidden_size
        router, _, _, up, down = self.names
        first = self._sources(up, self.expert_size, self.shared_size)
        if self.gated:  # [every gate | every up]
            first = self._sources(self.gate_name, self.expert_size, self.shared_size) + first
        specs = [
            ParamSpec(self.name + ".router", (self.num_experts, h), "matrix_f32",
                      (Source(self.prefix + router, self.num_experts),)),
            ParamSpec(self.name + ".up", (self.up.out_features, h), "matrix", first),
            ParamSpec(self.name + ".down", (h, self.inner), "matrix",
                      self._sources(down, self.expert_size, self.shared_size), axis=1),
        ]
        if self.router_bias_name:
            specs.append(ParamSpec(self.name + ".router_bias", (self.num_experts,), "vector",
                                   (Source(self.prefix + self.router_bias_name, self.num_experts),)))
        return specs

    def bind(self, params, runtime) -> None:
        if self.router_bias_name:
            self.router_bias = params[self.name + ".router_bias"]
        self.router.bind(params[self.name + ".router"])
        self.up.bind(params[self.name + ".up"])
        self.down.bind(params[self.name + ".down"])

    def forward(self, x, ctx):
        # float32 throughout
        weights = ops.router(x, self.router.weight, self.top, self.route_scale, self.router_bias, self.scores)
        hidden = self.up(x)
        if self.gated:
            act = torch.empty((x.shape[0], self.inner), dtype=hidden.dtype, device=x.device)
            ops.swiglu(hidden, act, self.limit, self.alpha, route=weights, expert_ff=self.expert_size,
                       route_input=self.scale_input)
            return self.down.deferred(act, ctx)
        ops.unary_act(hidden, hidden, self.activation, weights, self.expert_size)
        return self.down.deferred(hidden, ctx)


FEED_FORWARDS.register("two_layer", TwoLayer)
FEED_FORWARDS.register("routed_experts", RoutedExperts)
FEED_FORWARDS.register("swiglu", SwiGLU)
FEED_FORWARDS.register("gated", SwiGLU)  # the same part under the name that fits either activation
