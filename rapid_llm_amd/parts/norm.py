"""RMSNorm fused with the residual add in front of it.

``residual += delta`` in float32, then ``residual * rsqrt(mean(residual^2) + eps) * w``
(rapid_llm/kernels/ops/layernorm/skip_rmsnorm.py:41-47,:51-85).  The residual stream is
kept in float32 in every engine type; the reference rounds it to the activation type after
each add (:104-144), which this engine does not need to.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import NORMS, Norm, ParamSpec, Source
from .lazy import DeferredProduct, NormedDelta, SummedDeltas, plain


class RMSNorm(Norm):
    replayable = True
    fuses_products = True  # takes a DeferredProduct as delta, may return ScaledRows

    def __init__(self, size: int, eps: float, checkpoint_name: str, name: str = "norm",
                 single_weight: bool = False) -> None:
        self.size = size
        self.eps = float(eps)
        self.checkpoint_name = checkpoint_name
        self.name = name
        # one learned number for all coordinates instead of one a coordinate: the kernels get it
        # laid out as a vector, so every fused form of the norm serves both
        self.single_weight = bool(single_weight)
        self.weight: torch.Tensor | None = None

    def param_specs(self) -> list[ParamSpec]:
        if self.single_weight:
            return [ParamSpec(self.name + ".weight", (), "vector", (Source(self.checkpoint_name, 1),), init="norm")]
        return [
            ParamSpec(
                self.name + ".weight",
                (self.size,),
                "vector",
                (Source(self.checkpoint_name, self.size),),
                init="norm",
            )
        ]

    def bind(self, params, runtime) -> None:
        self.weight = params[self.name + ".weight"]
        if self.single_weight:
            self.weight = self.weight.reshape(1).expand(self.size).contiguous()
        self.dtype = runtime.dtype

    def forward(self, residual, delta, ctx, rows=None, scaled_ok=False):
        if isinstance(delta, NormedDelta):
            # the sub-layer's own norm, the add and this norm in one kernel
            n = residual.shape[0] if rows is None else rows.numel()
            out = torch.empty((n, self.size), dtype=self.dtype, device=residual.device)
            y = delta.y
            if y.dtype != self.dtype:
                y = y.to(self.dtype)
            ops.normed_add_rmsnorm(residual, y, delta.weight, delta.eps, self.weight, out, self.eps, rows)
            return out
        if isinstance(delta, SummedDeltas):
            delta.add_to(residual)
            delta = None
        if isinstance(delta, DeferredProduct):
            if (
                scaled_ok and rows is None and delta.linear.out_features == self.size
                and self.dtype == torch.bfloat16 and delta.linear.bias is None and delta.linear.skinny(delta.x)
            ):
                # the producer's kernel adds into the residual and leaves what the consumer's
                # kernel needs to finish the norm: no kernel of this norm's own runs
                return delta.linear.add_to_residual(delta.x, residual, self.weight, self.eps)
            if (
                rows is None and delta.linear.out_features == self.size and self.dtype == torch.bfloat16
                and self.size % 4 == 0 and self.size <= 16 * 1024 and delta.linear.bias is None
                and delta.linear.midsize(delta.x)
            ):
                # the product arrives as float32 runs of K, which this norm's kernel adds
                out = torch.empty((residual.shape[0], self.size), dtype=self.dtype, device=residual.device)
                ops.add_rmsnorm_parts(residual, delta.linear.partial_sums(delta.x), self.weight, out, self.eps)
                return out
            delta = delta.materialize()
        n = residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.size), dtype=self.dtype, device=residual.device)
        ops.add_rmsnorm(residual, delta, self.weight, out, self.eps, rows)
        return out


class LayerNorm(Norm):
    """Layer norm with weight and bias, fused with the residual add in front of it:
    ``(x - mean) / sqrt(var + eps) * w + b``, ``var`` the mean of the squared deviations, all in
    float32.  A pending pair of sub-layer outputs (:class:`SummedDeltas`) is added in the same
    kernel, and with ``second`` (another layer norm of the same rows, as a block has whose two
    sub-layers read the same stream) both outputs come from one pass: the statistics are shared."""

    replayable = True
    fuses_products = True  # receives lazy deltas as they are (it settles what it cannot fold)

    def __init__(self, size: int, eps: float, checkpoint_name: str, bias_checkpoint_name: str | None = None,
                 name: str = "norm") -> None:
        self.size = size
        self.eps = float(eps)
        self.checkpoint_name = checkpoint_name
        self.bias_checkpoint_name = bias_checkpoint_name or checkpoint_name + ".bias"
        self.name = name
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None

    def param_specs(self) -> list[ParamSpec]:
        return [
            ParamSpec(self.name + ".weight", (self.size,), "vector", (Source(self.checkpoint_name, self.size),),
                      init="norm"),
            ParamSpec(self.name + ".bias", (self.size,), "vector", (Source(self.bias_checkpoint_name, self.size),)),
        ]

    def bind(self, params, runtime) -> None:
        self.weight = params[self.name + ".weight"]
        self.bias = params[self.name + ".bias"]
        self.dtype = runtime.dtype

    def pairs_with(self, other) -> bool:
        """Whether ``other`` can be computed from this norm's statistics."""
        return isinstance(other, LayerNorm) and other.size == self.size and other.eps == self.eps

    def forward(self, residual, delta, ctx, rows=None, scaled_ok=False, second: "LayerNorm | None" = None):
        d1 = d2 = None
        if isinstance(delta, SummedDeltas):
            d1, d2 = delta.tensors()
        elif isinstance(delta, NormedDelta):
            delta.add_to(residual)
        else:
            d1 = plain(delta)

        def typed(d):
            return d if d is None or d.dtype == self.dtype else d.to(self.dtype)

        n = residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.size), dtype=self.dtype, device=residual.device)
        if second is None:
            ops.add_layernorm(residual, typed(d1), typed(d2), self.weight, self.bias, out, eps=self.eps, rows=rows)
            return out
        if not self.pairs_with(second):
            raise ValueError("two layer norms share a kernel only with the same width and epsilon")
        out2 = torch.empty_like(out)
        ops.add_layernorm(residual, typed(d1), typed(d2), self.weight, self.bias, out, second.weight, second.bias,
                          out2, eps=self.eps, rows=rows)
        return out, out2


NORMS.register("rmsnorm", RMSNorm)
NORMS.register("layernorm", LayerNorm)
