"""Values that a neighbouring part may still fold its own work into.

A decode step is a chain of small kernels, and the residual norm between two products is
the smallest: it only has to know every row's sum of squares.  Two lazy values let the
products on either side absorb it, without any part knowing its neighbours:

* :class:`DeferredProduct`: what a mixer or a feed-forward returns in place of its last
  product ``x W^T`` when that product's own kernels could absorb a norm (``Linear.deferred``
  decides: bfloat16 and few rows).  Whoever receives it may run the product with an epilogue
  of its own, or simply ``materialize()`` it.
* :class:`ScaledRows`: what a norm returns in place of normalised rows when its consumer
  says it accepts them: the rows times the norm's weight, and the pieces of every row's sum
  of squares; the factor ``rsqrt(mean + eps)`` is a scalar per row and commutes with the
  consumer's own product, which applies it to its result.

* :class:`NormedDelta`: what a block whose sub-layers pass a norm of their own on their way into
  the stream returns in place of that norm's result: the sub-layer's output as it is, with the
  norm's weight and epsilon.  A norm that declares ``fuses_products`` applies it, adds the result
  to the stream and computes its own rows in one kernel; anything else gets the normed rows in
  the stream's type from ``materialize()``.

* :class:`SummedDeltas`: what a block whose two sub-layers read the same stream returns: both
  outputs, not yet added to each other.  A norm that declares ``fuses_products`` and knows the
  type adds both into the stream in the kernel that computes its own rows; anything else gets
  their sum joined to the stream first (``add_to``) or as a tensor (``materialize``).

Blocks and models route these only between parts that declare them (``fuses_products`` on
a norm, ``accepts_scaled_rows`` on a mixer or feed-forward, ``accepts_deferred`` on a
block); everything else sees plain tensors.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch


class DeferredProduct:
    def __init__(self, linear: Any, x: torch.Tensor) -> None:
        self.linear = linear
        self.x = x

    @property
    def shape(self) -> tuple[int, int]:
        return (self.x.shape[0], self.linear.out_features)

    def materialize(self, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        return self.linear(self.x, out_dtype)


class NormedDelta:
    """``rmsnorm(y) * weight``, not yet computed."""

    def __init__(self, y: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
        self.y = y
        self.weight = weight
        self.eps = float(eps)

    @property
    def shape(self):
        return self.y.shape

    def add_to(self, residual: torch.Tensor) -> None:
        """``residual += rmsnorm(y) * weight`` in place (float32)."""
        from ..kernels import ops

        ops.normed_add_rmsnorm(residual, self.y, self.weight, self.eps, None, None, 0.0)

    def materialize(self, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        """The normed rows as a float32 tensor (what is added to the stream)."""
        out = torch.zeros(self.y.shape, dtype=torch.float32, device=self.y.device)
        self.add_to(out)
        return out


class SummedDeltas:
    """``first + second``, the outputs of two sub-layers that read the same stream, not yet added."""

    def __init__(self, first, second) -> None:
        self.first = first
        self.second = second

    @property
    def shape(self):
        return self.first.shape

    def tensors(self) -> tuple[torch.Tensor, torch.Tensor]:
        return plain(self.first), plain(self.second)

    def add_to(self, residual: torch.Tensor) -> None:
        """``residual += first + second`` in place (float32)."""
        from ..kernels import ops

        a, b = self.tensors()
        ops.add_layernorm(residual, a, b, None, None, None)

    def materialize(self, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        """The sum as a float32 tensor."""
        a, _ = self.tensors()
        out = torch.zeros(a.shape, dtype=torch.float32, device=a.device)
        self.add_to(out)
        return out


@dataclass
class ScaledRows:
    rows: torch.Tensor  # [M, size], the residual rows times the norm's weight
    partial: torch.Tensor  # [parts, 16] float32: pieces of every row's sum of squares
    size: int
    eps: float

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype

    @property
    def device(self):
        return self.rows.device


def plain(value):
    """A tensor, whatever lazy value it still was."""
    return value.materialize() if isinstance(value, (DeferredProduct, NormedDelta, SummedDeltas)) else value


def settle(residual, delta):
    """What is left to add once lazy values are settled: a pending normed delta joins the stream
    now, a deferred product becomes a tensor."""
    if isinstance(delta, (NormedDelta, SummedDeltas)):
        delta.add_to(residual)
        return None
    return plain(delta)


def run_norm(norm, residual, delta, ctx, consumer=None, rows=None):
    """``norm.forward`` with the lazy values routed as the two sides declare them."""
    if getattr(norm, "fuses_products", False):
        return norm.forward(
            residual, delta, ctx, rows, scaled_ok=bool(getattr(consumer, "accepts_scaled_rows", False))
        )
    if isinstance(delta, (NormedDelta, SummedDeltas)):
        # a norm that knows nothing of it: the stream takes it first
        delta.add_to(residual)
        delta = None
    return norm.forward(residual, plain(delta), ctx, rows)
