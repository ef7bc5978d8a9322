"""Token embedding (row gather into the float32 residual stream) and the output projection.

rapid_llm/modules/vocab_parallel.py:102-103 (``F.embedding``) and :125-126 (``F.linear(h, W)``);
a tied output projection is the embedding table under a second name
(rapid_llm/models/weights.py:197-214).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import EMBEDDINGS, OUTPUT_PROJECTIONS, Embedding, OutputProjection, ParamSpec, Source
from .linear import Linear


class TokenEmbedding(Embedding):
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int, checkpoint_name: str, name: str = "embed",
                 scale: float = 1.0, sinusoid_base: float | None = None,
                 position_table_name: str | None = None, positions: int = 0) -> None:
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        # a learned vector per position (``positions`` rows), added unscaled to the token's row
        self.position_table_name = position_table_name
        self.positions = int(positions)
        if position_table_name is not None and self.positions < 1:
            raise ValueError(f"a learned position table needs its number of positions, got {positions}")
        self.position_table: torch.Tensor | None = None
        self.scale = float(scale)  # every row is multiplied by it on its way into the stream
        # with a base b, the sinusoidal vector of the token's position p is added: channel 2i
        # gets sin(p * b^(-2i/hidden)), channel 2i + 1 the cosine of the same angle
        self.sinusoid_base = None if sinusoid_base is None else float(sinusoid_base)
        if self.sinusoid_base is not None and not self.sinusoid_base > 0:
            raise ValueError(f"the base of a sinusoidal position vector must be positive, got {sinusoid_base}")
        self.inv_freq: torch.Tensor | None = None
        self.checkpoint_name = checkpoint_name
        self.name = name
        self.table: torch.Tensor | None = None

    def param_specs(self):
        specs = [
            ParamSpec(
                self.name + ".weight",
                (self.vocab_size, self.hidden_size),
                "matrix",
                (Source(self.checkpoint_name, self.vocab_size),),
            )
        ]
        if self.position_table_name is not None:
            specs.append(ParamSpec(
                self.name + ".positions", (self.positions, self.hidden_size), "matrix",
                (Source(self.position_table_name, self.positions),),
            ))
        return specs

    def bind(self, params, runtime) -> None:
        self.table = params[self.name + ".weight"]
        self.max_seq_len = int(runtime.max_seq_len)
        if self.position_table_name is not None:
            self.position_table = params[self.name + ".positions"]
            if self.position_table.dtype != self.table.dtype:  # one stored wider than the other
                self.table = self.table.to(torch.float32)
                self.position_table = self.position_table.to(torch.float32)
        if self.sinusoid_base is not None:
            i = torch.arange((self.hidden_size + 1) // 2, dtype=torch.float64)
            inv = self.sinusoid_base ** (-2.0 * i / self.hidden_size)
            self.inv_freq = inv.to(torch.float32).to(runtime.device)

    def forward(self, token_ids: torch.Tensor, ctx) -> torch.Tensor:
        """Rows of the table for the ids; an id ``-(r + 1)`` takes ``ctx.fed_tokens[r]``."""
        out = torch.empty((token_ids.numel(), self.hidden_size), dtype=torch.float32, device=token_ids.device)
        learned = self.position_table is not None
        # (a recorded step names the end of its context bucket, which may lie beyond the longest
        # sequence the engine admits; no request's position does)
        if learned and min(ctx.max_position, self.max_seq_len - 1) >= self.positions:
            raise ops.KernelError(f"position {ctx.max_position} is beyond the {self.positions} learned positions")
        ops.embed(token_ids, self.table, out, getattr(ctx, "fed_tokens", None), self.scale,
                  ctx.positions if (self.inv_freq is not None or learned) else None, self.inv_freq,
                  self.position_table)
        return out


class LinearOutput(OutputProjection):
    """``logits = h W^T`` in float32, over the rows that were asked for only.  ``tied_to``
    names the parameter (the embedding's table) that stands in when the checkpoint ships no
    tensor of this part's own.  ``scale`` multiplies the logits; ``softcap`` c > 0 then turns them
    into ``c * tanh(logits / c)`` (both in float32, one kernel over the finished rows)."""

    replayable = True

    def __init__(
        self,
        vocab_size: int,
        hidden_size: int,
        checkpoint_name: str,
        tied_to: str | None,
        name: str = "output",
        scale: float = 1.0,
        softcap: float = 0.0,
    ) -> None:
        if softcap < 0:
            raise ValueError(f"the cap of the logits must not be negative, got {softcap}")
        self.scale, self.softcap = float(scale), float(softcap)
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.checkpoint_name = checkpoint_name
        self.tied_to = tied_to
        self.name = name
        self.proj = Linear(hidden_size, vocab_size)

    def param_specs(self):
        return [
            ParamSpec(
                self.name + ".weight",
                (self.vocab_size, self.hidden_size),
                "matrix",
                (Source(self.checkpoint_name, self.vocab_size),),
                fallback=self.tied_to,
            )
        ]

    def bind(self, params, runtime) -> None:
        self.proj.bind(params[self.name + ".weight"])

    def forward(self, h: torch.Tensor, ctx=None) -> torch.Tensor:
        logits = self.proj(h, out_dtype=torch.float32)
        if self.scale != 1.0 or self.softcap:
            ops.scale_cap(logits, self.scale, self.softcap)
        return logits


EMBEDDINGS.register("token_embedding", TokenEmbedding)
OUTPUT_PROJECTIONS.register("linear_output", LinearOutput)
