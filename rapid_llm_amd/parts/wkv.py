"""RWKV-style time mixing as a mixer with a fixed-size state per request.

With ``h'`` the previous token's input (zeros before a request's first token), each of the five
branches ``s`` in (r, k, v, g, w) reads its own mix ``h + (h' - h) * mu_s``.  ``r``, ``k``, ``v``
(``heads x head_dim`` each) and the gate ``silu(W_g mix_g)`` are projections of their mixes; the
decay of every head and key channel is ``w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0))``.  Per head,
with the state ``S [key channel, value channel]`` and the bonus ``u`` for the current token::

    o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t          S_t = diag(w_t) S_(t-1) + k_t v_t^T

Each head's ``o`` is divided by its root mean square; the concatenated heads are multiplied by a
weight and by the gate, and the output projection follows.

The four projections run in the compute type.  The mix of the decay branch, its two small
products (matrices held in float32 in every engine), the decay itself, the state and the head
norm are float32 (``csrc/recurrent.hip``).  The state and the previous token's input live in the
request's slot (``cache.states``), so portions, single tokens and batches of both continue where
the request's last step stopped.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Mixer, ParamSpec, Source, StateSpec
from .linear import Linear

BRANCHES = ("r", "k", "v", "g", "w")


class WKV(Mixer):
    replayable = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        head_dim: int,
        norm_eps: float,
        checkpoint_prefix: str,
        decay_rank: int = 0,  # 0: the size the checkpoint's tensors have
        position=None,  # the recurrence knows order by itself
        name: str = "mixer",
        mix_prefix: str = "mu.",
        r_name: str = "r",
        k_name: str = "k",
        v_name: str = "v",
        gate_name: str = "g",
        o_name: str = "o",
        decay_in_name: str = "w1",
        decay_out_name: str = "w2",
        decay_bias_name: str = "w0",
        bonus_name: str = "u",
        norm_name: str = "norm",
    ) -> None:
        if num_heads < 1 or not 1 <= head_dim <= ops.WKV_MAX_HEAD_DIM:
            raise ValueError(f"the recurrence's kernel takes heads of up to {ops.WKV_MAX_HEAD_DIM} channels, got {head_dim}")
        self.hidden_size, self.heads, self.d = hidden_size, num_heads, head_dim
        self.rank = int(decay_rank) if decay_rank else -1
        self.eps = float(norm_eps)
        self.prefix, self.name = checkpoint_prefix, name
        self.names = dict(mu=mix_prefix, r=r_name, k=k_name, v=v_name, g=gate_name, o=o_name, w1=decay_in_name,
                          w2=decay_out_name, w0=decay_bias_name, u=bonus_name, norm=norm_name)
        inner = num_heads * head_dim
        self.inner = inner
        self.proj = {s: Linear(hidden_size, inner) for s in ("r", "k", "v", "g")}
        self.o = Linear(inner, hidden_size)
        self.decay_in = self.decay_out = None  # sized when the tensors are bound

    def param_specs(self) -> list[ParamSpec]:
        p, n, h, inner = self.prefix, self.names, self.hidden_size, self.inner
        specs = [
            ParamSpec(self.name + ".mu", (5 * h,), "vector", tuple(Source(p + n["mu"] + s, h) for s in BRANCHES)),
        ]
        specs += [ParamSpec(f"{self.name}.{s}", (inner, h), "matrix", (Source(p + n[s], inner),)) for s in ("r", "k", "v", "g")]
        specs += [
            ParamSpec(self.name + ".decay_in", (self.rank, h), "matrix_f32", (Source(p + n["w1"], max(self.rank, 0)),)),
            ParamSpec(self.name + ".decay_out", (inner, self.rank), "matrix_f32", (Source(p + n["w2"], inner),)),
            ParamSpec(self.name + ".decay_bias", (inner,), "vector", (Source(p + n["w0"], inner),)),
            ParamSpec(self.name + ".bonus", (self.heads, self.d), "vector", (Source(p + n["u"], self.heads),)),
            ParamSpec(self.name + ".norm", (inner,), "vector", (Source(p + n["norm"], inner),), init="norm"),
            ParamSpec(self.name + ".o", (h, inner), "matrix", (Source(p + n["o"], h),)),
        ]
        return specs

    def bind(self, params, runtime) -> None:
        for s, linear in self.proj.items():
            linear.bind(params[f"{self.name}.{s}"])
        w1, w2 = params[self.name + ".decay_in"], params[self.name + ".decay_out"]
        if w1.shape[0] != w2.shape[1]:
            raise ValueError(f"the decay's two matrices do not meet: {tuple(w1.shape)} and {tuple(w2.shape)}")
        self.decay_in = Linear(self.hidden_size, w1.shape[0])
        self.decay_in.bind(w1)
        self.decay_out = Linear(w1.shape[0], self.inner)
        self.decay_out.bind(w2)
        self.mu = params[self.name + ".mu"]
        self.decay_bias = params[self.name + ".decay_bias"]
        self.bonus = params[self.name + ".bonus"]
        self.norm_weight = params[self.name + ".norm"]
        self.o.bind(params[self.name + ".o"])

    def cache_need(self) -> CacheNeed:
        return CacheNeed(
            "state",
            states=(
                StateSpec("shift", (self.hidden_size,), "float32"),
                StateSpec("S", (self.heads, self.d, self.d), "float32"),  # [value channel, key channel]
            ),
        )

    def forward(self, x, ctx, cache):
        tokens = x.shape[0]
        # the four mixes that feed projections, in the compute type, and the decay's in float32
        mixes = torch.empty((4, tokens, self.hidden_size), dtype=x.dtype, device=x.device)
        mix_w = torch.empty((tokens, self.hidden_size), dtype=torch.float32, device=x.device)
        ops.token_shift(x, self.mu, cache.states["shift"], mixes, mix_w, ctx)
        r, k, v, g = (self.proj[s](mixes[i]) for i, s in enumerate(("r", "k", "v", "g")))
        low = self.decay_in(mix_w)
        ops.unary_act(low, low, "tanh")
        decay = self.decay_out(low)  # float32: before the bias and the two exponentials
        out = torch.empty((tokens, self.inner), dtype=x.dtype, device=x.device)
        ops.wkv(r, k, v, g, decay, self.decay_bias, self.bonus, self.norm_weight, out, ctx, cache.states["S"],
                self.heads, self.d, self.eps)
        return self.o.deferred(out, ctx)


MIXERS.register("wkv", WKV)
