"""A plain, slow implementation of the Fomunex decoder in float64 torch on the CPU: the oracle of
the tests.  One function per mechanism, whole sequences only, no cache, no batching; it shares
no code with the package.

``cfg`` is the ``config.json`` dictionary, ``w`` maps checkpoint tensor names to tensors.  ``cast``
(optional) is applied wherever an engine that computes in a narrower type would round: the
normed rows, the projections' results, the activations; never to what the design keeps in 32-bit.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x`` divided by the root of (the mean of its squares over the last axis, plus eps)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    return rms(x, eps) * g


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# --------------------------------------------------------------------------- #
# mixers: h [T, width] -> [T, width]
# --------------------------------------------------------------------------- #


def same(x):
    return x


def attention(m: dict, w: dict, p: str, h: torch.Tensor, eps: float, cast=same) -> torch.Tensor:
    T = h.shape[0]
    H, G, d = m["heads"], m.get("kv_heads") or m["heads"], m["dim"]
    dv = m.get("vdim") or d
    q = cast(h @ w[p + "q"].T).view(T, H, d)
    k = cast(h @ w[p + "k"].T).view(T, G, d)
    v = cast(h @ w[p + "v"].T).view(T, G, dv)
    q, k = cast(rms(q, eps)), cast(rms(k, eps))
    cap = m.get("softcap")
    window = (m.get("mask") or {}).get("size") or 0
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    seen = (j <= i) if not window else ((j <= i) & (i - j < window))
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        kv = head // (H // G)
        s = (q[:, head] @ k[:, kv].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        slope = 2.0 ** (-8.0 * (head + 1) / H)
        s = s - slope * (i - j).to(F)
        s = s.masked_fill(~seen, -math.inf)
        sink = w[p + "sink"][head]
        top = torch.maximum(s.max(-1, keepdim=True).values, sink)
        e = torch.exp(s - top)
        den = e.sum(-1, keepdim=True) + torch.exp(sink - top)
        out[:, head] = (e / den) @ v[:, kv]
    return cast(out.reshape(T, H * dv)) @ w[p + "o"].T


def wkv(m: dict, w: dict, p: str, h: torch.Tensor, eps: float, cast=same) -> torch.Tensor:
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, h.shape[1], dtype=F), h[:-1]], 0)

    def mix(s):
        return h + (prev - h) * w[p + "mu." + s]

    r = cast(cast(mix("r")) @ w[p + "r"].T).view(T, H, d)
    k = cast(cast(mix("k")) @ w[p + "k"].T).view(T, H, d)
    v = cast(cast(mix("v")) @ w[p + "v"].T).view(T, H, d)
    gate = silu(cast(cast(mix("g")) @ w[p + "g"].T))
    decay = torch.exp(-torch.exp(torch.tanh(mix("w") @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).view(T, H, d)
    u = w[p + "u"]  # [H, d]
    S = torch.zeros(H, d, d, dtype=F)  # [head, key channel, value channel]
    out = torch.zeros(T, H, d, dtype=F)
    for t in range(T):
        kv = k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out[t] = torch.einsum("hkv,hk->hv", S + u.unsqueeze(-1) * kv, r[t])
        S = decay[t].unsqueeze(-1) * S + kv
    out = rms(out, eps).reshape(T, H * d) * w[p + "norm"] * gate
    return cast(out) @ w[p + "o"].T


def mamba2(m: dict, w: dict, p: str, h: torch.Tensor, eps: float, cast=same) -> torch.Tensor:
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    taps, parts = m["conv"], m["norm_groups"]
    inner = H * P
    zxbcdt = h @ w[p + "in"].T
    z = cast(zxbcdt[:, :inner])
    xbc = cast(zxbcdt[:, inner : 2 * inner + 2 * G * N])
    dt = zxbcdt[:, 2 * inner + 2 * G * N :]
    channels = xbc.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, channels, dtype=F), xbc], 0)
    conv = w[p + "conv"]  # [channels, taps], the last column meets the current token
    y = torch.zeros(T, channels, dtype=F)
    for tap in range(taps):
        y = y + padded[tap : tap + T] * conv[:, tap]
    xbc = silu(y + w[p + "conv.b"])
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner : inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N :].view(T, G, N)
    dt = softplus(dt + w[p + "dt_bias"])  # [T, H]
    A = -torch.exp(w[p + "A_log"])
    S = torch.zeros(H, N, P, dtype=F)
    out = torch.zeros(T, H, P, dtype=F)
    for t in range(T):
        for head in range(H):
            g = head // (H // G)
            S[head] = torch.exp(A[head] * dt[t, head]) * S[head] + dt[t, head] * torch.outer(B[t, g], x[t, head])
            out[t, head] = S[head].T @ C[t, g] + w[p + "D"][head] * x[t, head]
    y = out.reshape(T, inner) * silu(z)
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[p + "norm"]
    return cast(y) @ w[p + "o"].T


MIXERS = {"attention": attention, "wkv": wkv, "mamba2": mamba2}


# --------------------------------------------------------------------------- #
# feed-forwards
# --------------------------------------------------------------------------- #


def polynorm(z: torch.Tensor, coefficients: torch.Tensor, eps: float) -> torch.Tensor:
    a, b, c, e = coefficients
    return a * rms(z, eps) + b * rms(z**2, eps) + c * rms(z**3, eps) + e


def dense(f: dict, w: dict, p: str, h: torch.Tensor, eps: float, cast=same) -> torch.Tensor:
    z = cast(h @ w[p + "up"].T)
    return cast(polynorm(z, w[p + "act"], eps)) @ w[p + "down"].T


def expert(w: dict, p: str, h: torch.Tensor, limit: float, cast=same) -> torch.Tensor:
    g = torch.clamp(cast(h @ w[p + "gate"].T), max=limit)
    u = torch.clamp(cast(h @ w[p + "up"].T), -limit, limit)
    return cast(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def moe(f: dict, w: dict, p: str, h: torch.Tensor, eps: float, cast=same) -> torch.Tensor:
    experts, top = f["router"]["experts"], f["router"]["top"]
    limit = f["expert"]["limit"]
    scores = torch.sigmoid(h @ w[p + "router"].T)
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        chosen = torch.topk(scores[t], top).indices
        for e in chosen.tolist():
            out[t] += expert(w, f"{p}e{e}.", (scores[t, e] * h[t]).unsqueeze(0), limit, cast)[0]
    return out


FEED_FORWARDS = {"dense": dense, "moe": moe}


# --------------------------------------------------------------------------- #
# the model
# --------------------------------------------------------------------------- #


def forward(cfg: dict, w: dict, tokens: list[int], streams: list | None = None, cast=same) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence from its start.  ``streams``: a list that receives
    the residual stream after every layer."""
    w = {name: t.to(F) for name, t in w.items()}
    eps = cfg["norm"]["eps"]
    ids = torch.tensor(tokens, dtype=torch.long)
    x = w["embed"][ids] + w["pos"][: len(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of")
        p = f"l{i if src is None else src}."
        x = x + MIXERS[layer["type"]](layer["mixer"], w, p + "mix.", cast(scalar_norm(x, w[p + "norm1"], eps)), eps, cast)
        if layer.get("mlp") is not None:
            kind = layer["mlp"].get("kind", "dense")
            x = x + FEED_FORWARDS[kind](layer["mlp"], w, p + "mlp.", cast(scalar_norm(x, w[p + "norm2"], eps)), eps, cast)
        if streams is not None:
            streams.append(x.clone())
    x = cast(scalar_norm(x, w["final.norm"], eps))
    logits = (x @ w["head"].T) * cfg["logit_scale"]
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits


def greedy(cfg: dict, w: dict, prompt: list[int], steps: int) -> list[int]:
    ids, out = list(prompt), []
    for _ in range(steps):
        tok = int(forward(cfg, w, ids)[-1].argmax())
        out.append(tok)
        ids.append(tok)
    return out
