"""A plain, slow Miborax decoder: whole sequences, dense masks, no cache, one function per mechanism.

Written from the design's equations alone and sharing no code with the package.  ``cfg`` is the
body of a ``config.json`` of the design (a dict), ``w`` maps checkpoint tensor names to tensors.
Everything runs in the type of ``x`` (float64 for the sharpest comparison); ``cast`` is a hook
that rounds what a bfloat16 engine stores between its kernels (identity by default).

The design in this file's notation.  A layer is ``x += mix(LN1(x)) + ff(LN2(x))`` with two layer
norms (weight and bias) of the same ``x``.  ``mix`` is attention through a latent: per token one
row ``c`` (RMS-normed) and one rotated key part ``kr`` shared by all heads; head ``h`` scores a
key with ``(qn_h . (Uk_h c) + qr_h . kr) * scale``, takes values ``Uv_h c``, and its softmax has
``exp(sink_h)`` more in the denominator.  Queries come straight from a projection or through an
RMS-normed latent of their own; a mask limits a query to the last ``size`` positions; heads may
be gated by a sigmoid of a projection of the mixer's input; a layer may read another layer's
``c`` and ``kr``.  ``ff`` is a mixture of gated experts chosen by the largest router logits.
"""

from __future__ import annotations

import math

import torch


def identity(t: torch.Tensor) -> torch.Tensor:
    return t


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def layer_norm(x, weight, bias, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight + bias


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def rotate_pairs(x, positions, base, dims):
    """Rotate channel ``2i`` with ``2i + 1`` of the first ``dims`` channels of the last axis by the
    angle ``p * base^(-2i / dims)``; ``x [T, ..., d]``, ``positions [T]``."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = base ** (-2.0 * i / dims)
    # the angle as a float32 product, as an engine computes it
    angle = (positions.to(torch.float32)[:, None] * freq.to(torch.float32)[None, :]).to(torch.float64)
    cos, sin = torch.cos(angle).to(x.dtype), torch.sin(angle).to(x.dtype)
    while cos.dim() < x.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def visible(positions, size):
    """``[T, T]`` bool: query ``i`` sees key ``j`` when ``j <= i`` and, with a mask of ``size``,
    ``i - j < size``."""
    i = positions[:, None]
    j = positions[None, :]
    seen = j <= i
    if size:
        seen &= (i - j) < size
    return seen


def sink_softmax(scores, seen, sink):
    """Softmax weights over the seen keys whose denominator also holds ``exp(sink)``:
    ``scores [H, T, T]``, ``seen [T, T]``, ``sink [H]``."""
    s = scores.masked_fill(~seen[None], float("-inf"))
    top = torch.maximum(s.max(-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(s - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink[:, None, None] - top))


def latent_of(h, m, w, p, eps, positions, cast):
    """The cached pair of a layer with a projection of its own: the normed latent ``c [T, r]`` and
    the rotated shared key part ``kr [T, rot_dim]``."""
    r, rd = m["kv_rank"], m["rot_dim"]
    row = cast(h @ w[p + "dkv"].T)
    c = cast(rms_norm(row[:, :r], w[p + "dkv.norm"], eps))
    kr = cast(rotate_pairs(row[:, r : r + rd], positions, m["rot"]["base"], m["rot"]["dims"]))
    return c, kr


def latent_attention(h, m, w, p, eps, positions, latent, cast=identity):
    """One mixer.  ``latent`` is the ``(c, kr)`` pair it reads (its own or another layer's)."""
    T = h.shape[0]
    H, d, rd, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    if "q_rank" in m:
        cq = cast(rms_norm(cast(h @ w[p + "dq"].T), w[p + "dq.norm"], eps))
        q = cast(cq @ w[p + "uq"].T)
    else:
        q = cast(h @ w[p + "q"].T)
    q = q.view(T, H, d + rd)
    qn = q[..., :d]
    qr = cast(rotate_pairs(q[..., d:], positions, m["rot"]["base"], m["rot"]["dims"]))
    c, kr = latent
    kn = cast(c @ w[p + "uk"].T).view(T, H, d)
    v = cast(c @ w[p + "uv"].T).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", qn, kn) + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    size = (m.get("mask") or {}).get("size", 0)
    weights = sink_softmax(scores, visible(positions, size), w[p + "sink"].to(h.dtype))
    out = cast(torch.einsum("hij,jhd->ihd", weights, v))
    if (p + "g") in w:
        gate = torch.sigmoid(cast(h @ w[p + "g"].T))
        out = cast(out * gate[:, :, None])
    return cast(out.reshape(T, H * dv) @ w[p + "o"].T)


def route(h, ff, w, p):
    """Per token the chosen experts and their weights: the ``top`` largest router logits, softmax
    over those alone."""
    logits = h @ w[p + "router"].T + w[p + "router.b"]
    chosen = torch.topk(logits, ff["router"]["top"], dim=-1)
    return chosen.indices, torch.softmax(chosen.values, dim=-1)


def experts(h, ff, w, p, cast=identity):
    """The mixture, token by token and expert by expert."""
    index, weight = route(h, ff, w, p)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(index[t].tolist(), weight[t]):
            q = f"{p}e{e}."
            g = h[t] @ w[q + "gate"].T
            u = h[t] @ w[q + "up"].T
            hidden = cast(g * torch.sigmoid(g) * u)
            out[t] += a * (hidden @ w[q + "down"].T)
    return cast(out)


def forward(cfg, w, tokens, dtype=torch.float64, cast=identity, positions=None, streams=None):
    """Logits ``[T, vocab]`` of one sequence.  ``streams``: a list that receives the residual
    stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.numel()
    if positions is None:
        positions = torch.arange(T)
    eps = cfg["norm"]["eps"]
    x = w["embed"][tokens] * cfg["embedding"]["scale"]
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        h1 = cast(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps))
        if "kv_from" in m:
            latent = latents[m["kv_from"]]
        else:
            latent = latents[i] = latent_of(h1, m, w, p + "mix.", eps, positions, cast)
        delta = latent_attention(h1, m, w, p + "mix.", eps, positions, latent, cast)
        if layer.get("mlp") is not None:
            h2 = cast(layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps))
            delta = delta + experts(h2, layer["mlp"], w, p + "mlp.", cast)
        x = x + delta
        if streams is not None:
            streams.append(x.clone())
    h = cast(layer_norm(x, w["final.norm"], w["final.norm.b"], eps))
    return h @ w["embed"].T


def absorbed_attention(h, m, w, p, eps, positions, latent):
    """The same mixer written over the latent rows themselves: the query takes the key
    projection in (``Uk_h^T qn_h``), the weights average the rows ``c``, and the value projection
    comes last.  Equal to :func:`latent_attention` up to rounding."""
    T = h.shape[0]
    H, d, rd, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    if "q_rank" in m:
        q = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps) @ w[p + "uq"].T
    else:
        q = h @ w[p + "q"].T
    q = q.view(T, H, d + rd)
    qr = rotate_pairs(q[..., d:], positions, m["rot"]["base"], m["rot"]["dims"])
    c, kr = latent
    qa = torch.einsum("ihd,hdr->ihr", q[..., :d], w[p + "uk"].view(H, d, r))
    scores = (torch.einsum("ihr,jr->hij", qa, c) + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    size = (m.get("mask") or {}).get("size", 0)
    weights = sink_softmax(scores, visible(positions, size), w[p + "sink"].to(h.dtype))
    mean_c = torch.einsum("hij,jr->ihr", weights, c)
    out = torch.einsum("ihr,hvr->ihv", mean_c, w[p + "uv"].view(H, dv, r))
    if (p + "g") in w:
        out = out * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]
    return out.reshape(T, H * dv) @ w[p + "o"].T
