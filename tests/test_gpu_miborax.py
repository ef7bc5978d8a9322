"""The Miborax decoder in the engine against the plain implementation of ``plain_miborax.py``:
every mechanism alone, every way of cutting requests into steps, pages and slots that are used
again, the edges of windows, rows that another layer cached, long decoding, and greedy
generation through the entry point."""

import math
import random
from types import SimpleNamespace

import pytest
import torch

import parity
import plain_miborax as pm
import replay_util as ru
from miborax_configs import (
    BF16_ROWS_BEYOND,
    BF16_TIMES_ROUNDING,
    MIBO,
    load_plain,
    make_model_dir,
    random_tokens,
    rounding_figure,
    row_errors,
)

pytestmark = pytest.mark.gpu

DEV = "cuda"
# float32 rows against the plain implementation in float64: root mean square over a row,
# relative to the logits' spread
F32_ROW = 2e-4


def _ops():
    from rapid_llm_amd.kernels import ops

    return ops


def bf16_round(t):
    return t.bfloat16().to(t.dtype)


def _tol(dtype, f32=1e-5, bf16=1e-2):
    return dict(rtol=f32, atol=f32) if dtype == torch.float32 else dict(rtol=bf16, atol=bf16)


# --------------------------------------------------------------------------- #
# attention over one shared row a token, with a learned term in the denominator
# --------------------------------------------------------------------------- #


def _plain_rows(q, k, v, scale, window, sink, first_row):
    """Attention of the last ``q.shape[0]`` positions of one request over its shared rows:
    ``q [n, heads, d]``, ``k [t, d]``, ``v [t, dv]``, ``sink [heads]``."""
    t, n = k.shape[0], q.shape[0]
    seen = pm.visible(torch.arange(t), window)[first_row:]
    scores = torch.einsum("ihd,jd->hij", q.double(), k.double()) * scale
    weights = pm.sink_softmax(scores, seen, sink.double())
    return torch.einsum("hij,jv->ihv", weights, v.double()).reshape(n, -1).float()


def _paged(seqs, heads, d, dv, page, dtype, seed, window, scale, sink, spike=None):
    """``seqs`` = (tokens already cached, tokens in this step) per request.  Pages in shuffled
    order, everything unwritten NaN, and the pages before the window of the step's first token
    mapped to the null page, as after trimming."""
    rng = random.Random(seed)
    gen = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-(a + n) // page) for a, n in seqs) + 1
    order = list(range(1, total_pages))
    rng.shuffle(order)
    max_pages = max(-(-(a + n) // page) for a, n in seqs) + 2
    table = torch.zeros((len(seqs) + 3, max_pages), dtype=torch.int32)
    k_cache = torch.full((total_pages, 1, page, d), float("nan"))
    v_cache = torch.full((total_pages, 1, dv, page), float("nan"))
    slots = list(range(len(seqs) + 3))
    rng.shuffle(slots)
    q_rows, positions, token_slot, expect = [], [], [], []
    for i, (a, n) in enumerate(seqs):
        t = a + n
        k = torch.randn((t, d), generator=gen)
        v = torch.randn((t, dv), generator=gen)
        q = torch.randn((n, heads, d), generator=gen)
        if spike is not None and i == spike[0]:
            # one key carries nearly all of the softmax mass of every head of the request's last query
            far = spike[1]
            u = q[-1, 0].clone()
            q[-1, :] = u
            k[far] = u * (30.0 / scale / float(u @ u))
            v[far] = 7.0
        if dtype == torch.bfloat16:
            q, k, v = (x.bfloat16().float() for x in (q, k, v))
        slot = slots[i]
        first_needed = max(0, a - window + 1) // page if window else 0
        for p in range(-(-t // page)):
            pid = order.pop()
            if p < first_needed:
                continue  # given back: the table keeps the null page, whose content is NaN
            table[slot, p] = pid
            lo, hi = p * page, min(t, (p + 1) * page)
            k_cache[pid, 0, : hi - lo, :] = k[lo:hi]
            v_cache[pid, 0, :, : hi - lo] = v[lo:hi].T
        expect.append(_plain_rows(q, k, v, scale, window, sink, a))
        q_rows.append(q.reshape(n, heads * d))
        positions += list(range(a, t))
        token_slot += [slot] * n
    ctx = SimpleNamespace(
        positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
        token_slot=torch.tensor(token_slot, dtype=torch.int32, device=DEV),
        token_ids=torch.zeros(len(positions), dtype=torch.int32, device=DEV),
        h_seq_starts=[a for a, _ in seqs], h_seq_lens=[n for _, n in seqs],
        max_position=max(positions), extra={},
    )
    return (torch.cat(q_rows).to(DEV, dtype), k_cache.to(DEV, dtype), v_cache.to(DEV, dtype), table.to(DEV), ctx,
            torch.cat(expect))


ATTENTION_CASES = [
    # heads, key row, value row, page, window, seqs (cached, new)
    (4, 64, 32, 8, 19, [(0, 60), (45, 1), (200, 1), (30, 31), (0, 1)]),
    (3, 96, 80, 8, 0, [(300, 1), (5, 70), (0, 2)]),                    # every earlier key
    (5, 32, 16, 8, 7, [(0, 7), (6, 1), (7, 1), (8, 1), (14, 9), (0, 1)]),
    (1, 32, 16, 4, 0, [(0, 33), (33, 1), (34, 1)]),                    # one head
    (2, 48, 32, 4, 1, [(0, 9), (5, 1)]),                               # a window of the own key alone
    (1, 48, 32, 4, 5, [(0, 12), (4, 1), (5, 1), (3, 1)]),
    (8, 128, 96, 16, 0, [(990, 40), (0, 130), (3000, 1)]),             # long contexts
    (4, 128, 96, 16, 64, [(0, 140), (63, 1), (64, 1), (65, 1), (1000, 1)]),
    (2, 160, 144, 16, 130, [(0, 200), (129, 1), (130, 1), (131, 1)]),
    (3, 320, 256, 16, 50, [(0, 70), (49, 1), (50, 1), (400, 1)]),      # rows wider than a lane's registers were sized for
    (2, 576, 512, 16, 0, [(0, 40), (100, 1), (300, 2)]),               # the widest rows the kernel is built for
    (5, 24, 18, 8, 33, [(0, 50), (32, 1), (33, 1), (100, 1)]),         # sizes off the grid of 16
    (3, 36, 26, 8, 0, [(0, 40), (9, 1), (10, 1), (130, 2)]),
    (2, 24, 18, 8, 9, [(0, 30), (8, 1), (9, 1), (10, 1)]),
    (2, 64, 32, 4, 0, [(8300, 1), (8250, 60)]),  # more pages than a workgroup stages: the table is read
    (32, 64, 32, 16, 0, [(3000, 1), (1500, 1), (40, 1)]),  # more heads than a block of rows holds: single tokens far in,
    (32, 64, 32, 16, 0, [(40, 1), (7, 1)]),                # near the start,
    (20, 32, 16, 8, 19, [(45, 1), (0, 30), (200, 3)]),     # and a last block that is not full, beside portions
]


@pytest.mark.parametrize("case", ATTENTION_CASES, ids=lambda c: f"h{c[0]}d{c[1]}v{c[2]}p{c[3]}w{c[4]}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_attention_over_shared_rows_with_a_learned_term(case, dtype):
    ops = _ops()
    heads, d, dv, page, window, seqs = case
    scale = 0.8 / math.sqrt(d)
    sink = torch.linspace(-2.0, 3.0, heads) if heads > 1 else torch.tensor([1.5])
    q, kc, vc, table, ctx, want = _paged(seqs, heads, d, dv, page, dtype, d + dv + page, window, scale, sink)
    out = torch.full((q.shape[0], heads * dv), float("nan"), dtype=dtype, device=DEV)
    ops.paged_attention(q, kc, vc, out, ctx, table, page, heads, 1, d, window, scale, value_dim=dv,
                        sink_values=sink.to(DEV))
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-5, atol=3e-6)
    else:
        assert float((got - want).abs().max()) <= 0.03 * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("d,dv,page", [(64, 32, 8), (96, 80, 16), (24, 18, 8)])
def test_one_key_holds_the_mass_at_every_edge(dtype, d, dv, page):
    """One key among hundreds carries the last query's weight.  Inside the window the output is
    that key's value; one position further out the key is not seen and the output is far from
    it.  At a page's last and first place, far away without a window, for a single decoded token
    and for the last token of a portion."""
    ops = _ops()
    heads, scale = 4, 0.125
    length = 400
    sink = torch.tensor([-1.0, 0.0, 2.0, 4.0])
    for window in (50, 0):
        if window:
            edges = [(0, False), (200, False), (length - window - 1, False), (length - window, True),
                     (length - 1, True), (length - 2 * page, 2 * page <= window),
                     (length - 2 * page - 1, 2 * page + 1 <= window)]
        else:
            edges = [(0, True), (200, True), (length - 1, True), (length - 2 * page, True), (length - 2 * page - 1, True)]
        for far, visible in edges:
            for seqs, who in (([(length - 1, 1), (10, 1)], 0), ([(5, 1), (length - 120, 120)], 1)):
                q, kc, vc, table, ctx, want = _paged(seqs, heads, d, dv, page, dtype, far, window, scale, sink,
                                                     spike=(who, far))
                out = torch.empty((q.shape[0], heads * dv), dtype=dtype, device=DEV)
                ops.paged_attention(q, kc, vc, out, ctx, table, page, heads, 1, d, window, scale, value_dim=dv,
                                    sink_values=sink.to(DEV))
                got = out.float().cpu()
                row = 0 if who == 0 else got.shape[0] - 1
                assert bool((want[row] > 6.5).all()) == visible  # the construction works in the plain attention
                torch.testing.assert_close(got[row], want[row], rtol=2e-2, atol=3e-2)
                torch.testing.assert_close(got, want, rtol=2e-2, atol=3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("d,dv", [(32, 16), (24, 18)])
def test_the_learned_term_shows_when_scores_are_small(dtype, d, dv):
    """Keys with score 0: n seen keys have weight 1 / (n + exp(s_h)) each, head by head.  A kernel
    that leaves the term out returns the plain mean, one that scales it or adds 1 another share."""
    ops = _ops()
    heads, page = 3, 8
    sink = torch.tensor([-1.0, 0.0, 1.5])
    seqs = [(0, 1), (0, 3), (6, 1)]
    q, kc, vc, table, ctx, want = _paged(seqs, heads, d, dv, page, dtype, 7, 0, 0.0, sink)
    out = torch.empty((q.shape[0], heads * dv), dtype=dtype, device=DEV)
    ops.paged_attention(q, kc, vc, out, ctx, table, page, heads, 1, d, 0, 0.0, value_dim=dv, sink_values=sink.to(DEV))
    got = out.float().cpu()
    torch.testing.assert_close(got, want, rtol=1e-2, atol=1e-2)
    # the first token of a request sees itself alone: its value times 1 / (1 + exp(s_h))
    v0 = vc[int(table[ctx.token_slot[0], 0]), 0, :, 0].float().cpu()
    for h in range(heads):
        torch.testing.assert_close(got[0, h * dv:(h + 1) * dv], v0 / (1.0 + math.exp(float(sink[h]))), rtol=1e-2, atol=1e-2)


# --------------------------------------------------------------------------- #
# the row-wise mechanisms alone
# --------------------------------------------------------------------------- #


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("hidden", [96, 100, 64, 4100, 97, 18, 2050, 20000])
def test_layer_norms_with_the_residual_add_in_front(dtype, hidden):
    ops = _ops()
    tokens = 9
    residual = torch.randn(tokens, hidden) * 2.0 + 0.7  # a mean far from zero: the variance is about it
    d1, d2 = (torch.randn(tokens, hidden) * 3.0).to(dtype), torch.randn(tokens, hidden).to(dtype)
    w1, b1 = 1.0 + 0.2 * torch.randn(hidden), 0.5 * torch.randn(hidden)
    w2, b2 = 1.0 + 0.2 * torch.randn(hidden), 0.5 * torch.randn(hidden)
    eps = 3e-6
    new = residual.double() + d1.double() + d2.double()
    want1 = pm.layer_norm(new, w1.double(), b1.double(), eps).float()
    want2 = pm.layer_norm(new, w2.double(), b2.double(), eps).float()
    tol = _tol(dtype)
    # both sub-layers' outputs added, both norms from one pass
    res = residual.clone().to(DEV)
    out1 = torch.empty((tokens, hidden), dtype=dtype, device=DEV)
    out2 = torch.empty_like(out1)
    ops.add_layernorm(res, d1.to(DEV), d2.to(DEV), w1.to(DEV), b1.to(DEV), out1, w2.to(DEV), b2.to(DEV), out2, eps=eps)
    torch.testing.assert_close(res.cpu(), new.float(), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(out1.float().cpu(), want1, **tol)
    torch.testing.assert_close(out2.float().cpu(), want2, **tol)
    # one delta, one norm; no delta
    for deltas in ((d1, None), (None, d2), (None, None)):
        res = residual.clone().to(DEV)
        out = torch.empty((tokens, hidden), dtype=dtype, device=DEV)
        ops.add_layernorm(res, *(None if d is None else d.to(DEV) for d in deltas), w1.to(DEV), b1.to(DEV), out, eps=eps)
        now = residual.double() + sum(d.double() for d in deltas if d is not None)
        torch.testing.assert_close(res.cpu(), now.float(), rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(out.float().cpu(), pm.layer_norm(now, w1.double(), b1.double(), eps).float(), **tol)
    # chosen rows only (the last norm of a step): every row takes the add, the chosen ones are normed
    rows = torch.tensor([7, 2], dtype=torch.int32, device=DEV)
    res = residual.clone().to(DEV)
    out = torch.empty((2, hidden), dtype=dtype, device=DEV)
    ops.add_layernorm(res, d1.to(DEV), d2.to(DEV), w1.to(DEV), b1.to(DEV), out, eps=eps, rows=rows)
    torch.testing.assert_close(out.float().cpu(), want1[[7, 2]], **tol)
    # the add alone
    res = residual.clone().to(DEV)
    ops.add_layernorm(res, d1.to(DEV), d2.to(DEV), None, None, None)
    torch.testing.assert_close(res.cpu(), new.float(), rtol=1e-6, atol=1e-6)


def test_layer_norm_of_a_row_with_a_large_mean():
    """Deviations are taken from the mean, not from the mean of squares (whose float32 difference
    from the squared mean would be off by several percent here): a row of 1000 +- 1 keeps its shape."""
    ops = _ops()
    hidden = 256
    x = 1000.0 + torch.randn(3, hidden)
    w, b = torch.ones(hidden), torch.zeros(hidden)
    out = torch.empty((3, hidden), dtype=torch.float32, device=DEV)
    ops.add_layernorm(x.clone().to(DEV), None, None, w.to(DEV), b.to(DEV), out, eps=1e-12)
    want = pm.layer_norm(x.double(), w.double(), b.double(), 1e-12).float()
    torch.testing.assert_close(out.cpu(), want, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("q_rank,r,rd,rotating", [(48, 32, 32, 32), (0, 16, 16, 16), (14, 26, 10, 10), (0, 18, 6, 4),
                                                  (64, 144, 16, 16), (300, 520, 64, 32)])
@pytest.mark.parametrize("tokens", [1, 21])
def test_latent_rows_normed_rotated_and_cached(dtype, q_rank, r, rd, rotating, tokens):
    """From the packed row: the query latent normed; the cached row ``[normed latent | rotated
    shared part]`` at the token's place of its page, the latent once more transposed; the shared
    part is rotated and not normed, channels beyond the rotating ones pass."""
    ops = _ops()
    page, base, eps = 8, 300.0, 1e-5
    q_cols = q_rank if q_rank else 40
    width = q_cols + r + rd + 3
    width += -width % 8
    packed = (torch.randn(tokens, width) * 2.0).to(dtype)
    positions = torch.arange(5, 5 + tokens, dtype=torch.int32)
    table = torch.tensor([[0, 0, 0, 0, 0, 0], [2, 3, 1, 4, 0, 0]], dtype=torch.int32)
    k_cache = torch.zeros((5, 1, page, r + rd), dtype=dtype, device=DEV)
    v_cache = torch.zeros((5, 1, r, page), dtype=dtype, device=DEV)
    wq, wkv = 1.0 + 0.2 * torch.randn(max(q_rank, 1)), 1.0 + 0.2 * torch.randn(r)
    i = torch.arange(rotating // 2, dtype=torch.float64)
    angle = (torch.arange(64, dtype=torch.float32)[:, None] * (base ** (-2.0 * i / rotating)).float()[None, :]).double()
    cos, sin = torch.cos(angle).float(), torch.sin(angle).float()
    q_latent = torch.empty((tokens, q_rank), dtype=dtype, device=DEV) if q_rank else None
    ops.latent_rows(
        packed.to(DEV), q_rank, wq.to(DEV) if q_rank else None, q_latent, q_cols, r, rd, wkv.to(DEV), cos.to(DEV),
        sin.to(DEV), k_cache, v_cache, positions.to(DEV), torch.ones(tokens, dtype=torch.int32, device=DEV),
        table.to(DEV), page, eps, int(positions.max()),
    )
    x = packed.double()
    tol = _tol(dtype)
    if q_rank:
        torch.testing.assert_close(q_latent.float().cpu(), pm.rms_norm(x[:, :q_rank], wq.double(), eps).float(), **tol)
    c = pm.rms_norm(x[:, q_cols:q_cols + r], wkv.double(), eps).float()
    kr = pm.rotate_pairs(x[:, q_cols + r:q_cols + r + rd], positions.long(), base, rotating).float()
    for t in range(tokens):
        pos = int(positions[t])
        pg, slot = int(table[1, pos // page]), pos % page
        torch.testing.assert_close(k_cache[pg, 0, slot, :r].float().cpu(), c[t], **tol)
        torch.testing.assert_close(k_cache[pg, 0, slot, r:].float().cpu(), kr[t], **tol)
        assert torch.equal(v_cache[pg, 0, :, slot], k_cache[pg, 0, slot, :r])
        if rotating < rd:
            assert torch.equal(k_cache[pg, 0, slot, r + rotating:].cpu(), packed[t, q_cols + r + rotating:q_cols + r + rd])
    assert not k_cache[0].any() and not v_cache[0].any()  # nothing lands on the null page
    # a layer that reads another's rows norms its query latent and writes nothing
    if q_rank:
        again = torch.empty_like(q_latent)
        ops.latent_rows(packed.to(DEV), q_rank, wq.to(DEV), again, q_cols, r, rd, None, cos.to(DEV), sin.to(DEV), None,
                        None, positions.to(DEV), torch.ones(tokens, dtype=torch.int32, device=DEV), table.to(DEV),
                        page, eps, int(positions.max()))
        assert torch.equal(again, q_latent)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("heads,d,rd,rotating,r", [(4, 16, 32, 32, 32), (3, 12, 10, 10, 26), (5, 10, 6, 4, 18), (1, 64, 64, 64, 512)])
def test_rotated_query_part_behind_the_latent_part(dtype, heads, d, rd, rotating, r):
    ops = _ops()
    tokens, base = 11, 77.0
    q_row = heads * (d + rd) + 8  # rows may carry more behind the heads
    q = torch.randn(tokens, q_row).to(dtype)
    positions = torch.tensor([0, 1, 2, 50, 3, 63, 7, 8, 9, 10, 33], dtype=torch.int32)
    i = torch.arange(rotating // 2, dtype=torch.float64)
    angle = (torch.arange(64, dtype=torch.float32)[:, None] * (base ** (-2.0 * i / rotating)).float()[None, :]).double()
    out = torch.zeros((tokens, heads * (r + rd)), dtype=dtype, device=DEV)
    ops.rotate_tail(q.to(DEV), out, torch.cos(angle).float().to(DEV), torch.sin(angle).float().to(DEV),
                    positions.to(DEV), heads, d, rd, r + rd, r, 63)
    tails = q[:, : heads * (d + rd)].double().view(tokens, heads, d + rd)[..., d:]
    want = pm.rotate_pairs(tails, positions.long(), base, rotating).float()
    got = out.float().cpu().view(tokens, heads, r + rd)
    torch.testing.assert_close(got[..., r:], want, **_tol(dtype))
    assert not got[..., :r].any()  # the latent part is another kernel's
    torch.testing.assert_close(got[0, :, r:], tails[0].float(), rtol=0, atol=0)  # position 0 turns nothing


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("heads,I,O", [(4, 16, 32), (3, 80, 16), (1, 16, 16), (8, 96, 16), (2, 144, 128), (5, 10, 18),
                                       (3, 26, 6), (2, 520, 48), (2, 128, 80), (3, 256, 32), (1, 512, 16), (2, 32, 272),
                                       (2, 64, 64)])
@pytest.mark.parametrize("tokens", [1, 37, 300])
def test_one_small_matrix_a_head(dtype, heads, I, O, tokens):
    """Slices of every head of ``x`` through the head's own matrix into slices of every head of
    ``y``, with and without the sigmoid gate per head; few tokens (a wave an output tile) and many
    (a wave 16 tokens and all outputs of a head) give a token the same bits."""
    ops = _ops()
    x_head, y_head, x_off, y_off = I + 8, O + 12, 4, 8
    x = torch.randn(tokens, x_off + heads * x_head).to(dtype)
    w = (torch.randn(heads, O, I) / math.sqrt(I)).to(dtype)
    gate = torch.randn(tokens, heads + 5).to(dtype)
    want = torch.einsum("thi,hoi->tho", x[:, x_off:].double().view(tokens, heads, x_head)[..., :I], w.double())
    tol = _tol(dtype, f32=2e-5, bf16=2e-2)
    for gated in (False, True):
        y = torch.zeros((tokens, y_off + heads * y_head), dtype=dtype, device=DEV)
        ops.head_product(x.to(DEV), w.to(DEV), y, heads, x_head, x_off, y_head, y_off,
                         gate=gate.to(DEV) if gated else None, gate_col=3)
        got = y.float().cpu()[:, y_off:].view(tokens, heads, y_head)
        ref = want * torch.sigmoid(gate[:, 3:3 + heads].double())[:, :, None] if gated else want
        torch.testing.assert_close(got[..., :O], ref.float(), **tol)
        assert not got[..., O:].any() and not y[:, :y_off].any()  # nothing beside the slices
    if dtype == torch.float32 and tokens > 1:
        # a token alone gives the same bits as in a batch
        y = torch.zeros((tokens, y_off + heads * y_head), dtype=dtype, device=DEV)
        ops.head_product(x.to(DEV), w.to(DEV), y, heads, x_head, x_off, y_head, y_off)
        alone = torch.zeros((1, y_off + heads * y_head), dtype=dtype, device=DEV)
        ops.head_product(x[20:21].contiguous().to(DEV), w.to(DEV), alone, heads, x_head, x_off, y_head, y_off)
        assert torch.equal(alone[0], y[20])


@pytest.mark.parametrize("experts,top", [(6, 2), (3, 1), (4, 4), (70, 5), (1, 1), (5, 2)])
def test_router_with_a_bias_and_weights_over_the_chosen_logits(experts, top):
    ops = _ops()
    tokens, width = 37, 48
    h = torch.randn(tokens, width)
    w = {"router": torch.randn(experts, width) * 0.8, "router.b": torch.randn(experts) * 2.0}
    cfg = {"router": {"experts": experts, "top": top}}
    for dtype in (torch.float32, torch.bfloat16):
        hx = h.to(dtype)
        chosen, weight = pm.route(hx.double(), cfg, {k: v.double() for k, v in w.items()}, "")
        want = torch.zeros(tokens, experts, dtype=torch.float64).scatter_(1, chosen, weight).float()
        got = ops.router(hx.to(DEV), w["router"].to(DEV), top, 1.0, w["router.b"].to(DEV))
        torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-5)
        assert ((got.cpu() > 0).sum(dim=1) == top).all()
        torch.testing.assert_close(got.sum(dim=1).cpu(), torch.ones(tokens), rtol=1e-5, atol=1e-5)
        alone = ops.router(hx[5:6].contiguous().to(DEV), w["router"].to(DEV), top, 1.0, w["router.b"].to(DEV))
        assert torch.equal(alone[0], got[5])
    if experts > top:
        # the bias decides: without it other experts are chosen for some token
        bare = ops.router(h.to(DEV), w["router"].to(DEV), top, 1.0)
        assert not torch.equal(bare.cpu() > 0, want > 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("experts,ff", [(5, 27), (6, 40), (1, 16), (3, 9)])
def test_gated_hidden_units_times_the_experts_weights(dtype, experts, ff):
    """Packed rows ``[every expert's gate | every expert's up]``: ``silu(gate) * up`` times the
    token's weight for the expert, 0 where it is not chosen."""
    ops = _ops()
    tokens = 13
    inner = experts * ff
    x = (torch.randn(tokens, 2 * inner) * 2.0).to(dtype)
    route = (torch.rand(tokens, experts) * (torch.rand(tokens, experts) > 0.5)).float()
    out = torch.empty((tokens, inner), dtype=dtype, device=DEV)
    ops.swiglu(x.to(DEV), out, route=route.to(DEV), expert_ff=ff)
    g, u = x[:, :inner].double(), x[:, inner:].double()
    want = g * torch.sigmoid(g) * u * route.double().repeat_interleave(ff, dim=1)
    torch.testing.assert_close(out.float().cpu(), want.float(), **_tol(dtype, f32=1e-5, bf16=2e-2))
    assert not out[:, :ff][route[:, 0] == 0].any()


# --------------------------------------------------------------------------- #
# whole models: every way of cutting the requests
# --------------------------------------------------------------------------- #

LENGTHS = {
    "A": [1, 2, 3, 6, 7, 8, 18, 19, 20, 21, 40, 41, 42, 43, 57, 150],  # the first tokens; around the windows of 7, 19 and 41
    "B": [1, 2, 4, 5, 6, 7, 9, 33, 80],                               # around the window of 5 and the page of 4
    "C": [2, 15, 63, 64, 65, 66, 129, 130, 131, 132, 260],            # around the windows of 64 and 130
    "D": [1, 2, 3, 8, 9, 10, 11, 32, 33, 34, 35, 90],                 # around the windows of 9 and 33
}


def _requests(which):
    cfg, _page, seed = MIBO[which]
    return {f"q{i}": random_tokens(n, cfg["vocab"], seed * 100 + i) for i, n in enumerate(LENGTHS[which])}


def _oracles(pcfg, pw, requests):
    """Per request the plain logits in float64, and what rounding alone does: the figure that
    nine rows in ten stay under, and how many rows of the plain implementation with rounded
    activations lie beyond the bound themselves (tokens whose choice of experts rounding flips)."""
    want = {rid: pm.forward(pcfg, pw, toks, torch.float64) for rid, toks in requests.items()}
    rounded = {rid: pm.forward(pcfg, pw, toks, torch.float64, cast=bf16_round) for rid, toks in requests.items()}
    order = sorted(want)
    a, b = torch.cat([rounded[r] for r in order]), torch.cat([want[r] for r in order])
    figure = rounding_figure(a, b)
    return want, (figure, int((row_errors(a, b) > BF16_TIMES_ROUNDING * figure).sum()))


def _runner(model_dir, dtype, page, num_pages, max_seq_len, slots=4):
    from rapid_llm_amd import EngineConfig, ModelRunner

    runner = ModelRunner(
        model_dir,
        EngineConfig(dtype=dtype, max_seq_len=max_seq_len, page_size=page, num_pages=num_pages,
                     max_num_seqs=slots, use_graph=False),
    )
    for layer in runner.device_cache.layers:  # whatever is read before it is written shows
        for t in layer.pages.values() if layer.owns_pages else ():
            t.fill_(float("nan"))
    return runner


def _check(got, want, dtype, label, rounding=None):
    order = sorted(want)
    if dtype == "bfloat16":
        a, b = torch.cat([got[r] for r in order]), torch.cat([want[r] for r in order])
        assert a.shape == b.shape and torch.isfinite(a).all(), label
        rows = row_errors(a, b)
        rounding, flipped = rounding
        beyond = rows > BF16_TIMES_ROUNDING * rounding
        parity.record(label, float(rows.max()), float((a.double() - b.double()).abs().max() / b.double().std()))
        allowed = max(2, int(BF16_ROWS_BEYOND * rows.numel()), 2 * flipped)
        assert int(beyond.sum()) <= allowed, (
            f"{label}: {int(beyond.sum())} of {rows.numel()} rows are off by more than {BF16_TIMES_ROUNDING} times "
            f"what rounding does ({rounding:.4f} of the logits' spread); the first is row {int(torch.nonzero(beyond)[0])}"
        )
        return
    spread = float(torch.cat([want[r] for r in order]).double().std())
    for rid in order:
        assert got[rid].shape == want[rid].shape and torch.isfinite(got[rid]).all(), (label, rid)
        rows = (got[rid].double() - want[rid].double()).square().mean(dim=1).sqrt() / spread
        bad = rows > F32_ROW
        assert not bad.any(), (
            f"{label}: request {rid}, first wrong position {int(torch.nonzero(bad)[0])}, "
            f"worst row {float(rows.max()):.3e} of the spread"
        )


@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cut_matches_plain(tmp_path, which, dtype):
    cfg, page, seed = MIBO[which]
    model_dir = make_model_dir(tmp_path, which, sharp=3.0)
    pcfg, pw = load_plain(model_dir)
    requests = _requests(which)
    want, rounding = _oracles(pcfg, pw, requests)
    longest = max(LENGTHS[which])
    schedules = {
        "whole": ru.whole(requests),
        "decode": ru.prefill_then_decode(requests, 50),
        "token_by_token": ru.prefill_then_decode(requests, 10 ** 6),
        "portions": ru.changing_portions(requests),
        "portions_of_two": ru.changing_portions(requests, sizes=(2, 2, 3, 2, 64, 2)),
        "mixed": ru.mixed(requests, seed, max_tokens=None),
        "mixed_tight": ru.mixed(requests, seed + 1, max_tokens=2 * 64 * ((longest + 63) // 64)),
    }
    first = None
    for label, steps in schedules.items():
        pages = ru.pages_for(steps, requests, page) + 1
        runner = _runner(model_dir, dtype, page, pages + 1, longest + 8)
        got = ru.run_in_process(runner, steps)
        _check(got, want, dtype, f"{which}/{dtype}/{label}", rounding)
        if dtype == "float32":
            # one order of summation however the requests are cut: the same bits
            if first is None:
                first = got
            else:
                for rid in got:
                    assert torch.equal(got[rid], first[rid]), (label, rid)
        runner.cache.check_invariants()
        assert not runner.cache.live_requests()
        del runner


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_of_unequal_requests_equals_each_alone(tmp_path, dtype):
    """One step holds a long prompt, a short one, a single first token and decoded tokens of two
    requests at different depths; every row equals the row of the request run alone."""
    which = "A"
    cfg, page, seed = MIBO[which]
    model_dir = make_model_dir(tmp_path, which, sharp=3.0)
    requests = {f"u{i}": random_tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate((90, 5, 1, 61, 30))}
    runner = _runner(model_dir, dtype, page, 60, 100, slots=5)
    alone = ru.run_in_process(runner, ru.whole(requests))
    full = lambda r, a, b, end=(): {"id": r, "tokens": requests[r][a:b], "want": list(range(b - a))}  # noqa: E731
    steps = [
        {"step": 0, "entries": [full("u3", 0, 60), full("u4", 0, 29)], "end": []},
        {"step": 1, "entries": [full("u0", 0, 90), full("u3", 60, 61), full("u1", 0, 5), full("u2", 0, 1), full("u4", 29, 30)],
         "end": ["u0", "u1", "u2", "u3", "u4"]},
    ]
    got = ru.run_in_process(runner, steps)
    for rid in requests:
        if dtype == "float32":
            assert torch.equal(got[rid], alone[rid]), rid
        else:
            assert float(row_errors(got[rid], alone[rid]).max()) < 0.05, rid
    runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_slots_used_again(tmp_path, dtype):
    """Five requests through two slots, each a short prompt and then 300 tokens one by one, two
    at a time in a step: the windows pass over decoded tokens, their pages come back and are
    taken again by later requests; the layer that sees everything keeps its pages."""
    which = "A"
    cfg, page, seed = MIBO[which]
    model_dir = make_model_dir(tmp_path, which, sharp=3.0)
    pcfg, pw = load_plain(model_dir)
    requests = {f"d{i}": random_tokens(300 + 7 * i, cfg["vocab"], 40 + i) for i in range(5)}
    want, rounding = _oracles(pcfg, pw, requests)
    steps = ru.mixed(requests, 3, max_live=2, tail=295)
    runner = _runner(model_dir, dtype, page, 2 * (-(-340 // page) + 1) + 2, 340, slots=2)
    got = ru.run_in_process(runner, steps)
    _check(got, want, dtype, f"long decoding/{dtype}", rounding)
    runner.cache.check_invariants()


def test_windowed_groups_give_pages_back_while_decoding(tmp_path):
    """The cache of a windowed layer holds a window's pages and no more, however long the request;
    rows that a layer with a longer window reads are kept for that longer window."""
    from rapid_llm_amd import StepEntry

    which = "A"
    cfg, page, seed = MIBO[which]
    model_dir = make_model_dir(tmp_path, which)
    runner = _runner(model_dir, "float32", page, 80, 420, slots=1)
    toks = random_tokens(400, cfg["vocab"], 5)
    runner.step([StepEntry("r", toks[:100], [99])])
    for i in range(100, 400):
        runner.step([StepEntry("r", toks[i:i + 1], [0])])
    held = {g.window: int((runner.cache.tables[g.group_id][runner.cache.slot_of("r")] != 0).sum())
            for g in runner.cache.groups}
    assert held[0] == 400 // page
    assert held[41] <= -(-41 // page) + 1 and held[7] <= -(-7 // page) + 1
    runner.finish("r")
    runner.cache.check_invariants()


def test_trace_program(tmp_path):
    """``bin/trace_run`` as a child process on a mixed trace over a tight pool."""
    which = "B"
    cfg, page, seed = MIBO[which]
    model_dir = make_model_dir(tmp_path, which, sharp=3.0)
    pcfg, pw = load_plain(model_dir)
    requests = _requests(which)
    want, rounding = _oracles(pcfg, pw, requests)
    steps = ru.mixed(requests, seed + 5, max_tokens=256)
    got = ru.run_trace_program(model_dir, "float32", steps, tmp_path / "out", 256, cfg["vocab"])
    _check(got, want, "float32", "trace_run")
    assert rounding[0] > 0


@pytest.mark.parametrize("use_graph", [False, True])
@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("D", "float32"), ("C", "bfloat16")])
def test_greedy_generation_through_the_entry_point(tmp_path, which, dtype, use_graph):
    """``LLM.generate``: scheduler, chunked prompts beside decoding requests, sampling kernels;
    decode steps eagerly and replayed from graphs.  The plain implementation re-runs the whole
    sequence for every token; a bfloat16 engine may pick another of several nearly equal maxima."""
    from rapid_llm_amd import LLM, SamplingParams

    cfg, page, seed = MIBO[which]
    model_dir = make_model_dir(tmp_path, which)
    pcfg, pw = load_plain(model_dir)
    prompts = [random_tokens(n, cfg["vocab"], seed + n) for n in (1, 7, 30, 45)]
    llm = LLM(str(model_dir), dtype=dtype, page_size=page, num_pages=60, max_num_seqs=3, max_seq_len=96,
              max_chunk_size=16, max_num_batched_tokens=32, use_cuda_graph=use_graph)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_gen_len=24))
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for tok in out.token_ids:
            logits = pm.forward(pcfg, pw, ids)[-1]
            if dtype == "float32":
                assert float(logits.max() - logits[tok]) <= 1e-3, (len(prompt), len(ids))
            else:
                parity.assert_near_choice(logits, tok, f"generation/{which}/graph={use_graph}")
            ids.append(tok)
        assert len(out.token_ids) == 24
    llm.scheduler.cache.check_invariants()
    assert not llm.scheduler.cache.live_requests()
