"""Decode and prefill speed of the engine on one MI355X, random weights, synthetic token ids.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--dtype bfloat16]
                    [--shape NAME] [--batch B] [--prompt-len T] [--context C]
    python bench.py --workload qwen3-0.6b-256 | qwen3-32b-32
    python bench.py --design fokulorn|sikevik|miborax|fomunex [--design-size 2b,8b]

A "step" is one decode step of the whole batch through the engine's step function and the
greedy sampling kernel, tokens fed back.  The default run has the layer sizes of
Qwen3-8B (BASELINE.json ``configs[2]``), a batch of 8, every request with a 2,048-token
prompt, context 4,096.  One JSON line is printed: decoded tokens a second (``value``), the
2,048-token prefill (``prefill``), the decode step against the HBM roofline (``roofline``)
and decoding at batch 1 and 64 (``points``, which also holds the true 32-bit path's decode
and prefill speed, measured in a second process).  ``--shape``, ``--prompt-len`` and
``--context`` measure the same at other sizes of the model family and other lengths; the
line then names them in ``metric`` and ``config``.

``points`` also holds the two scheduler workloads of BASELINE.json (``configs[3]``: the
Qwen3-0.6B shape, 256 requests at once, prompts uniform in 64 to 1,024 tokens, 128 tokens each;
``configs[4]``: the Qwen3-32B shape, 32 requests, prompts uniform in 4,096 to 16,384, context
16,384, cache pages from the memory that is free, 128 tokens each): time per output token,
generated tokens a second and the decode step's share of the HBM roofline, each measured in a
process of its own through the continuous-batching scheduler (``--workload NAME`` runs one
alone; ``--no-workloads`` leaves them out).

``--design fokulorn`` measures another architecture of the engine, the Fokulorn decoder
(matrix-memory recurrences beside windowed attention whose values are its keys), at layer
sizes of real models, beside the Qwen3 decoder of the same width, depth, heads and
feed-forward width: prefill of one prompt and decode at batch 8 through the same step
function, and the design's own kernels alone against their rooflines.  It prints one line of
its own and leaves the default run as it is.

``--design sikevik`` does the same for the Sikevik decoder (windowed attention that keeps a
request's first positions, with a sink term and value heads of half the key heads' size; norms
before and behind every sub-layer; one dense two-layer feed-forward, then mixtures of eight
experts with a shared one; the last six layers in two passes of three), whose feed-forward
matrices hold as many weights a layer as Qwen3's.

``--design miborax`` does the same for the Miborax decoder (attention through a latent row that
all heads share, half of the layers windowed, a quarter reading the rows another layer cached; both
sub-layers of a layer behind layer norms of the same stream; mixtures of eight gated experts with a
router bias), beside the Sikevik decoder, the engine's closest (a sink term, windows, routed
experts), and Qwen3 of equal size.

``--design fomunex`` does the same for the Fomunex decoder (layers in turn: capped windowed
attention with a distance term and learned sinks, a token-shift time mixing, a state-space mixer
behind a short convolution, attention again; dense feed-forwards with a polynomial activation in
the even layers, mixtures of eight clamped gated experts behind a sigmoid router in the odd ones),
beside the Fokulorn decoder, the engine's closest (recurrent layers with a state per request
beside windowed attention), and Qwen3 of equal size.

Metric definitions follow rapid_llm's docs/benchmark_models.md:141-149: decode tok/s is
batch / mean step time; prefill tok/s is prompt tokens / prefill latency; both timed
between device synchronisations after warm-up.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBPS = 8000.0
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}


def load_shape() -> dict:
    """Layer sizes of BASELINE.json configs[2], parsed from its text."""
    import re

    with open(os.path.join(ROOT, "BASELINE.json")) as fh:
        text = json.load(fh)["configs"][2]

    def num(pattern: str) -> int:
        m = re.search(pattern, text)
        if m is None:
            raise SystemExit(f"BASELINE.json configs[2] does not state {pattern!r}")
        return int(m.group(1).replace(",", ""))

    theta = re.search(r"rope_theta ([0-9.e+]+)", text).group(1)
    eps = re.search(r"rms_norm_eps ([0-9.e+-]+)", text).group(1)
    return dict(
        architectures=["Qwen3ForCausalLM"],
        model_type="qwen3",
        num_hidden_layers=num(r"(\d+) layers"),
        hidden_size=num(r"hidden (\d+)"),
        num_attention_heads=num(r"(\d+) query heads"),
        num_key_value_heads=num(r"(\d+) KV heads"),
        head_dim=num(r"head_dim (\d+)"),
        intermediate_size=num(r"intermediate (\d+)"),
        vocab_size=num(r"vocab (\d+)"),
        rope_theta=float(theta),
        rms_norm_eps=float(eps),
        tie_word_embeddings="untied" not in text,
        max_position_embeddings=40960,
        context=num(r"context (\d+)"),
        prompt_len=num(r"one ([\d,]+)-token prompt"),
    )


# Other members of the model family (layer sizes as their model cards give them), for
# measurements beside the default run's.
FAMILY = {
    "qwen3-0.6b": dict(num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8,
                       intermediate_size=3072, tie_word_embeddings=True),
    "qwen3-1.7b": dict(num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, num_key_value_heads=8,
                       intermediate_size=6144, tie_word_embeddings=True),
    "qwen3-4b": dict(num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
                     intermediate_size=9728, tie_word_embeddings=True),
    "qwen3-14b": dict(num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                      intermediate_size=17408, tie_word_embeddings=False),
    "qwen3-32b": dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                      intermediate_size=25600, tie_word_embeddings=False),
}


def weight_bytes(cfg, elem: int) -> int:
    h, i = cfg.hidden_size, cfg.intermediate_size
    per_layer = (cfg.q_size + 2 * cfg.kv_size) * h + h * cfg.q_size + 2 * i * h + h * i
    return (per_layer * cfg.num_hidden_layers + cfg.vocab_size * h) * elem


def kv_bytes_per_token(cfg, elem: int) -> int:
    return 2 * cfg.kv_size * cfg.num_hidden_layers * elem


def prefill_flops(cfg, tokens: int) -> float:
    h, i = cfg.hidden_size, cfg.intermediate_size
    per_layer = (cfg.q_size + 2 * cfg.kv_size) * h + h * cfg.q_size + 2 * i * h + h * i
    linear = 2.0 * tokens * per_layer * cfg.num_hidden_layers + 2.0 * cfg.vocab_size * h  # one logits row
    attn = 2.0 * 2.0 * cfg.q_size * (tokens * (tokens + 1) / 2) * cfg.num_hidden_layers  # causal QK^T and PV
    return linear + attn


def measured_peaks() -> int:
    """Practical peaks of this device, beside the published ones the fractions are quoted
    against: a 4 GiB read by a plain streaming kernel, a 2 GiB library copy, and the library's square
    products of 8,192."""
    import torch

    def timed(fn, n=10) -> float:
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / n

    from rapid_llm_amd.kernels import ops

    out = {}
    x = torch.ones(1 << 31, dtype=torch.bfloat16, device="cuda")  # 4 GiB
    out["read_gbps"] = round(
        max(x.numel() * 2 / timed(lambda: ops.read_buffer(x, blocks)) for blocks in (1024, 2048, 4096, 8192, 32768)) / 1e9, 1
    )
    half = x[: 1 << 30]
    y = torch.empty_like(half)
    out["copy_gbps_read_plus_write"] = round(2 * half.numel() * 2 / timed(lambda: y.copy_(half)) / 1e9, 1)
    del x, y, half
    n = 8192
    for name, dtype in (("bf16", torch.bfloat16), ("fp32", torch.float32)):
        a = torch.randn(n, n, device="cuda", dtype=dtype)
        b = torch.randn(n, n, device="cuda", dtype=dtype)
        torch.backends.cuda.matmul.allow_tf32 = False
        out[f"gemm_{name}_tflops"] = round(2 * n**3 / timed(lambda: torch.matmul(a, b.t())) / 1e12, 1)
    # What a kernel of a decode step can hope for: plain reads of the sizes of a layer's four
    # weight matrices (Qwen3-8B: 34, 50, 100 and 201 MB) and of 400 MB, forty in a row replayed
    # from a graph, every one over memory that no earlier one touched.  Microseconds a kernel;
    # the rate is what a product of that size can reach at most, start and end included.
    pool = torch.ones(1 << 30, dtype=torch.bfloat16, device="cuda")  # 2 GiB
    chain = {}
    for mb in (34, 50, 100, 201, 400):
        n = int(mb * 1e6 / 2)
        views = [pool[i * n : (i + 1) * n] for i in range(pool.numel() // n)]
        best = None
        for blocks in (256, 512, 2048):
            graph = torch.cuda.CUDAGraph()
            ops.read_buffer(views[0], blocks)
            torch.cuda.synchronize()
            with torch.cuda.graph(graph):
                for i in range(40):
                    ops.read_buffer(views[i % len(views)], blocks)
            sec = timed(graph.replay, 5) / 40
            best = sec if best is None else min(best, sec)
        chain[f"{mb}MB"] = {"us": round(best * 1e6, 1), "gbps": round(mb * 1e6 / best / 1e9, 1)}
    out["read_chain"] = chain
    out["published"] = {"hbm_gbps": HBM_GBPS, "bf16_tflops": PEAK_TFLOPS["bfloat16"], "fp32_tflops": PEAK_TFLOPS["float32"]}
    print(json.dumps(out), flush=True)
    return 0


# The scheduler workloads of BASELINE.json configs[3] and configs[4].
WORKLOADS = {
    "qwen3-0.6b-256": dict(shape="qwen3-0.6b", requests=256, low=64, high=1024, gen=128, context=2048, key="w06b",
                           passes=2),
    # one pass: its 300,000 prompt tokens take 25 s, and recording the decode graphs in the
    # first steps changes the mean of 127 steps by under 1%
    "qwen3-32b-32": dict(shape="qwen3-32b", requests=32, low=4096, high=16384, gen=128, context=16384 + 128, key="w32b",
                         passes=1),
}


def run_workload(name: str, seed: int = 1234) -> int:
    """One workload through the scheduler; prints one JSON line of its own."""
    import torch

    from rapid_llm_amd.cli import measure_offline, sample_prompt_lengths
    from rapid_llm_amd.engine.llm import build_engine

    w = WORKLOADS[name]
    shape = load_shape()
    shape.pop("context"), shape.pop("prompt_len")
    shape.update(FAMILY[w["shape"]])
    t0 = time.time()
    engine = build_engine(
        shape, load_format="random", dtype="bfloat16", max_seq_len=w["context"], max_num_seqs=w["requests"],
        max_num_batched_tokens=8192, max_chunk_size=8192, page_size=16, seed=seed,
    )
    cfg = engine.runner.config
    torch.cuda.synchronize()
    print(f"[bench] {name}: model ready in {time.time() - t0:.1f} s, "
          f"{engine.cache.capacity_tokens()} tokens of cache", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(seed)
    rows = []
    for it in range(w["passes"]):  # with two, the first records the graphs and warms the allocator
        lengths = sample_prompt_lengths(w["requests"], w["low"], w["high"], seed + it)
        prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for n in lengths]
        row = measure_offline(engine, prompts, w["gen"])
        row["mean_prompt"] = sum(lengths) / len(lengths)
        rows.append(row)
        print(f"[bench] {name} pass {it}: {row}", file=sys.stderr, flush=True)
    row = rows[-1]
    tpot = row["tpot_s"]
    mean_ctx = row["mean_prompt"] + w["gen"] / 2.0
    step_bytes = weight_bytes(cfg, 2) + w["requests"] * mean_ctx * kv_bytes_per_token(cfg, 2)
    k = w["key"]
    print(json.dumps({
        f"{k}_tpot_ms": round(tpot * 1e3, 3),
        f"{k}_decode_tok_s": round(w["requests"] / tpot, 1),
        f"{k}_tok_s": round(row["output_tokens"] / row["latency_s"], 1),
        f"{k}_prefill_tok_s": round(row["prompt_tokens"] / row["ttft_s"], 1),
        f"{k}_hbm_frac": round(step_bytes / tpot / 1e9 / HBM_GBPS, 4),
        f"{k}_preemptions": row["preemptions"],
    }), flush=True)
    return 0


def workload_points(names) -> dict:
    """Each workload in a process of its own (the 32B shape needs the whole device)."""
    import subprocess

    out = {}
    for name in names:
        try:
            done = subprocess.run(
                [sys.executable, os.path.abspath(__file__), "--workload", name], capture_output=True, text=True, timeout=900
            )
            out.update(json.loads(done.stdout.strip().splitlines()[-1]))
            print(f"[bench] workload {name}: {done.stdout.strip().splitlines()[-1]}", file=sys.stderr, flush=True)
        except Exception as err:  # the main line must not be lost to a workload
            tail = "" if "done" not in locals() else done.stderr[-800:]
            print(f"[bench] workload {name} gave no result: {err!r} {tail}", file=sys.stderr, flush=True)
    return out


def float32_points(args) -> dict:
    """The same model through the true 32-bit path, in a process of its own (the float32
    weights need their own 33 GB): decode tok/s at the main batch size and prefill tok/s."""
    import subprocess

    cmd = [
        sys.executable, os.path.abspath(__file__), "--dtype", "float32", "--batch", str(args.batch),
        "--steps", "16", "--warmup", "4", "--points", "",
    ]
    if args.layers is not None:
        cmd += ["--layers", str(args.layers)]
    cmd += ["--shape", args.shape]
    if args.prompt_len is not None:
        cmd += ["--prompt-len", str(args.prompt_len)]
    if args.context is not None:
        cmd += ["--context", str(args.context)]
    try:
        done = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        line = json.loads(done.stdout.strip().splitlines()[-1])
        out = {f"fp32_decode_b{args.batch}": line["value"]}
        if line.get("prefill"):
            out["fp32_prefill"] = line["prefill"]["value"]
        print(f"[bench] float32 path: {out}", file=sys.stderr, flush=True)
        return out
    except Exception as err:  # the main line must not be lost to the float32 run
        print(f"[bench] the float32 run gave no result: {err!r}", file=sys.stderr, flush=True)
        return {}


# Layer sizes for ``--design fokulorn``: three recurrent layers to one of attention, the
# attention as in the Qwen3 shape of that width, the recurrence with half the width in keys and
# the whole width in values (heads of 128 / 256 and of 256 / 512 channels).
DESIGN_SIZES = {
    "2b": dict(width=2048, layers=8, heads=16, kv_heads=8, head_dim=128, ff=6144, vocab=151936,
               mem_heads=8, mem_dk=128, mem_dv=256, window=1024),
    "8b": dict(width=4096, layers=8, heads=32, kv_heads=8, head_dim=128, ff=12288, vocab=151936,
               mem_heads=8, mem_dk=256, mem_dv=512, window=1024),
}


def fokulorn_body(z: dict) -> dict:
    layers = []
    for i in range(z["layers"]):
        if i % 4 == 3:
            layers.append({"type": "attention", "mixer": {
                "heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["head_dim"], "vdim": z["head_dim"],
                "scale": z["head_dim"] ** -0.5, "mask": {"size": z["window"]},
                "rot": {"dims": z["head_dim"] // 2, "base": 10000.0}},
                "mlp": {"kind": "dense", "ff": z["ff"], "limit": 7.0}})
        else:
            layers.append({"type": "mlstm", "mixer": {
                "heads": z["mem_heads"], "dim": z["mem_dk"], "vdim": z["mem_dv"], "gate_cap": 15.0},
                "mlp": {"kind": "dense", "ff": z["ff"], "limit": 7.0}})
    return {"architecture": "Fokulorn", "width": z["width"], "vocab": z["vocab"], "embedding": {"scale": 1.0},
            "norm": {"eps": 1e-6}, "layers": layers}


def sikevik_body(z: dict) -> dict:
    """Eight layer runs as five layers, the last three twice; a layer's feed-forward matrices
    hold what Qwen3's three do (two matrices of 1.5 x the width for the dense one; eight experts
    of an eighth and a shared one of half the width for the others)."""
    ff = z["ff"]
    mixer = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["head_dim"], "vdim": z["head_dim"] // 2,
             "scale": z["head_dim"] ** -0.5, "mask": {"size": z["window"], "keep_first": 64}}
    moe = {"kind": "moe", "expert": {"ff": ff // 8}, "router": {"experts": 8, "top": 2, "scale": 1.0},
           "shared": {"ff": ff // 2}}
    n = z["layers"] - 3
    layers = [{"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff * 3 // 2} if i == 0 else moe}
              for i in range(n)]
    return {"architecture": "Sikevik", "width": z["width"], "vocab": z["vocab"], "embedding": {"scale": 1.0},
            "norm": {"eps": 1e-6}, "layers": layers, "loop": {"start": n - 3, "stop": n, "times": 2}}


def _time_sikevik_kernels(z: dict, prompt_len: int, batch: int) -> dict:
    """The design's attention kernel alone: one prompt from its start (matrix rate over the keys
    every query sees) and ``batch`` single tokens behind ``prompt_len`` (bytes of the keys and
    values read), microseconds and share of the roofline."""
    import types

    import torch

    from rapid_llm_amd.kernels import ops

    nq, nkv, d, dv, page = z["heads"], z["kv_heads"], z["head_dim"], z["head_dim"] // 2, 16
    window, keep, dev = z["window"], 64, "cuda"

    def run(seqs):
        tokens = sum(n for _, n in seqs)
        per = -(-max(a + n for a, n in seqs) // page)
        pages = len(seqs) * per + 1
        table = (1 + torch.arange(len(seqs) * per, dtype=torch.int32, device=dev)).view(len(seqs), per).contiguous()
        kc = (torch.randn(pages, nkv, page, d, device=dev) * 0.5).bfloat16()
        vc = (torch.randn(pages, nkv, dv, page, device=dev) * 0.5).bfloat16()
        q = (torch.randn(tokens, nq * d, device=dev) * 0.5).bfloat16()
        out = torch.empty((tokens, nq * dv), dtype=torch.bfloat16, device=dev)
        pos = torch.cat([torch.arange(a, a + n, dtype=torch.int32) for a, n in seqs]).to(dev)
        slot = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, (_, n) in enumerate(seqs)]).to(dev)
        ctx = types.SimpleNamespace(positions=pos, token_slot=slot, token_ids=pos, h_seq_starts=[a for a, _ in seqs],
                                    h_seq_lens=[n for _, n in seqs], max_position=int(pos.max()), extra={})

        def call():
            ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, window, d ** -0.5,
                                value_dim=dv, keep_first=keep, sink=True)

        for _ in range(3):
            call()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(10):
            call()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / 10

    sec_p = run([(0, prompt_len)])
    seen = sum(min(p + 1, window) + (min(keep, p + 1 - window) if p + 1 > window else 0) for p in range(prompt_len))
    flops = 2.0 * nq * seen * (d + dv)
    sec_d = run([(prompt_len, 1)] * batch)
    keys = min(prompt_len + 1, window) + (keep if prompt_len + 1 > window + keep else 0)
    kv_bytes = 2.0 * batch * nkv * keys * (d + dv)
    return {
        "attention_prefill_us": round(sec_p * 1e6, 1),
        "attention_prefill_frac_bf16_matrix": round(flops / sec_p / (PEAK_TFLOPS["bfloat16"] * 1e12), 4),
        "attention_decode_us": round(sec_d * 1e6, 1),
        "attention_decode_frac_hbm": round(kv_bytes / sec_d / 1e9 / HBM_GBPS, 4),
    }


def qwen3_body(z: dict) -> dict:
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=z["layers"],
                hidden_size=z["width"], num_attention_heads=z["heads"], num_key_value_heads=z["kv_heads"],
                head_dim=z["head_dim"], intermediate_size=z["ff"], vocab_size=z["vocab"], rope_theta=1e6,
                rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960)


def _time_model(body: dict, prompt_len: int, batch: int, steps: int, context: int) -> dict:
    """Prefill of one prompt and decode at ``batch`` through ``ModelRunner.step``."""
    import torch

    from rapid_llm_amd import EngineConfig, ModelRunner, StepEntry

    pages = batch * (-(-(prompt_len + steps + 40) // 16)) + 1
    runner = ModelRunner(body, EngineConfig(dtype="bfloat16", max_seq_len=context, page_size=16, num_pages=pages,
                                            max_num_seqs=batch, max_num_batched_tokens=8192, seed=1234),
                         load_format="random")
    gen = torch.Generator().manual_seed(7)
    vocab = runner.vocab_size

    def prompt():
        return torch.randint(0, vocab, (prompt_len,), generator=gen).tolist()

    times = []
    for _ in range(4):
        toks = prompt()
        torch.cuda.synchronize()
        t = time.perf_counter()
        runner.step([StepEntry("p", toks, [prompt_len - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t)
        runner.finish("p")
    prefill = statistics.median(times[1:])
    ids = [f"d{i}" for i in range(batch)]
    for rid in ids:
        runner.step([StepEntry(rid, prompt(), [prompt_len - 1])])
    entries = [StepEntry(rid, [1 + i], [0]) for i, rid in enumerate(ids)]
    for _ in range(12):
        runner.step(entries)
    torch.cuda.synchronize()
    t = time.perf_counter()
    for _ in range(steps):
        runner.step(entries)
    torch.cuda.synchronize()
    decode = (time.perf_counter() - t) / steps
    out = {"prefill_tok_s": round(prompt_len / prefill, 1), "prefill_ms": round(prefill * 1e3, 3),
           "decode_tok_s": round(batch / decode, 1), "decode_ms": round(decode * 1e3, 4)}
    del runner
    torch.cuda.empty_cache()
    return out


def _time_kernels(z: dict, prompt_len: int, batch: int) -> dict:
    """The design's own kernels alone, microseconds and share of the roofline each: the
    recurrence over one prompt (float32 matrix rate) and over ``batch`` single tokens (bytes
    of state read and written), and the two row-wise kernels (bytes)."""
    import types

    import torch

    from rapid_llm_amd.kernels import ops

    h, dk, dv = z["mem_heads"], z["mem_dk"], z["mem_dv"]
    width = 2 * h * dk + 2 * h * dv
    cols = (0, h * dk, 2 * h * dk, 2 * h * dk + h * dv)
    dev = "cuda"
    S = torch.zeros((batch + 1, h, dk, dv), device=dev)
    n = torch.zeros((batch + 1, h, dk), device=dev)
    m = torch.zeros((batch + 1, h), device=dev)
    weight = torch.ones(h * dv, device=dev)

    def run(lens):
        tokens = sum(lens)
        packed = (torch.randn(tokens, width, device=dev) * 0.5).bfloat16()
        pre = torch.randn(tokens, 2 * h, device=dev)
        out = torch.empty((tokens, h * dv), dtype=torch.bfloat16, device=dev)
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
        ctx = types.SimpleNamespace(num_seqs=len(lens), h_seq_lens=lens, h_seq_slots=list(range(len(lens))),
                                    cu_seqlens=cu, seq_slots=torch.arange(len(lens), dtype=torch.int32, device=dev))

        def call():
            ops.mlstm(packed, cols, pre, None, weight, out, ctx, S, n, m, h, dk, dv, 15.0, 1e-6)

        for _ in range(3):
            call()
        torch.cuda.synchronize()
        if max(lens) == 1:
            # single tokens: replayed from a graph, as a decode step runs them (launched one
            # by one the three kernels cost the host more than the device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(10):
                    call()
            graph.replay()
            torch.cuda.synchronize()
            t = time.perf_counter()
            for _ in range(5):
                graph.replay()
            torch.cuda.synchronize()
            return (time.perf_counter() - t) / 50
        t = time.perf_counter()
        for _ in range(10):
            call()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / 10

    sec_p = run([prompt_len])
    # per token and head: S^T q and the update k v^T over dk x (dv + 1), and the chunk's own
    # scores and their products with the values at chunks of 64
    flops = prompt_len * h * (4.0 * dk * (dv + 1) + 2.0 * 64 * (dk + dv + 1))
    sec_d = run([1] * batch)
    state_bytes = 2.0 * batch * h * dk * (dv + 1) * 4
    return {
        "recurrence_prefill_us": round(sec_p * 1e6, 1),
        "recurrence_prefill_frac_fp32_matrix": round(flops / sec_p / (PEAK_TFLOPS["float32"] * 1e12), 4),
        "recurrence_decode_us": round(sec_d * 1e6, 1),
        "recurrence_decode_frac_hbm": round(state_bytes / sec_d / 1e9 / HBM_GBPS, 4),
    }


# Latent sizes for ``--design miborax``: a row of 256 channels and a rotated part of 64 that all
# heads share, heads of 128 + 64 query channels and 128 value channels, queries through a latent of
# three quarters of the width in the layers that see everything.
MIBORAX_LATENT = dict(kv_rank=256, rot_dim=64, dim=128, vdim=128)


def miborax_body(z: dict) -> dict:
    """Of every four layers the first and last are windowed with rows of their own, the second sees
    everything and takes its queries through a latent, the third is windowed and reads the first's
    rows.  Eight gated experts of an eighth of Qwen3's feed-forward width each (two of eight used):
    a layer's feed-forward matrices hold what Qwen3's three do."""
    lat = MIBORAX_LATENT
    scale = (lat["dim"] + lat["rot_dim"]) ** -0.5

    def mixer(**more):
        return {"heads": z["heads"], "dim": lat["dim"], "rot_dim": lat["rot_dim"], "vdim": lat["vdim"],
                "kv_rank": lat["kv_rank"], "scale": scale, "rot": {"base": 10000.0, "dims": lat["rot_dim"]}, **more}

    moe = {"kind": "moe", "expert": {"ff": z["ff"] // 8}, "router": {"experts": 8, "top": 2}}
    layers = []
    for i in range(z["layers"]):
        if i % 4 == 1:
            layers.append({"type": "latent_attention", "mixer": mixer(q_rank=z["width"] * 3 // 4), "mlp": moe})
        elif i % 4 == 2:
            layers.append({"type": "latent_attention_2", "mixer": mixer(mask={"size": z["window"]}, kv_from=i - 2), "mlp": moe})
        else:
            layers.append({"type": "latent_attention_2", "mixer": mixer(mask={"size": z["window"]}), "mlp": moe})
    return {"architecture": "Miborax", "width": z["width"], "vocab": z["vocab"], "embedding": {"scale": 1.0},
            "norm": {"eps": 1e-6}, "layers": layers}


def _time_calls(call, graph: bool) -> float:
    """Seconds a call.  ``graph``: ten calls recorded and replayed, as a decode step runs them
    (launched one by one, short kernels cost the host more than the device)."""
    import torch

    for _ in range(3):
        call()
    torch.cuda.synchronize()
    if graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(10):
                call()
        g.replay()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(5):
            g.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / 50
    t = time.perf_counter()
    for _ in range(10):
        call()
    torch.cuda.synchronize()
    return (time.perf_counter() - t) / 10


def _time_miborax_kernels(z: dict, prompt_len: int, batch: int) -> dict:
    """The design's own kernels alone, microseconds and share of the roofline each.  Attention over
    the shared rows: one prompt from its start (matrix rate over the keys every query sees, each a
    row of ``kv_rank + rot_dim`` channels against ``heads`` queries, and ``kv_rank`` channels of
    values) and ``batch`` single tokens behind ``prompt_len`` (bytes of the rows read: the latent
    twice, once as keys and once transposed as values), windowed and over everything.  The heads'
    key and value matrices (matrix rate in a prompt step, bytes of the matrices in a decode step)
    and the pair of layer norms with the residual add (bytes)."""
    import types

    import torch

    from rapid_llm_amd.kernels import ops

    lat = MIBORAX_LATENT
    nq, r, rd, dn, dv, page, dev = z["heads"], lat["kv_rank"], lat["rot_dim"], lat["dim"], lat["vdim"], 16, "cuda"
    d = r + rd
    sink = torch.zeros(nq, device=dev)
    out = {}

    def attention(seqs, window):
        tokens = sum(n for _, n in seqs)
        per = -(-max(a + n for a, n in seqs) // page)
        pages = len(seqs) * per + 1
        table = (1 + torch.arange(len(seqs) * per, dtype=torch.int32, device=dev)).view(len(seqs), per).contiguous()
        kc = (torch.randn(pages, 1, page, d, device=dev) * 0.5).bfloat16()
        vc = (torch.randn(pages, 1, r, page, device=dev) * 0.5).bfloat16()
        q = (torch.randn(tokens, nq * d, device=dev) * 0.5).bfloat16()
        res = torch.empty((tokens, nq * r), dtype=torch.bfloat16, device=dev)
        pos = torch.cat([torch.arange(a, a + n, dtype=torch.int32) for a, n in seqs]).to(dev)
        slot = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, (_, n) in enumerate(seqs)]).to(dev)
        ctx = types.SimpleNamespace(positions=pos, token_slot=slot, token_ids=pos, h_seq_starts=[a for a, _ in seqs],
                                    h_seq_lens=[n for _, n in seqs], max_position=int(pos.max()), extra={})
        return _time_calls(lambda: ops.paged_attention(q, kc, vc, res, ctx, table, page, nq, 1, d, window, d ** -0.5,
                                                       value_dim=r, sink_values=sink), graph=False)

    for name, window in (("windowed", z["window"]), ("causal", 0)):
        sec = attention([(0, prompt_len)], window)
        seen = sum(min(p + 1, window) if window else p + 1 for p in range(prompt_len))
        out[f"attention_{name}_prefill_us"] = round(sec * 1e6, 1)
        out[f"attention_{name}_prefill_frac_bf16_matrix"] = round(
            2.0 * nq * seen * (d + r) / sec / (PEAK_TFLOPS["bfloat16"] * 1e12), 4)
        sec = attention([(prompt_len, 1)] * batch, window)
        keys = min(prompt_len + 1, window) if window else prompt_len + 1
        out[f"attention_{name}_decode_us"] = round(sec * 1e6, 1)
        out[f"attention_{name}_decode_frac_hbm"] = round(2.0 * batch * keys * (d + r) / sec / 1e9 / HBM_GBPS, 4)

    # the heads' key matrices (queries into the latent's channels) and value matrices
    uk = (torch.randn(nq, r, dn, device=dev) * 0.05).bfloat16()
    uv = (torch.randn(nq, dv, r, device=dev) * 0.05).bfloat16()
    for what, tokens in (("prefill", prompt_len), ("decode", batch)):
        q = (torch.randn(tokens, nq * (dn + rd), device=dev) * 0.5).bfloat16()
        full = torch.empty((tokens, nq * d), dtype=torch.bfloat16, device=dev)
        mean = (torch.randn(tokens, nq * r, device=dev) * 0.5).bfloat16()
        heads_out = torch.empty((tokens, nq * dv), dtype=torch.bfloat16, device=dev)
        small = what == "decode"
        sec_k = _time_calls(lambda: ops.head_product(q, uk, full, nq, dn + rd, 0, d, 0), graph=small)
        sec_v = _time_calls(lambda: ops.head_product(mean, uv, heads_out, nq, r, 0, dv, 0), graph=small)
        flops = 2.0 * tokens * nq * r * dn
        moved = 2.0 * (nq * r * dn + tokens * nq * (dn + r))
        for tag, sec, io in (("key", sec_k, moved), ("value", sec_v, 2.0 * (nq * r * dv + tokens * nq * (r + dv)))):
            out[f"head_{tag}_matrices_{what}_us"] = round(sec * 1e6, 1)
            if small:
                out[f"head_{tag}_matrices_{what}_frac_hbm"] = round(io / sec / 1e9 / HBM_GBPS, 4)
            else:
                out[f"head_{tag}_matrices_{what}_frac_bf16_matrix"] = round(flops / sec / (PEAK_TFLOPS["bfloat16"] * 1e12), 4)

    # both layer norms of a layer with the add of the two sub-layers' outputs in front
    width = z["width"]
    for what, tokens in (("prefill", prompt_len), ("decode", batch)):
        res = torch.randn(tokens, width, device=dev)
        d1 = torch.randn(tokens, width, device=dev).bfloat16()
        d2 = torch.randn(tokens, width, device=dev).bfloat16()
        w1, b1, w2, b2 = (torch.randn(width, device=dev) for _ in range(4))
        o1 = torch.empty((tokens, width), dtype=torch.bfloat16, device=dev)
        o2 = torch.empty_like(o1)
        sec = _time_calls(lambda: ops.add_layernorm(res, d1, d2, w1, b1, o1, w2, b2, o2, eps=1e-6), graph=what == "decode")
        out[f"add_two_layernorms_{what}_us"] = round(sec * 1e6, 1)
        out[f"add_two_layernorms_{what}_frac_hbm"] = round(tokens * width * (4 + 4 + 2 + 2 + 2 + 2) / sec / 1e9 / HBM_GBPS, 4)
    return out


def fomunex_body(z: dict) -> dict:
    """Layers in turn attention, time mixing, state-space, attention; the recurrent mixers with
    heads of 64 channels (the time mixing as wide as the model, the state-space mixer twice as
    wide with states of 128); a layer's feed-forward matrices hold what Qwen3's three do."""
    w, ff = z["width"], z["ff"]
    attention = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["head_dim"], "vdim": z["head_dim"],
                 "scale": z["head_dim"] ** -0.5, "softcap": 50.0, "mask": {"size": z["window"]}}
    mixing = {"heads": w // 64, "dim": 64, "rank": 64}
    space = {"heads": 2 * w // 64, "vdim": 64, "state": 128, "groups": 8, "conv": 4, "norm_groups": 8}
    dense = {"kind": "dense", "ff": ff * 3 // 2}
    moe = {"kind": "moe", "expert": {"ff": ff // 8, "limit": 7.0}, "router": {"experts": 8, "top": 2}}
    kinds = [("attention", attention), ("wkv", mixing), ("mamba2", space), ("attention", attention)]
    layers = [{"type": kinds[i % 4][0], "mixer": kinds[i % 4][1], "mlp": dense if i % 2 == 0 else moe}
              for i in range(z["layers"])]
    return {"architecture": "Fomunex", "width": w, "vocab": z["vocab"], "max_positions": 4096, "norm": {"eps": 1e-6},
            "logit_scale": 1.0, "logit_softcap": 30.0, "layers": layers}


def _time_fomunex_kernels(z: dict, prompt_len: int, batch: int) -> dict:
    """The design's own kernels alone, microseconds and share of the roofline each.  The two scans
    over one prompt (float32 operations: per token and head four a state element for the time
    mixing, whose output reads the state before and its update after, and four for the state-space
    one) and over ``batch`` single tokens (bytes of state read and written); the mixes, the
    convolution and the polynomial activation (bytes); attention with cap, distance term and
    learned sinks over one prompt from its start (matrix rate over the keys every query sees) and
    over ``batch`` single tokens behind ``prompt_len`` (bytes of keys and values)."""
    import types

    import torch

    from rapid_llm_amd.kernels import ops

    dev, width = "cuda", z["width"]
    bf = torch.bfloat16
    out: dict = {}

    def step(lens):
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
        return types.SimpleNamespace(num_seqs=len(lens), h_seq_lens=list(lens), h_seq_slots=list(range(len(lens))),
                                     cu_seqlens=cu, seq_slots=torch.arange(len(lens), dtype=torch.int32, device=dev))

    # ---- time mixing
    h, d = width // 64, 64
    inner = h * d
    S = torch.zeros((batch + 1, h, d, d), device=dev)
    shift = torch.zeros((batch + 1, width), device=dev)
    for what, lens in (("prefill", [prompt_len]), ("decode", [1] * batch)):
        tokens, ctx = sum(lens), step(lens)
        r, k, v, g = ((torch.randn(tokens, inner, device=dev) * 0.5).to(bf) for _ in range(4))
        pre = torch.randn(tokens, inner, device=dev)
        bias, u, nw = torch.full((inner,), -2.5, device=dev), torch.zeros((h, d), device=dev), torch.ones(inner, device=dev)
        o = torch.empty((tokens, inner), dtype=bf, device=dev)
        sec = _time_calls(lambda: ops.wkv(r, k, v, g, pre, bias, u, nw, o, ctx, S, h, d, 1e-6), what == "decode")
        out[f"time_mixing_scan_{what}_us"] = round(sec * 1e6, 1)
        if what == "prefill":
            out["time_mixing_scan_prefill_frac_fp32_matrix"] = round(
                tokens * h * 4.0 * d * d / sec / (PEAK_TFLOPS["float32"] * 1e12), 4)
        else:
            out["time_mixing_scan_decode_frac_hbm"] = round(2.0 * batch * h * d * d * 4 / sec / 1e9 / HBM_GBPS, 4)
        x = (torch.randn(tokens, width, device=dev)).to(bf)
        mu = torch.rand(5 * width, device=dev)
        mixes, last = torch.empty((4, tokens, width), dtype=bf, device=dev), torch.empty((tokens, width), device=dev)
        sec = _time_calls(lambda: ops.token_shift(x, mu, shift, mixes, last, ctx), what == "decode")
        out[f"token_shift_{what}_us"] = round(sec * 1e6, 1)
        out[f"token_shift_{what}_frac_hbm"] = round(tokens * width * (2 + 4 * 2 + 4) / sec / 1e9 / HBM_GBPS, 4)
    # ---- state-space mixer
    hs, P, N, G, taps = 2 * width // 64, 64, 128, 8, 4
    inner = hs * P
    channels = inner + 2 * G * N
    S2 = torch.zeros((batch + 1, hs, P, N), device=dev)
    conv_state = torch.zeros((batch + 1, taps - 1, channels), device=dev)
    conv_w, conv_b = torch.randn(channels, taps, device=dev) * 0.5, torch.zeros(channels, device=dev)
    for what, lens in (("prefill", [prompt_len]), ("decode", [1] * batch)):
        tokens, ctx = sum(lens), step(lens)
        packed = (torch.randn(tokens, inner + channels, device=dev) * 0.5).to(bf)
        mixed = torch.empty((tokens, channels), device=dev)
        sec = _time_calls(lambda: ops.causal_conv(packed, inner, conv_w, conv_b, conv_state, mixed, ctx), what == "decode")
        out[f"convolution_{what}_us"] = round(sec * 1e6, 1)
        out[f"convolution_{what}_frac_hbm"] = round(tokens * channels * (2 + 4) / sec / 1e9 / HBM_GBPS, 4)
        dt = torch.randn(tokens, hs, device=dev)
        vec = torch.zeros(hs, device=dev)
        y = torch.empty((tokens, inner), device=dev)
        sec = _time_calls(lambda: ops.state_space_scan(mixed, dt, vec - 1.0, vec - 1.0, vec + 1.0, packed, y, ctx, S2,
                                                       hs, P, N, G), what == "decode")
        out[f"state_space_scan_{what}_us"] = round(sec * 1e6, 1)
        if what == "prefill":
            out["state_space_scan_prefill_frac_fp32_matrix"] = round(
                tokens * hs * 4.0 * N * P / sec / (PEAK_TFLOPS["float32"] * 1e12), 4)
        else:
            out["state_space_scan_decode_frac_hbm"] = round(2.0 * batch * hs * N * P * 4 / sec / 1e9 / HBM_GBPS, 4)
        o = torch.empty((tokens, inner), dtype=bf, device=dev)
        sec = _time_calls(lambda: ops.group_rmsnorm(y, torch.ones(inner, device=dev), o, 8, 1e-6), what == "decode")
        out[f"norm_in_parts_{what}_us"] = round(sec * 1e6, 1)
        out[f"norm_in_parts_{what}_frac_hbm"] = round(tokens * inner * (4 + 2) / sec / 1e9 / HBM_GBPS, 4)
    # ---- the polynomial activation over a prompt's hidden rows
    ff = z["ff"] * 3 // 2
    hidden = (torch.randn(prompt_len, ff, device=dev)).to(bf)
    coef = torch.tensor([0.7, 0.2, 0.1, 0.0], device=dev)
    sec = _time_calls(lambda: ops.polynorm(hidden, hidden, coef, 1e-6), False)
    out["polynomial_activation_prefill_us"] = round(sec * 1e6, 1)
    out["polynomial_activation_prefill_frac_hbm"] = round(prompt_len * ff * 4 / sec / 1e9 / HBM_GBPS, 4)
    # ---- attention
    nq, nkv, dh, window, page = z["heads"], z["kv_heads"], z["head_dim"], z["window"], 16
    sink = torch.zeros(nq, device=dev)
    slopes = torch.exp2(-8.0 * torch.arange(1, nq + 1, device=dev, dtype=torch.float32) / nq)

    def attention(seqs, plain):
        tokens = sum(n for _, n in seqs)
        pages_per = [-(-(a + n) // page) for a, n in seqs]
        table = torch.zeros((len(seqs), max(pages_per)), dtype=torch.int32)
        at = 1
        for i, n in enumerate(pages_per):
            table[i, :n] = torch.arange(at, at + n, dtype=torch.int32)
            at += n
        kc = (torch.randn(at, nkv, page, dh, device=dev) * 0.3).to(bf)
        vc = (torch.randn(at, nkv, dh, page, device=dev) * 0.3).to(bf)
        q = (torch.randn(tokens, nq * dh, device=dev) * 0.3).to(bf)
        o = torch.empty((tokens, nq * dh), dtype=bf, device=dev)
        positions = torch.cat([torch.arange(a, a + n) for a, n in seqs]).to(torch.int32).to(dev)
        slot = torch.cat([torch.full((n,), i) for i, (_, n) in enumerate(seqs)]).to(torch.int32).to(dev)
        ctx = types.SimpleNamespace(positions=positions, token_slot=slot, token_ids=positions,
                                    h_seq_starts=[a for a, _ in seqs], h_seq_lens=[n for _, n in seqs],
                                    max_position=max(a + n for a, n in seqs) - 1, extra={}, static={})
        table = table.to(dev)
        more = dict(sink=True) if plain else dict(sink_values=sink, score_cap=50.0, slopes=slopes)
        return _time_calls(lambda: ops.paged_attention(q, kc, vc, o, ctx, table, page, nq, nkv, dh, window,
                                                       dh ** -0.5, **more), max(n for _, n in seqs) == 1)

    seen = sum(min(p + 1, window) for p in range(prompt_len))
    for label, plain in (("", False), ("_without_cap_and_distance", True)):
        sec = attention([(0, prompt_len)], plain)
        out[f"attention_prefill{label}_us"] = round(sec * 1e6, 1)
        out[f"attention_prefill{label}_frac_bf16_matrix"] = round(4.0 * nq * dh * seen / sec / (PEAK_TFLOPS["bfloat16"] * 1e12), 4)
        sec = attention([(prompt_len, 1)] * batch, plain)
        out[f"attention_decode{label}_us"] = round(sec * 1e6, 1)
        out[f"attention_decode{label}_frac_hbm"] = round(
            batch * min(prompt_len + 1, window) * nkv * dh * 2 * 2 / sec / 1e9 / HBM_GBPS, 4)
    return out


# design -> (name, its configuration at a size, its kernels alone, the engine's closest other
# architecture measured beside it and Qwen3)
DESIGNS = {
    "fokulorn": ("Fokulorn", fokulorn_body, _time_kernels, None),
    "sikevik": ("Sikevik", sikevik_body, _time_sikevik_kernels, None),
    "miborax": ("Miborax", miborax_body, _time_miborax_kernels, ("sikevik", sikevik_body)),
    "fomunex": ("Fomunex", fomunex_body, _time_fomunex_kernels, ("fokulorn", fokulorn_body)),
}


def run_design(args) -> int:
    if args.design not in DESIGNS:
        print(f"unknown design {args.design!r}; known: {', '.join(sorted(DESIGNS))}")
        return 2
    title, design_body, design_kernels, closest = DESIGNS[args.design]
    prompt_len = args.prompt_len or 2048
    beside = "Qwen3 of equal width, depth, heads and feed-forward width"
    if closest is not None:
        beside = f"{closest[0]} and " + beside
    out = {"design": title, "beside": beside,
           "dtype": "bf16", "data": "synthetic (uniform random token ids, random N(0,0.02) weights)",
           "prompt_len": prompt_len, "batch": args.batch, "sizes": {}}
    for name in [x for x in args.design_size.split(",") if x]:
        z = DESIGN_SIZES[name]
        row = {"config": z}
        row[args.design] = _time_model(design_body(z), prompt_len, args.batch, args.point_steps, prompt_len + 512)
        print(f"[bench] {name} {args.design} {row[args.design]}", file=sys.stderr, flush=True)
        if closest is not None:
            row[closest[0]] = _time_model(closest[1](z), prompt_len, args.batch, args.point_steps, prompt_len + 512)
            print(f"[bench] {name} {closest[0]} {row[closest[0]]}", file=sys.stderr, flush=True)
        row["qwen3"] = _time_model(qwen3_body(z), prompt_len, args.batch, args.point_steps, prompt_len + 512)
        print(f"[bench] {name} qwen3 {row['qwen3']}", file=sys.stderr, flush=True)
        row["kernels"] = design_kernels(z, prompt_len, args.batch)
        print(f"[bench] {name} kernels {row['kernels']}", file=sys.stderr, flush=True)
        out["sizes"][name] = row
    print(json.dumps(out), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256,
                    help="timed decode steps (BASELINE.json's decode workload: 256 tokens a request)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--shape", default="qwen3-8b", choices=["qwen3-8b", *FAMILY],
                    help="layer sizes: qwen3-8b is BASELINE.json configs[2], the others its family's")
    ap.add_argument("--prompt-len", type=int, default=None, help="tokens of every prompt (default 2,048)")
    ap.add_argument("--context", type=int, default=None, help="longest sequence the engine is sized for")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64", help="other decode batch sizes to measure ('' for none)")
    ap.add_argument("--point-steps", type=int, default=64)
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-pipeline", action="store_true", help="read every step's tokens before queueing the next")
    ap.add_argument("--no-fp32", action="store_true", help="skip the float32 points (a second process)")
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help="run one scheduler workload of BASELINE.json alone and print its own line")
    ap.add_argument("--no-workloads", action="store_true", help="skip the scheduler workloads (processes of their own)")
    ap.add_argument("--peaks", action="store_true",
                    help="measure what the device reaches with library kernels (a large read, copy and square products) and exit")
    ap.add_argument("--design", default=None,
                    help="measure another architecture of the engine beside Qwen3 at equal size (fokulorn, sikevik, miborax, fomunex) and exit")
    ap.add_argument("--design-size", default="2b,8b", help=f"sizes for --design: {', '.join(DESIGN_SIZES)}")
    args = ap.parse_args()
    if args.peaks:
        return measured_peaks()
    if args.design is not None:
        return run_design(args)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU engine")
        return 2
    if args.workload is not None:
        return run_workload(args.workload)

    import torch

    from rapid_llm_amd import EngineConfig, ModelRunner, StepEntry
    from rapid_llm_amd.engine.feed import fed_token
    from rapid_llm_amd.engine.llm import GpuExecutor
    from rapid_llm_amd.engine.scheduler import SamplingPlan
    from rapid_llm_amd.sampling.sampler import RowSampling, Sampler

    shape = load_shape()
    context, prompt_len = shape.pop("context"), shape.pop("prompt_len")
    if args.shape != "qwen3-8b":
        shape.update(FAMILY[args.shape])
    if args.prompt_len is not None:
        prompt_len = args.prompt_len
        context = max(context, prompt_len + 2048)
    if args.context is not None:
        context = args.context
    room = max(args.steps + args.warmup, args.point_steps + max(2, args.warmup // 2)) + 2
    if prompt_len < 1 or prompt_len + room > context:
        print(f"a prompt of {prompt_len} tokens and {room} decoded ones do not fit a context of {context}")
        return 2
    full_layers = shape["num_hidden_layers"]
    if args.layers is not None:
        shape["num_hidden_layers"] = args.layers
    points = [int(p) for p in args.points.split(",") if p]
    elem = 2 if args.dtype == "bfloat16" else 4

    # batch sizes whose caches do not fit beside the weights are left out, and said so: the
    # pool is made for the largest batch that is measured
    from rapid_llm_amd.config.registry import config_from_dict

    _, sized = config_from_dict(shape)
    per_request = (-(-(prompt_len + room) // 16)) * 16 * kv_bytes_per_token(sized, elem)
    free, _ = torch.cuda.mem_get_info()
    most = int((0.92 * free - weight_bytes(sized, elem)) // per_request)
    if args.batch > most:
        print(f"a batch of {args.batch} requests of {prompt_len + room} tokens does not fit this device "
              f"beside the weights ({most} do)")
        return 2
    for b in [b for b in points if b > most]:
        print(f"[bench] batch {b} left out: {most} requests of {prompt_len + room} tokens fit beside the weights",
              file=sys.stderr, flush=True)
    points = [b for b in points if b <= most]
    max_batch = max([args.batch] + points)

    engine = EngineConfig(
        dtype=args.dtype,
        max_seq_len=context,
        page_size=16,
        num_pages=max_batch * (-(-(prompt_len + room) // 16)) + 1,
        max_num_seqs=max_batch,
        max_num_batched_tokens=8192,
        use_graph=not args.no_graph,
        seed=1234,
    )
    t0 = time.time()
    runner = ModelRunner(shape, engine, load_format="random")
    cfg = runner.config
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(7)
    vocab = cfg.vocab_size

    def prompt() -> list[int]:
        return torch.randint(0, vocab, (prompt_len,), generator=gen).tolist()

    def portions(rid: str, toks: list[int]) -> list[StepEntry]:
        """The prompt as the steps that run it: whole if the step's token budget holds it, else
        in portions of that budget; the last one asks for the logits of its last token."""
        budget = engine.max_num_batched_tokens
        cuts = [toks[lo : lo + budget] for lo in range(0, len(toks), budget)]
        return [StepEntry(rid, part, [len(part) - 1] if i == len(cuts) - 1 else []) for i, part in enumerate(cuts)]

    # ---- prefill of one prompt (2,048 tokens unless asked otherwise) ----------
    prefill = None
    if not args.no_prefill:
        times = []
        for i in range(4):
            cuts = portions("p", prompt())
            torch.cuda.synchronize()
            t = time.perf_counter()
            for entry in cuts:
                runner.step([entry])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            runner.finish("p")
        sec = statistics.median(times[1:])
        flops = prefill_flops(cfg, prompt_len)
        prefill = {
            "value": round(prompt_len / sec, 1),
            "tokens": prompt_len,
            "ms": round(sec * 1e3, 3),
            "frac": round(flops / sec / (PEAK_TFLOPS[args.dtype] * 1e12), 4),
        }
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ---- decode ----------------------------------------------------------------
    executor = GpuExecutor(runner, Sampler(runner.device))

    def greedy(rows: int) -> SamplingPlan:
        return SamplingPlan(
            rows=[RowSampling() for _ in range(rows)], logits_rows=list(range(rows)), logprob_ks=[None] * rows
        )

    def decode(batch: int, steps: int, warmup: int) -> tuple[float, float]:
        """Mean seconds per decode step and the mean context length over the timed steps.
        A step is what the engine's loop does for one token of every request: queue the
        forward pass and the choice of the tokens, read the chosen tokens back.  Pipelined
        (the engine's default), the next step is queued, fed from the device, before the
        last one's tokens are read."""
        ids = [f"d{i}" for i in range(batch)]
        tokens = []
        for rid in ids:  # prompts, one request a step
            cuts = portions(rid, prompt())
            for entry in cuts[:-1]:
                executor.execute([entry], greedy(0))
            tokens += executor.execute([cuts[-1]], greedy(1)).token_ids
        plan = greedy(batch)
        fed = [StepEntry(rid, [fed_token(i)], [0]) for i, rid in enumerate(ids)]
        inflight = executor.launch([StepEntry(rid, [tok], [0]) for rid, tok in zip(ids, tokens)], plan)

        def one_step():
            nonlocal inflight
            if args.no_pipeline:
                tokens = inflight.result().token_ids  # the step's one host synchronisation
                inflight = executor.launch([StepEntry(rid, [tok], [0]) for rid, tok in zip(ids, tokens)], plan)
            else:
                queued = executor.launch(fed, plan)
                inflight.result()
                inflight = queued

        for _ in range(warmup):
            one_step()
        inflight.result()
        torch.cuda.synchronize()
        ctx_start = runner.tokens_cached(ids[0]) - 1  # one step is in flight
        t = time.perf_counter()
        for _ in range(steps):
            one_step()
        inflight.result()
        torch.cuda.synchronize()
        sec = (time.perf_counter() - t) / steps
        mean_ctx = ctx_start + (steps - 1) / 2.0 + 1
        for rid in ids:
            runner.finish(rid)
        return sec, mean_ctx

    model_name = "Qwen3-" + args.shape.split("-")[1].upper()
    sec, mean_ctx = decode(args.batch, args.steps, args.warmup)
    step_bytes = weight_bytes(cfg, elem) + args.batch * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / sec / 1e9
    result = {
        "metric": f"{model_name} {'bf16' if args.dtype == 'bfloat16' else 'fp32'} decode tok/s (batch {args.batch}, "
                  f"{prompt_len}-token prompts); prefill tok/s at {prompt_len} tokens",
        "value": round(args.batch / sec, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (uniform random token ids, random N(0,0.02) weights, norm weights 1)",
        "config": {
            "model": f"{model_name} shape",
            "layers": cfg.num_hidden_layers,
            "layers_full": full_layers,
            "hidden": cfg.hidden_size,
            "q_heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate": cfg.intermediate_size,
            "vocab": cfg.vocab_size,
            "rope_theta": cfg.rope_theta,
            "rms_norm_eps": cfg.rms_norm_eps,
            "tied": cfg.tie_word_embeddings,
            "global_batch": args.batch,
            "seq_len": prompt_len,
            "context": context,
            "page_size": engine.page_size,
            "graph": engine.use_graph,
            "pipeline": not args.no_pipeline,
            "parallelism": "single GPU",
        },
        "prefill": prefill,
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_GBPS, 4),
        },
    }
    pts = {}
    for b in points:
        s, _ = decode(b, args.point_steps, max(2, args.warmup // 2))
        pts[f"decode_b{b}"] = round(b / s, 2)
        print(f"[bench] decode batch {b}: {pts[f'decode_b{b}']} tok/s", file=sys.stderr, flush=True)
    if args.dtype == "bfloat16" and not args.no_fp32 and points:
        pts.update(float32_points(args))
    default_run = args.shape == "qwen3-8b" and args.layers is None and args.prompt_len is None and args.context is None
    if args.dtype == "bfloat16" and not args.no_workloads and points and default_run:
        del runner, executor  # the workloads need the device's memory
        torch.cuda.empty_cache()
        pts.update(workload_points(sorted(WORKLOADS)))
    result["points"] = pts
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
