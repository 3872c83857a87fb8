#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, Qwen3-8B layer sizes, bfloat16,
random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 8192] [--shape 8B|14B|32B] [--layers L]

A step is one decode step of the whole batch: the step function over one token per request,
greedy choice of the next token on the device, and feeding it back.  The requests' caches are
brought to the benchmark's context length by filling their pages with random keys and values
(decode time does not depend on their content); the prefill figure is measured separately
on a 2,048-token prompt through the same step function.  One JSON line is printed.

    python bench.py --workload mixed16|concurrent32 [--shape ...] [--decode-tokens T]

runs requests through the serving loop instead (scheduler, prompt portions beside decode tokens, greedy
choice): `mixed16` is 16 requests with prompts of 128 to 4,096 random tokens in portions of 512 at the
14B shape, `concurrent32` 32 requests of 1,024 prompt tokens at the 32B shape; every request decodes
`--decode-tokens` tokens.  Its JSON line gives tokens a second over the whole run, the prompts' and the
decoded tokens' rates apart, and the time to a request's first token.

The reference measures the same quantities with `inferrs bench` (`inferrs/src/bench.rs:40-224`,
`Engine::bench_generate`, `inferrs/src/engine.rs:2557-2641`): synthetic prompt, stop tokens
ignored, device-synchronised wall time.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

# Qwen3-8B as its config.json gives it.
QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=151936,
                hidden_size=4096, intermediate_size=12288, num_hidden_layers=36,
                num_attention_heads=32, num_key_value_heads=8, head_dim=128, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960)
# The larger dense models of the family differ in these sizes only.
QWEN3_14B = dict(QWEN3_8B, hidden_size=5120, intermediate_size=17408, num_hidden_layers=40, num_attention_heads=40)
QWEN3_32B = dict(QWEN3_8B, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64)
# The smallest shape is the one that the reference's defaults describe (`inferrs/src/config.rs:468-502`: width 1,024, 28 layers,
# 16 query and 8 key/value heads, feed-forward 3,072, tied embeddings); two more small ones between it and the 8B shape.
QWEN3_0_6B = dict(QWEN3_8B, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16,
                  tie_word_embeddings=True)
QWEN3_1_7B = dict(QWEN3_0_6B, hidden_size=2048, intermediate_size=6144)
QWEN3_4B = dict(QWEN3_0_6B, hidden_size=2560, intermediate_size=9728, num_hidden_layers=36, num_attention_heads=32)
SHAPES = {"0.6B": QWEN3_0_6B, "1.7B": QWEN3_1_7B, "4B": QWEN3_4B, "8B": QWEN3_8B, "14B": QWEN3_14B, "32B": QWEN3_32B}
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PREFILL_TOKENS = 2048
PAGE = 16


def matmul_params(c) -> int:
    """Weights of one layer's matrix products."""
    h, d = c["hidden_size"], c["head_dim"]
    qkv = (c["num_attention_heads"] + 2 * c["num_key_value_heads"]) * d * h
    return qkv + c["num_attention_heads"] * d * h + 3 * h * c["intermediate_size"]


def prefill_flops(c, t: int, rows_of_logits: int = 1) -> float:
    linear = 2.0 * t * matmul_params(c) * c["num_hidden_layers"]
    # causal scores and weighted values: 2 products of t(t+1)/2 x head_dim per query head
    attn = 4.0 * (t * (t + 1) / 2) * c["head_dim"] * c["num_attention_heads"] * c["num_hidden_layers"]
    return linear + attn + 2.0 * rows_of_logits * c["vocab_size"] * c["hidden_size"]


def decode_bytes(c, batch: int, context: float, esize: int = 2) -> float:
    """What one decode step has to read: every weight it uses once, and the cache of the live requests."""
    weights = (matmul_params(c) + 2 * c["hidden_size"] + 2 * c["head_dim"]) * c["num_hidden_layers"]
    weights += c["vocab_size"] * c["hidden_size"] + c["hidden_size"]          # logits head, final norm
    kv = 2 * c["num_key_value_heads"] * c["head_dim"] * c["num_hidden_layers"] * context * batch
    return float(weights * esize + kv * esize + batch * c["hidden_size"] * esize)


def fill_storage(engine) -> None:
    """Random keys and values in every page of the cache (decode time does not depend on their content)."""
    import torch
    gen = torch.Generator(device=engine.device).manual_seed(1)
    for arr in engine.storage.arrays:
        flat = arr.view(-1)
        step = 1 << 28
        for i in range(0, flat.numel(), step):
            part = flat[i:i + step]
            part.copy_(torch.randn(part.numel(), generator=gen, device=engine.device, dtype=torch.float32)
                       .mul_(0.5).to(arr.dtype))


def fill_context(engine, ids, context: int) -> None:
    """Gives each request `context` cached tokens without running them: pages are reserved (they hold the
    random keys and values of `fill_storage`)."""
    for sid in ids:
        engine.add_request(sid)
        if not engine.cache.reserve(sid, context):
            raise RuntimeError("the cache pool is too small for the benchmark's context")
        engine.cache.commit(sid, context)


def time_decode(engine, batch: int, context: int, steps: int, warmup: int, decode_run: int = 8, sampled: bool = False):
    """(seconds for `steps` steps, mean context length during them).  The steps go through the
    serving loop: scheduler, step function, greedy choice on the device; with `sampled` the choice is a draw
    with the reference's default parameters (temperature 0.7, top_k 50, top_p 0.9, repetition penalty 1.1
    over 64 tokens: `inferrs/src/main.rs:144-154`, `inferrs/src/sampler.rs:96-97`) and a fixed seed."""
    import torch
    from inferrs_amd.engine import GenerationLoop
    from inferrs_amd.engine.scheduler import Request
    from inferrs_amd.sampling import SamplingParams
    start_len = context - steps - warmup
    loop = GenerationLoop(engine, max_batch_size=batch, max_tokens_per_step=max(batch, 16), decode_run=decode_run)
    if sampled:
        params = SamplingParams(max_tokens=steps + warmup + 8, bypass_stop_tokens=True, seed=7)
    else:
        params = SamplingParams.greedy(max_tokens=steps + warmup + 8, bypass_stop_tokens=True)
    ids = [f"d{i}" for i in range(batch)]
    # the requests enter as if their contexts had been run: random keys and values, and one generated token
    fill_context(engine, ids, start_len)
    for i, sid in enumerate(ids):
        loop.scheduler.adopt(Request(sid, [1] * start_len, params, output=[1 + i]))
    done_steps = 0
    while done_steps < warmup:
        loop.step(max_steps=warmup - done_steps)
        done_steps = loop.steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while loop.steps < warmup + steps:
        loop.step(max_steps=warmup + steps - loop.steps)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    for sid in ids:
        if engine.has_request(sid):
            engine.end_request(sid)
    return elapsed, start_len + warmup + (steps - 1) / 2.0


def time_prefill(engine, n_tokens: int, runs: int, vocab: int):
    """Seconds of each of `runs` prefills of one prompt of `n_tokens` tokens, after three that are not counted: a shape's
    first steps run eagerly and, where the host is their bound, the third is captured into a graph (prompts of up to
    `Engine.GRAPH_MAX_TOKENS` tokens), so the counted runs are what a repeated shape settles at (the reference's own
    bench counts five runs after one warm-up, `inferrs/src/bench.rs:27-33`)."""
    import torch
    from inferrs_amd.engine import Entry
    g = torch.Generator().manual_seed(2)
    prompt = torch.randint(0, vocab, (n_tokens,), generator=g).tolist()
    times = []
    for r in range(runs + 3):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([Entry("p", prompt, [n_tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.end_request("p")
        if r > 2:
            times.append(dt)
    return times


def mean_std(values):
    m = sum(values) / len(values)
    var = sum((v - m) ** 2 for v in values) / max(len(values) - 1, 1)
    return m, var ** 0.5


def measured_roofs(engine):
    """(GB/s of a pure streaming read over at least 4 GB, TFLOP/s of a large bfloat16 product through the vendor's
    GEMM): what this GPU gives in practice, beside the published peaks."""
    import torch
    from inferrs_amd import ops
    src = max(engine.storage.arrays, key=lambda a: a.numel() * a.element_size()).view(-1)
    want = 8 << 30
    n = min(src.numel(), want // src.element_size()) // 64 * 64
    if n * src.element_size() < (4 << 30):                  # a small cache: a buffer of its own
        src = torch.empty(4 << 30, dtype=torch.uint8, device=engine.device).random_(0, 255)
        n = src.numel()
    part = src[:n]
    best = None
    for blocks in (8192, 16384, 65536):
        for _ in range(3):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            ops.stream_read(part, blocks)
            b.record()
            torch.cuda.synchronize()
            gbs = n * part.element_size() / (a.elapsed_time(b) * 1e-3) / 1e9
            best = gbs if best is None else max(best, gbs)
    m = 8192
    x = torch.randn(m, m, device=engine.device, dtype=torch.bfloat16)
    w = torch.randn(m, m, device=engine.device, dtype=torch.bfloat16)
    torch.nn.functional.linear(x, w)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(10):
        torch.nn.functional.linear(x, w)
    b.record()
    torch.cuda.synchronize()
    tflops = 10 * 2.0 * m ** 3 / (a.elapsed_time(b) * 1e-3) / 1e12
    return best, tflops


def kernel_breakdown(engine, batch: int, context: int, prefill_tokens: int, vocab: int):
    """Microseconds by kernel entry point for one decode step (batch, context) and one prefill, each kernel call
    bracketed by events (eager steps, no graph; an event pair adds a few microseconds to a short kernel)."""
    import torch
    from inferrs_amd import ops
    from inferrs_amd.engine import Entry
    out = {}
    ids = [f"k{i}" for i in range(batch)]
    fill_context(engine, ids, context - 4)
    graphs, engine.use_graphs = engine.use_graphs, False
    try:
        entries = [Entry(sid, [1 + i], [0]) for i, sid in enumerate(ids)]
        engine.step(entries)                                   # once without the timer
        with ops.KernelTimer() as timer:
            engine.step(entries)
        out["decode"] = timer.summary()
        for sid in ids:
            engine.end_request(sid)
        g = torch.Generator().manual_seed(3)
        prompt = torch.randint(0, vocab, (prefill_tokens,), generator=g).tolist()
        engine.step([Entry("kp", prompt, [prefill_tokens - 1])])
        engine.end_request("kp")
        with ops.KernelTimer() as timer:
            engine.step([Entry("kp", prompt, [prefill_tokens - 1])])
        out["prefill"] = timer.summary()
        engine.end_request("kp")
    finally:
        engine.use_graphs = graphs
    return {phase: {name: {"calls": calls, "us": round(us, 1)} for name, (calls, us) in sorted(table.items(), key=lambda kv: -kv[1][1])}
            for phase, table in out.items()}


def host_gap(engine, entries_of, repeats: int = 3):
    """One eager step as the host sees it: (wall milliseconds from the call to the synchronised end, milliseconds of
    the same step's kernels replayed from a captured graph, kernel calls of the step).  What is between the two is the
    host: Python between the kernel calls, where the GPU waits for the next launch.  `entries_of()` sets the step's
    requests up and returns (entries, clean-up)."""
    import torch
    from inferrs_amd import ops
    graphs, engine.use_graphs = engine.use_graphs, False
    try:
        walls = []
        for _ in range(repeats + 1):
            entries, cleanup = entries_of()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.step(entries)
            torch.cuda.synchronize()
            walls.append(time.perf_counter() - t0)
            cleanup()
        # the same step's kernels without the host between them: captured once, replayed
        entries, cleanup = entries_of()
        for e in entries:
            if not engine.has_request(e.seq_id):
                engine.add_request(e.seq_id)
        if not engine.cache.ensure_reserved([(e.seq_id, len(e.tokens)) for e in entries]):
            raise RuntimeError("the cache pool is too small for this step")
        ctx = engine.builder.build([(e.seq_id, e.tokens, e.want) for e in entries])
        with ops.KernelTimer() as timer:
            engine.model.forward(ctx, engine.storage)
        n_calls = sum(calls for calls, _us in timer.summary().values())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            engine.model.forward(ctx, engine.storage)
        replays = []
        for _ in range(repeats + 1):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            torch.cuda.synchronize()
            replays.append(a.elapsed_time(b))
        del graph
        cleanup()
    finally:
        engine.use_graphs = graphs
    return min(walls[1:]) * 1e3, min(replays[1:]), n_calls


WORKLOADS = {
    # name: (shape, requests, shortest prompt, longest prompt, portion, decode tokens)
    "mixed16": ("14B", 16, 128, 4096, 512, 128),
    "concurrent32": ("32B", 32, 1024, 1024, 1024, 256),
}


def run_workload(engine, lengths, portion: int, decode_tokens: int, budget: int, vocab: int, seed: int, row_multiple: int = 256):
    """All requests arrive at once and run to their last token.  Returns (seconds, seconds to each
    request's first token, loop steps, seconds until the last prompt was through)."""
    import torch
    from inferrs_amd.engine import GenerationLoop
    from inferrs_amd.sampling import SamplingParams
    loop = GenerationLoop(engine, max_batch_size=len(lengths), max_tokens_per_step=budget, prefill_chunk=portion,
                          row_multiple=row_multiple)
    g = torch.Generator().manual_seed(seed)
    params = SamplingParams.greedy(max_tokens=decode_tokens, bypass_stop_tokens=True)
    requests = [loop.add(torch.randint(0, vocab, (n,), generator=g).tolist(), params) for n in lengths]
    first = {}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while loop.scheduler.has_work():
        loop.step()
        now = time.perf_counter() - t0          # (a step's tokens are on the host when it returns)
        for r in requests:
            if r.output and r.request_id not in first:
                first[r.request_id] = now
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    if any(len(r.output) != decode_tokens for r in requests):
        raise RuntimeError("a request ended early")
    return elapsed, [first[r.request_id] for r in requests], loop.steps, max(first.values())


def workload_main(args, raw, engine_factory) -> int:
    import random
    _, n_req, lo, hi, portion, _ = WORKLOADS[args.workload]
    rnd = random.Random(0)
    lengths = [rnd.randint(lo, hi) for _ in range(n_req)]
    decode_tokens = args.decode_tokens
    budget = max(2048, portion)
    pages = sum(-(-(n + decode_tokens + 1) // PAGE) + 1 for n in lengths) + 8
    note(f"{args.workload}: {n_req} requests, {sum(lengths)} prompt tokens, {decode_tokens} decoded tokens each")
    engine = engine_factory(pages, n_req + 1)
    run_workload(engine, lengths, portion, min(decode_tokens, 16), budget, raw["vocab_size"], seed=1, row_multiple=args.row_multiple)      # warm-up
    runs = [run_workload(engine, lengths, portion, decode_tokens, budget, raw["vocab_size"], seed=2 + i, row_multiple=args.row_multiple)
            for i in range(max(1, args.steps if args.steps < 16 else 3))]
    elapsed, firsts, steps, prompts_done = min(runs, key=lambda r: r[0])
    p_tok, d_tok = sum(lengths), n_req * decode_tokens
    print(json.dumps({
        "metric": f"tokens/s of the serving loop, workload {args.workload} (Qwen3-{args.shape})",
        "value": round((p_tok + d_tok) / elapsed, 1), "unit": "tok/s", "n_gpus": 1, "runs": len(runs),
        "seconds": round(elapsed, 4), "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random-init weights, uniform-random token ids, stop tokens ignored",
        "config": {"model": f"Qwen3-{args.shape} shape", "layers": args.layers, "requests": n_req,
                   "prompt_tokens": p_tok, "shortest_prompt": min(lengths), "longest_prompt": max(lengths),
                   "portion": portion, "tokens_per_step": budget, "decode_tokens": decode_tokens, "kv_page_size": PAGE,
                   "row_multiple": args.row_multiple},
        "loop_steps": steps,
        "first_token_s": {"mean": round(sum(firsts) / len(firsts), 4), "max": round(max(firsts), 4)},
        # until the last request has its first token the steps are mostly prompt portions, after it only decode steps
        "prompt_phase": {"seconds": round(prompts_done, 4), "prompt_tok_s": round(p_tok / prompts_done, 1)},
        "decode_phase": {"seconds": round(elapsed - prompts_done, 4),
                         "tok_s": round(n_req * (decode_tokens - 1) / max(elapsed - prompts_done, 1e-9), 1)},
    }))
    return 0


def note(msg: str) -> None:
    """Progress goes to stderr; the one JSON line is all that stdout carries."""
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--shape", default=None, choices=sorted(SHAPES), help="layer sizes of this Qwen3 model (8B)")
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help="run requests through the serving loop instead of timing decode steps")
    ap.add_argument("--decode-tokens", type=int, default=None, help="tokens every request of a workload decodes")
    ap.add_argument("--layers", type=int, default=None,
                    help="run fewer layers than the model has (recorded in the config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    ap.add_argument("--sampled", action="store_true",
                    help="the timed steps draw with the reference's default sampling parameters instead of the arg max (for profiles)")
    ap.add_argument("--prefill-only", action="store_true", help="time the prefill alone (for profiles)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS, help="length of the prompt of the prefill")
    ap.add_argument("--runs", type=int, default=5, help="times the decode steps and the prefill are measured (mean and deviation)")
    ap.add_argument("--no-extra-points", dest="extra_points", action="store_false",
                    help="only batch 1 and 64 and the prefill beside the headline (no further batches and contexts, "
                         "no per-kernel times, no 32-bit path)")
    ap.add_argument("--row-multiple", type=int, default=256,
                    help="workloads: cut prompt portions so that a step's tokens are a multiple of this (0: off)")
    ap.add_argument("--decode-run", type=int, default=8,
                    help="decode steps that the serving loop queues on the GPU at once (1: one at a time)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from inferrs_amd.config import Qwen3Config
    from inferrs_amd.engine import Engine

    if args.shape is None:
        args.shape = WORKLOADS[args.workload][0] if args.workload else "8B"
    full_layers = SHAPES[args.shape]["num_hidden_layers"]
    if args.layers is None:
        args.layers = full_layers
    raw = dict(SHAPES[args.shape], num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    dtype_key = "bf16" if args.dtype == "bfloat16" else "fp32"
    esize = 2 if args.dtype == "bfloat16" else 4
    if args.workload:
        if args.decode_tokens is None:
            args.decode_tokens = WORKLOADS[args.workload][5]
        note(f"random weights of {args.layers} layers")
        return workload_main(args, raw, lambda pages, seqs: Engine.from_random(
            config, seed=0, dtype=args.dtype, page_size=PAGE, num_pages=pages, max_seqs=seqs))
    points_batches = [] if args.no_points or args.prefill_only else [1, 64]
    # a point whose cache would not fit beside the weights is left out (batch 64 at a context of 32 k and more)
    per_token = 2 * raw["num_key_value_heads"] * raw["head_dim"] * args.layers * esize
    weights = (matmul_params(raw) * args.layers + 2 * raw["vocab_size"] * raw["hidden_size"]) * esize
    room = 0.9 * torch.cuda.get_device_properties(0).total_memory - weights
    for b in list(points_batches):
        if b * (args.context + PAGE) * per_token > room:
            note(f"batch {b} at context {args.context} does not fit this GPU's memory: point left out")
            points_batches.remove(b)
    biggest = max([args.batch] + points_batches)
    num_pages = biggest * (-(-args.context // PAGE) + 1) + 8
    note(f"random weights of {args.layers} layers and a cache of {num_pages} pages")
    engine = Engine.from_random(config, seed=0, dtype=args.dtype, page_size=PAGE, num_pages=num_pages,
                                max_seqs=biggest + 1)
    fill_storage(engine)
    vocab = raw["vocab_size"]

    def prefill_record(tokens: int, runs: int, roof_tflops=None):
        times = time_prefill(engine, tokens, runs, vocab)
        mean, std = mean_std(times)
        flops = prefill_flops(raw, tokens)
        rec = {"value": round(tokens / mean, 1), "tokens": tokens, "ms": round(mean * 1e3, 3),
               "frac": round(flops / mean / PEAK_FLOPS[dtype_key], 4), "runs": len(times),
               "ms_std": round(std * 1e3, 3), "ms_best": round(min(times) * 1e3, 3)}
        if roof_tflops:
            rec["measured_peak_tflops"] = round(roof_tflops, 1)
            rec["frac_of_measured"] = round(flops / mean / (roof_tflops * 1e12), 4)
        return rec

    if args.prefill_only:
        print(json.dumps({"prefill": prefill_record(args.prefill_tokens, max(1, args.steps))}))
        return 0
    note(f"decode at batch {args.batch}, context {args.context}: {args.warmup} + {args.steps} steps, {args.runs} times")
    elapsed, mean_ctx = time_decode(engine, args.batch, args.context, args.steps, args.warmup, args.decode_run, args.sampled)
    ms_per_step = elapsed / args.steps * 1e3
    value = args.batch * args.steps / elapsed
    nbytes = decode_bytes(raw, args.batch, mean_ctx, esize)
    achieved = nbytes / (elapsed / args.steps) / 1e9
    # the same K steps again, for the spread (the reference's bench: warm-up, then runs, mean and standard
    # deviation, inferrs/src/bench.rs:159-173,226-248); the headline stays the first K steps
    repeats = [ms_per_step] + [time_decode(engine, args.batch, args.context, args.steps, args.warmup, args.decode_run, args.sampled)[0]
                               / args.steps * 1e3 for _ in range(max(0, args.runs - 1))]
    rep_mean, rep_std = mean_std(repeats)

    record = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} (Qwen3-{args.shape})", "value": round(value, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype_key,
        "data": "synthetic: random-init weights, uniform-random token ids, cache pages of the context "
                "filled with random keys and values",
        "config": {
            "model": f"Qwen3-{args.shape} shape", "global_batch": args.batch, "seq_len": args.context,
            "parallelism": "single GPU", "layers": args.layers, "layers_of_model": full_layers,
            "hidden_size": raw["hidden_size"], "intermediate_size": raw["intermediate_size"],
            "num_attention_heads": raw["num_attention_heads"], "num_key_value_heads": raw["num_key_value_heads"],
            "head_dim": raw["head_dim"], "vocab_size": raw["vocab_size"], "rope_theta": raw["rope_theta"],
            "rms_norm_eps": raw["rms_norm_eps"], "tie_word_embeddings": raw["tie_word_embeddings"],
            "kv_page_size": PAGE, "prefill_tokens": args.prefill_tokens,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "decode_runs": {"runs": len(repeats), "ms_per_step_mean": round(rep_mean, 4), "ms_per_step_std": round(rep_std, 4),
                        "tok_s_mean": round(args.batch / rep_mean * 1e3, 2)},
    }
    if not args.no_points:
        note("measured roofs: a streaming read and a large bfloat16 product")
        read_gbs, gemm_tflops = measured_roofs(engine)
        record["roofline"]["measured_peak"] = round(read_gbs, 1)
        record["roofline"]["frac_of_measured"] = round(achieved / read_gbs, 4)
        points = {}

        def decode_point(name: str, b: int, context: int, sampled: bool = False):
            steps = max(8, args.steps // 2)
            note(f"decode at batch {b}, context {context}: {steps} steps" + (", default sampling parameters" if sampled else ""))
            el, ctx_mean = time_decode(engine, b, context, steps, min(args.warmup, 4), args.decode_run, sampled)
            points[name] = round(b * steps / el, 2)
            fractions[name] = round(decode_bytes(raw, b, ctx_mean, esize) / (el / steps) / 1e9 / PEAK_HBM_GBS, 4)

        fractions = {}
        for b in points_batches:
            decode_point(f"decode_b{b}", b, args.context)
        if args.extra_points:
            for b in (16, 32):
                if b <= biggest:
                    decode_point(f"decode_b{b}", b, args.context)
            long_ctx = 4 * args.context
            if args.batch * (long_ctx // PAGE + 1) + 8 <= num_pages and long_ctx <= raw["max_position_embeddings"]:
                decode_point(f"decode_b{args.batch}_ctx{long_ctx}", args.batch, long_ctx)
        record["points"] = points
        record["points_hbm_frac"] = fractions
        note(f"prefill of {args.prefill_tokens} tokens")
        record["prefill"] = prefill_record(args.prefill_tokens, args.runs, gemm_tflops)
        # the time to a request's first token through the serving loop (scheduler, step, choice, copy to the host)
        from inferrs_amd.engine import GenerationLoop
        from inferrs_amd.sampling import SamplingParams
        g = torch.Generator().manual_seed(4)
        prompt = torch.randint(0, vocab, (args.prefill_tokens,), generator=g).tolist()
        firsts = []
        for _ in range(3):
            loop = GenerationLoop(engine, max_batch_size=1, max_tokens_per_step=args.prefill_tokens)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            loop.add(prompt, SamplingParams.greedy(max_tokens=1, bypass_stop_tokens=True))
            loop.run()
            firsts.append(time.perf_counter() - t0)
        record["prefill"]["first_token_ms"] = round(min(firsts) * 1e3, 3)
        if args.extra_points:
            # shorter contexts and prompts, where a step is short and the host's share of it largest: the reference's
            # own bench times a prompt of 128 tokens (inferrs/src/bench.rs:35-37)
            for context in (512, 2048):
                if context < args.context:
                    for b in sorted(set([1, args.batch] + ([64] if 64 in points_batches else []))):
                        decode_point(f"decode_b{b}_ctx{context}", b, context)
            # the same steps when every request draws with the reference's default parameters instead of the arg max
            if 2048 < args.context:
                decode_point(f"decode_b{args.batch}_ctx2048_sampled", args.batch, 2048, sampled=True)
            for tokens in (128, 512):
                if tokens < args.prefill_tokens:
                    rec = prefill_record(tokens, 3)
                    points[f"prefill_{tokens}"] = rec["value"]
                    fractions[f"prefill_{tokens}_mfma"] = rec["frac"]
            # eager steps as the host sees them: wall time against the sum of the kernels' own times
            from inferrs_amd.engine import Entry
            note("eager steps: wall time against the kernels' times")
            gp = torch.Generator().manual_seed(5)
            portion = torch.randint(0, vocab, (512,), generator=gp).tolist()
            mixed_context = min(2048, args.context)

            def mixed_step():
                ids = [f"m{i}" for i in range(args.batch)]
                fill_context(engine, ids, mixed_context - 1)
                def cleanup():
                    for sid in ids + ["mp"]:
                        if engine.has_request(sid):
                            engine.end_request(sid)
                return [Entry(sid, [1 + i], [0]) for i, sid in enumerate(ids)] + [Entry("mp", portion, [511])], cleanup

            def short_prompt(tokens):
                def setup():
                    return [Entry("hp", portion[:tokens], [tokens - 1])], lambda: engine.end_request("hp")
                return setup

            host = {}
            for name, setup in ((f"mixed_{args.batch}_decodes_and_512", mixed_step), ("prefill_128", short_prompt(128)),
                                ("prefill_512", short_prompt(512))):
                wall, kernels, calls = host_gap(engine, setup)
                host[name] = {"wall_ms": round(wall, 3), "graph_ms": round(kernels, 3), "kernel_calls": calls,
                              "host_frac": round(max(0.0, 1.0 - kernels / wall), 4)}
            record["eager_steps"] = host
            long_prompt = 4 * args.prefill_tokens
            note(f"prefill of {long_prompt} tokens")
            rec = prefill_record(long_prompt, 3)
            points[f"prefill_{long_prompt}"] = rec["value"]
            fractions[f"prefill_{long_prompt}_mfma"] = rec["frac"]
            note("per-kernel times of one decode step and one prefill")
            record["kernels"] = kernel_breakdown(engine, args.batch, args.context, args.prefill_tokens, vocab)
            # the true 32-bit path at the same layer sizes, four layers of them
            if args.dtype == "bfloat16":
                f32_layers = min(4, args.layers)
                note(f"the 32-bit path: {f32_layers} layers")
                del loop
                raw32 = dict(raw, num_hidden_layers=f32_layers)
                eng32 = Engine.from_random(Qwen3Config.from_dict(raw32), seed=0, dtype="float32", page_size=PAGE,
                                           num_pages=max(args.batch * (-(-args.context // PAGE) + 1),
                                                         -(-args.prefill_tokens // PAGE)) + 8, max_seqs=args.batch + 1)
                fill_storage(eng32)
                el, ctx_mean = time_decode(eng32, args.batch, args.context, 8, 3, args.decode_run)
                points[f"f32_decode_b{args.batch}_layers{f32_layers}"] = round(args.batch * 8 / el, 2)
                fractions[f"f32_decode_b{args.batch}_layers{f32_layers}"] = round(
                    decode_bytes(raw32, args.batch, ctx_mean, 4) / (el / 8) / 1e9 / PEAK_HBM_GBS, 4)
                times = time_prefill(eng32, args.prefill_tokens, 2, vocab)
                points[f"f32_prefill_{args.prefill_tokens}_layers{f32_layers}"] = round(args.prefill_tokens / min(times), 1)
                fractions[f"f32_prefill_{args.prefill_tokens}_layers{f32_layers}_fma"] = round(
                    prefill_flops(raw32, args.prefill_tokens) / min(times) / PEAK_FLOPS["fp32"], 4)
                del eng32
            # the smallest shape of the family, all its layers (the model that the reference's command line names as its
            # example, inferrs/src/run.rs:35): steps so short that the kernels' fixed costs and, in eager steps, the host set the pace; prompts of
            # a repeated length run from captured graphs there
            if args.dtype == "bfloat16" and args.shape != "0.6B":
                small = SHAPES["0.6B"]
                note("the 0.6B shape: decode at batch 1 and 8 at a context of 2,048, prompts of 128 and 512 tokens")
                eng_s = Engine.from_random(Qwen3Config.from_dict(small), seed=0, dtype="bfloat16", page_size=PAGE,
                                           num_pages=8 * (2048 // PAGE + 2) + 8, max_seqs=9)
                fill_storage(eng_s)
                for b in (1, 8):
                    el, ctx_mean = time_decode(eng_s, b, 2048, 16, 4, args.decode_run)
                    points[f"shape0.6B_decode_b{b}_ctx2048"] = round(b * 16 / el, 2)
                    fractions[f"shape0.6B_decode_b{b}_ctx2048"] = round(decode_bytes(small, b, ctx_mean, 2) / (el / 16) / 1e9 / PEAK_HBM_GBS, 4)
                for tokens in (128, 512):
                    times = time_prefill(eng_s, tokens, 3, small["vocab_size"])
                    points[f"shape0.6B_prefill_{tokens}"] = round(tokens / (sum(times) / len(times)), 1)
                    fractions[f"shape0.6B_prefill_{tokens}_mfma"] = round(
                        prefill_flops(small, tokens) / (sum(times) / len(times)) / PEAK_FLOPS["bf16"], 4)
                del eng_s
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
