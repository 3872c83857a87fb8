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
SHAPES = {"8B": QWEN3_8B, "14B": QWEN3_14B, "32B": QWEN3_32B}
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


def fill_context(engine, ids, context: int) -> None:
    """Gives each request `context` cached tokens without running them: pages are reserved and
    filled with random keys and values."""
    import torch
    for sid in ids:
        engine.add_request(sid)
        if not engine.cache.reserve(sid, context):
            raise RuntimeError("the cache pool is too small for the benchmark's context")
        engine.cache.commit(sid, context)
    gen = torch.Generator(device=engine.device).manual_seed(1)
    for arr in engine.storage.arrays:
        flat = arr.view(-1)
        step = 1 << 28
        for i in range(0, flat.numel(), step):
            part = flat[i:i + step]
            part.copy_(torch.randn(part.numel(), generator=gen, device=engine.device, dtype=torch.float32)
                       .mul_(0.5).to(arr.dtype))


def time_decode(engine, batch: int, context: int, steps: int, warmup: int, decode_run: int = 8):
    """(seconds for `steps` steps, mean context length during them).  The steps go through the
    serving loop: scheduler, step function, greedy choice on the device."""
    import torch
    from inferrs_amd.engine import GenerationLoop
    from inferrs_amd.engine.scheduler import Request
    from inferrs_amd.sampling import SamplingParams
    start_len = context - steps - warmup
    loop = GenerationLoop(engine, max_batch_size=batch, max_tokens_per_step=max(batch, 16), decode_run=decode_run)
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
    import torch
    from inferrs_amd.engine import Entry
    g = torch.Generator().manual_seed(2)
    prompt = torch.randint(0, vocab, (n_tokens,), generator=g).tolist()
    best = None
    for r in range(runs + 1):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([Entry("p", prompt, [n_tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.end_request("p")
        if r > 0:
            best = dt if best is None else min(best, dt)
    return best


WORKLOADS = {
    # name: (shape, requests, shortest prompt, longest prompt, portion, decode tokens)
    "mixed16": ("14B", 16, 128, 4096, 512, 128),
    "concurrent32": ("32B", 32, 1024, 1024, 1024, 256),
}


def run_workload(engine, lengths, portion: int, decode_tokens: int, budget: int, vocab: int, seed: int):
    """All requests arrive at once and run to their last token.  Returns (seconds, seconds to each
    request's first token, loop steps, seconds until the last prompt was through)."""
    import torch
    from inferrs_amd.engine import GenerationLoop
    from inferrs_amd.sampling import SamplingParams
    loop = GenerationLoop(engine, max_batch_size=len(lengths), max_tokens_per_step=budget, prefill_chunk=portion)
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
    run_workload(engine, lengths, portion, min(decode_tokens, 16), budget, raw["vocab_size"], seed=1)      # warm-up
    runs = [run_workload(engine, lengths, portion, decode_tokens, budget, raw["vocab_size"], seed=2 + i)
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
                   "portion": portion, "tokens_per_step": budget, "decode_tokens": decode_tokens, "kv_page_size": PAGE},
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
    ap.add_argument("--prefill-only", action="store_true", help="time the prefill alone (for profiles)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS, help="length of the prompt of the prefill")
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
    note(f"decode at batch {args.batch}, context {args.context}: {args.warmup} + {args.steps} steps")

    if args.prefill_only:
        t = time_prefill(engine, args.prefill_tokens, max(1, args.steps), raw["vocab_size"])
        print(json.dumps({"prefill": {"value": round(args.prefill_tokens / t, 1), "tokens": args.prefill_tokens,
                                      "ms": round(t * 1e3, 3),
                                      "frac": round(prefill_flops(raw, args.prefill_tokens) / t / PEAK_FLOPS[dtype_key], 4)}}))
        return 0
    elapsed, mean_ctx = time_decode(engine, args.batch, args.context, args.steps, args.warmup, args.decode_run)
    ms_per_step = elapsed / args.steps * 1e3
    value = args.batch * args.steps / elapsed
    nbytes = decode_bytes(raw, args.batch, mean_ctx, esize)
    achieved = nbytes / (elapsed / args.steps) / 1e9

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
    }
    if not args.no_points:
        points = {}
        for b in points_batches:
            steps = max(8, args.steps // 2)
            note(f"decode at batch {b}: {steps} steps")
            el, _ = time_decode(engine, b, args.context, steps, min(args.warmup, 4), args.decode_run)
            points[f"decode_b{b}"] = round(b * steps / el, 2)
        record["points"] = points
        note(f"prefill of {args.prefill_tokens} tokens")
        t = time_prefill(engine, args.prefill_tokens, 3, raw["vocab_size"])
        flops = prefill_flops(raw, args.prefill_tokens)
        record["prefill"] = {"value": round(args.prefill_tokens / t, 1), "tokens": args.prefill_tokens,
                             "ms": round(t * 1e3, 3), "frac": round(flops / t / PEAK_FLOPS[dtype_key], 4)}
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
