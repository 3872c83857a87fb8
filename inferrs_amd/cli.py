"""Command line in the reference's manner: `run MODEL [PROMPT]` generates, `bench MODEL` times
prefill and decode.  Option names, defaults and meanings are the reference's where it has them
(`inferrs/src/main.rs:91-204`, `inferrs/src/run.rs:33-146`, `inferrs/src/bench.rs:22-38`).
MODEL is a folder with config.json and safetensors weights (`inferrs/src/hub.rs:94-101`: an
existing path is loaded locally; nothing is downloaded here).  Servers are not part of this
engine: `serve` says so and exits.

A prompt is text when the folder holds a tokenizer.json, else token ids separated by commas or
blanks; `--random-weights` draws seeded random weights for MODEL's config.json instead of
reading its safetensors.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from typing import List, Optional

from . import __version__


def _add_engine_options(p: argparse.ArgumentParser) -> None:
    p.add_argument("model", help="folder with config.json and safetensors weights")
    p.add_argument("--dtype", default="bf16", choices=["f32", "bf16", "float32", "bfloat16"],
                   help="weight and compute data type (f16 is not built)")
    p.add_argument("--max-seq-len", type=int, default=0, help="maximum sequence length (0 = model default)")
    p.add_argument("--device", default="auto", choices=["auto", "hip", "cuda"],
                   help="the one AMD GPU (there is no CPU path)")
    p.add_argument("--block-size", type=int, default=16, help="KV cache block size in tokens")
    p.add_argument("--initial-blocks", type=int, default=16,
                   help="initial KV cache blocks (the pool is allocated whole at the start: it never has fewer than this)")
    p.add_argument("--max-blocks", type=int, default=0, help="KV cache blocks (0 = from --paged-attention)")
    p.add_argument("--max-batch-size", type=int, default=32, help="maximum concurrent sequences")
    p.add_argument("--max-tokens-per-step", type=int, default=2048, help="token budget per scheduler step")
    p.add_argument("--paged-attention", type=float, default=0.9, metavar="FRACTION",
                   help="fraction of free GPU memory for KV blocks when --max-blocks is 0")
    p.add_argument("--temperature", type=float, default=0.7)
    p.add_argument("--top-p", type=float, default=0.9)
    p.add_argument("--top-k", type=int, default=50)
    p.add_argument("--max-tokens", type=int, default=2048, help="max tokens to generate")
    p.add_argument("--random-weights", action="store_true",
                   help="seeded random weights for the folder's config.json instead of its safetensors")
    p.add_argument("--seed", type=int, default=None, help="sampling seed (and weight seed with --random-weights)")
    p.add_argument("--allow-ignored-keys", action="store_true",
                   help="load a config.json that asks for what the architecture does not do (attention bias, scaled "
                        "rotation, a sliding window, another activation) and ignore those keys, as the reference does")


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="inferrs-amd", description=__doc__.split("\n\n")[0])
    ap.add_argument("-v", "--version", action="version", version=f"inferrs-amd {__version__}")
    sub = ap.add_subparsers(dest="command", required=True)

    run = sub.add_parser("run", help="generate from a prompt, or read prompts line by line")
    _add_engine_options(run)
    run.add_argument("prompt", nargs="?", default=None)
    run.add_argument("--system", default=None, help="system prompt (needs a tokenizer)")
    run.add_argument("--min-p", type=float, default=0.0)
    run.add_argument("--repetition-penalty", type=float, default=1.1)
    run.add_argument("--repeat-last-n", type=int, default=64)
    run.add_argument("--frequency-penalty", type=float, default=0.0)
    run.add_argument("--presence-penalty", type=float, default=0.0)
    run.add_argument("--ignore-eos", action="store_true", help="generate max-tokens whatever comes")

    bench = sub.add_parser("bench", help="time prefill and decode on a synthetic prompt")
    _add_engine_options(bench)
    bench.add_argument("--warmup", type=int, default=1)
    bench.add_argument("--runs", type=int, default=5)
    bench.add_argument("--prompt-len", type=int, default=128)

    serve = sub.add_parser("serve", help="not built: this engine has no server")
    serve.add_argument("rest", nargs=argparse.REMAINDER)
    return ap


def load_engine(args):
    from .config import load_config
    from .engine import Engine
    if not os.path.isdir(args.model):
        raise SystemExit(f"inferrs-amd: '{args.model}' is not a folder; models are loaded from local folders only")
    dtype = {"f32": "float32", "bf16": "bfloat16"}.get(args.dtype, args.dtype)
    options = dict(dtype=dtype, page_size=args.block_size, max_seqs=args.max_batch_size)
    if args.max_blocks > 0:
        options["num_pages"] = max(args.max_blocks, args.initial_blocks)
    else:
        options["memory_fraction"] = args.paged_attention
    print(f"inferrs-amd: loading {args.model} ({dtype})", file=sys.stderr, flush=True)
    if args.random_weights:
        return Engine.from_random(load_config(args.model, allow_ignored_keys=args.allow_ignored_keys),
                                  seed=args.seed or 0, **options)
    return Engine.from_folder(args.model, allow_ignored_keys=args.allow_ignored_keys, **options)


class TokenCodec:
    """Text <-> token ids through the folder's tokenizer.json when there is one; plain ids else."""

    def __init__(self, model_dir: str, config=None):
        from .chat import detect_template
        self.tokenizer = None
        self.template = "plain"
        path = os.path.join(model_dir, "tokenizer.json")
        if os.path.isfile(path):
            from tokenizers import Tokenizer
            self.tokenizer = Tokenizer.from_file(path)
            self.template = detect_template(model_dir, config)

    def encode(self, text: str, system: Optional[str] = None) -> List[int]:
        if self.tokenizer is not None:
            from .chat import render
            return self.tokenizer.encode(render(self.template, text, system)).ids
        if system:
            raise SystemExit("inferrs-amd: --system needs a tokenizer.json in the model folder")
        try:
            return [int(t) for t in text.replace(",", " ").split()]
        except ValueError:
            raise SystemExit("inferrs-amd: the model folder has no tokenizer.json, so the prompt must be "
                             "token ids separated by commas or blanks") from None

    def decode(self, ids: List[int]) -> str:
        if self.tokenizer is not None:
            return self.tokenizer.decode(ids)
        return " ".join(str(i) for i in ids)


def cmd_run(args) -> int:
    from .engine import GenerationLoop
    from .sampling import SamplingParams
    engine = load_engine(args)
    codec = TokenCodec(args.model, getattr(engine, "config", None))
    params = SamplingParams(
        temperature=args.temperature, top_p=args.top_p, top_k=args.top_k, min_p=args.min_p,
        repetition_penalty=args.repetition_penalty, repeat_last_n=args.repeat_last_n,
        frequency_penalty=args.frequency_penalty, presence_penalty=args.presence_penalty,
        max_tokens=args.max_tokens, seed=args.seed, bypass_stop_tokens=args.ignore_eos)

    def answer(text: str) -> None:
        loop = GenerationLoop(engine, max_batch_size=args.max_batch_size,
                              max_tokens_per_step=args.max_tokens_per_step, max_seq_len=args.max_seq_len or None,
                              detokenize=codec.decode)
        req = loop.add(codec.encode(text, args.system), params)
        t0 = time.perf_counter()
        if codec.tokenizer is None:
            loop.run(on_token=lambda r, t: print(t, end=" ", flush=True))
        else:
            shown = 0

            def show(r, _t):
                nonlocal shown
                text_now = codec.decode(r.output)
                print(text_now[shown:], end="", flush=True)
                shown = len(text_now)
            loop.run(on_token=show)
        dt = time.perf_counter() - t0
        print()
        if req.finish_reason == "error":
            print(f"inferrs-amd: {req.error}", file=sys.stderr)
        print(f"[{len(req.output)} tokens, {len(req.output) / max(dt, 1e-9):.1f} tok/s, finish: {req.finish_reason}]",
              file=sys.stderr, flush=True)

    if args.prompt is not None:
        answer(args.prompt)
        return 0
    return prompt_lines(answer)


def prompt_lines(answer) -> int:
    """Without a prompt on the command line: one prompt a line from standard input until it ends, each
    answered on its own (nothing of an earlier answer is context for the next).  Blank lines are skipped."""
    print("inferrs-amd: one prompt a line; end of input ends the run", file=sys.stderr, flush=True)
    for line in sys.stdin:
        line = line.strip()
        if line:
            answer(line)
            sys.stdout.flush()
    return 0


def cmd_bench(args) -> int:
    """Like `inferrs bench` (`inferrs/src/bench.rs:40-224`): a prompt of `--prompt-len` copies of
    one token, stop tokens bypassed, `--warmup` unmeasured runs and `--runs` measured ones; prints
    mean and deviation of prefill and decode throughput."""
    import statistics

    import torch

    from .engine import GenerationLoop
    from .sampling import SamplingParams
    engine = load_engine(args)
    prompt = [min(1, engine.spec.vocab_size - 1)] * args.prompt_len
    params = SamplingParams.greedy(max_tokens=args.max_tokens, bypass_stop_tokens=True)
    prefill, decode = [], []
    for run in range(args.warmup + args.runs):
        loop = GenerationLoop(engine, max_batch_size=args.max_batch_size,
                              max_tokens_per_step=max(args.max_tokens_per_step, args.prompt_len))
        req = loop.add(prompt, params)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        loop.step()                                   # the whole prompt, and the first token
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        loop.run()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        if run >= args.warmup:
            prefill.append(args.prompt_len / (t1 - t0))
            decode.append(max(len(req.output) - 1, 1) / max(t2 - t1, 1e-9))
    def fmt(xs):
        return f"{statistics.mean(xs):.1f} ± {statistics.pstdev(xs):.1f} tok/s"
    print(json.dumps({"prompt_len": args.prompt_len, "max_tokens": args.max_tokens, "runs": args.runs,
                      "prefill_tok_s": statistics.mean(prefill), "decode_tok_s": statistics.mean(decode)}))
    print(f"prefill: {fmt(prefill)}   decode: {fmt(decode)}", file=sys.stderr)
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    if args.command == "serve":
        print("inferrs-amd: servers are not part of this engine; use `run` or the Python entry point "
              "inferrs_amd.Engine", file=sys.stderr)
        return 2
    return {"run": cmd_run, "bench": cmd_bench}[args.command](args)


if __name__ == "__main__":
    sys.exit(main())
