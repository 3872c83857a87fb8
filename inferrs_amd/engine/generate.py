"""Generation: requests go through the scheduler, the step function and the sampler until
they finish.  This is the loop behind `Engine.generate` and the command line; the reference's
counterpart is `run_engine_loop` (`inferrs/src/engine.rs:1380-1912`)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Hashable, List, Optional, Sequence

from ..sampling import Sampler, SamplingParams, fresh_seed
from .engine import Engine, Entry
from .scheduler import Plan, Request, Scheduler


@dataclass
class Generation:
    request_id: Hashable
    prompt: List[int]
    tokens: List[int]
    finish_reason: str
    error: Optional[str] = None
    preemptions: int = 0
    logprobs: Optional[list] = None     # a TokenLogprob per token when the parameters asked for them


class GenerationLoop:
    def __init__(self, engine: Engine, *, max_batch_size: int = 32, max_tokens_per_step: int = 2048,
                 prefill_chunk: Optional[int] = None, max_seq_len: Optional[int] = None,
                 stop_token_ids: Optional[Sequence[int]] = None, decode_run: int = 8,
                 detokenize: Optional[Callable[[List[int]], str]] = None, row_multiple: int = 256):
        """`decode_run`: when every running request decodes and nobody waits, up to this many decode
        steps are queued on the GPU at once (`Engine.decode_chain`; draws included, their random
        numbers and penalty windows kept on the device); 1 switches it off.
        `detokenize`: output token ids -> text, for requests with stop strings.
        `row_multiple`: see `Scheduler` (cut prompt portions so that a step's tokens are a multiple of it)."""
        self.engine = engine
        self.detokenize = detokenize
        self.decode_run = max(1, decode_run)
        limit = engine.spec.max_position if not max_seq_len else min(max_seq_len, engine.spec.max_position)
        self.scheduler = Scheduler(
            engine.cache, max_batch_size=min(max_batch_size, engine.max_seqs),
            max_tokens_per_step=max_tokens_per_step, prefill_chunk=prefill_chunk, max_seq_len=limit,
            stop_token_ids=engine.stop_token_ids if stop_token_ids is None else stop_token_ids, row_multiple=row_multiple)
        self.sampler = Sampler(engine.device)
        self.steps = 0
        self._next_id = 0

    def add(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
            request_id: Optional[Hashable] = None) -> Request:
        params = params or SamplingParams()
        if request_id is None:
            request_id = f"req-{self._next_id}"
            self._next_id += 1
        vocab = self.engine.spec.vocab_size
        if any((not isinstance(t, int)) or t < 0 or t >= vocab for t in prompt):
            raise ValueError(f"request {request_id!r}: token ids must be integers in 0..{vocab - 1}")
        if any(params.stop_strings) and self.detokenize is None:
            raise ValueError(f"request {request_id!r}: stop strings need a detokenizer (GenerationLoop(detokenize=...))")
        seed = params.seed if params.seed is not None else fresh_seed()
        req = Request(request_id, list(prompt), params, seed=seed)
        self.scheduler.add(req)
        return req

    def _try_decode_run(self, max_steps: int) -> Optional[List[Request]]:
        """Several decode steps at once, when nothing else could happen in them anyway."""
        sched = self.scheduler
        running = list(sched.running)
        if max_steps < 2 or not running or sched.waiting or len(running) > sched.max_tokens_per_step:
            return None
        # (log-probabilities and stop strings are looked at step by step)
        if any(r.total - r.computed != 1 or not r.output or r.params.logprobs or any(r.params.stop_strings)
               for r in running):
            return None
        k = min(max_steps, min(min(r.params.max_tokens - len(r.output), sched.max_seq_len - r.total) for r in running))
        ids = [r.request_id for r in running]
        if k < 2 or not self.engine.chain_ready(ids, k) or not self.engine.cache.can_reserve([(i, k) for i in ids]):
            return None
        for i in ids:
            self.engine.cache.reserve(i, k)
        draw = self.sampler.begin_chain([r.params for r in running], [r.tokens for r in running],
                                        [r.seed for r in running], k)
        tokens = self.engine.decode_chain(ids, [r.tokens[-1] for r in running], k,
                                          pick=None if draw.greedy else draw.pick)
        if tokens is None:
            # (the shape's graph wanted rows of the engine's hidden request, and the pages reserved above were the last:
            # single steps then, which find their pages reserved)
            return None
        done: List[Request] = []
        for i in range(k):
            done += sched.commit_decode(running, tokens[i])
            self.steps += 1
        return done

    def step(self, max_steps: Optional[int] = None) -> List[Request]:
        """One scheduler step, or a run of up to `decode_run` decode steps (at most `max_steps`);
        returns the requests that finished (failed ones included)."""
        run = self._try_decode_run(min(self.decode_run, max_steps if max_steps is not None else self.decode_run))
        if run is not None:
            return run
        plan: Plan = self.scheduler.plan()
        done = list(plan.failed)
        if not plan.entries:
            return done
        for e in plan.entries:
            if e.request.computed == 0:
                self.engine.storage.clear_state_slot(self.engine.cache.sequences[e.request.request_id].state_slot)
        entries = [Entry(e.request.request_id, e.tokens, [len(e.tokens) - 1] if e.samples else [])
                   for e in plan.entries]
        logits = self.engine.step(entries, commit=False)
        drawing = [e.request for e in plan.entries if e.samples]
        tokens, infos = self.sampler.sample_with_logprobs(logits, [r.params for r in drawing],
                                                          [r.tokens for r in drawing], [r.seed for r in drawing])
        for r, info in zip(drawing, infos):
            if info is not None:
                # a request that was preempted draws its tokens again while it is recomputed: the same ones
                del r.logprobs[len(r.output):]
                r.logprobs.append(info)
        sampled: Dict[Hashable, int] = {r.request_id: t for r, t in zip(drawing, tokens)}
        done += self.scheduler.commit(plan, sampled)
        # stop strings: the decoded output ends with one (`check_stop`, inferrs/src/engine.rs:866-887, where
        # they come after the stop tokens and before the length)
        for r in drawing:
            if any(r.params.stop_strings) and r.finish_reason in (None, "length"):
                text = self.detokenize(list(r.output))
                if any(s and text.endswith(s) for s in r.params.stop_strings):
                    if r.finish_reason is None:
                        self.scheduler.finish(r, "stop")
                        done.append(r)
                    else:
                        r.finish_reason = "stop"
        self.steps += 1
        return done

    def cancel(self, request: Request) -> None:
        """Nobody waits for this request any more: it ends with "cancelled" and gives back what it holds."""
        self.scheduler.finish(request, "cancelled")

    def run(self, on_token: Optional[Callable[[Request, int], None]] = None) -> List[Request]:
        """Steps until nothing is waiting or running; returns everything that finished."""
        finished: List[Request] = []
        emitted: Dict[Hashable, int] = {}
        while self.scheduler.has_work():
            live = list(self.scheduler.running) + list(self.scheduler.waiting)
            done = self.step()
            if on_token is not None:
                for r in live:
                    for t in r.output[emitted.get(r.request_id, 0):]:
                        on_token(r, t)
                    emitted[r.request_id] = len(r.output)
            finished += done
        return finished


def generate(engine: Engine, prompts: Sequence[Sequence[int]], params=None, **loop_options) -> List[Generation]:
    """Generates for every prompt (lists of token ids); `params` is one `SamplingParams` for all
    or one per prompt.  Results come in the order of the prompts."""
    loop = GenerationLoop(engine, **loop_options)
    if params is None or isinstance(params, SamplingParams):
        params = [params] * len(prompts)
    if len(params) != len(prompts):
        raise ValueError("one SamplingParams for all prompts, or one per prompt")
    requests = [loop.add(p, sp, request_id=i) for i, (p, sp) in enumerate(zip(prompts, params))]
    loop.run()
    return [Generation(r.request_id, r.prompt, list(r.output), r.finish_reason or "error", r.error, r.preemptions,
                       list(r.logprobs) if r.params.logprobs else None)
            for r in requests]
