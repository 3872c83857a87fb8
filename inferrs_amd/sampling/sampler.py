"""Turns rows of logits into tokens on the device, one row per request, in the reference's
order of operations (`inferrs/src/sampler.rs:146-335`): logit bias, repetition, frequency and
presence penalties over the last `repeat_last_n` tokens, temperature, softmax, top-k, top-p,
min-p, and the walk to a random number that depends on the request's seed and step only."""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from .params import SAMPLING_EPS, SamplingParams, TokenLogprob
from .rng import rand_f32


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)

    def _dev(self, array: np.ndarray) -> torch.Tensor:
        return torch.from_numpy(array).to(self.device, non_blocking=False)

    def begin_chain(self, params: Sequence[SamplingParams], previous: Sequence[Sequence[int]],
                    seeds: Sequence[int], steps: int) -> "ChainDraw":
        """The draws of the next `steps` decode steps of these requests, prepared for the device."""
        return ChainDraw(self, params, previous, seeds, steps)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], previous: Sequence[Sequence[int]],
               seeds: Sequence[int]) -> List[int]:
        """`logits` float32 [rows, vocab] on the device; row i belongs to a request with
        `params[i]`, whose prompt and output so far are `previous[i]` and whose seed is `seeds[i]`."""
        return self.sample_with_logprobs(logits, params, previous, seeds)[0]

    def sample_with_logprobs(self, logits: torch.Tensor, params: Sequence[SamplingParams],
                             previous: Sequence[Sequence[int]], seeds: Sequence[int]):
        """(tokens, per row a `TokenLogprob` or None): the log-probabilities for the rows whose
        parameters ask for them (`sampler.rs:285-352`)."""
        rows = logits.shape[0]
        if not (len(params) == len(previous) == len(seeds) == rows):
            raise ValueError("one parameter set, token history and seed per row of logits")
        if rows == 0:
            return [], []
        if all(p.is_plain_greedy for p in params):
            return ops.argmax(logits).cpu().tolist(), [None] * rows

        # penalties and bias, on a copy only if something is changed
        width = max((min(p.repeat_last_n, len(prev)) if p.has_penalty else 0) for p, prev in zip(params, previous))
        n_bias = max(len(p.logit_bias) for p in params)
        if width or n_bias:
            logits = logits.clone()
            window = np.full((rows, max(width, 1)), -1, dtype=np.int32)
            rep = np.ones(rows, dtype=np.float32)
            freq = np.zeros(rows, dtype=np.float32)
            pres = np.zeros(rows, dtype=np.float32)
            for i, (p, prev) in enumerate(zip(params, previous)):
                if p.has_penalty and prev:
                    tail = list(prev[-p.repeat_last_n:])
                    window[i, :len(tail)] = tail
                    rep[i], freq[i], pres[i] = p.repetition_penalty, p.frequency_penalty, p.presence_penalty
            bias_ids = bias_vals = None
            if n_bias:
                ids = np.full((rows, n_bias), -1, dtype=np.int32)
                vals = np.zeros((rows, n_bias), dtype=np.float32)
                for i, p in enumerate(params):
                    for j, (tid, b) in enumerate(sorted(p.logit_bias.items())):
                        ids[i, j], vals[i, j] = int(tid), float(b)
                bias_ids, bias_vals = self._dev(ids), self._dev(vals)
            ops.penalize(logits, self._dev(window) if width else None, self._dev(rep), self._dev(freq),
                         self._dev(pres), bias_ids, bias_vals)

        temperature = np.asarray([p.draw_temperature(len(prev)) for p, prev in zip(params, previous)], dtype=np.float32)
        top_k = np.asarray([p.top_k for p in params], dtype=np.int32)
        top_p = np.asarray([p.top_p for p in params], dtype=np.float32)
        min_p = np.asarray([p.min_p for p in params], dtype=np.float32)
        # the step of a draw is the number of tokens before it (`sampler.rs:323-325`)
        u = np.asarray([rand_f32(seed, len(prev)) if p.draw_temperature(len(prev)) >= SAMPLING_EPS else 0.0
                        for p, prev, seed in zip(params, previous, seeds)], dtype=np.float32)
        if not any(p.logprobs for p in params):
            out = ops.sample(logits, self._dev(temperature), self._dev(top_k), self._dev(top_p), self._dev(min_p),
                             self._dev(u))
            return out.cpu().tolist(), [None] * rows
        n_top = np.asarray([p.top_logprobs if p.logprobs else -1 for p in params], dtype=np.int32)
        out, lp, ids = ops.sample(logits, self._dev(temperature), self._dev(top_k), self._dev(top_p), self._dev(min_p),
                                  self._dev(u), self._dev(n_top))
        tokens, lp, ids = out.cpu().tolist(), lp.cpu().tolist(), ids.cpu().tolist()
        infos = []
        for i, p in enumerate(params):
            if not p.logprobs:
                infos.append(None)
                continue
            top = tuple((t, v) for t, v in zip(ids[i], lp[i][1:]) if t >= 0)[:p.top_logprobs]
            infos.append(TokenLogprob(tokens[i], lp[i][0], top))
        return tokens, infos


class ChainDraw:
    """The draws of a run of decode steps that are queued without the host in between: what
    `Sampler.sample` works out from the token lists at every step is kept on the device here, the
    random numbers of all steps (they depend on seed and step only) and every row's penalty window,
    which takes the row's new token after each draw.  The tokens are those of single steps."""

    def __init__(self, sampler: "Sampler", params: Sequence[SamplingParams], previous: Sequence[Sequence[int]],
                 seeds: Sequence[int], steps: int):
        if any(p.logprobs for p in params):
            raise ValueError("log-probabilities are reported step by step, not from a run of steps")
        rows = len(params)
        self.greedy = all(p.is_plain_greedy for p in params)
        if self.greedy:
            return
        dev = sampler._dev
        caps = np.asarray([p.repeat_last_n if p.has_penalty else 0 for p in params], dtype=np.int32)
        width = int(caps.max()) if rows else 0
        n_bias = max(len(p.logit_bias) for p in params)
        self.window = self.caps = self.bias_ids = self.bias_vals = None
        self.penalized = bool(width or n_bias)
        if self.penalized:
            rep, freq, pres = np.ones(rows, np.float32), np.zeros(rows, np.float32), np.zeros(rows, np.float32)
            window = np.full((rows, max(width, 1)), -1, dtype=np.int32)
            for i, (p, prev) in enumerate(zip(params, previous)):
                if p.has_penalty:
                    tail = list(prev[-p.repeat_last_n:])
                    window[i, :len(tail)] = tail
                    rep[i], freq[i], pres[i] = p.repetition_penalty, p.frequency_penalty, p.presence_penalty
            if width:
                self.window, self.caps = dev(window), dev(caps)
            self.rep, self.freq, self.pres = dev(rep), dev(freq), dev(pres)
            if n_bias:
                ids = np.full((rows, n_bias), -1, dtype=np.int32)
                vals = np.zeros((rows, n_bias), dtype=np.float32)
                for i, p in enumerate(params):
                    for j, (tid, b) in enumerate(sorted(p.logit_bias.items())):
                        ids[i, j], vals[i, j] = int(tid), float(b)
                self.bias_ids, self.bias_vals = dev(ids), dev(vals)
        # (a window that holds a token at the run's start holds one at every step of it)
        self.temperature = dev(np.asarray([p.draw_temperature(len(prev)) for p, prev in zip(params, previous)], dtype=np.float32))
        self.top_k = dev(np.asarray([p.top_k for p in params], dtype=np.int32))
        self.top_p = dev(np.asarray([p.top_p for p in params], dtype=np.float32))
        self.min_p = dev(np.asarray([p.min_p for p in params], dtype=np.float32))
        # the step of a draw is the number of tokens before it (`sampler.rs:323-325`)
        self.u = dev(np.asarray([[rand_f32(seed, len(prev) + i) if p.draw_temperature(len(prev)) >= SAMPLING_EPS else 0.0
                                  for p, prev, seed in zip(params, previous, seeds)] for i in range(steps)],
                                dtype=np.float32).reshape(steps, rows))

    def pick(self, logits: torch.Tensor, step: int, out: torch.Tensor) -> None:
        """The tokens of the run's `step`-th step from its logits, into `out` (int32 [rows], on the device).
        The penalties are applied to `logits` in place: inside a run they are the captured step's own output buffer,
        which the next step overwrites and nobody else reads."""
        if self.greedy:
            ops.argmax(logits, out=out)
            return
        if self.penalized:
            ops.penalize(logits, self.window, self.rep, self.freq, self.pres, self.bias_ids, self.bias_vals)
        out.copy_(ops.sample(logits, self.temperature, self.top_k, self.top_p, self.min_p, self.u[step]))
        if self.window is not None:
            ops.window_push(self.window, self.caps, out)
