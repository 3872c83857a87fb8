"""The step function: one call runs a batch of (request, its next tokens) through the model,
from the cache and into it, and returns the logits at the wanted places.

The reference's model interface takes one sequence per call, either a whole prompt or one
decode token (`forward(input_ids, seqlen_offset)`, `forward_paged(...)`,
`inferrs-models/src/models/mod.rs:172,214-220`; the engine's only two call shapes are
`inferrs/src/engine.rs:2074-2109` and `:2121-2150`).  Here a step holds any mix: portions
of prompts beside single decoded tokens, cut anywhere.  Only the tokens given are run;
everything earlier comes from the cache that previous steps left.
"""
from __future__ import annotations

import logging
import time
from collections import OrderedDict
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import torch

from .. import ops
from ..cache import CacheError, CacheManager, CacheStorage, OutOfPages
from ..config.base import folder_stop_ids
from ..config.registry import load_config
from ..parts.assemble import generated_tensors, model_tensors
from ..weights.loader import load_weights
from ..weights.random_init import random_tensors
from .batch import StepBuilder, StepError
from .model import DecoderModel, parse_dtype


log = logging.getLogger("inferrs_amd")


class Entry:
    """One request's share of a step: its next `tokens` and the places among them whose
    logits are wanted."""
    __slots__ = ("seq_id", "tokens", "want")

    def __init__(self, seq_id: Hashable, tokens: Sequence[int], want: Sequence[int] = ()):
        self.seq_id, self.tokens, self.want = seq_id, list(tokens), list(want)


# The hidden request whose rows fill a decode step up to the next of the batch sizes that graphs are captured for.
_PAD = ("inferrs_amd", "rows that fill a decode step")


class Engine:
    GRAPH_BUCKET_TOKENS = 1024      # a captured step serves context lengths up to a multiple of this
    GRAPH_MAX_TOKENS = 1024         # steps of more tokens run eagerly: their kernels outlast the host, and a graph would hold their buffers
    MAX_GRAPHS = 48                 # captured graphs kept (the one replayed longest ago goes first)
    MAX_SHAPES_SEEN = 512           # shapes remembered as seen, with what was measured of them
    GRAPH_HOST_SHARE = 0.8          # steps other than decode steps are captured where the host took this share of a step's time (0: always)

    def __init__(self, model: DecoderModel, *, page_size: int = 16, num_pages: Optional[int] = None,
                 max_seqs: int = 32, cache_tokens: Optional[int] = None, memory_fraction: float = 0.9,
                 use_graphs: bool = True):
        """`num_pages` pages per cache group, or enough for `cache_tokens` tokens, or, when
        neither is given, `memory_fraction` of the GPU memory that is free now (the reference
        sizes by a fraction of total memory, `inferrs-models/src/kv_cache.rs:44-65`)."""
        ops.require_gpu()
        self.model = model
        self.spec = model.spec
        self.device = model.device
        self.page_size = page_size
        needs = model.cache_needs()
        probe = CacheManager(needs, page_size, 0, max_seqs + 1)
        if num_pages is None and cache_tokens is not None:
            num_pages = -(-cache_tokens // page_size)
        if num_pages is None:
            # the budget pays for the fixed-size state of every request slot first, pages get the rest
            per_page = CacheStorage.page_bytes(probe, model.dtype)
            free, _total = torch.cuda.mem_get_info(self.device)
            budget = int(free * memory_fraction) - CacheStorage.state_bytes(probe)
            if budget < per_page:
                raise OutOfPages(f"{memory_fraction:.2f} of the free GPU memory ({free >> 20} MiB) does not hold the "
                                 f"per-request state of {max_seqs} requests and one page of {per_page} bytes")
            num_pages = max(1, budget // max(per_page, 1))
            # more than every request slot at the longest sequence is never used
            num_pages = min(num_pages, max_seqs * -(-model.spec.max_position // page_size))
        # (one request slot more than asked for: the hidden request of the rows that fill a decode step takes none of the callers')
        self.max_seqs = max_seqs
        self.cache = CacheManager(needs, page_size, num_pages, max_seqs + 1)
        self.storage = CacheStorage(self.cache, model.dtype, self.device)
        self.builder = StepBuilder(self.cache, self.device)
        # Decode steps (one token a request) and steps of few tokens are bound by their launches: each distinct
        # shape is captured into a HIP graph the second time it is seen and replayed from then on.
        self.use_graphs = use_graphs and model.graph_safe
        self.unused_tensors: List[str] = []
        self.stop_token_ids: Tuple[int, ...] = tuple(model.spec.eos_token_ids)
        # a part that will run off its fast path says so once, here, and not at every step
        self.load_notes: List[str] = model.load_notes(page_size)
        for note in self.load_notes:
            log.warning("%s", note)
        self._graphs: "OrderedDict[Tuple[int, ...], object]" = OrderedDict()      # shape -> (graph, its logits)
        self._seen: "OrderedDict[Tuple[int, ...], object]" = OrderedDict()        # shapes that ran eagerly: "once", a measurement, or "eager" for good
        self._graphs_generation = self.builder.generation    # the staging buffer the graphs were captured over
        self.graph_replays = 0

    # ---- construction -----------------------------------------------------------------------
    @classmethod
    def from_folder(cls, model_dir: str, dtype="bfloat16", device="cuda:0", strict: bool = False,
                    allow_ignored_keys: bool = False, **kw) -> "Engine":
        """`strict`: tensors of the folder that the model does not read are an error instead of a warning.
        `allow_ignored_keys`: config.json values that the architecture does not honour are ignored, as the
        reference ignores them, instead of refused."""
        config = load_config(model_dir, allow_ignored_keys=allow_ignored_keys)
        spec = config.to_spec()
        expected, optional = model_tensors(spec)
        unused: List[str] = []
        tensors = load_weights(model_dir, expected, optional, strict=strict, unused=unused)
        if unused:
            log.warning("%s: %d tensors are not read by %s: %s", model_dir, len(unused), spec.architecture,
                     ", ".join(unused[:8]) + (" ..." if len(unused) > 8 else ""))
        model = DecoderModel(spec, tensors, parse_dtype(dtype), device)
        eng = cls(model, **kw)
        eng.config = config
        eng.unused_tensors = unused
        # what ends a request of this folder's model: config.json's ids and what the files beside it declare
        eng.stop_token_ids = folder_stop_ids(model_dir, spec.eos_token_ids)
        return eng

    @classmethod
    def from_random(cls, config, seed: int = 0, dtype="bfloat16", device="cuda:0", **kw) -> "Engine":
        """Random weights drawn on the device, without a folder in between."""
        spec = config.to_spec()
        wanted = generated_tensors(spec)
        dt = parse_dtype(dtype)
        tensors = random_tensors(wanted, seed, torch.bfloat16 if dt == torch.bfloat16 else torch.float32,
                                 device=device)
        model = DecoderModel(spec, tensors, dt, device)
        eng = cls(model, **kw)
        eng.config = config
        return eng

    def generate(self, prompts, params=None, **loop_options):
        """Token ids in, token ids out: see `inferrs_amd.engine.generate.generate`."""
        from .generate import generate
        return generate(self, prompts, params, **loop_options)

    # ---- requests ---------------------------------------------------------------------------
    def add_request(self, seq_id: Hashable) -> None:
        seq = self.cache.add_sequence(seq_id)
        self.storage.clear_state_slot(seq.state_slot)

    def has_request(self, seq_id: Hashable) -> bool:
        return seq_id in self.cache.sequences

    def end_request(self, seq_id: Hashable) -> None:
        self.cache.free_sequence(seq_id)

    def cached_length(self, seq_id: Hashable) -> int:
        return self.cache.length(seq_id)

    # ---- the step ---------------------------------------------------------------------------
    def step(self, entries: Sequence[Entry], commit: bool = True) -> torch.Tensor:
        """Run one batch; returns float32 logits `[wanted, vocab]` on the device, in the order
        of the entries and of each entry's `want`.  Pages that the entries need beyond what is
        reserved for them are reserved here.  With `commit` the requests' cached lengths advance;
        a caller that passes False (the scheduler) does that itself.

        The tensor that a step returns under `use_graphs` may be a captured graph's own output buffer (decode
        steps and steps of up to `GRAPH_MAX_TOKENS` tokens whose shape has been seen before): it holds this
        step's logits until the next step of the same shape overwrites them.  Read or `.clone()` it before
        stepping again."""
        if not entries:
            raise StepError("a step needs at least one entry")
        vocab = self.spec.vocab_size
        seen = set()
        for e in entries:
            if e.seq_id in seen:
                raise StepError(f"request {e.seq_id!r} appears twice in one step")
            seen.add(e.seq_id)
            if not e.tokens:
                raise StepError(f"request {e.seq_id!r}: a step entry needs at least one token")
            if min(e.tokens) < 0 or max(e.tokens) >= vocab:
                raise StepError(f"request {e.seq_id!r}: token ids must lie in 0..{vocab - 1}")
            if any(not (0 <= w < len(e.tokens)) for w in e.want):
                raise StepError(f"request {e.seq_id!r}: 'want' {e.want} outside its {len(e.tokens)} tokens")
        ids = [e.seq_id for e in entries]
        fresh = [] if self.cache.all_live(ids) else [s for s in ids if s not in self.cache.sequences]
        try:
            for sid in fresh:
                self.add_request(sid)
            if not self.cache.ensure_reserved([(e.seq_id, len(e.tokens)) for e in entries]):
                raise OutOfPages("paged attention: out of KV blocks for this step "
                                 f"({[g.pool.num_free for g in self.cache.groups]} pages free)")
        except Exception:
            for sid in fresh:
                if sid in self.cache.sequences:
                    self.cache.free_sequence(sid)
            raise

        triples = [(e.seq_id, e.tokens, e.want) for e in entries]
        n_tokens = sum(len(e.tokens) for e in entries)
        if self.use_graphs and (n_tokens == len(entries) or n_tokens <= self.GRAPH_MAX_TOKENS):
            logits = self._graphed_step(triples)
        else:
            logits = self.model.forward(self.builder.build(triples), self.storage)
        if commit:
            self.cache.commit_many([(e.seq_id, len(e.tokens)) for e in entries])
        return logits

    @staticmethod
    def padded_batch(n: int) -> int:
        """The batch size whose graph a decode step of `n` requests runs on: every size up to 8 (where the products
        change their kernels row by row), then in steps of 2 up to 16, of 4 up to 32, of 8 up to 64, of 16 up to
        128 and of 32 beyond.  A batch that grows and shrinks request by request then walks through a few shapes
        and not through one for every size."""
        if n <= 8:
            return n
        step = 2 if n <= 16 else 4 if n <= 32 else 8 if n <= 64 else 16 if n <= 128 else 32
        return -(-n // step) * step

    def _pad_rows(self, n: int, tokens_ahead: int) -> int:
        """Rows of the hidden request that a decode step of `n` requests gets on top, 0 when its size is one of
        `padded_batch` or the rows cannot be had (no page free for them).  The hidden request has no cached token
        and never gets one: each of its rows is token 0 at the first positions, written to its pages with the same
        values by every row, and attends to itself alone; its logits are dropped.  It lives for the length of the
        call that asked for it (`_drop_pad_rows` at that call's end): between steps nobody sees its pages missing,
        and what its rows write reaches the pages before anything that a later step queues."""
        extra = self.padded_batch(n) - n
        if extra == 0:
            return 0
        try:
            if not self.has_request(_PAD):
                self.add_request(_PAD)
            if not self.cache.ensure_reserved([(_PAD, tokens_ahead)]):
                self._drop_pad_rows()
                return 0
        except CacheError:
            return 0
        return extra

    def _drop_pad_rows(self) -> None:
        if self.has_request(_PAD):
            self.cache.free_sequence(_PAD)

    def _bucket_pages(self, longest: int) -> int:
        bucket_pages = max(1, self.GRAPH_BUCKET_TOKENS // self.page_size)
        return -(-(-(-longest // self.page_size)) // bucket_pages) * bucket_pages

    def chain_ready(self, seq_ids: Sequence[Hashable], steps: int) -> bool:
        """Whether `decode_chain` can run these requests for `steps` steps: their shape has a
        captured graph whose context bucket holds them to the end."""
        if not self.use_graphs or steps < 1 or not seq_ids:
            return False
        self._drop_stale_graphs()
        pad_pages = self._bucket_pages(self.cache.max_length(seq_ids) + steps)
        try:
            n = len(seq_ids) + self._pad_rows(len(seq_ids), steps)
        finally:
            self._drop_pad_rows()
        return self._decode_key(n, pad_pages) in self._graphs

    def decode_chain(self, seq_ids: Sequence[Hashable], tokens: Sequence[int], steps: int,
                     pick=None) -> Optional[List[List[int]]]:
        """`steps` decode steps of the same requests, queued back to back: every step's choice
        (the arg max, or `pick(logits, step, out)` writing int32 tokens into `out` on the device; it may change `logits`, the
        captured step's own buffer) is
        written on the device where the next step reads its token ids, so the host prepares and
        queues step i+1 while step i runs and waits once at the end.  The requests hold reserved
        pages for `steps` more tokens; nothing is committed here.  Returns the chosen tokens
        `[steps][requests]`, or None when this shape has no captured graph yet (the caller then
        takes single steps)."""
        if not self.chain_ready(seq_ids, steps):
            return None
        pad_pages = self._bucket_pages(self.cache.max_length(seq_ids) + steps)
        n_real = len(seq_ids)
        try:
            extra = self._pad_rows(n_real, steps)     # (as in chain_ready: rows of the hidden request up to the graph's batch size)
            key = self._decode_key(n_real + extra, pad_pages)
            if key not in self._graphs:               # (the hidden request found pages a moment ago and finds none now)
                return None
            graph, logits = self._graphs[key]
            self._graphs.move_to_end(key)
            generation = self.builder.generation
            # (zeros: the hidden request's rows take token 0 where `pick` chooses for the callers' rows only)
            chosen = torch.zeros((steps, n_real + extra), dtype=torch.int32, device=self.device)
            for i in range(steps):
                triples = [(sid, [tok if i == 0 else 0], [0]) for sid, tok in zip(seq_ids, tokens)] + [(_PAD, [0], [0])] * extra
                ctx = self.builder.build(triples, pad_pages=pad_pages, advance=i, skip_tokens=i > 0)
                if self.builder.generation != generation:
                    raise RuntimeError("the staging buffer moved under a captured graph")
                graph.replay()
                if pick is None:
                    ops.argmax(logits, out=chosen[i])
                else:
                    pick(logits[:n_real], i, chosen[i, :n_real])
                ctx.token_ids.copy_(chosen[i])            # the next step's token ids, on the device
                self.graph_replays += 1
        finally:
            self._drop_pad_rows()
        return chosen[:, :n_real].cpu().tolist()

    @staticmethod
    def _decode_key(n_seqs: int, pad_pages: int) -> Tuple[int, ...]:
        """The shape of a decode step of `n_seqs` requests that all want their logits."""
        return (n_seqs, n_seqs, n_seqs, n_seqs, 1, pad_pages)

    def _drop_stale_graphs(self) -> None:
        """Captured graphs hold the address of the step builder's device buffer.  Any step, also one
        that runs eagerly (a long prompt portion), may have made that buffer grow and move
        since: graphs captured over the old one are dropped before any of them is looked up."""
        if self._graphs_generation != self.builder.generation:
            self._graphs.clear()
            self._seen.clear()
            self._graphs_generation = self.builder.generation

    def _graphed_step(self, triples) -> torch.Tensor:
        try:
            return self._step_of_a_shape(triples)
        finally:
            self._drop_pad_rows()

    def _step_of_a_shape(self, triples) -> torch.Tensor:
        """A step through a captured graph when its shape has been seen before.  The shape is what the launches
        of a step depend on: the counts of requests, of tokens, of requests with a single token and of wanted
        rows, the longest portion, and the width of the block tables.  The tables are padded to the bucket's
        width and the bounds of the key lengths are the bucket's, so that every kernel argument is the same for
        all context lengths of the bucket; lengths, positions and pages are read from device memory.  A shape's
        eager steps run with the same arguments, so a step's logits do not depend on whether it was replayed.

        Decode steps repeat by their nature and are captured the second time their shape is seen; their batch is
        filled up to the next size of `padded_batch` with rows of a hidden request, so that a batch which changes
        request by request meets few shapes.  A capture
        costs about one more step, which other steps only earn back where the host is their bound (small models,
        few tokens): a shape's second step is timed, on the host and on the GPU, and its third is captured if
        the host's share was `GRAPH_HOST_SHARE` or more; otherwise the shape stays eager.

        The logits that a replayed step returns are the graph's own buffer: they hold until the next step of
        the shape."""
        singles = [t[0] for t in triples if len(t[1]) == 1]
        n_want = sum(len(t[2]) for t in triples)
        extra = self._pad_rows(len(triples), 1) if len(singles) == len(triples) else 0
        if extra:
            triples = list(triples) + [(_PAD, [0], [0])] * extra
        longest = self.cache.max_length(singles) + 1 if singles else 0
        for t in triples:
            if len(t[1]) > 1:
                longest = max(longest, self.cache.length(t[0]) + len(t[1]))
        pad_pages = self._bucket_pages(longest)
        self._drop_stale_graphs()
        ctx = self.builder.build(triples, pad_pages=pad_pages)
        self._drop_stale_graphs()                       # (the buffer may have moved in this very build)
        key = (ctx.n_seqs, ctx.n_tokens, ctx.n_single, int(ctx.want_rows.shape[0]), ctx.max_q_len, pad_pages)
        entry = self._graphs.get(key)
        if entry is not None:
            self._graphs.move_to_end(key)
        else:
            state = self._seen.get(key)
            if state is None:
                if len(self._seen) >= self.MAX_SHAPES_SEEN:
                    self._seen.popitem(last=False)
                self._seen[key] = "once"
                return self.model.forward(ctx, self.storage)[:n_want]
            if ctx.max_q_len > 1:
                if state == "eager":
                    return self.model.forward(ctx, self.storage)
                if state == "once":
                    # (the first step of a shape also pays for what is set up once; this one is the measure)
                    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    begin.record()
                    t0 = time.perf_counter()
                    out = self.model.forward(ctx, self.storage)
                    host_ms = (time.perf_counter() - t0) * 1e3
                    end.record()
                    self._seen[key] = (host_ms, begin, end)
                    return out
                host_ms, begin, end = state
                # (a step that the GPU has not finished by now was not bound by the host either)
                if self.GRAPH_HOST_SHARE > 0.0 and (not end.query() or host_ms < self.GRAPH_HOST_SHARE * begin.elapsed_time(end)):
                    self._seen[key] = "eager"
                    return self.model.forward(ctx, self.storage)
            del self._seen[key]
            while len(self._graphs) >= max(self.MAX_GRAPHS, 1):
                self._graphs.popitem(last=False)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                out = self.model.forward(ctx, self.storage)
            entry = self._graphs[key] = (graph, out)
        graph, out = entry
        graph.replay()
        self.graph_replays += 1
        return out[:n_want] if extra else out
