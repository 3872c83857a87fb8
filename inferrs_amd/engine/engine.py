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

from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import ops
from ..cache import RELEASED, CacheManager, CacheStorage, OutOfPages
from ..config.registry import load_config
from ..parts.assemble import model_tensors
from ..weights.loader import load_weights
from ..weights.random_init import random_tensors
from .batch import GroupStep, StepContext
from .model import DecoderModel, parse_dtype


class StepError(ValueError):
    pass


class Entry:
    """One request's share of a step: its next `tokens` and the places among them whose
    logits are wanted."""
    __slots__ = ("seq_id", "tokens", "want")

    def __init__(self, seq_id: Hashable, tokens: Sequence[int], want: Sequence[int] = ()):
        self.seq_id, self.tokens, self.want = seq_id, list(tokens), list(want)


class Engine:
    def __init__(self, model: DecoderModel, *, page_size: int = 16, num_pages: Optional[int] = None,
                 max_seqs: int = 32, cache_tokens: Optional[int] = None, memory_fraction: float = 0.9):
        """`num_pages` pages per cache group, or enough for `cache_tokens` tokens, or, when
        neither is given, `memory_fraction` of the GPU memory that is free now (the reference
        sizes by a fraction of total memory, `inferrs-models/src/kv_cache.rs:44-65`)."""
        ops.require_gpu()
        self.model = model
        self.spec = model.spec
        self.device = model.device
        self.page_size = page_size
        needs = model.cache_needs()
        probe = CacheManager(needs, page_size, 0, max_seqs)
        if num_pages is None and cache_tokens is not None:
            num_pages = -(-cache_tokens // page_size)
        if num_pages is None:
            esize = 4 if model.dtype == torch.float32 else 2
            per_page = sum(len(g.layers) * 2 * g.need.n_kv_heads * g.need.head_dim * page_size * esize
                           for g in probe.groups)
            free, _total = torch.cuda.mem_get_info(self.device)
            num_pages = max(1, int(free * memory_fraction) // max(per_page, 1))
            # more than every request slot at the longest sequence is never used
            num_pages = min(num_pages, max_seqs * -(-model.spec.max_position // page_size))
        self.cache = CacheManager(needs, page_size, num_pages, max_seqs)
        self.storage = CacheStorage(self.cache, model.dtype, self.device)
        self._stage_host: Optional[torch.Tensor] = None
        self._stage_dev: Optional[torch.Tensor] = None
        self._stage_event: Optional[torch.cuda.Event] = None

    # ---- construction -----------------------------------------------------------------------
    @classmethod
    def from_folder(cls, model_dir: str, dtype="bfloat16", device="cuda:0", **kw) -> "Engine":
        config = load_config(model_dir)
        spec = config.to_spec()
        expected, optional = model_tensors(spec)
        tensors = load_weights(model_dir, expected, optional)
        model = DecoderModel(spec, tensors, parse_dtype(dtype), device)
        eng = cls(model, **kw)
        eng.config = config
        return eng

    @classmethod
    def from_random(cls, config, seed: int = 0, dtype="bfloat16", device="cuda:0", **kw) -> "Engine":
        """Random weights drawn on the device, without a folder in between."""
        spec = config.to_spec()
        expected, optional = model_tensors(spec)
        wanted = {n: s for n, s in expected.items() if n not in optional}
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
        return self.cache.sequences[seq_id].length

    # ---- the step ---------------------------------------------------------------------------
    def _staging(self, n: int) -> Tuple[torch.Tensor, torch.Tensor]:
        if self._stage_host is None or self._stage_host.numel() < n:
            size = 1 << max(12, (n - 1).bit_length())
            self._stage_host = torch.empty(size, dtype=torch.int32, pin_memory=True)
            self._stage_dev = torch.empty(size, dtype=torch.int32, device=self.device)
            self._stage_event = None
        if self._stage_event is not None:
            self._stage_event.synchronize()      # the previous step's copy has left the host buffer
        return self._stage_host, self._stage_dev

    def step(self, entries: Sequence[Entry], commit: bool = True) -> torch.Tensor:
        """Run one batch; returns float32 logits `[wanted, vocab]` on the device, in the order
        of the entries and of each entry's `want`.  Pages that the entries need beyond what is
        reserved for them are reserved here.  With `commit` the requests' cached lengths advance;
        a caller that passes False (the scheduler) does that itself."""
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
        fresh = [e.seq_id for e in entries if e.seq_id not in self.cache.sequences]
        try:
            for sid in fresh:
                self.add_request(sid)
            asks = [(e.seq_id, max(0, len(e.tokens) - self.cache.sequences[e.seq_id].reserved))
                    for e in entries]
            if not self.cache.can_reserve(asks):
                raise OutOfPages("paged attention: out of KV blocks for this step "
                                 f"({[g.pool.num_free for g in self.cache.groups]} pages free)")
            for sid, n in asks:
                if n and not self.cache.reserve(sid, n):
                    raise OutOfPages("paged attention: out of KV blocks")
        except Exception:
            for sid in fresh:
                if sid in self.cache.sequences:
                    self.cache.free_sequence(sid)
            raise

        ctx = self._build_context(entries)
        logits = self.model.forward(ctx, self.storage)
        if commit:
            for e in entries:
                self.cache.commit(e.seq_id, len(e.tokens))
        return logits

    def _build_context(self, entries: Sequence[Entry]) -> StepContext:
        ps = self.page_size
        seqs = [self.cache.sequences[e.seq_id] for e in entries]
        q_lens = [len(e.tokens) for e in entries]
        starts = [s.length for s in seqs]
        n, s_count = sum(q_lens), len(entries)
        n_groups = len(self.cache.groups)
        max_pages = max(1, max(-(-(st + q) // ps) for st, q in zip(starts, q_lens)))
        cu = np.zeros(s_count + 1, dtype=np.int64)
        np.cumsum(q_lens, out=cu[1:])
        token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
        positions = np.concatenate([np.arange(st, st + q, dtype=np.int32) for st, q in zip(starts, q_lens)])
        token_seq = np.repeat(np.arange(s_count, dtype=np.int32), q_lens)
        want = np.asarray([cu[i] + w for i, e in enumerate(entries) for w in e.want], dtype=np.int32)
        state_slots = np.asarray([s.state_slot for s in seqs], dtype=np.int32)
        tables, slots = [], []
        for g in range(n_groups):
            bt = np.zeros((s_count, max_pages), dtype=np.int32)
            for i, s in enumerate(seqs):
                row = s.tables[g][:max_pages]
                bt[i, :len(row)] = row
            pages_of_token = bt[token_seq, positions // ps]
            if n and (pages_of_token == RELEASED).any():
                raise StepError("a new token falls into a page that was already released")
            slots.append((pages_of_token * ps + positions % ps).astype(np.int32))
            np.maximum(bt, 0, out=bt)                 # released pages are never read
            tables.append(bt)

        parts = [token_ids, positions, token_seq, cu.astype(np.int32), state_slots, want]
        for g in range(n_groups):
            parts += [slots[g], tables[g].reshape(-1)]
        sizes = [p.size for p in parts]
        total = sum(sizes)
        host, dev = self._staging(max(total, 1))
        flat = host.numpy()
        off, views = 0, []
        for p, sz in zip(parts, sizes):
            flat[off:off + sz] = p
            views.append(dev[off:off + sz])
            off += sz
        dev[:total].copy_(host[:total], non_blocking=True)
        self._stage_event = torch.cuda.Event()
        self._stage_event.record()
        groups = [GroupStep(ps, views[6 + 2 * g], views[7 + 2 * g].view(s_count, max_pages))
                  for g in range(n_groups)]
        return StepContext(
            n_tokens=n, n_seqs=s_count, token_ids=views[0], positions=views[1], token_seq=views[2],
            cu_tokens=views[3], state_slots=views[4], want_rows=views[5], groups=groups,
            q_lens=q_lens, kv_starts=starts, state_slots_host=[int(x) for x in state_slots],
            max_q_len=max(q_lens), max_kv_len=max(st + q for st, q in zip(starts, q_lens)))
