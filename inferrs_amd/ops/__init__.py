"""Python face of the HIP kernels: shape checks on the host, then one C call per kernel.

There is no other implementation behind these functions: without a GPU, or
without the compiled library, they raise.  Tensors are torch tensors on the
GPU; torch serves as the allocator and, for large bfloat16 matrix products,
as the door to the vendor's GEMM library (the reference uses cuBLAS there,
`candle-core/src/cuda_backend/mod.rs:2260-2305`).
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Optional, Tuple

import torch

from . import build as _build

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


_LIBS: Dict[str, ctypes.CDLL] = {}
_LIB_PATHS: Dict[str, str] = {}


class KernelTimer:
    """Times every kernel call of this module with a pair of events while it is active:

        with ops.KernelTimer() as timer: ...steps...
        timer.summary() -> {entry point: (calls, microseconds)}

    For measurement only: each call is bracketed on the current stream, so launches are not overlapped."""
    active: Optional["KernelTimer"] = None

    def __init__(self):
        self.records = []                 # (name, start event, end event)

    def __enter__(self):
        KernelTimer.active = self
        return self

    def __exit__(self, *exc):
        KernelTimer.active = None

    def call(self, name, fn, *args):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        out = fn(*args)
        b.record()
        self.records.append((name, a, b))
        return out

    def summary(self) -> Dict[str, Tuple[int, float]]:
        torch.cuda.synchronize()
        out: Dict[str, Tuple[int, float]] = {}
        for name, a, b in self.records:
            calls, us = out.get(name, (0, 0.0))
            out[name] = (calls + 1, us + a.elapsed_time(b) * 1e3)
        return out


class _Timed:
    """A kernel library whose entry points report to the active `KernelTimer`, if there is one."""
    __slots__ = ("_lib", "_short")

    def __init__(self, lib: ctypes.CDLL):
        object.__setattr__(self, "_lib", lib)
        object.__setattr__(self, "_short", {})

    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        if KernelTimer.active is None or not name.startswith("ia_") or name.endswith(("_workspace", "_blocks", "_block_rows",
                                                                                      "_error", "_version", "_capacity", "_top",
                                                                                      "_splits", "_tune", "_target", "_counters", "_fills", "_plan")):
            return fn
        timer = KernelTimer.active
        return lambda *args: timer.call(name[3:], fn, *args)


_C_TYPES = {"int": ctypes.c_int, "long long": ctypes.c_longlong, "unsigned long long": ctypes.c_ulonglong,
            "float": ctypes.c_float, "double": ctypes.c_double, "hipStream_t": ctypes.c_void_p, "size_t": ctypes.c_size_t}
_DECLARATIONS: Dict[str, Tuple[object, list]] = {}


def _declarations() -> Dict[str, Tuple[object, list]]:
    """Entry point -> (result type, argument types), read from the header that declares them (`csrc/api.h`): with the
    types known, ctypes converts plain integers to pointers itself, and a call's arguments need no objects around them
    (0.3 us each, a thousand a step)."""
    if _DECLARATIONS:
        return _DECLARATIONS
    import re
    with open(os.path.join(_build.CSRC, "api.h")) as f:
        text = re.sub(r"//[^\n]*", "", f.read())

    def ctype(decl: str):
        decl = decl.strip()
        if "*" in decl:
            return ctypes.c_char_p if decl.replace("const", "").replace("*", "").split()[0] == "char" else ctypes.c_void_p
        words = [w for w in decl.replace("const", "").split()]
        for n in (3, 2, 1):                                 # the type's words, with or without a parameter's name behind them
            for cut in (words[:n],):
                if " ".join(cut) in _C_TYPES and len(words) - n <= 1:
                    return _C_TYPES[" ".join(cut)]
        raise KernelError(f"api.h: no ctypes type for {decl!r}")

    for m in re.finditer(r"\b(int|long long|void|const char\s*\*)\s+(ia_\w+)\s*\(([^)]*)\)\s*;", text):
        result, name, params = m.group(1), m.group(2), m.group(3).strip()
        args = [] if params in ("", "void") else [ctype(a) for a in params.split(",")]
        restype = None if result == "void" else (ctypes.c_char_p if "char" in result else _C_TYPES[result])
        _DECLARATIONS[name] = (restype, args)
    for must in ("ia_last_error", "ia_add_rmsnorm", "ia_gemm_skinny_bf16", "ia_attention_mfma", "ia_sample"):
        if must not in _DECLARATIONS:
            _DECLARATIONS.clear()
            raise KernelError(f"api.h: the declaration of {must} was not found (the header's form has changed?)")
    return _DECLARATIONS


def _declare(lib: ctypes.CDLL) -> None:
    for name, (restype, args) in _declarations().items():
        try:
            fn = getattr(lib, name)
        except AttributeError:                              # (an entry point of another library)
            continue
        fn.restype, fn.argtypes = restype, args


def library(target: str = "core"):
    """A compiled kernel library; compiled on first use when no built one is found."""
    lib = _LIBS.get(target)
    if lib is not None:
        return lib if KernelTimer.active is None else _Timed(lib)
    path = _build.library_path(target)
    if path is None:
        path = _build.build(target, verbose=True)
    lib = ctypes.CDLL(path)
    lib.ia_last_error.restype = ctypes.c_char_p
    if lib.ia_abi_version() != 1:
        raise KernelError(f"{path}: unexpected ABI version {lib.ia_abi_version()}")
    _declare(lib)
    _LIBS[target], _LIB_PATHS[target] = lib, path
    return lib if KernelTimer.active is None else _Timed(lib)


def _raw_library(target: str = "core") -> ctypes.CDLL:
    """The library without the timer around its entry points (for calls that a caller times under a name of its own)."""
    library(target)
    return _LIBS[target]


def library_files() -> Dict[str, str]:
    """The libraries loaded so far: target -> file."""
    return dict(_LIB_PATHS)


def require_gpu() -> None:
    if not torch.cuda.is_available():
        raise KernelError("inferrs_amd runs on an AMD GPU through its HIP kernels; "
                          "no GPU is visible and there is no CPU fallback")
    library()


def _check(code: int, target: str = "core") -> None:
    if code:
        raise KernelError(library(target).ia_last_error().decode("utf-8", "replace"))


def _stream() -> int:
    # (the raw handle straight from the runtime: `torch.cuda.current_stream()` builds a Python object around it, 3 us
    # a kernel call)
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    """A tensor's address as the entry points take it (their argument types are declared: see `_declarations`)."""
    return None if t is None else t.data_ptr()


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}") from None


def _dev(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is not None and (not t.is_cuda or not t.is_contiguous()):
            raise KernelError("kernel operands must be contiguous GPU tensors "
                              f"(got device={t.device}, contiguous={t.is_contiguous()}, shape={tuple(t.shape)})")


def _i32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32:
        raise KernelError(f"{name} must be int32, got {t.dtype}")


def _f32(t: Optional[torch.Tensor], name: str) -> None:
    if t is not None and t.dtype != torch.float32:
        raise KernelError(f"{name} must be float32, got {t.dtype}")


# ---- embedding, gathers ---------------------------------------------------------------------

def embed_gather(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    _dev(table, ids); _i32(ids, "ids")
    vocab, hidden = table.shape
    n = ids.numel()
    out = torch.empty((n, hidden), dtype=table.dtype, device=table.device)
    _check(library().ia_embed_gather(_p(out), _p(table), _p(ids), n, hidden, vocab, _dt(table), _stream()))
    return out


def gather_rows(x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    _dev(x, rows); _i32(rows, "rows")
    n, cols = rows.numel(), x.shape[-1]
    out = torch.empty((n, cols), dtype=x.dtype, device=x.device)
    _check(library().ia_gather_rows(_p(out), _p(x), _p(rows), n, cols, _dt(x), _stream()))
    return out


# ---- norms ----------------------------------------------------------------------------------

def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, add_one: bool = False) -> torch.Tensor:
    _dev(x, w); _f32(w, "norm weight")
    cols = x.shape[-1]
    if w.numel() != cols:
        raise KernelError(f"rmsnorm: weight has {w.numel()} entries, rows have {cols}")
    rows = x.numel() // cols
    out = torch.empty_like(x)
    _check(library().ia_rmsnorm(_p(out), _p(x), _p(w), ctypes.c_float(eps), rows, cols, int(add_one),
                                _dt(x), _stream()))
    return out


def add_rmsnorm(x: torch.Tensor, delta: torch.Tensor, w: torch.Tensor, eps: float,
                add_one: bool = False) -> torch.Tensor:
    """x += delta in place (summed in 32-bit); returns rmsnorm(x)."""
    _dev(x, delta, w); _f32(w, "norm weight")
    if x.shape != delta.shape or x.dtype != delta.dtype:
        raise KernelError(f"add_rmsnorm: x {tuple(x.shape)} {x.dtype} and delta {tuple(delta.shape)} {delta.dtype} differ")
    cols = x.shape[-1]
    if w.numel() != cols:
        raise KernelError(f"add_rmsnorm: weight has {w.numel()} entries, rows have {cols}")
    rows = x.numel() // cols
    out = torch.empty_like(x)
    _check(library().ia_add_rmsnorm(_p(out), _p(x), _p(delta), _p(w), ctypes.c_float(eps), rows, cols,
                                    int(add_one), _dt(x), _stream()))
    return out


def add_inplace(x: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _dev(x, delta)
    if x.shape != delta.shape or x.dtype != delta.dtype:
        raise KernelError("add_inplace: operands differ in shape or dtype")
    _check(library().ia_add_inplace(_p(x), _p(delta), ctypes.c_longlong(x.numel()), _dt(x), _stream()))
    return x


# The activations a gated feed-forward may name, and their numbers in the kernels' `dual` / `act` argument
# (0 there: a plain product).  "gelu_tanh" is GELU in its tanh form, x / 2 * (1 + tanh(sqrt(2 / pi) * (x + 0.044715 x^3))).
ACTIVATIONS: Dict[str, int] = {"silu": 1, "gelu_tanh": 2}


def activation_code(activation: str) -> int:
    try:
        return ACTIVATIONS[activation]
    except KeyError:
        raise KernelError(f"no kernel has the activation {activation!r}; known: {sorted(ACTIVATIONS)}") from None


def gate_mul(gu: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """rows of [gate | up] -> act(gate) * up."""
    _dev(gu)
    if gu.shape[-1] % 2:
        raise KernelError(f"gate_mul: last dimension {gu.shape[-1]} must be even")
    inter = gu.shape[-1] // 2
    rows = gu.numel() // (2 * inter)
    out = torch.empty((*gu.shape[:-1], inter), dtype=gu.dtype, device=gu.device)
    _check(library().ia_gate_mul(_p(out), _p(gu), rows, inter, activation_code(activation), _dt(gu), _stream()))
    return out


def silu_mul(gu: torch.Tensor) -> torch.Tensor:
    """rows of [gate | up] -> silu(gate) * up."""
    return gate_mul(gu, "silu")


def add_bias(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x[row] += bias in place, for products whose kernel has no place for a bias."""
    _dev(x, bias)
    cols = x.shape[-1]
    if bias.numel() != cols or bias.dtype != x.dtype:
        raise KernelError(f"add_bias: a bias of {bias.numel()} {bias.dtype} entries for rows of {cols} {x.dtype}")
    _check(library().ia_add_bias(_p(x), _p(bias), x.numel() // cols, cols, _dt(x), _stream()))
    return x


# ---- position encoding ----------------------------------------------------------------------

def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    _dev(positions, inv_freq); _i32(positions, "positions"); _f32(inv_freq, "inv_freq")
    n, half = positions.numel(), inv_freq.numel()
    cos = torch.empty((n, half), dtype=torch.float32, device=positions.device)
    sin = torch.empty_like(cos)
    _check(library().ia_rope_table(_p(cos), _p(sin), _p(positions), _p(inv_freq), n, half, _stream()))
    return cos, sin


def qk_rope_kv(qkv: torch.Tensor, nq: int, nkv: int, d: int, *,
               q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor],
               eps: float, add_one: bool, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
               rot: int, interleaved: bool, k_cache: Optional[torch.Tensor],
               v_cache: Optional[torch.Tensor], slots: Optional[torch.Tensor],
               page_size: int) -> torch.Tensor:
    """Norm and rotate q and k, write k and v at `slots` of the cache; returns q [n, nq, d]."""
    _dev(qkv, q_norm_w, k_norm_w, cos, sin, k_cache, v_cache, slots)
    _f32(q_norm_w, "q_norm weight"); _f32(k_norm_w, "k_norm weight"); _f32(cos, "cos"); _f32(sin, "sin")
    n = qkv.shape[0]
    if qkv.dim() != 2 or qkv.shape[1] != (nq + 2 * nkv) * d:
        raise KernelError(f"qk_rope_kv: qkv has shape {tuple(qkv.shape)}, expected [n, {(nq + 2 * nkv) * d}]")
    for w, name in ((q_norm_w, "q_norm"), (k_norm_w, "k_norm")):
        if w is not None and w.numel() != d:
            raise KernelError(f"qk_rope_kv: {name} weight has {w.numel()} entries, head_dim is {d}")
    if cos is not None:
        if sin is None or cos.shape != (n, rot // 2) or sin.shape != cos.shape:
            raise KernelError(f"qk_rope_kv: rotary tables must be [{n}, {rot // 2}]")
    if slots is not None:
        _i32(slots, "slots")
        if k_cache is None or v_cache is None:
            raise KernelError("qk_rope_kv: slots given without a cache")
        if slots.numel() != n:
            raise KernelError(f"qk_rope_kv: {slots.numel()} slots for {n} tokens")
        _check_cache(k_cache, v_cache, nkv, page_size, d, qkv.dtype, "qk_rope_kv")
    q_out = torch.empty((n, nq, d), dtype=qkv.dtype, device=qkv.device)
    _check(library().ia_qk_rope_kv(
        _p(q_out), _p(k_cache if slots is not None else None), _p(v_cache if slots is not None else None),
        _p(qkv), _p(q_norm_w), _p(k_norm_w), _p(cos), _p(sin), _p(slots), n, nq, nkv, d, rot,
        int(interleaved), page_size, ctypes.c_float(eps), int(add_one), _dt(qkv), _stream()))
    return q_out


# ---- attention --------------------------------------------------------------------------------

def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, page_size: int, d: int,
                 dtype: torch.dtype, who: str) -> None:
    """Keys [pages, nkv, page_size, d]; values transposed inside a page, [pages, nkv, d, page_size]."""
    if (k_cache.dtype != dtype or v_cache.dtype != dtype or k_cache.dim() != 4 or v_cache.dim() != 4
            or tuple(k_cache.shape[1:]) != (nkv, page_size, d) or tuple(v_cache.shape[1:]) != (nkv, d, page_size)
            or k_cache.shape[0] != v_cache.shape[0]):
        raise KernelError(f"{who}: cache has shapes {tuple(k_cache.shape)} {k_cache.dtype} and "
                          f"{tuple(v_cache.shape)} {v_cache.dtype}, expected [pages, {nkv}, {page_size}, {d}] "
                          f"and [pages, {nkv}, {d}, {page_size}] {dtype}")


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      positions: torch.Tensor, token_seq: torch.Tensor, block_table: torch.Tensor,
                      *, window: Optional[int], scale: float, max_kv_len: Optional[int] = None,
                      split: Optional[bool] = None) -> torch.Tensor:
    """q [n, nq, d] against the paged cache; token i sees the keys at positions <= positions[i]
    (and > positions[i] - window) of row token_seq[i] of the table.  Any head size up to 512, any
    page size, 32-bit or bfloat16 storage, all arithmetic in 32-bit.  `max_kv_len`: an upper bound of
    positions + 1 (default: what the table can hold).  Steps of few tokens run a wave a segment of 512 keys
    and a merge kernel (`split`; None: the kernel's own rule); the bits are the same either way."""
    _dev(q, k_cache, v_cache, positions, token_seq, block_table)
    _i32(positions, "positions"); _i32(token_seq, "token_seq"); _i32(block_table, "block_table")
    n, nq, d = q.shape
    nkv, page_size = k_cache.shape[1], k_cache.shape[2]
    _check_cache(k_cache, v_cache, nkv, page_size, d, q.dtype, "attention")
    if positions.numel() != n or token_seq.numel() != n or block_table.dim() != 2:
        raise KernelError("attention: positions, token_seq and block_table do not fit the batch")
    capacity = block_table.shape[1] * page_size
    max_kv_len = capacity if max_kv_len is None else min(int(max_kv_len), capacity)
    out = torch.empty_like(q)
    lib = library()
    ws_floats = lib.ia_attention_generic_workspace(n, nq, nkv, d, max_kv_len) if split is not False else 0
    if split and not ws_floats:
        raise KernelError("attention: a step of this many tokens, or of so few keys, is not split")
    ws = torch.empty((ws_floats,), dtype=torch.float32, device=q.device) if ws_floats else None
    _check(lib.ia_attention_generic(
        _p(out), _p(q), _p(k_cache), _p(v_cache), _p(positions), _p(token_seq), _p(block_table), n,
        block_table.shape[1], nq, nkv, d, page_size, int(window or 0), ctypes.c_float(scale), _dt(q),
        _p(ws), max_kv_len, _stream()))
    return out


ATTN_TARGET_WAVES = 2048       # waves wanted in flight before the keys stop being split
ATTN_MIN_CHUNK = 64            # fewest keys a split is worth


def attention_mfma_fits(dtype: torch.dtype, d: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and d in _build.ATTN_HEAD_DIMS and page_size % 16 == 0


ATTN_TILE_COLS = 128           # head size 128, prompt portions: columns a block of four waves
ATTN_TILE_BLOCKS = 256         # blocks wanted (one a compute unit: eight waves) before the keys stop being split
ATTN_TILE_MIN_CHUNK = 512      # fewest keys a block's share is worth (eight stages of 64)
ATTN_TILE_WHOLE_UP_TO = 2048   # contexts up to this length are not split


def attention_split(n_seqs: int, nkv: int, g: int, max_q_len: int, max_kv_len: int, d: int = 0) -> Tuple[int, int]:
    """(splits, keys per split) for the matrix-core kernel: the keys are split between waves
    when the batch alone has too few (request, kv head, column block) items to fill the chip."""
    cols = max_q_len * g
    if d == 128 and cols >= ATTN_TILE_COLS:
        if 2 * max_q_len > max_kv_len or max_kv_len <= ATTN_TILE_WHOLE_UP_TO:
            # whole prompts and portions that span most of their context: a block's walk ends at its own tokens, so
            # the later splits of the early blocks are empty and the partial sums of every row go through memory for
            # nothing (16 query and 8 key/value heads, 1,024 tokens, 128 blocks: 25.6 us whole against 28.2 in two
            # splits; 2,048 tokens 44 against 63; 32 query heads, 512 tokens 18 against 26); short contexts likewise: the
            # walks are short, and where the blocks are few the kernel halves them instead (a portion of 512 tokens at
            # a context of 2,048, 32 query heads: 29.7 us whole in blocks of 64 columns against 36.8 in two splits)
            return 1, -(-max_kv_len // 64) * 64
        items = n_seqs * nkv * -(-cols // ATTN_TILE_COLS)
        splits = 1
        while items * splits < ATTN_TILE_BLOCKS and max_kv_len >= 2 * splits * ATTN_TILE_MIN_CHUNK and splits < 128:
            splits *= 2
        chunk = -(-max_kv_len // splits)
        return splits, -(-chunk // 64) * 64
    col_blocks = 1 if cols <= 16 else -(-cols // 32)
    items = n_seqs * nkv * col_blocks
    splits = 1
    while items * splits < ATTN_TARGET_WAVES and max_kv_len >= 2 * splits * ATTN_MIN_CHUNK and splits < 128:
        splits *= 2
    chunk = -(-max_kv_len // splits)
    chunk = -(-chunk // 32) * 32
    return splits, chunk


DECODE_WAVES = 1024            # the decode kernel holds a wave a SIMD: as many waves as the chip has SIMDs, no more
DECODE_MIN_CHUNK = 64          # fewest keys a wave's share is worth (two steps of 32); 128 up to a context of 512
DECODE_MANY_SPLITS = 32        # more splits than these only where a split would still hold more than 128 keys


def decode_split(n_seqs: int, nkv: int, g: int, max_kv_len: int) -> Tuple[int, int]:
    """(splits, keys per split) for the decode kernel: the largest power of two that keeps the step's waves
    (request x kv head x 16 query heads x split) within one round of the chip and a wave's share at 64 keys
    or more; beyond 32 splits (eight blocks to merge) only where a share would exceed 128 keys.  Measured at head
    size 128, 32 query and 8 kv heads, context 8,192 (microseconds a layer): batch 1
    18.0 with 64 splits against 20.0 with 128, batch 3 27.6 with 32 against 34.1 with 64, batch 8 52.4 with 16
    against 55.5 with 32, batch 64 358 with 2 against 375 with 4.  Shares of 64 keys against 128, the kernel called
    back to back in a graph: batch 1 at a context of 1,024 11.3 against 13.0, of 2,048 12.4 against 13.7; batch 4
    at 2,048 14.3 against 15.9; batch 8 at 1,024 13.3 against 14.6; at a context of 512 four splits are as good as
    any (10.8), and 64 splits of 64 keys at 4,096 lose to 32 of 128 (batch 2: 17.0 against 16.0)."""
    items = n_seqs * nkv * -(-g // 16)
    min_chunk = DECODE_MIN_CHUNK if max_kv_len > 512 else 128
    splits = 1
    while items * splits * 2 <= DECODE_WAVES and max_kv_len >= 2 * splits * min_chunk and splits < 128:
        if splits >= DECODE_MANY_SPLITS and max_kv_len <= splits * 128:
            break
        splits *= 2
    chunk = -(-max_kv_len // splits)
    return splits, -(-chunk // 32) * 32


def attention_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, positions: torch.Tensor,
                   cu_tokens: torch.Tensor, block_table: torch.Tensor, *, max_q_len: int, max_kv_len: int,
                   window: Optional[int], scale: float, splits: Optional[int] = None,
                   seqs: Optional[Tuple[int, int]] = None, tokens: Optional[Tuple[int, int]] = None,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The matrix-core kernel: bfloat16, head sizes in steps of 16 up to 256, page sizes in steps
    of 16.  Request s owns tokens cu_tokens[s]..cu_tokens[s+1] at consecutive positions.  `seqs` =
    (first, count) and `tokens` = (first, count) restrict the call to a run of requests and their
    tokens (the whole step by default); `max_q_len` and `max_kv_len` are the largest token count of
    one of these requests in this step and their largest length after it.  `out` receives the result
    (rows outside `tokens` are left alone)."""
    _dev(q, k_cache, v_cache, positions, cu_tokens, block_table, out)
    _i32(positions, "positions"); _i32(cu_tokens, "cu_tokens"); _i32(block_table, "block_table")
    n, nq, d = q.shape
    nkv, page_size = k_cache.shape[1], k_cache.shape[2]
    _check_cache(k_cache, v_cache, nkv, page_size, d, q.dtype, "attention")
    if not attention_mfma_fits(q.dtype, d, page_size):
        raise KernelError(f"attention_mfma: takes bfloat16, head sizes {_build.ATTN_HEAD_DIMS[0]}.."
                          f"{_build.ATTN_HEAD_DIMS[-1]} in steps of 16 and page sizes in steps of 16; got "
                          f"{q.dtype}, head size {d}, page size {page_size}")
    all_seqs = cu_tokens.numel() - 1
    seq_begin, n_seqs = seqs if seqs is not None else (0, all_seqs)
    token_begin, n_tokens = tokens if tokens is not None else (0, n)
    if (positions.numel() != n or block_table.dim() != 2 or block_table.shape[0] < all_seqs or nq % nkv
            or seq_begin < 0 or seq_begin + n_seqs > all_seqs or token_begin < 0 or token_begin + n_tokens > n):
        raise KernelError("attention_mfma: positions, cu_tokens, block_table and the ranges do not fit the batch")
    if max_kv_len > block_table.shape[1] * page_size or max_q_len < 1 or max_q_len > max(n_tokens, 1):
        raise KernelError(f"attention_mfma: max_kv_len {max_kv_len} / max_q_len {max_q_len} do not fit "
                          f"{block_table.shape[1]} pages of {page_size} and {n_tokens} tokens")
    if out is None:
        out = torch.empty_like(q)
    elif out.shape != q.shape or out.dtype != q.dtype:
        raise KernelError("attention_mfma: `out` must have the shape and dtype of q")
    if splits is None:
        splits, chunk = attention_split(n_seqs, nkv, nq // nkv, max_q_len, max_kv_len, d)
    else:
        chunk = -(-(-(-max_kv_len // splits)) // 64) * 64
    target = _build.attn_target(d)
    lib = library(target)
    ws_floats = lib.ia_attention_mfma_workspace(n, nq, splits)
    ws = torch.empty((ws_floats,), dtype=torch.float32, device=q.device) if ws_floats else None
    _check(lib.ia_attention_mfma(
        _p(out), _p(ws), _p(q), _p(k_cache), _p(v_cache), _p(block_table), _p(cu_tokens), _p(positions),
        n, seq_begin, n_seqs, token_begin, n_tokens, max_q_len, max_kv_len, block_table.shape[1], nq, nkv, d,
        page_size, int(window or 0), ctypes.c_float(scale), splits, chunk, _stream()), target)
    return out


# The decode kernel's counters: zero between calls (the kernel puts them back).  One array a device: calls that
# share it must follow each other (one stream, or a graph replayed on it), as an engine's steps do.
_DECODE_COUNTERS: Dict[int, torch.Tensor] = {}
_DECODE_COUNTERS_OUTGROWN: list = []                # captured graphs may still hold their addresses: never freed
DECODE_COUNTERS_MIN = 1 << 16


def _decode_counters(device: torch.device, needed: int) -> Optional[torch.Tensor]:
    if needed <= 0:
        return None
    key = device.index if device.index is not None else torch.cuda.current_device()
    have = _DECODE_COUNTERS.get(key)
    if have is None or have.numel() < needed:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("attention_decode_fused: the counters of the decode kernel cannot be allocated under "
                              "graph capture; run a step of this size once before capturing it")
        if have is not None:
            _DECODE_COUNTERS_OUTGROWN.append(have)
        have = torch.zeros((max(DECODE_COUNTERS_MIN, 2 * needed),), dtype=torch.int32, device=device)
        _DECODE_COUNTERS[key] = have
    return have


def attention_decode_fused_fits(dtype: torch.dtype, d: int, page_size: int, rot: int, interleaved: bool,
                                has_rotation: bool) -> bool:
    """Whether decode steps can take `attention_decode_fused`: what the matrix-core kernel takes, head sizes
    in steps of 64, and a rotation (if any) of whole heads with halves paired."""
    return (attention_mfma_fits(dtype, d, page_size) and d % 64 == 0
            and (not has_rotation or (rot == d and not interleaved)))


def attention_decode_fused(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, positions: torch.Tensor,
                           cu_tokens: torch.Tensor, block_table: torch.Tensor, *, nq: int, nkv: int, d: int,
                           slots: Optional[torch.Tensor], q_norm_w: Optional[torch.Tensor],
                           k_norm_w: Optional[torch.Tensor], eps: float, add_one: bool,
                           cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], max_kv_len: int,
                           window: Optional[int], scale: float, splits: Optional[int] = None,
                           seqs: Optional[Tuple[int, int]] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Decode steps (one token a request) in one kernel: per-head norm of q and k, rotation, the write
    of the new key and value at `slots` (None: the cache is only read) and the attention over the pages.
    `qkv` [n, (nq + 2 nkv) * d] is the projections' output; request s owns token s.  Returns [n, nq, d]."""
    _dev(qkv, k_cache, v_cache, positions, cu_tokens, block_table, slots, q_norm_w, k_norm_w, cos, sin, out)
    _i32(positions, "positions"); _i32(cu_tokens, "cu_tokens"); _i32(block_table, "block_table")
    _f32(q_norm_w, "q_norm weight"); _f32(k_norm_w, "k_norm weight"); _f32(cos, "cos"); _f32(sin, "sin")
    n = qkv.shape[0]
    page_size = k_cache.shape[2]
    _check_cache(k_cache, v_cache, nkv, page_size, d, qkv.dtype, "attention_decode_fused")
    if not attention_decode_fused_fits(qkv.dtype, d, page_size, d, False, cos is not None):
        raise KernelError(f"attention_decode_fused: takes bfloat16, head sizes in steps of 64 and page sizes in "
                          f"steps of 16; got {qkv.dtype}, head size {d}, page size {page_size}")
    if qkv.dim() != 2 or qkv.shape[1] != (nq + 2 * nkv) * d or nq % nkv:
        raise KernelError(f"attention_decode_fused: qkv has shape {tuple(qkv.shape)}, expected [n, {(nq + 2 * nkv) * d}]")
    all_seqs = cu_tokens.numel() - 1
    seq_begin, n_seqs = seqs if seqs is not None else (0, all_seqs)
    if (positions.numel() != n or block_table.dim() != 2 or block_table.shape[0] < all_seqs or seq_begin < 0
            or seq_begin + n_seqs > all_seqs or seq_begin + n_seqs > n):
        raise KernelError("attention_decode_fused: positions, cu_tokens, block_table and the range do not fit the batch")
    if max_kv_len > block_table.shape[1] * page_size:
        raise KernelError(f"attention_decode_fused: max_kv_len {max_kv_len} does not fit {block_table.shape[1]} pages")
    for w, name in ((q_norm_w, "q_norm"), (k_norm_w, "k_norm")):
        if w is not None and w.numel() != d:
            raise KernelError(f"attention_decode_fused: {name} weight has {w.numel()} entries, head_dim is {d}")
    if (q_norm_w is None) != (k_norm_w is None) or (cos is None) != (sin is None):
        raise KernelError("attention_decode_fused: norm weights and angle tables come in pairs")
    if cos is not None and (cos.shape != (n, d // 2) or sin.shape != cos.shape):
        raise KernelError(f"attention_decode_fused: rotary tables must be [{n}, {d // 2}]")
    if slots is not None:
        _i32(slots, "slots")
        if slots.numel() != n:
            raise KernelError(f"attention_decode_fused: {slots.numel()} slots for {n} tokens")
    if out is None:
        out = torch.empty((n, nq, d), dtype=qkv.dtype, device=qkv.device)
    elif tuple(out.shape) != (n, nq, d) or out.dtype != qkv.dtype:
        raise KernelError("attention_decode_fused: `out` must be [n, nq, d] in the dtype of qkv")
    if splits is None:
        splits, chunk = decode_split(n_seqs, nkv, nq // nkv, max_kv_len)
    else:
        chunk = -(-(-(-max_kv_len // splits)) // 32) * 32
    if splits & (splits - 1):
        raise KernelError(f"attention_decode_fused: the keys are split 2^k ways, not {splits}")
    target = _build.attn_target(d)
    lib = library(target)
    ws_floats = lib.ia_attention_decode_workspace(n, nq, nkv, splits)
    ws = torch.empty((ws_floats,), dtype=torch.float32, device=qkv.device) if ws_floats else None
    counters = _decode_counters(qkv.device, lib.ia_attention_decode_counters(n, nq, nkv, splits))
    _check(lib.ia_attention_mfma_decode_fused(
        _p(out), _p(ws), _p(qkv), _p(k_cache), _p(v_cache), _p(block_table), _p(cu_tokens), _p(positions), _p(slots),
        _p(q_norm_w), _p(k_norm_w), _p(cos), _p(sin), ctypes.c_float(eps), int(add_one), n, seq_begin, n_seqs,
        seq_begin, n_seqs, max_kv_len, block_table.shape[1], nq, nkv, d, page_size, int(window or 0),
        ctypes.c_float(scale), splits, chunk, _p(counters), counters.numel() if counters is not None else 0,
        _stream()), target)
    return out


# ---- matrix products --------------------------------------------------------------------------

# Beyond this many rows (one tile of MFMA columns) the vendor's GEMM reads the weights faster.  Up to 16 rows the
# skinny products also take over the sums and norms of the residual stream; a decode step at a context of 2,048
# and the sizes of an 8 B model takes 5.02 ms with 12 requests, 5.20 with 13 and 5.22 with 16 (5.54 and 5.44 with
# the vendor's GEMM and norm kernels of their own from 13 rows on; at the 14B shape 9.7 against 10.9 ms at 14 rows).
SKINNY_MAX_ROWS = 16


# Who multiplies more bfloat16 rows than the skinny kernel takes: "library" (the vendor's GEMM, as the reference's
# products go to cuBLAS) or "own" (the tiled matrix-core kernel of this package, where the width is a multiple of
# 64).  The library is faster at the sizes of an 8 B model (2,048 rows: 84, 60, 335 with SiLU and 168 us for qkv, o,
# gate|up and down against 125, 119, 435 and 323 us), so it is the default; INFERRS_AMD_LARGE_PRODUCTS=own
# runs the model without it.
LARGE_PRODUCTS = os.environ.get("INFERRS_AMD_LARGE_PRODUCTS", "library")


# How the vendor's GEMM is called: "direct" (hipBLASLt through this package's own entry point, which keeps descriptors,
# layouts and the library's choice of kernel for every shape: 7 us of host time a product) or "torch" (`F.linear`:
# 18 us a product whatever its size, more than the GPU needs for the products of a small model).  "direct" falls back
# to "torch", with a warning, where the library cannot be opened.
VENDOR_GEMM = os.environ.get("INFERRS_AMD_VENDOR_GEMM", "direct")
VENDOR_WORKSPACE_BYTES = 128 << 20
_VENDOR_STATE: Dict[str, object] = {}


def _vendor_library_path() -> Optional[str]:
    """The hipBLASLt that this process has loaded (torch brings its own copy), else torch's, else the system's."""
    try:
        with open("/proc/self/maps") as f:
            for line in f:
                if "libhipblaslt.so" in line:
                    return line.split(None, 5)[-1].strip()
    except OSError:
        pass
    for path in (os.path.join(os.path.dirname(torch.__file__), "lib", "libhipblaslt.so"), "/opt/rocm/lib/libhipblaslt.so"):
        if os.path.exists(path):
            return path
    return None


def _vendor_direct() -> bool:
    if VENDOR_GEMM not in ("direct", "torch"):
        raise KernelError(f"INFERRS_AMD_VENDOR_GEMM / ops.VENDOR_GEMM: 'direct' or 'torch', not {VENDOR_GEMM!r}")
    if VENDOR_GEMM == "torch":
        return False
    if "ready" not in _VENDOR_STATE:
        path = _vendor_library_path()
        lib = _raw_library()
        ok = path is not None and lib.ia_vendor_gemm_init(path.encode()) == 0
        if not ok:
            import logging
            logging.getLogger("inferrs_amd").warning(
                "the vendor's GEMM library could not be opened directly (%s): its products go through torch",
                lib.ia_last_error().decode() if path is not None else "libhipblaslt.so not found")
        _VENDOR_STATE["ready"] = ok
    return bool(_VENDOR_STATE["ready"])


def vendor_gemm_bf16(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x [m, k] . w[n, k]^T in bfloat16 through the vendor's GEMM library."""
    if not _vendor_direct() or x.shape[0] == 0:
        return torch.nn.functional.linear(x, w)
    _dev(x, w)
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"vendor_gemm: x {tuple(x.shape)} {x.dtype} does not fit w {tuple(w.shape)} {w.dtype}")
    if not (x.is_contiguous() and w.is_contiguous()):
        raise KernelError("vendor_gemm: operands must be contiguous")
    key = ("workspace", x.device.index)
    ws = _VENDOR_STATE.get(key)
    if ws is None:
        if torch.cuda.is_current_stream_capturing():
            # (the library's handle and the workspace are made outside a capture: a product that is the first of its
            # process and is being captured goes through torch)
            return torch.nn.functional.linear(x, w)
        ws = _VENDOR_STATE[key] = torch.empty((VENDOR_WORKSPACE_BYTES,), dtype=torch.uint8, device=x.device)
        warm = torch.zeros((16, 64), dtype=torch.bfloat16, device=x.device)
        if _raw_library().ia_vendor_gemm_bf16(_p(torch.empty((16, 16), dtype=torch.bfloat16, device=x.device)), _p(warm),
                                              _p(warm), 16, 16, 64, _p(ws), ws.numel(), _stream()) == 1:
            _check(1)
    refused = _VENDOR_STATE.setdefault("refused", set())
    if (m, n, k) in refused:
        return torch.nn.functional.linear(x, w)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    code = _raw_library().ia_vendor_gemm_bf16(_p(out), _p(x), _p(w), m, n, k, _p(ws), ws.numel(), _stream())
    if code == 2:                                    # the library's search names no kernel for this shape (an odd k)
        refused.add((m, n, k))
        return torch.nn.functional.linear(x, w)
    _check(code)
    return out


def _own_large(x: torch.Tensor, w: torch.Tensor) -> bool:
    if LARGE_PRODUCTS not in ("library", "own"):
        raise KernelError(f"INFERRS_AMD_LARGE_PRODUCTS / ops.LARGE_PRODUCTS: 'library' or 'own', not {LARGE_PRODUCTS!r}")
    return (LARGE_PRODUCTS == "own" and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] % 64 == 0
            and x.is_contiguous() and w.is_contiguous())


def gemm_mfma_bf16(x: torch.Tensor, w: torch.Tensor, dual: bool = False, activation: str = "silu") -> torch.Tensor:
    """x [m, k] . w[n, k]^T in bfloat16 by the tiled matrix-core kernel (k a multiple of 64); with `dual`
    w is [gate; up] and the result act(x . gate^T) * (x . up^T)."""
    _dev(x, w)
    m, k = x.shape
    rows, k2 = w.shape
    if k2 != k or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or k % 64 or (dual and rows % 2):
        raise KernelError(f"gemm_mfma: x {tuple(x.shape)} {x.dtype} does not fit w {tuple(w.shape)} {w.dtype}")
    if not (x.is_contiguous() and w.is_contiguous()):
        raise KernelError("gemm_mfma: operands must be contiguous")
    n = rows // 2 if dual else rows
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    if m:
        _check(library().ia_gemm_mfma_bf16(_p(out), _p(x), _p(w), m, n, k, activation_code(activation) if dual else 0,
                                           _stream()))
    return out


def gemm_tiled(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    _dev(x, w)
    m, k = x.shape
    n, k2 = w.shape
    if k != k2 or x.dtype != w.dtype:
        raise KernelError(f"gemm: x {tuple(x.shape)} {x.dtype} does not fit w {tuple(w.shape)} {w.dtype}")
    out_dtype = out_dtype or x.dtype
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _check(library().ia_gemm_tiled(_p(out), _p(x), _p(w), m, n, k, _dt(x), _DT[out_dtype], _stream()))
    return out


def _skinny_bias(bias: Optional[torch.Tensor], rows: int) -> None:
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != rows or not bias.is_cuda
                             or not bias.is_contiguous()):
        raise KernelError(f"gemm_skinny: the bias must be a contiguous bfloat16 vector of {rows} entries on the GPU")


def gemm_skinny_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                     dual: bool = False, activation: str = "silu", bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [m, k] . w[n, k]^T (+ bias) on the matrix cores, made for few rows.  `dual`: w is [gate; up]
    stacked along its rows and the result is act(x . gate^T + bias[:n]) * (x . up^T + bias[n:])."""
    _dev(x, w)
    _skinny_bias(bias, w.shape[0])
    m, k = x.shape
    n, k2 = w.shape
    if k != k2 or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"gemm_skinny: x {tuple(x.shape)} {x.dtype} does not fit w {tuple(w.shape)} {w.dtype}")
    if dual:
        if n % 2:
            raise KernelError(f"gemm_skinny: a stacked [gate; up] weight needs an even row count, got {n}")
        n //= 2
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _check(library().ia_gemm_skinny_bf16(_p(out), _p(x), _p(w), _p(bias), m, n, k, _DT[out_dtype],
                                         activation_code(activation) if dual else 0, _stream()))
    return out


def skinny_fits(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and (x.data_ptr() | w.data_ptr()) % 16 == 0)


def fill_normal(shape, seed: int, mean: float, std: float, dtype: torch.dtype, device) -> torch.Tensor:
    """A tensor of mean + std * N(0, 1), element i a function of (seed, i) alone; the same values
    as the host fill of `inferrs_amd.weights.random_init`."""
    require_gpu()
    out = torch.empty(tuple(shape), dtype=dtype, device=device)
    _check(library().ia_fill_normal(_p(out), ctypes.c_longlong(out.numel()), ctypes.c_ulonglong(seed & (2**64 - 1)),
                                    ctypes.c_double(mean), ctypes.c_double(std), _dt(out), _stream()))
    return out


def stream_read(x: torch.Tensor, blocks: int = 4096) -> torch.Tensor:
    """Reads all of `x` once (a multiple of 16 bytes), a contiguous range a block: the measurement script times it for
    the memory's practical read rate.  (The returned words are scratch.)"""
    _dev(x)
    nbytes = x.numel() * x.element_size()
    out = torch.zeros((blocks,), dtype=torch.int32, device=x.device)
    _check(library().ia_stream_read(_p(out), _p(x), ctypes.c_longlong(nbytes), blocks, _stream()))
    return out


def widen(x: torch.Tensor) -> torch.Tensor:
    """bfloat16 -> float32, exactly."""
    _dev(x)
    if x.dtype != torch.bfloat16:
        raise KernelError(f"widen: takes bfloat16, got {x.dtype}")
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _check(library().ia_widen_bf16(_p(out), _p(x), ctypes.c_longlong(x.numel()), _stream()))
    return out


# ---- a residual stream around the skinny product ---------------------------------------------
# Decode steps have a few rows, and a kernel of its own that adds a product to the stream and norms the
# sum is all launch and latency.  The product before such a norm can add itself to the stream
# (`linear_add`): it leaves every row's sum of squares, block by block, and the new rows times the
# norm's weight; the product after the norm (`linear` / `gated_silu_linear` given `NormedRows`) takes
# those rows and multiplies its sums by the row's scale, rsqrt(mean of squares + eps).

STREAM_MAX_ROWS = 16          # rows up to which the products take over the sums and norms of a step


class Added:
    """What a part returns instead of its output when it has added it to the step's stream itself:
    `sums` [rows, blocks] are the partial sums of squares of the stream's new rows and `scaled` the
    new rows times the weight of `norm` (the norm part that comes next), or None."""
    __slots__ = ("sums", "scaled", "norm")

    def __init__(self, sums: torch.Tensor, scaled: Optional[torch.Tensor] = None, norm=None):
        self.sums, self.scaled, self.norm = sums, scaled, norm


class NormedRows:
    """Rows of a stream `x` whose norm, rmsnorm(x; weight, eps), is left to the product that reads them:
    `scaled` = x * weight (rounded once) and `sums` [rows, blocks] the rows' sums of squares."""
    __slots__ = ("x", "scaled", "sums", "weight", "eps", "add_one")

    def __init__(self, x: torch.Tensor, scaled: torch.Tensor, sums: torch.Tensor, weight: torch.Tensor, eps: float,
                 add_one: bool):
        self.x, self.scaled, self.sums, self.weight = x, scaled, sums, weight
        self.eps, self.add_one = float(eps), bool(add_one)

    @property
    def shape(self):
        return self.x.shape

    @property
    def dtype(self):
        return self.x.dtype

    def materialize(self) -> torch.Tensor:
        return rmsnorm(self.x, self.weight, self.eps, self.add_one)


def _stream_product(x: torch.Tensor, w: torch.Tensor, n: int, out_dtype, dual: bool, resid=None, sums_out=None,
                    scaled_out=None, next_w=None, add_one: bool = False, sums_in=None, eps: float = 0.0,
                    activation: str = "silu", bias: Optional[torch.Tensor] = None):
    m, k = x.shape
    _skinny_bias(bias, w.shape[0])
    out = None if resid is not None else torch.empty((m, n), dtype=out_dtype, device=x.device)
    _check(library().ia_gemm_skinny_stream(
        _p(out), _p(x), _p(w), _p(bias), m, n, k, _DT[out_dtype], activation_code(activation) if dual else 0, _p(resid),
        _p(sums_out), _p(scaled_out), _p(next_w),
        int(add_one), _p(sums_in), sums_in.shape[1] if sums_in is not None else 0, ctypes.c_float(eps), _stream()))
    return out


def _takes_normed_rows(x: NormedRows, w: torch.Tensor, n: int) -> bool:
    m, k = x.scaled.shape
    return (m <= SKINNY_MAX_ROWS and x.scaled.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.shape[1] == k
            and skinny_fits(x.scaled, w) and n < 65536 and x.sums.dtype == torch.float32 and x.sums.shape[0] == m
            and x.sums.is_contiguous() and x.scaled.is_contiguous())


def linear_add(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, next_norm=None,
               bias: Optional[torch.Tensor] = None):
    """resid += x . w^T (+ bias) in place, as `add_rmsnorm` would add the product (rounded, then summed in 32-bit
    and rounded), by the skinny kernel itself.  Returns (sums, scaled): the partial sums of squares of the
    new rows [rows, blocks], and the new rows times the weight of `next_norm` (a norm part with `weight`
    and `add_one`; None: no such rows); or None when this product cannot (the caller then forms it and
    lets the norm add it)."""
    m, k = x.shape
    n = w.shape[0]
    if (m > SKINNY_MAX_ROWS or m == 0 or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != k
            or not skinny_fits(x, w) or n >= 65536 or resid.dtype != torch.bfloat16 or tuple(resid.shape) != (m, n)
            or not resid.is_contiguous() or (bias is not None and bias.dtype != torch.bfloat16)):
        return None
    next_w = getattr(next_norm, "weight", None)
    if next_w is not None and (next_w.dtype != torch.float32 or next_w.numel() != n):
        next_w = None
    _dev(x, w, resid, next_w)
    sums = torch.empty((m, library().ia_gemm_skinny_blocks(n)), dtype=torch.float32, device=x.device)
    scaled = torch.empty_like(resid) if next_w is not None else None
    _stream_product(x, w, n, torch.bfloat16, False, resid=resid, sums_out=sums, scaled_out=scaled, next_w=next_w,
                    add_one=bool(getattr(next_norm, "add_one", False)), bias=bias)
    return sums, scaled


# ---- products of 17 to 128 rows ------------------------------------------------------------------
# Decode steps of many requests and short prompt portions: still bound by reading the weights once, which the vendor's
# GEMM does at 2 to 3.4 TB/s and the kernel of gemm_mid.hip faster.  (Sizes of an 8B model, a prompt of 128 tokens, the four
# products of a layer inside the model: 129 us against 174 through the vendor's GEMM; of 65 tokens: 108 against 182.)  Weights with few rows (the output projection, the
# feed-forward's second product) are split along k between blocks, and the splits' sums are added up by the reader:
# `Partials` stands for a product in that state.

MID_MAX_ROWS = 128            # rows up to which the products of gemm_mid.hip take over from the vendor's GEMM
# Rows from which a layer's products go to gemm_mid.hip, with kernels of their own for the sums of the splits and the norms,
# instead of the skinny products that take over the stream's sums and norms: None = by the rule of `mid_from_rows`.
MID_FROM_ROWS: Optional[int] = None
MID_MIN_ROWS = 5              # fewest rows for which a split product is worth the kernel that adds it up


def mid_from_rows(width: int) -> int:
    """Rows of a step from which the products of a model of this width (the residual stream's) run on gemm_mid.hip.
    Measured, decode steps at a context of 2,048 (ms a step, skinny products against gemm_mid.hip): width 4,096 (8B
    shape) 6 rows 4.72 / 4.89, 8 rows 3.99 / 4.00, 9 rows 4.27 / 4.22, 12 rows 4.40 / 4.34, 16 rows 4.69 / 4.56; width
    5,120, where the skinny product's blocks are no whole tiles and its waves' shares of k are uneven (14B shape): 4 rows
    6.50 / 6.52, 6 rows 6.85 / 6.71, 8 rows 7.13 / 6.94, 12 rows 8.12 / 7.39, 16 rows 9.49 / 7.78 (32B shape: 8 rows 15.09 /
    14.26, 16 rows 19.10 / 15.42)."""
    if MID_FROM_ROWS is not None:
        return MID_FROM_ROWS
    return 9 if width & (width - 1) == 0 else MID_MIN_ROWS
# [gate; up] weights beyond this many bytes go to the vendor's GEMM and the SiLU kernel also at 17 to 64 rows.  Measured at 32
# rows (kernel after kernel, launch gaps included): 2 x 12,288 x 4,096 (201 MB) 49 us here against 49 + 5 us there,
# 2 x 25,600 x 5,120 (524 MB) 125 us here against 96 + 5 us there; the plain products are faster here at every size
# (5,120 x 25,600: 57 us against 147).
MID_DUAL_MAX_BYTES = 256 << 20
MID_PRODUCTS = os.environ.get("INFERRS_AMD_MID_PRODUCTS", "own")      # "own" or "library"


class Partials:
    """A product [rows, features] as the 32-bit sums of each split of k, `parts` [splits, rows, features]; whoever
    needs it adds them up in the order of the splits (`materialize()`, or `add_rmsnorm_partials`)."""
    __slots__ = ("parts",)

    def __init__(self, parts: torch.Tensor):
        self.parts = parts

    @property
    def shape(self):
        return self.parts.shape[1:]

    def materialize(self) -> torch.Tensor:
        splits, m, n = self.parts.shape
        out = torch.empty((m, n), dtype=torch.bfloat16, device=self.parts.device)
        _check(library().ia_sum_partials(_p(out), _p(self.parts), splits, m, n, _stream()))
        return out


def mid_fits(x: torch.Tensor, w: torch.Tensor, few_rows: bool = False) -> bool:
    """Whether x . w^T goes to gemm_mid.hip: from `mid_from_rows(k)` to `MID_MAX_ROWS` rows (`few_rows`: from 1 row on)."""
    if MID_PRODUCTS not in ("own", "library"):
        raise KernelError(f"INFERRS_AMD_MID_PRODUCTS / ops.MID_PRODUCTS: 'own' or 'library', not {MID_PRODUCTS!r}")
    return (MID_PRODUCTS == "own" and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and (1 if few_rows else mid_from_rows(x.shape[1])) <= x.shape[0] <= MID_MAX_ROWS
            and x.shape[1] % 128 == 0 and w.shape[1] == x.shape[1]
            and x.is_contiguous() and w.is_contiguous() and (x.data_ptr() | w.data_ptr()) % 16 == 0)


def gemm_mid_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, dual: bool = False,
                  partial: bool = False, sums_in: Optional[torch.Tensor] = None, eps: float = 0.0,
                  activation: str = "silu"):
    """x [m, k] . w[n, k]^T for 1 to 128 bfloat16 rows and k a multiple of 128 (gemm_mid.hip).  `dual`: w = [gate; up],
    the result act(x . gate^T) * (x . up^T).  `partial`: the result stays split along k, as `Partials` (a weight that
    needs no split gives a plain tensor).  `sums_in` [m, blocks] (up to 16 rows): the rows are a norm's input times its
    weight and these their sums of squares; every sum is multiplied by the row's rsqrt(mean of squares + eps)."""
    _dev(x, w)
    m, k = x.shape
    rows, k2 = w.shape
    if (k2 != k or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or k % 128 or not (1 <= m <= MID_MAX_ROWS)
            or (dual and (rows % 2 or partial or out_dtype != torch.bfloat16))):
        raise KernelError(f"gemm_mid: x {tuple(x.shape)} {x.dtype} does not fit w {tuple(w.shape)} {w.dtype} "
                          f"(1 to {MID_MAX_ROWS} rows, k a multiple of 128)")
    n = rows // 2 if dual else rows
    lib = library()
    act = activation_code(activation) if dual else 0
    if partial:
        splits = lib.ia_gemm_mid_splits(n, k)
        if splits > 1 and (m * n) % 4 == 0:
            parts = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            _check(lib.ia_gemm_mid_bf16(_p(parts), _p(x), _p(w), m, n, k, 2, 0, _stream()))
            return Partials(parts)
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    if sums_in is not None:
        _dev(sums_in); _f32(sums_in, "sums of squares")
        if partial or m > 16 or sums_in.dim() != 2 or sums_in.shape[0] != m or not sums_in.is_contiguous():
            raise KernelError(f"gemm_mid: sums of squares {tuple(sums_in.shape)} for {m} rows (up to 16, whole sums)")
        _check(lib.ia_gemm_mid_bf16_scaled(_p(out), _p(x), _p(w), m, n, k, 0 if out_dtype == torch.bfloat16 else 1,
                                           act, _p(sums_in), sums_in.shape[1], ctypes.c_float(eps), _stream()))
        return out
    _check(lib.ia_gemm_mid_bf16(_p(out), _p(x), _p(w), m, n, k, 0 if out_dtype == torch.bfloat16 else 1,
                                act, _stream()))
    return out


def linear_partials(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None):
    """x . w^T for a reader that takes `Partials` (the norm that adds the product to the stream): split along k where the
    weight has few rows.  None when the product of 17 to 64 rows does not take these operands (a bias among them: the
    caller then forms the whole product, and `linear` adds the bias)."""
    # (whoever asks is in a step whose products go to gemm_mid.hip: the rule has been asked with the stream's width, and a
    # product of another width follows it)
    if bias is None and isinstance(x, torch.Tensor) and x.shape[0] >= MID_MIN_ROWS and mid_fits(x, w, few_rows=True):
        return gemm_mid_bf16(x, w, partial=True)
    return None


def add_rmsnorm_partials(x: torch.Tensor, delta: Partials, w: torch.Tensor, eps: float, add_one: bool = False) -> torch.Tensor:
    """x += delta in place, delta's splits added up and rounded to bfloat16 first (as a stored product would be);
    returns rmsnorm(x)."""
    parts = delta.parts
    _dev(x, parts, w); _f32(w, "norm weight")
    splits, rows, cols = parts.shape
    if x.dtype != torch.bfloat16 or tuple(x.shape) != (rows, cols) or w.numel() != cols:
        raise KernelError(f"add_rmsnorm_partials: x {tuple(x.shape)} {x.dtype} does not fit the product {tuple(parts.shape)}")
    if cols % 4 or cols > 8192:
        return add_rmsnorm(x, delta.materialize(), w, eps, add_one)
    out = torch.empty_like(x)
    _check(library().ia_add_rmsnorm_partials(_p(out), _p(x), _p(parts), splits, _p(w), ctypes.c_float(eps), rows, cols,
                                             int(add_one), _stream()))
    return out


def linear(x, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None, mid: bool = True,
           bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [m, k] . w[n, k]^T (+ bias [n], in the precision of w).  32-bit: the tiled kernel (true 32-bit, fixed
    order).  bfloat16: the skinny MFMA kernel for up to SKINNY_MAX_ROWS rows, the vendor's GEMM beyond that (the
    reference uses cuBLAS for all of them).  A 32-bit result of bfloat16 operands (logits) comes straight from
    the skinny kernel's accumulators for those few rows; beyond that it is the vendor's bfloat16
    result widened, which is what the reference does for every row (its logits are computed in
    the model's precision and cast for sampling, `inferrs/src/sampler.rs:182`).  From `mid_from_rows(k)` rows on (and up to
    `MID_MAX_ROWS`) a bfloat16 result comes from gemm_mid.hip; `mid=False`: from the skinny product or the vendor's GEMM.  The skinny kernel adds a bias to its sums before it rounds them; behind every
    other product a kernel of its own adds it to the stored rows."""
    out_dtype = out_dtype or x.dtype
    if bias is not None and (bias.dtype != w.dtype or bias.numel() != w.shape[0]):
        raise KernelError(f"linear: a bias of {bias.numel()} {bias.dtype} entries for a weight {tuple(w.shape)} {w.dtype}")
    if isinstance(x, NormedRows):
        if _takes_normed_rows(x, w, w.shape[0]):
            _dev(x.scaled, w, x.sums)
            return _stream_product(x.scaled, w, w.shape[0], out_dtype, False, sums_in=x.sums, eps=x.eps, bias=bias)
        x = x.materialize()
    if x.dtype == torch.bfloat16 and skinny_fits(x, w) and x.shape[0] <= SKINNY_MAX_ROWS:
        # (rows that both kernels take: a 32-bit result, the logits head's, stays with the skinny product)
        if out_dtype != torch.bfloat16 or bias is not None or not mid or not mid_fits(x, w):
            return gemm_skinny_bf16(x, w, out_dtype, bias=bias)
    y = _linear_no_bias(x, w, out_dtype if bias is None else x.dtype, mid)
    if bias is None:
        return y
    add_bias(y, bias)
    return widen(y) if out_dtype == torch.float32 and y.dtype != torch.float32 else y


def _linear_no_bias(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, mid: bool) -> torch.Tensor:
    """The products of `linear` beyond the skinny kernel's rows."""
    if x.dtype == torch.float32:
        return gemm_tiled(x, w, out_dtype)
    m, k = x.shape
    if not skinny_fits(x, w):
        return gemm_tiled(x, w, out_dtype)
    if mid and mid_fits(x, w):
        if out_dtype == torch.float32:
            return gemm_mid_bf16(x, w, torch.float32)
        y = gemm_mid_bf16(x, w, partial=True)
        return y.materialize() if isinstance(y, Partials) else y
    _dev(x, w)
    if w.shape[1] != k or w.dtype != x.dtype:
        raise KernelError(f"gemm: x {tuple(x.shape)} {x.dtype} does not fit w {tuple(w.shape)} {w.dtype}")
    if _own_large(x, w):
        y = gemm_mfma_bf16(x, w)
    elif KernelTimer.active is not None:
        y = KernelTimer.active.call("vendor_gemm", vendor_gemm_bf16, x, w)
    else:
        y = vendor_gemm_bf16(x, w)
    return widen(y) if out_dtype == torch.float32 else y


# ---- sampling ---------------------------------------------------------------------------------

def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The lowest index among each row's maxima, int32 [rows] (into `out` when given)."""
    _dev(logits, out); _f32(logits, "logits")
    rows, vocab = logits.shape
    if out is None:
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    elif out.dtype != torch.int32 or out.numel() != rows:
        raise KernelError(f"argmax: `out` must be int32 [{rows}]")
    words = library().ia_argmax_workspace(rows, vocab)
    ws = torch.empty((words,), dtype=torch.int32, device=logits.device) if words else None
    _check(library().ia_argmax(_p(out), _p(logits), _p(ws), rows, vocab, _stream()))
    return out


def penalize(logits: torch.Tensor, window: Optional[torch.Tensor], repetition: torch.Tensor,
             frequency: torch.Tensor, presence: torch.Tensor, bias_ids: Optional[torch.Tensor] = None,
             bias_vals: Optional[torch.Tensor] = None) -> torch.Tensor:
    """In place on float32 logits [rows, vocab]: logit bias, then repetition, frequency and presence
    penalties over each row's `window` of earlier tokens (int32 [rows, w], -1 = none)."""
    _dev(logits, window, repetition, frequency, presence, bias_ids, bias_vals)
    _f32(logits, "logits"); _f32(repetition, "repetition"); _f32(frequency, "frequency"); _f32(presence, "presence")
    rows, vocab = logits.shape
    w = 0 if window is None else window.shape[1]
    nb = 0 if bias_ids is None else bias_ids.shape[1]
    if window is not None:
        _i32(window, "window")
        if window.shape[0] != rows:
            raise KernelError("penalize: one window row per row of logits")
    if (bias_ids is None) != (bias_vals is None):
        raise KernelError("penalize: bias ids and values come together")
    if bias_ids is not None:
        _i32(bias_ids, "bias_ids"); _f32(bias_vals, "bias_vals")
        if bias_ids.shape != bias_vals.shape or bias_ids.shape[0] != rows:
            raise KernelError("penalize: bias arrays must be [rows, entries]")
    for t in (repetition, frequency, presence):
        if t.numel() != rows:
            raise KernelError("penalize: one penalty value per row of logits")
    _check(library().ia_penalize(_p(logits), rows, vocab, _p(window), w, _p(repetition), _p(frequency),
                                 _p(presence), _p(bias_ids), _p(bias_vals), nb, _stream()))
    return logits


def window_push(window: torch.Tensor, caps: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """In place: every row's penalty window [rows, w] (int32, -1 = empty) takes the row's new token; row i
    keeps its last caps[i] tokens (0: no window)."""
    _dev(window, caps, tokens)
    _i32(window, "window"); _i32(caps, "caps"); _i32(tokens, "tokens")
    rows, w = window.shape
    if caps.numel() != rows or tokens.numel() != rows or not window.is_contiguous():
        raise KernelError("window_push: one cap and one token per row of a contiguous window")
    _check(library().ia_window_push(_p(window), rows, w, _p(caps), _p(tokens), _stream()))
    return window


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, u: torch.Tensor, n_top: Optional[torch.Tensor] = None):
    """One token per row of float32 logits: greedy where temperature < 1e-5, else temperature,
    top-k, top-p, min-p and the walk to the row's random number u in [0, 1).  With `n_top` (int32
    per row: -1 none, else 0..20) also returns the log-probabilities within the kept list, float32
    [rows, 1 + 20] (the drawn token's, then the list's first entries'), and those entries' ids, int32
    [rows, 20] (-1: no entry): the result is then (tokens, log-probabilities, ids)."""
    _dev(logits, temperature, top_k, top_p, min_p, u, n_top)
    _f32(logits, "logits"); _f32(temperature, "temperature"); _f32(top_p, "top_p"); _f32(min_p, "min_p"); _f32(u, "u")
    _i32(top_k, "top_k")
    rows, vocab = logits.shape
    for t in (temperature, top_k, top_p, min_p, u) + ((n_top,) if n_top is not None else ()):
        if t.numel() != rows:
            raise KernelError("sample: one parameter value per row of logits")
    lib = library()
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    ws = torch.empty((lib.ia_sample_workspace(rows, vocab),), dtype=torch.int32, device=logits.device)
    lp = ids = None
    if n_top is not None:
        _i32(n_top, "n_top")
        most = lib.ia_sample_max_top()
        lp = torch.empty((rows, 1 + most), dtype=torch.float32, device=logits.device)
        ids = torch.empty((rows, most), dtype=torch.int32, device=logits.device)
    _check(lib.ia_sample(_p(out), _p(logits), _p(ws), rows, vocab, _p(temperature), _p(top_k), _p(top_p),
                         _p(min_p), _p(u), _p(n_top), _p(lp), _p(ids), _stream()))
    return out if n_top is None else (out, lp, ids)


def _mid_dual_fits(x: torch.Tensor, w_gate_up: torch.Tensor) -> bool:
    """[gate; up] at up to 16 rows on gemm_mid.hip: where the weight makes a block for every compute unit."""
    return (w_gate_up.shape[0] % 2 == 0 and mid_fits(x, w_gate_up, few_rows=True)
            and w_gate_up.numel() * w_gate_up.element_size() <= MID_DUAL_MAX_BYTES
            and bool(library().ia_gemm_mid_fills(w_gate_up.shape[0] // 2, w_gate_up.shape[1], 1)))


def gated_linear(x, w_gate_up: torch.Tensor, activation: str = "silu",
                 bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """act(x . gate^T) * (x . up^T) for w_gate_up = [gate; up] (`activation`: a name of `ACTIVATIONS`; `bias`
    [2 n]: added to both products before the activation): one fused kernel for few bfloat16 rows, else the
    product followed by the element-wise kernel."""
    # (few rows too go to gemm_mid.hip where its blocks fill the chip evenly: inside a decode step the pair of this product
    # and the next takes 58.0 us against 60.6 at 8 rows and 60.4 against 67.2 at 16, sizes of an 8B model)
    activation_code(activation)
    even = w_gate_up.shape[0] % 2 == 0
    if isinstance(x, NormedRows):
        if even and _takes_normed_rows(x, w_gate_up, w_gate_up.shape[0] // 2):
            _dev(x.scaled, w_gate_up, x.sums)
            if bias is None and _mid_dual_fits(x.scaled, w_gate_up):
                return gemm_mid_bf16(x.scaled, w_gate_up, dual=True, sums_in=x.sums, eps=x.eps, activation=activation)
            return _stream_product(x.scaled, w_gate_up, w_gate_up.shape[0] // 2, x.scaled.dtype, True,
                                   sums_in=x.sums, eps=x.eps, activation=activation, bias=bias)
        x = x.materialize()
    if x.shape[0] <= SKINNY_MAX_ROWS and skinny_fits(x, w_gate_up):
        if bias is None and (_mid_dual_fits(x, w_gate_up) or (
                even and mid_fits(x, w_gate_up) and w_gate_up.numel() * w_gate_up.element_size() <= MID_DUAL_MAX_BYTES)):
            return gemm_mid_bf16(x, w_gate_up, dual=True, activation=activation)
        return gemm_skinny_bf16(x, w_gate_up, x.dtype, dual=True, activation=activation, bias=bias)
    if bias is None:
        if (even and mid_fits(x, w_gate_up)
                and w_gate_up.numel() * w_gate_up.element_size() <= MID_DUAL_MAX_BYTES):
            return gemm_mid_bf16(x, w_gate_up, dual=True, activation=activation)
        if even and x.dtype == torch.bfloat16 and skinny_fits(x, w_gate_up) and _own_large(x, w_gate_up):
            return gemm_mfma_bf16(x, w_gate_up, dual=True, activation=activation)
    # (a [gate; up] beyond MID_DUAL_MAX_BYTES at 17 to 64 rows: the vendor's GEMM, not the plain product of gemm_mid.hip)
    return gate_mul(linear(x, w_gate_up, mid=bias is not None, bias=bias), activation)


def gated_silu_linear(x, w_gate_up: torch.Tensor) -> torch.Tensor:
    """`gated_linear` with SiLU and no bias."""
    return gated_linear(x, w_gate_up, "silu")
