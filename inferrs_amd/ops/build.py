"""Compiles the sources under `inferrs_amd/csrc` into shared libraries.

Three kinds of library:
  * "core": every HIP kernel (gfx950) whose code does not depend on a model size;
  * "attn_d<N>": the matrix-core attention kernel built for head size N (`-DIA_HEAD_DIM=N`),
    so that a model compiles only the head size it has;
  * "runtime": the host runtime (cache manager, step assembly, scheduler), plain C++ that
    touches no GPU and is compiled with the host compiler.

A library's file name carries a hash of its sources and flags, so a library that is found
is never stale.  `build(target)` always compiles; `library_path(target)` returns a built
library or None.  Libraries live beside the package when that folder can be written, else
under the temporary directory.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, List, Optional, Sequence, Tuple

ARCH = "gfx950"
_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(_PKG, "csrc")
# Packed 32-bit float instructions are switched off: some of their forms have given wrong
# results on this hardware.
FLAGS = ["-O3", "-fPIC", "-std=c++17", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-pass-failed"]

HOST_FLAGS = ["-O2", "-fPIC", "-std=c++17", "-Wall"]
# Flags of single sources.  The attention kernels take the maximum of scores that come out of matrix products:
# told that no NaN reaches an arithmetic instruction (masked scores are replaced, never computed with), the
# compiler leaves out the instruction that would quiet a signalling NaN in front of every maximum (a prompt of
# 8,192 tokens 650 -> 614 us a layer).
SOURCE_FLAGS = {"attention_mfma.hip": ["-fno-honor-nans"]}

PER_HEAD_DIM = ("attention_mfma.hip",)
SHARED = ("error.hip",)
RUNTIME_SOURCES = ("runtime.cpp",)
RUNTIME_HEADERS = ("runtime.h",)
ATTN_HEAD_DIMS = tuple(range(16, 257, 16))


def attn_target(head_dim: int) -> str:
    return f"attn_d{head_dim}"


def all_targets() -> List[str]:
    return ["runtime", "core"] + [attn_target(d) for d in ATTN_HEAD_DIMS]


def _is_host(target: str) -> bool:
    return target == "runtime"


def _plan(target: str) -> Tuple[List[str], List[str]]:
    """(sources, extra defines) of a target."""
    names = sorted(n for n in os.listdir(CSRC) if n.endswith(".hip"))
    if target == "runtime":
        return [os.path.join(CSRC, n) for n in RUNTIME_SOURCES], []
    if target == "core":
        return [os.path.join(CSRC, n) for n in names if n not in PER_HEAD_DIM], []
    if target.startswith("attn_d"):
        d = int(target[len("attn_d"):])
        if d not in ATTN_HEAD_DIMS:
            raise ValueError(f"no matrix-core attention kernel for head size {d}")
        return [os.path.join(CSRC, n) for n in PER_HEAD_DIM + SHARED], [f"-DIA_HEAD_DIM={d}"]
    raise ValueError(f"unknown kernel library {target!r}")


def _digest(target: str) -> str:
    srcs, defines = _plan(target)
    h = hashlib.sha256()
    host = _is_host(target)
    headers = sorted(os.path.join(CSRC, n) for n in os.listdir(CSRC)
                     if n.endswith(".h") and (n in RUNTIME_HEADERS) == host)
    for p in srcs + headers:
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join((HOST_FLAGS if host else FLAGS) + defines).encode())
    for p in srcs:
        h.update(" ".join(SOURCE_FLAGS.get(os.path.basename(p), [])).encode())
    return h.hexdigest()[:12]


def _lib_name(target: str) -> str:
    return f"libinferrs_amd_{target}_{_digest(target)}.so"


def _candidate_dirs() -> List[str]:
    return [os.path.join(_PKG, "_lib"),
            os.path.join(tempfile.gettempdir(), f"inferrs_amd_lib_{os.getuid()}")]


def library_path(target: str = "core") -> Optional[str]:
    name = _lib_name(target)
    for d in _candidate_dirs():
        p = os.path.join(d, name)
        if os.path.isfile(p):
            return p
    return None


def _writable_dir() -> str:
    for d in _candidate_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe_{os.getpid()}_{threading.get_ident()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise RuntimeError("no writable folder for the kernel libraries: tried " + ", ".join(_candidate_dirs()))


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), shutil.which("hipcc"),
              os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")):
        if c and os.path.isfile(c):
            return c
    raise RuntimeError("hipcc not found: the HIP kernels cannot be compiled (looked at $HIPCC, PATH, "
                       "$ROCM_PATH/bin and /opt/rocm/bin)")


def _host_compiler() -> str:
    for c in (os.environ.get("CXX"), "g++", "c++", "clang++",
              os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "llvm", "bin", "clang++")):
        found = shutil.which(c) if c else None
        if found:
            return found
    raise RuntimeError("no C++ compiler found for the host runtime (looked at $CXX, g++, c++, clang++ and "
                       "$ROCM_PATH/llvm/bin/clang++)")


def _say(msg: str) -> None:
    print(f"[inferrs_amd build] {msg}", file=sys.stderr, flush=True)


def build(target: str = "core", verbose: bool = True, workers: Optional[int] = None) -> str:
    """Compile the sources of `target` and link its library; returns the path."""
    host = _is_host(target)
    hipcc = _host_compiler() if host else _hipcc()
    flags = HOST_FLAGS if host else FLAGS
    link_flags = [] if host else [f"--offload-arch={ARCH}"]
    out_dir = _writable_dir()
    name = _lib_name(target)
    srcs, defines = _plan(target)
    obj_dir = os.path.join(out_dir, "_build", f"{name[:-3]}_{os.getpid()}")
    os.makedirs(obj_dir, exist_ok=True)
    t0 = time.time()
    if verbose:
        _say(f"{target}: compiling {len(srcs)} {'C++ sources' if host else f'HIP sources for {ARCH}'} into {out_dir}")

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.splitext(os.path.basename(src))[0] + ".o")
        r = subprocess.run([hipcc, *flags, *SOURCE_FLAGS.get(os.path.basename(src), []), *defines, "-I", CSRC, "-c", src, "-o", obj],
                           capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"{os.path.basename(hipcc)} failed on {src}:\n{r.stdout}\n{r.stderr}")
        if verbose:
            _say(f"  {target}: {os.path.basename(src)} done ({time.time() - t0:.0f} s)")
        return obj

    n = workers or max(1, min(len(srcs), (os.cpu_count() or 2), 8))
    with ThreadPoolExecutor(n) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp = os.path.join(out_dir, f".{name}.{os.getpid()}.tmp")
    r = subprocess.run([hipcc, "-shared", "-fPIC", *link_flags, "-o", tmp, *objs],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"{os.path.basename(hipcc)} failed to link {name}:\n{r.stdout}\n{r.stderr}")
    lib = os.path.join(out_dir, name)
    os.replace(tmp, lib)
    prefix = f"libinferrs_amd_{target}_"
    for old in os.listdir(out_dir):          # libraries of older sources of the same target
        if old.startswith(prefix) and old.endswith(".so") and old != name:
            try:
                os.remove(os.path.join(out_dir, old))
            except OSError:
                pass
    shutil.rmtree(obj_dir, ignore_errors=True)
    try:
        os.rmdir(os.path.join(out_dir, "_build"))
    except OSError:
        pass
    if verbose:
        _say(f"{target}: linked {lib} ({time.time() - t0:.0f} s)")
    return lib


def build_all(verbose: bool = True, targets: Optional[Sequence[str]] = None) -> Dict[str, str]:
    """Compile every library (or `targets`), a few at a time."""
    targets = list(targets or all_targets())
    jobs = max(1, min(len(targets), (os.cpu_count() or 2), 8))
    with ThreadPoolExecutor(jobs) as pool:
        paths = list(pool.map(lambda t: build(t, verbose=verbose, workers=2), targets))
    return dict(zip(targets, paths))
