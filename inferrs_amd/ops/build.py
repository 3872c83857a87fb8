"""Compiles the HIP sources under `inferrs_amd/csrc` for gfx950 into one shared library.

The library's file name carries a hash of the sources and flags, so a library
that is found is never stale.  `build()` always compiles; `library_path()`
returns a built library or None.  The library lives beside the package when
that folder can be written, else under the temporary directory.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

ARCH = "gfx950"
_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(_PKG, "csrc")
# -packed-fp32-ops is switched off on purpose: some packed 32-bit forms have given wrong results.
FLAGS = ["-O3", "-fPIC", "-std=c++17", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-pass-failed"]


def _sources() -> List[str]:
    return sorted(os.path.join(CSRC, n) for n in os.listdir(CSRC) if n.endswith(".hip"))


def _digest() -> str:
    h = hashlib.sha256()
    for p in sorted(os.path.join(CSRC, n) for n in os.listdir(CSRC) if n.endswith((".hip", ".h"))):
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:12]


def _lib_name() -> str:
    return f"libinferrs_amd_{_digest()}.so"


def _candidate_dirs() -> List[str]:
    dirs = [os.path.join(_PKG, "_lib")]
    dirs.append(os.path.join(tempfile.gettempdir(), f"inferrs_amd_lib_{os.getuid()}"))
    return dirs


def library_path() -> Optional[str]:
    name = _lib_name()
    for d in _candidate_dirs():
        p = os.path.join(d, name)
        if os.path.isfile(p):
            return p
    return None


def _writable_dir() -> str:
    for d in _candidate_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe_{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise RuntimeError("no writable folder for the kernel library: tried " + ", ".join(_candidate_dirs()))


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), shutil.which("hipcc"),
              os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")):
        if c and os.path.isfile(c):
            return c
    raise RuntimeError("hipcc not found: the HIP kernels cannot be compiled (looked at $HIPCC, PATH, "
                       "$ROCM_PATH/bin and /opt/rocm/bin)")


def _say(msg: str) -> None:
    print(f"[inferrs_amd build] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True) -> str:
    """Compile every source and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = _writable_dir()
    name = _lib_name()
    obj_dir = os.path.join(out_dir, "_build", name[:-3])
    os.makedirs(obj_dir, exist_ok=True)
    srcs = _sources()
    t0 = time.time()
    if verbose:
        _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        r = subprocess.run([hipcc, *FLAGS, "-I", CSRC, "-c", src, "-o", obj],
                           capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
        if verbose:
            _say(f"  {os.path.basename(src)} done ({time.time() - t0:.0f} s)")
        return obj

    workers = max(1, min(len(srcs), (os.cpu_count() or 2), 8))
    with ThreadPoolExecutor(workers) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp = os.path.join(out_dir, f".{name}.{os.getpid()}.tmp")
    r = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *objs],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed to link the kernel library:\n{r.stdout}\n{r.stderr}")
    lib = os.path.join(out_dir, name)
    os.replace(tmp, lib)
    for old in os.listdir(out_dir):          # libraries of older sources
        if old.startswith("libinferrs_amd_") and old.endswith(".so") and old != name:
            try:
                os.remove(os.path.join(out_dir, old))
            except OSError:
                pass
    shutil.rmtree(os.path.join(out_dir, "_build"), ignore_errors=True)
    if verbose:
        _say(f"linked {lib} ({time.time() - t0:.0f} s)")
    return lib
