"""The reference's per-step random number: a function of (seed, step) alone, so that what a
request draws does not depend on what else is in the batch (`inferrs/src/sampler.rs:370-397`)."""
from __future__ import annotations

import os
import struct

_M64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15


def _mix(x: int) -> int:
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _M64
    return x ^ (x >> 31)


def rand_f32(seed: int, step: int) -> float:
    """Uniform in [0, 1] as a float32 value: splitmix64 of the seed, mixed with the step,
    one xorshift round, the high 32 bits of a multiply, divided by 2**32."""
    x = _mix((seed + _GOLDEN) & _M64)
    x = _mix((x + (((step + 1) * _GOLDEN) & _M64)) & _M64)
    if x == 0:
        x = 0x1234567890ABCDEF
    x ^= (x << 13) & _M64
    x ^= x >> 7
    x ^= (x << 17) & _M64
    hi = ((x * 0x2545F4914F6CDD1D) & _M64) >> 32
    as_f32 = struct.unpack("<f", struct.pack("<f", float(hi)))[0]       # u64 -> f32 rounds to nearest
    return struct.unpack("<f", struct.pack("<f", as_f32 / 4294967296.0))[0]


def fresh_seed() -> int:
    """A seed for a request that names none (the reference seeds a thread-local generator
    from the clock, `sampler.rs:540-579`)."""
    return int.from_bytes(os.urandom(8), "little")
