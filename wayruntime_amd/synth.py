"""Seeded synthetic inputs for the attention path (tests and benchmark).

The workload definitions say "N(0,1) from a seed" without fixing a generator,
so this module fixes one, used for both the device path and the CPU checker:

* ``normal``      splitmix64 counter stream -> two uniforms -> Box-Muller in
                  float64 -> float32.  Used for live comparisons, where both
                  sides read the very same array.
* ``hash_unit`` / ``hash_bell``
                  integer-hash fills that are exactly reproducible on any
                  IEEE-754 machine (integer arithmetic plus one correctly
                  rounded float32 operation).  Used for fixtures whose expected
                  outputs are stored in the repository, so the inputs can be
                  regenerated bit-for-bit instead of being stored.

Seeds for the numbered workloads: ``0x5EED0000 + 0x100 * config + tensor_id``.
"""
from __future__ import annotations

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def config_seed(config: int, tensor_id: int) -> int:
    return 0x5EED0000 + 0x100 * config + tensor_id


def splitmix64(seed: int, n: int, offset: int = 0) -> np.ndarray:
    """n outputs of the splitmix64 stream started at ``seed`` (counter form)."""
    with np.errstate(over="ignore"):
        idx = np.arange(offset + 1, offset + n + 1, dtype=np.uint64)
        z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + idx * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        z = z ^ (z >> np.uint64(31))
    return z


def normal(seed: int, shape, std: float = 1.0, chunk: int = 1 << 22) -> np.ndarray:
    """float32 N(0, std^2) array of ``shape`` (Box-Muller over splitmix64)."""
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float32)
    pairs = (n + 1) // 2
    done = 0
    while done < pairs:
        m = min(chunk, pairs - done)
        r = splitmix64(seed, 2 * m, offset=2 * done)
        # 53-bit uniforms; u1 in (0,1], u2 in [0,1)
        u1 = ((r[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
        u2 = (r[1::2] >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
        rad = np.sqrt(-2.0 * np.log(u1))
        ang = (2.0 * np.pi) * u2
        z = np.empty(2 * m, dtype=np.float64)
        z[0::2] = rad * np.cos(ang)
        z[1::2] = rad * np.sin(ang)
        lo = 2 * done
        hi = min(n, lo + 2 * m)
        out[lo:hi] = (z[: hi - lo] * std).astype(np.float32)
        done += m
    return out.reshape(shape)


def _hash32(seed: int, n: int) -> np.ndarray:
    """Per-index 32-bit integer hash (two rounds of multiply-xorshift)."""
    with np.errstate(over="ignore"):
        x = np.arange(n, dtype=np.uint32) * np.uint32(2654435761) + np.uint32(seed & 0xFFFFFFFF)
        x ^= x >> np.uint32(16)
        x *= np.uint32(0x7FEB352D)
        x ^= x >> np.uint32(15)
        x *= np.uint32(0x846CA68B)
        x ^= x >> np.uint32(16)
    return x


def hash_unit(seed: int, shape, amp: float = 1.0) -> np.ndarray:
    """float32 values on a 16-bit grid in [-amp, amp): exactly reproducible."""
    n = int(np.prod(shape))
    h = _hash32(seed, n)
    v = (h & np.uint32(0xFFFF)).astype(np.float32) / np.float32(32768.0) - np.float32(1.0)
    return (v * np.float32(amp)).reshape(shape)


def hash_bell(seed: int, shape) -> np.ndarray:
    """float32, unit variance, bell shaped (sum of four 16-bit uniforms):
    exactly reproducible, support about +-3.46."""
    n = int(np.prod(shape))
    a = _hash32(seed, n)
    b = _hash32(seed ^ 0xA5A5A5A5, n)
    s = ((a & np.uint32(0xFFFF)).astype(np.int64) + (a >> np.uint32(16)).astype(np.int64)
         + (b & np.uint32(0xFFFF)).astype(np.int64) + (b >> np.uint32(16)).astype(np.int64))
    centred = (s - 2 * 65535).astype(np.float32)          # exact: |.| < 2^18
    return (centred / np.float32(37837.227)).reshape(shape)


def ragged_contexts(seed: int, n: int, lo: int = 256, hi: int = 4096) -> np.ndarray:
    """n context lengths uniform on [lo, hi] (inclusive)."""
    r = splitmix64(seed, n)
    return (lo + (r % np.uint64(hi - lo + 1))).astype(np.uint32)


def f32_to_f16_trunc(x: np.ndarray) -> np.ndarray:
    """Truncating float32 -> binary16 bit patterns (uint16), vectorised.

    Same rule as the cache append: drop the low 13 mantissa bits, flush
    exponents at or below the half subnormal range to signed zero, saturate
    overflow (NaN included) to signed infinity.
    """
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    sign = ((bits >> np.uint32(16)) & np.uint32(0x8000)).astype(np.uint32)
    e = ((bits >> np.uint32(23)) & np.uint32(0xFF)).astype(np.int32) - 112
    mant = (bits >> np.uint32(13)) & np.uint32(0x3FF)
    body = (e.clip(0, 31).astype(np.uint32) << np.uint32(10)) | mant
    out = np.where(e <= 0, sign, np.where(e >= 31, sign | np.uint32(0x7C00), sign | body))
    return out.astype(np.uint16)
