"""Synthetic inputs for tests, smoke and bench: a counter-based generator that
does not depend on NumPy's RNG state or version, plus bf16 bit conversions.

normal(seed, n): splitmix64(seed, index // 2) -> two 32-bit uniforms -> Box-Muller in
float64 (cosine branch for even indices, sine branch for odd ones) -> float32.  The same
seed and index give the same value everywhere.
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(seed, n, offset=0):
    """uint64[n]: splitmix64 output for counters offset..offset+n-1 of stream `seed`."""
    with np.errstate(over="ignore"):
        idx = np.arange(offset, offset + n, dtype=np.uint64)
        z = (np.uint64(seed) * np.uint64(0x9E3779B97F4A7C15)) + (idx + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform(seed, n, offset=0):
    """float64[n] in (0, 1)."""
    z = splitmix64(seed, n, offset)
    return ((z >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def _normal_chunk(args):
    seed, out, o, m = args
    # element i comes from counter i // 2: the cosine branch for even i, the sine branch for odd i
    p0, p1 = o // 2, (o + m + 1) // 2
    z = splitmix64(seed, p1 - p0, p0)
    u1 = ((z >> np.uint64(32)).astype(np.float64) + 0.5) * (1.0 / 4294967296.0)
    u2 = ((z & np.uint64(0xFFFFFFFF)).astype(np.float64) + 0.5) * (1.0 / 4294967296.0)
    r = np.sqrt(-2.0 * np.log(u1))
    t = (2.0 * np.pi) * u2
    both = np.empty(2 * (p1 - p0), dtype=np.float32)
    both[0::2] = r * np.cos(t)
    both[1::2] = r * np.sin(t)
    out[o:o + m] = both[o - 2 * p0:o - 2 * p0 + m]


def normal(seed, shape, chunk=1 << 21):
    """float32 N(0,1) of the given shape (chunks are generated on a few threads; the values do
    not depend on the chunking)."""
    import concurrent.futures
    import os
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float32)
    jobs = [(seed, out, o, min(chunk, n - o)) for o in range(0, n, chunk)]
    workers = max(1, min(16, os.cpu_count() or 1, len(jobs)))
    if workers == 1:
        for j in jobs:
            _normal_chunk(j)
    else:
        with concurrent.futures.ThreadPoolExecutor(workers) as ex:
            list(ex.map(_normal_chunk, jobs))
    return out.reshape(shape)


def randint(seed, n, lo, hi):
    """int32[n] uniform in [lo, hi]."""
    z = splitmix64(seed, n)
    return (lo + (z % np.uint64(hi - lo + 1)).astype(np.int64)).astype(np.int32)


def fill(n, seed):
    """The reference tests' closed-form data: ((i + seed) % 37) * 0.01 - 0.18
    (tests/flash_cuda_bf16.rs:19-23), evaluated in float32 like the Rust expression."""
    i = (np.arange(n, dtype=np.int64) + seed) % 37
    return i.astype(np.float32) * np.float32(0.01) - np.float32(0.18)


def seq(shape, scale=0.3, off=-0.4):
    """arange * scale + off in float32 (py/dump_attention_golden.py:16-20)."""
    n = int(np.prod(shape))
    return (np.arange(n, dtype=np.float32) * np.float32(scale) + np.float32(off)).reshape(shape)


def to_bf16_bits(x):
    """float32 -> bf16 bit pattern (uint16), round-to-nearest-even."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    lsb = (b >> np.uint32(16)) & np.uint32(1)
    r = (b + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    nan = (b & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    r = np.where(nan, (b >> np.uint32(16)) | np.uint32(0x40), r)
    return r.astype(np.uint16)


def from_bf16_bits(b):
    """bf16 bit pattern (uint16) -> float32."""
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)
