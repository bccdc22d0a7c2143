"""Counter-based synthetic tensors (splitmix64), identical on every machine and numpy version.

Used by the tests, the fixtures generator and the benchmark so that "seeded synthetic tensor"
means the same bytes everywhere, without depending on a library's random-stream internals.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def splitmix64(seed: int, n: int) -> np.ndarray:
    """n 64-bit words: word i is splitmix64's finaliser applied to seed + (i+1)*golden."""
    with np.errstate(over="ignore"):
        z = (np.arange(1, n + 1, dtype=np.uint64) * _GOLDEN) + np.uint64(seed & 0xFFFFFFFFFFFFFFFF)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform_int(seed: int, shape, lo: int, hi: int, dtype) -> np.ndarray:
    """Integers uniform on [lo, hi] (inclusive)."""
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    span = np.uint64(hi - lo + 1)
    v = (splitmix64(seed, n) >> np.uint64(11)) % span
    return (v.astype(np.int64) + lo).astype(dtype).reshape(shape)


def uniform_f32(seed: int, shape, lo: float, hi: float) -> np.ndarray:
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    u = (splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
    return (lo + (hi - lo) * u).astype(np.float32).reshape(shape)


def normal_f32(seed: int, shape) -> np.ndarray:
    """N(0,1) by Box-Muller over two splitmix64 streams."""
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    m = (n + 1) // 2
    w = splitmix64(seed, 2 * m)
    u1 = ((w[:m] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / (1 << 53))
    u2 = (w[m:] >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
    r = np.sqrt(-2.0 * np.log(u1))
    out = np.concatenate([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)])[:n]
    return out.astype(np.float32).reshape(shape)
