"""Seeded synthetic inputs for the GEMM workloads (numpy only, no oracle dependency).

A counter-based generator: element ``i`` of stream ``seed`` is a pure function of
``(seed, i)`` (splitmix64 finaliser), so any sub-block can be regenerated without
the rest and the C and numpy implementations agree bit for bit.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(seed: int, count: int, start: int = 0) -> np.ndarray:
    with np.errstate(over="ignore"):
        i = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        z = np.uint64(seed) + i * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def uniform_f32(rows: int, cols: int, seed: int) -> np.ndarray:
    """iid uniform in [-1, 1), fp32, shape (rows, cols), row-major and dense."""
    out = np.empty((rows, cols), np.float32)
    step = max(1, (1 << 22) // max(cols, 1))
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        u = _mix(seed, (r1 - r0) * cols, r0 * cols) >> np.uint64(40)
        out[r0:r1] = (u.astype(np.float32) * np.float32(1.0 / 8388608.0) - np.float32(1.0)).reshape(r1 - r0, cols)
    return out


def uniform_f64(rows: int, cols: int, seed: int) -> np.ndarray:
    """iid uniform in [-1, 1), fp64 (52 random mantissa bits), shape (rows, cols), row-major and dense."""
    out = np.empty((rows, cols), np.float64)
    step = max(1, (1 << 22) // max(cols, 1))
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        u = _mix(seed, (r1 - r0) * cols, r0 * cols) >> np.uint64(12)
        out[r0:r1] = (u.astype(np.float64) * (1.0 / 2251799813685248.0) - 1.0).reshape(r1 - r0, cols)
    return out


def normal_half(rows: int, cols: int, seed: int, sigma: float = 0.5, clip: float = 4.0) -> np.ndarray:
    """iid N(0, sigma) drawn in fp32 (Box-Muller on two counter streams), clipped to
    [-clip, clip], rounded to nearest-even binary16.  Returns float16, shape (rows, cols)."""
    out = np.empty((rows, cols), np.float16)
    step = max(1, (1 << 22) // max(cols, 1))
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        n = (r1 - r0) * cols
        u1 = (_mix(seed, n, r0 * cols) >> np.uint64(40)).astype(np.float32)
        u2 = (_mix(seed ^ 0x5DEECE66D, n, r0 * cols) >> np.uint64(40)).astype(np.float32)
        u1 = (u1 + np.float32(1.0)) * np.float32(1.0 / 16777216.0)     # (0, 1]
        u2 = u2 * np.float32(1.0 / 16777216.0)                          # [0, 1)
        g = np.sqrt(np.float32(-2.0) * np.log(u1)) * np.cos(np.float32(2.0 * np.pi) * u2)
        g = np.clip(g * np.float32(sigma), -clip, clip).astype(np.float32)
        out[r0:r1] = g.astype(np.float16).reshape(r1 - r0, cols)
    return out


def seeds(cfg: int):
    """(seed_A, seed_B, seed_C) for workload number ``cfg``."""
    return 0xA000 + cfg, 0xB000 + cfg, 0xC000 + cfg
