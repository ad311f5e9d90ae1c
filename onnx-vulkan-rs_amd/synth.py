"""Seeded synthetic operands for the benchmark configurations and the parity tests.

One generator for everything: the 64-bit LCG the reference's own tests and harness use
(``state * 6364136223846793005 + 1442695040888963407``, high bits taken;
crates/onnx-vulkan-core/tests/conv_integer_im2col.rs:14-24,
crates/model-runner/src/main.rs:264-280), vectorised with numpy by its closed form.
Tensor ``i`` of a configuration is seeded ``base_seed + i``.
"""
from __future__ import annotations

import numpy as np

_A = np.uint64(6364136223846793005)
_C = np.uint64(1442695040888963407)
_CHUNK = 1 << 20
_pow = None
_geo = None


def _tables():
    """a^i and 1 + a + .. + a^(i-1) for i = 1.._CHUNK, modulo 2^64."""
    global _pow, _geo
    if _pow is None:
        with np.errstate(over="ignore"):
            p = np.cumprod(np.full(_CHUNK, _A, dtype=np.uint64), dtype=np.uint64)
            g = np.empty(_CHUNK, np.uint64)
            g[0] = 1
            g[1:] = np.cumsum(p[:-1], dtype=np.uint64) + np.uint64(1)
        _pow, _geo = p, g
    return _pow, _geo


def lcg_states(n: int, seed: int) -> np.ndarray:
    """The n states after `seed` (the state itself is not emitted), as uint64."""
    p, g = _tables()
    out = np.empty(n, np.uint64)
    s = np.uint64(seed & 0xFFFFFFFFFFFFFFFF)
    with np.errstate(over="ignore"):
        for lo in range(0, n, _CHUNK):
            m = min(_CHUNK, n - lo)
            out[lo:lo + m] = p[:m] * s + _C * g[:m]
            s = out[lo + m - 1]
    return out


def uniform_ints(n: int, seed: int, lo: int, hi: int) -> np.ndarray:
    """Integers uniform in [lo, hi] (inclusive) from the top 32 bits of each state."""
    top = (lcg_states(n, seed) >> np.uint64(32)).astype(np.uint64)
    span = np.uint64(hi - lo + 1)
    return ((top * span) >> np.uint64(32)).astype(np.int64) + lo


def uniform_f32(n: int, seed: int, lo: float, hi: float) -> np.ndarray:
    u = (lcg_states(n, seed) >> np.uint64(40)).astype(np.float64) / float(1 << 24)
    return (lo + (hi - lo) * u).astype(np.float32)


def normal_f32(n: int, seed: int) -> np.ndarray:
    """N(0, 1) by Box-Muller on consecutive pairs of states."""
    m = (n + 1) // 2
    s = lcg_states(2 * m, seed)
    u1 = ((s[0::2] >> np.uint64(40)).astype(np.float64) + 1.0) / float(1 << 24)
    u2 = (s[1::2] >> np.uint64(40)).astype(np.float64) / float(1 << 24)
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.empty(2 * m, np.float64)
    z[0::2] = r * np.cos(2.0 * np.pi * u2)
    z[1::2] = r * np.sin(2.0 * np.pi * u2)
    return z[:n].astype(np.float32)


# ----------------------------------------------------------- MatMulNBits packing

def pack_nibbles(q: np.ndarray, block_size: int) -> np.ndarray:
    """q [N, K] values 0..15 -> [N, n_blocks, block_size/2] bytes, element 2i in the low nibble
    (crates/onnx-vulkan-core/tests/matmul_nbits.rs:18-35)."""
    n, k = q.shape
    n_blocks = -(-k // block_size)
    padded = np.zeros((n, n_blocks * block_size), np.uint8)
    padded[:, :k] = q
    lo, hi = padded[:, 0::2], padded[:, 1::2]
    return (lo | (hi << 4)).astype(np.uint8).reshape(n, n_blocks, block_size // 2)


def pack_zero_points(z: np.ndarray) -> np.ndarray:
    """z [N, n_blocks] values 0..15 -> [N, ceil(n_blocks/2)] bytes, block 2j in the low nibble
    (tests/matmul_nbits.rs:37-46)."""
    n, nb = z.shape
    padded = np.zeros((n, 2 * ((nb + 1) // 2)), np.uint8)
    padded[:, :nb] = z
    return (padded[:, 0::2] | (padded[:, 1::2] << 4)).astype(np.uint8)


def nbits_weight(N: int, K: int, block_size: int, seed: int, with_zp: bool = True, scale_dtype=np.float32):
    """Uniform nibbles, scales U(0.005, 0.05), uniform zero points. Returns (B, scales, zp)."""
    n_blocks = -(-K // block_size)
    q = uniform_ints(N * K, seed, 0, 15).astype(np.uint8).reshape(N, K)
    B = pack_nibbles(q, block_size)
    scales = uniform_f32(N * n_blocks, seed + 1, 0.005, 0.05).astype(scale_dtype)
    zp = None
    if with_zp:
        zp = pack_zero_points(uniform_ints(N * n_blocks, seed + 2, 0, 15).astype(np.uint8).reshape(N, n_blocks))
    return B, scales, zp


def fast_nbits_weight(N: int, K: int, block_size: int, seed: int, with_zp: bool = True, scale_dtype=np.float32):
    """Same distributions from numpy's PCG64, for weights too large for the LCG to be worth it
    (hundreds of MB); still seeded and reproducible."""
    rng = np.random.default_rng(seed)
    n_blocks = -(-K // block_size)
    B = rng.integers(0, 256, size=(N, n_blocks, block_size // 2), dtype=np.uint8)
    scales = rng.uniform(0.005, 0.05, size=N * n_blocks).astype(np.float32).astype(scale_dtype)
    zp = rng.integers(0, 256, size=(N, (n_blocks + 1) // 2), dtype=np.uint8) if with_zp else None
    return B, scales, zp


def int8_weight(K: int, N: int, seed: int) -> np.ndarray:
    """int8 [K, N] uniform in -127..127 (symmetric per-tensor weights)."""
    return uniform_ints(K * N, seed, -127, 127).astype(np.int8).reshape(K, N)
