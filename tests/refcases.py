"""Inputs of the reference's own tests for the hot path, regenerated from their closed forms.

Only inputs live here (and independent, slow ways to the expected outputs that do not go
through the oracle): both the oracle pins and the GPU parity tests draw from this file.
Paths are relative to crates/onnx-vulkan-core in the reference tree.
"""
from __future__ import annotations

from fractions import Fraction

import numpy as np

# ---------------------------------------------------------------- MatMulNBits

# tests/matmul_nbits.rs:167-252 -- (M, K, N, block_size), in the order of the file
MATMUL_NBITS_CASES = [
    (1, 1152, 256, 32),   # decode_step_matches_the_unpacked_reference
    (5, 256, 48, 32),     # several_rows_share_the_weight
    (2, 100, 17, 32),     # a_partial_last_block_is_not_read_past_k
    (1, 128, 4096, 32),   # a_wide_decode_step_takes_the_wide_kernel
    (1, 96, 65536, 32),   # an_unembedding_width_takes_the_wide_kernel
    (3, 128, 4096, 32),   # a_wide_prefill_stays_on_the_row_kernel
    (1, 80, 33, 16),      # an_odd_block_count_misaligns_the_zero_point_rows
]


def matmul_nbits_case(m, k, n, block_size):
    """The closed-form operands of tests/matmul_nbits.rs:64-83, unpacked: returns
    (a [m,k] f32, nibbles [n,k] u8, zero points [n,n_blocks] u8, scales [n,n_blocks] f32)."""
    n_blocks = -(-k // block_size)
    col = np.arange(n)[:, None]
    kk = np.arange(k)[None, :]
    b = np.arange(n_blocks)[None, :]
    nib = ((col * 7 + kk * 3) % 16).astype(np.uint8)
    zp = ((col + b * 5) % 16).astype(np.uint8)
    scale = (((col * 3 + b) % 11).astype(np.float32) / np.float32(32.0) - np.float32(0.15)).astype(np.float32)
    i = np.arange(m * k)
    a = (((i * 13 % 29).astype(np.float32) - np.float32(14.0)) / np.float32(8.0)).reshape(m, k)
    return a, nib, zp, scale


def matmul_nbits_f64(a, nib, zp, scale, block_size):
    """Dense dequantised product in float64 -- the mathematics, not the oracle's f32 loop."""
    n, k = nib.shape
    blk = np.arange(k) // block_size
    w = (nib.astype(np.float64) - zp[:, blk].astype(np.float64)) * scale[:, blk].astype(np.float64)
    return a.astype(np.float64) @ w.T


# ------------------------------------------------------ DynamicQuantizeLinear

def dql_symmetric(r, n=2048):
    """tests/dynamic_quantize.rs:78-88: -r + 2 r i / (n-1) evaluated in f32, left to right."""
    i = np.arange(n, dtype=np.float32)
    r = np.float32(r)
    return (-r + np.float32(2.0) * r * i / np.float32(n - 1)).astype(np.float32)


def dql_xorshift(count=1 << 20, seed=0x9E3779B97F4A7C15):
    """tests/dynamic_quantize.rs:91-102."""
    mask = (1 << 64) - 1
    s = seed
    out = np.empty(count, np.float32)
    vals = np.empty(count, np.uint64)
    for i in range(count):
        s ^= (s << 13) & mask
        s ^= s >> 7
        s ^= (s << 17) & mask
        vals[i] = s >> 40
    out[:] = (vals.astype(np.float32) / np.float32(1 << 24)) * np.float32(5.3) - np.float32(1.9)
    return out


# -------------------------------------------------------------- MatMulInteger

def pseudo_plus1(n, seed):
    """tests/matmul_integer_variants.rs:29-37: LCG with increment 1, byte = state >> 33."""
    mask = (1 << 64) - 1
    s = seed | 1
    out = np.empty(n, np.uint8)
    for i in range(n):
        s = (s * 6364136223846793005 + 1) & mask
        out[i] = (s >> 33) & 0xFF
    return out


def pseudo_top_byte(n, seed):
    """tests/conv_integer_im2col.rs:14-24: LCG with the Knuth increment, byte = state >> 56."""
    mask = (1 << 64) - 1
    s = seed | 1
    out = np.empty(n, np.uint8)
    for i in range(n):
        s = (s * 6364136223846793005 + 1442695040888963407) & mask
        out[i] = s >> 56
    return out


def matmul_integer_bigint(A, B, a_zp, b_zp):
    """Python integers: no width, no wrap."""
    M, K = A.shape
    N = B.shape[1]
    a = [[int(v) - a_zp for v in row] for row in A]
    b = [[int(v) - b_zp for v in row] for row in B]
    return np.array([[sum(a[m][k] * b[k][n] for k in range(K)) for n in range(N)] for m in range(M)], dtype=np.int64)


# ----------------------------------------------------------------- Requantize

def f32(x) -> np.float32:
    return np.float32(x)


def requantize_exact(acc: int, x_scale, w_scale, y_scale, y_zp: int, signed: bool) -> int:
    """tests/qlinear.rs:94-102 evaluated with exact rationals and explicit f32 roundings:
    ratio = fl(fl(x_scale * w_scale) / y_scale); q = rte(fl(fl(acc) * ratio)) + y_zp, saturated.
    A product of two f32 is exact in f64 and an f64 quotient of two f32 rounds to the same f32 as
    the exact quotient (53 >= 2*24 + 2), so float64 followed by one cast is the f32 operation."""
    t = np.float32(np.float64(f32(x_scale)) * np.float64(f32(w_scale)))
    ratio = np.float32(np.float64(t) / np.float64(f32(y_scale)))
    prod = np.float32(np.float64(np.float32(acc)) * np.float64(ratio))
    fr = Fraction(float(prod))
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    q = fl + y_zp
    lo, hi = (-128, 127) if signed else (0, 255)
    return max(lo, min(hi, q))


# ---------------------------------------------------------------- ConvInteger

# tests/conv_integer_im2col.rs:185-247
CONV_CASES = [
    dict(c_in=64, c_out=32, h=20, w=20, k=3, stride=1, dilation=1, pads=(1, 1, 1, 1), x_signed=False, w_signed=False),
    dict(c_in=32, c_out=48, h=18, w=22, k=3, stride=2, dilation=2, pads=(2, 0, 1, 3), x_signed=True, w_signed=True),
    dict(c_in=32, c_out=16, h=15, w=15, k=3, stride=1, dilation=1, pads=(1, 1, 1, 1), x_signed=False, w_signed=True),
]


def conv_case_operands(case):
    """Operands as tests/conv_integer_im2col.rs:96-100 builds them. pads = (top, left, bottom, right)."""
    x = pseudo_top_byte(case["c_in"] * case["h"] * case["w"], 11)
    w = pseudo_top_byte(case["c_out"] * case["c_in"] * case["k"] * case["k"], 5)
    x_zp_byte = 0xFB if case["x_signed"] else 129
    w_zp_byte = 0x07
    xd = np.int8 if case["x_signed"] else np.uint8
    wd = np.int8 if case["w_signed"] else np.uint8
    X = x.view(xd).reshape(1, case["c_in"], case["h"], case["w"])
    W = w.view(wd).reshape(case["c_out"], case["c_in"], case["k"], case["k"])
    x_zp = int(np.array([x_zp_byte], np.uint8).view(xd)[0])
    w_zp = int(np.array([w_zp_byte], np.uint8).view(wd)[0])
    return X, W, x_zp, w_zp


def conv_integer_dense(X, W, x_zp, w_zp, strides, dilations, pads, group=1):
    """ConvInteger by explicit padding with the zero point, gathering columns and one int64
    matrix product per group -- a different route from the oracle's six nested loops."""
    n, c_in, h, w = X.shape
    c_out, cpg, kh, kw = W.shape
    pt, pl, pb, pr = pads
    xp = np.full((n, c_in, h + pt + pb, w + pl + pr), x_zp, np.int64)
    xp[:, :, pt:pt + h, pl:pl + w] = X.astype(np.int64)
    xp -= x_zp
    wz = W.astype(np.int64) - w_zp
    ho = (h + pt + pb - (dilations[0] * (kh - 1) + 1)) // strides[0] + 1
    wo = (w + pl + pr - (dilations[1] * (kw - 1) + 1)) // strides[1] + 1
    out = np.zeros((n, c_out, ho, wo), np.int64)
    opg = c_out // group
    for g in range(group):
        cols = np.empty((n, cpg, kh, kw, ho, wo), np.int64)
        for r in range(kh):
            for s in range(kw):
                hs, ws = r * dilations[0], s * dilations[1]
                cols[:, :, r, s] = xp[:, g * cpg:(g + 1) * cpg, hs:hs + strides[0] * (ho - 1) + 1:strides[0],
                                      ws:ws + strides[1] * (wo - 1) + 1:strides[1]]
        wm = wz[g * opg:(g + 1) * opg].reshape(opg, -1)
        out[:, g * opg:(g + 1) * opg] = np.einsum("ok,nkp->nop", wm, cols.reshape(n, cpg * kh * kw, ho * wo)).reshape(
            n, opg, ho, wo)
    return out
