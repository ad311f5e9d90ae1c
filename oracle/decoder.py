"""numpy restatement of one decoder-only decode step -- TEST INFRASTRUCTURE ONLY.

Follows the reference operators a gemma3-1b graph is made of (paths relative to
crates/onnx-vulkan-core/src in the reference tree):
  SimplifiedLayerNormalization  shaders/normalization.rs:109-181   x * rsqrt(mean(x^2) + eps) * w
  GroupQueryAttention           shaders/attention.rs:128-317       half-split rotary (:157-167), cache
                                                                   append, scale * q.k^T (:264), softmax, p.V
  Gelu approximate="tanh"       interp.rs:9020-9027
  GatherBlockQuantized          shaders/gather_block_quantized.rs:26-57
  MatMulNBits                   oracle.matmul_nbits (the C oracle)
All arithmetic is float32; the KV cache is rounded to float16 as the configuration asks.
Pin status: the glue pieces (norm, rotary, masked softmax, gelu, gather) are checked in
tests/test_oracle_pins.py against float64 closed forms; the step's composition (which norm feeds which
product, residual order, gate before up, head to kv-head map, cache write before attention, the state
rule) against an independent float64 route written from the operator definitions and against a
closed form with silenced branches. No reference vector exists for a whole step.
"""
from __future__ import annotations

import numpy as np

from . import matmul_nbits

QKV, O, GATE_UP, DOWN, LM_HEAD = 0, 1, 2, 3, 4
NORM_INPUT, NORM_POST_ATTN, NORM_PRE_FFN, NORM_POST_FFN, NORM_Q, NORM_K, NORM_FINAL = range(7)

f32 = np.float32


def rmsnorm(x, w, eps):
    x = x.astype(f32)
    ms = f32(np.sum(x * x, dtype=f32) / f32(x.size))
    return (x * f32(1.0 / np.sqrt(ms + f32(eps))) * w).astype(f32)


def rope_half(x, pos, theta):
    """Half-split rotary: channel j of the first half pairs with j + half (attention.rs:157-167)."""
    hd = x.size
    half = hd // 2
    j = np.arange(half, dtype=f32)
    ang = (f32(pos) * np.power(f32(theta), f32(-2.0) * j / f32(hd))).astype(f32)
    c, s = np.cos(ang).astype(f32), np.sin(ang).astype(f32)
    out = np.empty(hd, f32)
    out[:half] = x[:half] * c - x[half:] * s
    out[half:] = x[half:] * c + x[:half] * s
    return out


def gelu_tanh(v):
    v = v.astype(f32)
    return (f32(0.5) * v * (f32(1.0) + np.tanh(f32(0.79788456080286536) * (f32(0.044715) * v * v * v + v)))).astype(f32)


def gather_block_quantized(table, row, hidden, bs):
    B, scales, zp = table
    nb = -(-hidden // bs)
    q = B[row].reshape(-1)
    nib = np.empty(nb * bs, np.int32)
    nib[0::2], nib[1::2] = q & 15, q >> 4
    z = np.empty(2 * ((nb + 1) // 2), np.int32)
    z[0::2], z[1::2] = zp[row] & 15, zp[row] >> 4
    blk = np.arange(hidden) // bs
    return ((nib[:hidden] - z[blk]).astype(f32) * scales.reshape(-1, nb)[row][blk]).astype(f32)


def attend(q, K, V, pos, window, scale):
    """One query head at position `pos` over the cache rows K, V [>= pos + 1, hd] (float16):
    softmax(scale * K q) V over the visible keys. Key t is visible iff t <= pos and, with a window,
    pos - t < window (attention.rs:202-214, :250)."""
    first = max(0, pos + 1 - window) if window > 0 else 0
    Kf, Vf = K[first: pos + 1].astype(f32), V[first: pos + 1].astype(f32)
    s = (Kf @ q) * f32(scale)
    p = np.exp(s - s.max()).astype(f32)
    return (p @ Vf) / f32(p.sum(dtype=f32))


class Decoder:
    def __init__(self, weights, max_seq):
        self.w, self.cfg = weights, weights.cfg
        c = self.cfg
        self.k = np.zeros((c["n_layers"], c["n_kv_heads"], max_seq, c["head_dim"]), np.float16)
        self.v = np.zeros_like(self.k)
        # per layer: sliding window (0 = the whole context) and rotary base. Key t is visible from
        # position pos iff t <= pos and pos - t < window (attention.rs:202-214, :250): `window`
        # keys, the step's own included.
        self.window = [0] * c["n_layers"]
        self.theta = [c["rope_theta"]] * c["n_layers"]

    def set_layer_attention(self, li, window=0, rope_theta=0.0):
        self.window[li] = window if window > 0 else 0
        self.theta[li] = rope_theta if rope_theta > 0 else self.cfg["rope_theta"]

    def _lin(self, x, li, which):
        B, scales, zp = self.w.linears[(li, which)]
        n_rows = B.shape[0]
        return matmul_nbits(x.reshape(1, -1).astype(f32), B, scales, zp, x.size, n_rows, self.cfg["block_size"]).reshape(-1)

    def step(self, token, pos):
        c, w = self.cfg, self.w
        hd, nq, nkv = c["head_dim"], c["n_q_heads"], c["n_kv_heads"]
        scale = f32(c["attn_scale"] if c["attn_scale"] > 0 else 1.0 / np.sqrt(hd))
        x = (gather_block_quantized(w.embedding, token, c["hidden"], c["block_size"]) * f32(c["embed_scale"])).astype(f32)
        xn = rmsnorm(x, w.norms[(0, NORM_INPUT)], c["rms_eps"])
        for li in range(c["n_layers"]):
            qkv = self._lin(xn, li, QKV)
            q = qkv[: nq * hd].reshape(nq, hd)
            k = qkv[nq * hd: (nq + nkv) * hd].reshape(nkv, hd)
            v = qkv[(nq + nkv) * hd:].reshape(nkv, hd)
            theta = self.theta[li]
            q = np.stack([rope_half(rmsnorm(q[h], w.norms[(li, NORM_Q)], c["rms_eps"]), pos, theta) for h in range(nq)])
            for h in range(nkv):
                self.k[li, h, pos] = rope_half(rmsnorm(k[h], w.norms[(li, NORM_K)], c["rms_eps"]), pos, theta).astype(np.float16)
                self.v[li, h, pos] = v[h].astype(np.float16)
            attn = np.empty((nq, hd), f32)
            g = nq // nkv
            for h in range(nq):
                attn[h] = attend(q[h], self.k[li, h // g], self.v[li, h // g], pos, self.window[li], scale)
            y = self._lin(attn.reshape(-1), li, O)
            x = (x + rmsnorm(y, w.norms[(li, NORM_POST_ATTN)], c["rms_eps"])).astype(f32)
            xn = rmsnorm(x, w.norms[(li, NORM_PRE_FFN)], c["rms_eps"])
            gu = self._lin(xn, li, GATE_UP)
            h_ = (gelu_tanh(gu[: c["ffn"]]) * gu[c["ffn"]:]).astype(f32)
            y = self._lin(h_, li, DOWN)
            x = (x + rmsnorm(y, w.norms[(li, NORM_POST_FFN)], c["rms_eps"])).astype(f32)
            nxt = w.norms[(li + 1, NORM_INPUT)] if li + 1 < c["n_layers"] else w.norms[(0, NORM_FINAL)]
            xn = rmsnorm(x, nxt, c["rms_eps"])
        logits = self._lin(xn, 0, LM_HEAD)
        return logits, int(np.argmax(logits))


def advance_state(token, pos, logits, max_seq):
    """The loop state after one step: (token, pos, overflow).

    ArgMax keeps the smallest index among equal maxima (shaders/reduction.rs:76-191); a row in which
    no comparison succeeds (every logit NaN) yields index 0. A step asked for with the cache full
    (pos == max_seq: row `pos` does not exist) changes nothing and reports overflow; the caller must
    not have run the step's writes in that case.
    """
    if pos >= max_seq:
        return token, pos, True
    best, bi = -np.inf, None
    for i, v in enumerate(np.asarray(logits, np.float32)):
        if v > best:
            best, bi = v, i
    if bi is None:
        bi = 0
    return int(bi), pos + 1, False
