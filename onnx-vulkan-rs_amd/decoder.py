"""The decode-step object over the C ABI (``hipc_decoder_*``) and a seeded synthetic model.

Weights of a synthetic decoder are random int4 (block 32, with zero points) at the shape the
configuration names; ``build_weights`` keeps them on the host too, so the oracle can run the
same model.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field

import numpy as np

from . import synth
from .runtime import Context, DecoderConfig

QKV, O, GATE_UP, DOWN, LM_HEAD = 0, 1, 2, 3, 4
NORM_INPUT, NORM_POST_ATTN, NORM_PRE_FFN, NORM_POST_FFN, NORM_Q, NORM_K, NORM_FINAL = range(7)

GEMMA3_1B = dict(n_layers=26, hidden=1152, ffn=6912, n_q_heads=4, n_kv_heads=1, head_dim=256, vocab=262144,
                 block_size=32, rms_eps=1e-6, rope_theta=10000.0, attn_scale=1.0 / 16.0, embed_scale=float(np.sqrt(1152.0)))


@dataclass
class Weights:
    """Host copy of a synthetic model: linears as (B, scales, zp) in the ONNX layout."""
    cfg: dict
    linears: dict = field(default_factory=dict)   # (layer, which) -> (B, scales, zp)
    norms: dict = field(default_factory=dict)     # (layer, which) -> float32 vector
    embedding: tuple = None


def _shape(cfg, which):
    qd, kvd = cfg["n_q_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    return {QKV: (cfg["hidden"], qd + 2 * kvd), O: (qd, cfg["hidden"]), GATE_UP: (cfg["hidden"], 2 * cfg["ffn"]),
            DOWN: (cfg["ffn"], cfg["hidden"]), LM_HEAD: (cfg["hidden"], cfg["vocab"])}[which]


def build_weights(cfg: dict, seed: int, fast: bool = True) -> Weights:
    """Random int4 linears (uniform nibbles, scales U(0.005, 0.05)/sqrt(K/1152) so activations stay O(1),
    uniform zero points), norm weights near 1."""
    rng = np.random.default_rng(seed)
    w = Weights(cfg)
    bs = cfg["block_size"]

    def linear(K, N, s):
        B, scales, zp = synth.fast_nbits_weight(N, K, bs, s)
        return B, (scales * np.float32(np.sqrt(1152.0 / K) * 0.5)).astype(np.float32), zp

    s = seed * 1000
    for li in range(cfg["n_layers"]):
        for which in (QKV, O, GATE_UP, DOWN):
            K, N = _shape(cfg, which)
            w.linears[(li, which)] = linear(K, N, s)
            s += 1
        for which in (NORM_INPUT, NORM_POST_ATTN, NORM_PRE_FFN, NORM_POST_FFN):
            w.norms[(li, which)] = (1.0 + 0.1 * rng.standard_normal(cfg["hidden"])).astype(np.float32)
        for which in (NORM_Q, NORM_K):
            w.norms[(li, which)] = (1.0 + 0.1 * rng.standard_normal(cfg["head_dim"])).astype(np.float32)
    K, N = _shape(cfg, LM_HEAD)
    w.linears[(0, LM_HEAD)] = linear(K, N, s)
    w.norms[(0, NORM_FINAL)] = (1.0 + 0.1 * rng.standard_normal(cfg["hidden"])).astype(np.float32)
    w.embedding = synth.fast_nbits_weight(cfg["vocab"], cfg["hidden"], bs, s + 1)
    return w


class Decoder:
    def __init__(self, ctx: Context, cfg: dict, max_seq: int):
        self.ctx, self.cfg, self.max_seq = ctx, dict(cfg), max_seq
        c = DecoderConfig(cfg["n_layers"], cfg["hidden"], cfg["ffn"], cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"],
                          cfg["vocab"], max_seq, cfg["block_size"], cfg["rms_eps"], cfg["rope_theta"], cfg["attn_scale"],
                          cfg["embed_scale"])
        h = C.c_void_p()
        ctx._check(ctx.lib.hipc_decoder_create(ctx.handle, C.byref(c), C.byref(h)))
        self.handle = h

    def load(self, w: Weights):
        ctx = self.ctx
        for (li, which), (B, scales, zp) in w.linears.items():
            dB, dS, dZ = ctx.upload(B), ctx.upload(scales), ctx.upload(zp)
            ctx._check(ctx.lib.hipc_decoder_set_linear(ctx.handle, self.handle, li, which, dB.ptr, B.size, dS.ptr,
                                                       scales.size, dZ.ptr, zp.size))
            ctx.flush()
            for b in (dB, dS, dZ):
                b.free()
        for (li, which), v in w.norms.items():
            dV = ctx.upload(v)
            ctx._check(ctx.lib.hipc_decoder_set_norm(ctx.handle, self.handle, li, which, dV.ptr))
            ctx.flush()
            dV.free()
        B, scales, zp = w.embedding
        dB, dS, dZ = ctx.upload(B), ctx.upload(scales), ctx.upload(zp)
        ctx._check(ctx.lib.hipc_decoder_set_embedding(ctx.handle, self.handle, dB.ptr, B.size, dS.ptr, scales.size, dZ.ptr,
                                                      zp.size))
        ctx.flush()
        for b in (dB, dS, dZ):
            b.free()

    def reset(self, token: int, pos: int = 0):
        self.ctx._check(self.ctx.lib.hipc_decoder_reset(self.ctx.handle, self.handle, token, pos))

    def set_layer_attention(self, layer: int, window: int = 0, rope_theta: float = 0.0):
        """``window`` > 0: the layer sees its last ``window`` positions only (GroupQueryAttention's
        local_window_size); ``rope_theta`` > 0: this layer's rotary base."""
        self.ctx._check(self.ctx.lib.hipc_decoder_set_layer_attention(self.ctx.handle, self.handle, layer, window, rope_theta))

    def kv_cache(self, layer: int):
        k, v = C.c_void_p(), C.c_void_p()
        self.ctx._check(self.ctx.lib.hipc_decoder_kv_cache(self.ctx.handle, self.handle, layer, C.byref(k), C.byref(v)))
        return k.value, v.value

    def fill_cache(self, layer: int, k_rows: np.ndarray, v_rows: np.ndarray):
        """Write the first positions of a layer's cache from ``[n_kv_heads, n, head_dim]`` f16 rows
        (what a prefill would leave): keys as they are, values transposed into the library's
        ``[n_kv_heads, head_dim, v_stride]`` layout."""
        nkv, hd = self.cfg["n_kv_heads"], self.cfg["head_dim"]
        n = k_rows.shape[1]
        assert k_rows.shape == (nkv, n, hd) and v_rows.shape == (nkv, n, hd) and n <= self.max_seq
        kptr, vptr = self.kv_cache(layer)
        stride = (self.max_seq + 63) // 64 * 64
        up = self.ctx.lib.hipc_upload
        for h in range(nkv):
            rows = np.ascontiguousarray(k_rows[h], np.float16)
            self.ctx._check(up(self.ctx.handle, kptr, h * self.max_seq * hd * 2, rows.ctypes.data, rows.nbytes))
        vt = np.zeros((nkv, hd, stride), np.float16)
        vt[:, :, :n] = np.transpose(v_rows, (0, 2, 1))
        self.ctx._check(up(self.ctx.handle, vptr, 0, vt.ctypes.data, vt.nbytes))

    def step(self):
        self.ctx._check(self.ctx.lib.hipc_decoder_step(self.ctx.handle, self.handle))

    def read(self, want_logits: bool = False, n_history: int = 0):
        tok, pos = C.c_int32(), C.c_int32()
        logits = np.empty(self.cfg["vocab"], np.float32) if want_logits else None
        hist = np.empty(n_history, np.int32) if n_history else None
        self.ctx._check(self.ctx.lib.hipc_decoder_read(
            self.ctx.handle, self.handle, C.byref(tok), C.byref(pos), None if logits is None else logits.ctypes.data,
            None if hist is None else hist.ctypes.data, n_history))
        return tok.value, pos.value, logits, hist

    def destroy(self):
        if self.handle:
            self.ctx.lib.hipc_decoder_destroy(self.ctx.handle, self.handle)
            self.handle = None


def bytes_per_token(cfg: dict, context: int) -> int:
    """Compulsory HBM bytes of one decode step: every linear once (packed weight + scales + zero
    points, block 32) plus the f16 KV cache over `context` positions (the accounting of the
    reference's work model, crates/onnx-vulkan-core/src/work.rs:263-301)."""
    bs = cfg["block_size"]

    def lin(K, N):
        nb = -(-K // bs)
        return N * nb * bs // 2 + N * nb * 4 + N * ((nb + 1) // 2)

    per_layer = sum(lin(*_shape(cfg, w)) for w in (QKV, O, GATE_UP, DOWN))
    kv = cfg["n_layers"] * 2 * cfg["n_kv_heads"] * context * cfg["head_dim"] * 2
    return cfg["n_layers"] * per_layer + lin(*_shape(cfg, LM_HEAD)) + kv
