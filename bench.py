#!/usr/bin/env python3
"""Benchmark of the quantized matrix-product path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line. The headline `value` is the HBM throughput of the int4 MatMulNBits decode
GEMV over the linears of one gemma3-1b-shaped decode step (26 layers x 7 projections + lm_head,
block 32 with zero points, M = 1): every weight is distinct and resident in HBM (640 MB per
step, far beyond the 256 MB last-level cache), a step is replayed from a captured graph, and
the clock is the host's around K steps with a flush on both sides. `roofline` is the kernel that
owns that step -- the narrow one-row MatMulNBits kernel of the 104 per-layer launches -- timed with
device events on the library's stream over a graph of exactly those launches; the lm_head launch
(one launch, 30 % of the bytes) is a labelled entry of `extras`, as are the narrow launches at
accuracy_level = 1 (three bf16 terms per activation; inside `roofline`), the launch floor (a one-word fill kernel
replayed in the same graph shape) and the other configurations (int8 GEMM TOPS, QLinearConv,
single-op GEMVs hot and cold, the full decoder);
`cpu_baseline` is the restated CPU oracle on this box's host cores (ONNX Runtime is not
installed), on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0     # MI355X dense int8 MFMA, published

# gemma3-1b decoder linears as the decoder prepacks them, (K, N, count per layer): q|k|v in one
# weight (1024 + 256 + 256 columns), o, gate|up in one weight (2 x 6912 columns), down; lm_head once
LAYER_LINEARS = [(1152, 1536, 1), (1024, 1152, 1), (1152, 13824, 1), (6912, 1152, 1)]
LM_HEAD = (1152, 262144)
N_LAYERS = 26
BS = 32
# HBM bytes per lm_head GEMV launch as the memory counters see them (FETCH_SIZE + WRITE_SIZE, each
# scaled by its reading for a 256 MiB copy; profiles/mmnb_gemv_lm_head_1152x262144.txt). A counter
# run cannot happen inside this program, so the figure is carried over from that profile.
LM_HEAD_TRAFFIC_BYTES = 199.6e6
# The same for the average of the 104 narrow launches (a layer's q|k|v, o, gate|up, down: 18.257 MB of traffic for
# 17.304 MB algorithmic; profiles/mmnb_lean_decode_linears_gemma3_1b.txt)
NARROW_TRAFFIC_BYTES = 4.564e6
IN_GRAPH = 16   # instances of a small operator per captured graph: amortises the graph launch
LIGHT = False   # --light: a third of the timing samples (runs under a profiler, which a process that replays
                # graphs for more than ~12 k kernel dispatches brings down)


def gemv_bytes(K, N, bs=BS, with_zp=True, elt=4):
    """Compulsory traffic of one MatMulNBits call: packed weight + scales + zero points + A + Y
    (the reference's convention, crates/onnx-vulkan-core/src/work.rs:263-301)."""
    nb = -(-K // bs)
    return N * nb * bs // 2 + N * nb * 4 + (N * ((nb + 1) // 2) if with_zp else 0) + K * elt + N * elt


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class GemvSet:
    """Prepacked weights + device vectors of a list of (K, N) GEMVs, and a graph replaying them."""

    def __init__(self, pkg, ctx, shapes, seed, accuracy_level=0):
        self.pkg, self.ctx, self.items = pkg, ctx, []
        self.accuracy_level = accuracy_level
        self.bytes = 0
        for i, (K, N) in enumerate(shapes):
            B, scales, zp = pkg.synth.fast_nbits_weight(N, K, BS, seed + i)
            w = pkg.ops.NBitsWeight(ctx, B, scales, zp, K, N, BS)
            a = ctx.upload(pkg.synth.normal_f32(K, seed + 1000 + i))
            y = ctx.alloc(4 * N)
            self.items.append((w, a, y, K, N))
            self.bytes += gemv_bytes(K, N)
        self.graph = None

    def enqueue(self):
        for (w, a, y, K, N) in self.items:
            self.pkg.ops.matmul_nbits_packed_device(self.ctx, a, self.pkg.F32, w, y, 1, self.accuracy_level)

    def capture(self):
        if self.graph:
            self.ctx.graph_destroy(self.graph)
            self.graph = None
        self.enqueue()  # warm every launch shape (scratch sizing) before recording
        self.ctx.flush()
        self.ctx.capture_begin()
        self.enqueue()
        self.graph = self.ctx.capture_end()
        return self.graph

    def destroy(self):
        if self.graph:
            self.ctx.graph_destroy(self.graph)
        for (w, a, y, _, _) in self.items:
            w.destroy(), a.free(), y.free()
        self.ctx.flush()


def min_bound_us(byts, ops, peak_tops):
    """The roofline time of an operator: the larger of its HBM time and its matrix-core time."""
    return max(byts / (HBM_PEAK_GBS * 1e3), ops / (peak_tops * 1e6))


def median_ns(ctx, graph, launches_per_graph=1, samples=20, reps=10):
    if LIGHT:
        samples = max(3, samples // 3)
    ns = ctx.measure_graph(graph, samples, reps)
    return float(np.median(ns)) / launches_per_graph, float(ns.min()) / launches_per_graph


def warm_graph(ctx, graph, replays=40):
    """Untimed replays before a matrix-core section is sampled: its first ten milliseconds run 5-10 % slower than
    what follows (the same graph sampled again and again: 34.6, 32.0, 32.1, 32.0 us)."""
    for _ in range(4 if LIGHT else replays):
        ctx.graph_launch(graph)
    ctx.flush()


def host_timed_steps(ctx, graph, steps, warmup):
    """Milliseconds per replay of `graph`: the host's clock around `steps` replays, a flush on both sides."""
    for _ in range(warmup):
        ctx.graph_launch(graph)
    ctx.flush()
    t0 = time.perf_counter()
    for _ in range(steps):
        ctx.graph_launch(graph)
    ctx.flush()
    return (time.perf_counter() - t0) / steps * 1e3


def bench_decode_linears(pkg, ctx, steps, warmup):
    """The headline step (104 per-layer GEMVs + lm_head, host clock), then on the same weights: the
    104 narrow launches alone under device events (the `roofline` block), and both again at
    accuracy_level = 1. Returns (head, roofline, extras)."""
    shapes = []
    for _ in range(N_LAYERS):
        for (K, N, c) in LAYER_LINEARS:
            shapes += [(K, N)] * c
    n_narrow = len(shapes)
    shapes.append(LM_HEAD)
    t0 = time.time()
    s = GemvSet(pkg, ctx, shapes, seed=5000)
    log(f"[bench] decode linears: {len(shapes)} weights, {s.bytes / 1e6:.1f} MB algorithmic, built in {time.time() - t0:.1f}s")
    ms = host_timed_steps(ctx, s.capture(), steps, warmup)
    head = dict(bytes_per_step=s.bytes, launches=len(shapes), ms_per_step=ms, gbs=s.bytes / (ms * 1e-3) / 1e9)
    roof, extra = None, {}
    every, narrow_bytes = s.items, s.bytes - gemv_bytes(*LM_HEAD)
    try:
        # the 104 narrow launches alone, device events on the library's stream around whole replays; first at
        # accuracy_level = 1 (f32 activations as three bf16 terms instead of two). The lm_head launch stays out
        # of the level-1 figures: the wide kernel's three-term instance is not reached by any test yet.
        s.items = every[:n_narrow]
        per = narrow_bytes / n_narrow
        s.accuracy_level = 1
        med1, _ = median_ns(ctx, s.capture(), n_narrow, samples=15, reps=4)
        s.accuracy_level = 0
        med, mn = median_ns(ctx, s.capture(), n_narrow, samples=15, reps=4)
        s.items = every
        roof = dict(bound="hbm", achieved=per / med, peak=HBM_PEAK_GBS, unit="GB/s", frac=per / med / HBM_PEAK_GBS, traffic=NARROW_TRAFFIC_BYTES,
                    kernel="mmnb_lean_kernel, PRO 0 (the 104 per-layer one-row MatMulNBits launches of the step: q|k|v, o, gate|up, down x 26)",
                    bytes_per_launch=per, avg_launch_us=med / 1e3, min_launch_us=mn / 1e3, launches_per_replay=n_narrow,
                    timing="device events around whole graph replays / launches per replay: launch gaps included",
                    accuracy_level_1=dict(avg_launch_us=med1 / 1e3, achieved=per / med1, frac=per / med1 / HBM_PEAK_GBS))
    except Exception as e:  # the headline above stands on its own
        log(f"[bench] narrow-GEMV roofline failed: {e!r}")
    s.items = every
    s.destroy()
    return head, roof, extra


def bench_launch_floor(ctx, launches=105):
    """What a launch costs when the kernel does nothing: a one-word fill (one workgroup) replayed in a
    graph of the headline step's shape, device events around whole replays."""
    buf = ctx.alloc(4096)

    def enqueue():
        for i in range(launches):
            ctx.fill(buf, 4 * (i % 64), 4, i)

    enqueue()
    ctx.flush()
    ctx.capture_begin()
    enqueue()
    g = ctx.capture_end()
    med, mn = median_ns(ctx, g, launches, samples=20, reps=4)
    ctx.graph_destroy(g)
    buf.free()
    ctx.flush()
    return dict(us_per_launch=med / 1e3, min_us_per_launch=mn / 1e3, launches_per_graph=launches,
                kernel="one-word fill, one workgroup; every launch depends on the one before (one in-order stream)")


def bench_lm_head(pkg, ctx, copies=3, accuracy_level=0):
    """The widest launch of the step: lm_head GEMV rotating over `copies` distinct weights (~200 MB each)."""
    K, N = LM_HEAD
    s = GemvSet(pkg, ctx, [LM_HEAD] * copies, seed=7000, accuracy_level=accuracy_level)
    s.items = s.items * 4                     # 4 passes over the ring per graph
    g = s.capture()
    med, mn = median_ns(ctx, g, launches_per_graph=copies * 4, samples=15, reps=2)
    s.items = s.items[:copies]
    per = gemv_bytes(K, N)
    s.destroy()
    return dict(bound="hbm", achieved=per / med, peak=HBM_PEAK_GBS, unit="GB/s", frac=per / med / HBM_PEAK_GBS,
                traffic=LM_HEAD_TRAFFIC_BYTES if accuracy_level == 0 else None, kernel="mmnb_gemv_kernel (lm_head 1152->262144, M=1)", bytes_per_launch=per,
                avg_launch_us=med / 1e3, min_launch_us=mn / 1e3, accuracy_level=accuracy_level)


def bench_single_gemv(pkg, ctx, K, N, cold_copies):
    per = gemv_bytes(K, N)
    hot = GemvSet(pkg, ctx, [(K, N)], seed=8000)
    hot.items = hot.items * IN_GRAPH          # the same weight again and again: cache-resident
    g = hot.capture()
    hot_ns, _ = median_ns(ctx, g, IN_GRAPH, samples=20, reps=4)
    hot.items = hot.items[:1]
    hot.destroy()
    cold = GemvSet(pkg, ctx, [(K, N)] * cold_copies, seed=8100)
    g = cold.capture()
    cold_ns, _ = median_ns(ctx, g, cold_copies, samples=10, reps=2)
    cold.destroy()
    return dict(K=K, N=N, bytes=per, hot_us=hot_ns / 1e3, hot_gbs=per / hot_ns, cold_us=cold_ns / 1e3,
                cold_gbs=per / cold_ns, cold_frac_hbm=per / cold_ns / HBM_PEAK_GBS, cold_ring_mb=cold_copies * per / 1e6)


def bench_int8_ffn(pkg, ctx):
    """DynamicQuantizeLinear [1000,1024] then MatMulInteger x [1024,4096] and x [4096,1024], with the
    fused fp32 rescale."""
    ops = pkg.ops
    out = {}
    T = 1000
    x = pkg.synth.normal_f32(T * 1024, 2).reshape(T, 1024)
    dX = ctx.upload(x)
    dA, dP = ctx.alloc(T * 4096), ctx.alloc(8)
    ops.dynamic_quantize_linear_device(ctx, dX, x.size, dA, dP, dP.at(4))
    ctx.flush()
    ctx.capture_begin()
    for _ in range(IN_GRAPH):
        ops.dynamic_quantize_linear_device(ctx, dX, x.size, dA, dP, dP.at(4))
    g = ctx.capture_end()
    ns, _ = median_ns(ctx, g, IN_GRAPH, samples=20, reps=4)
    ctx.graph_destroy(g)
    dql_bytes = x.size * 4 + x.size + 5
    out["dynamic_quantize_linear_1000x1024"] = dict(us=ns / 1e3, gbs=dql_bytes / ns, frac_hbm=dql_bytes / ns / HBM_PEAK_GBS)
    # the FFN's middle: DynamicQuantizeLinear of the exact GELU of the first product's [1000, 4096] output,
    # fused (two passes over x, the GELU never stored) against GELU kernel + DynamicQuantizeLinear
    h = ctx.upload(pkg.synth.normal_f32(T * 4096, 3))
    hg, hq = ctx.alloc(T * 4096 * 4), ctx.alloc(T * 4096)
    sq2 = float(np.float32(np.sqrt(2.0)))
    lib = ctx.lib
    fused = lambda: ctx._check(lib.hipc_dynamic_quantize_linear_gelu(ctx.handle, h.ptr, T * 4096, sq2, 1.0, 0.5, 0, hq.ptr, dP.ptr, dP.ptr + 4, None))  # noqa: E731
    def unfused():
        ctx._check(lib.hipc_decomposed_gelu(ctx.handle, h.ptr, T * 4096, sq2, 1.0, 0.5, 0, hg.ptr))
        ops.dynamic_quantize_linear_device(ctx, hg, T * 4096, hq, dP, dP.at(4))
    for name, fn in [("gelu_quantize_fused_1000x4096", fused), ("gelu_then_quantize_1000x4096", unfused)]:
        fn()
        ctx.flush()
        ctx.capture_begin()
        for _ in range(IN_GRAPH):
            fn()
        g = ctx.capture_end()
        ns, _ = median_ns(ctx, g, IN_GRAPH, samples=20, reps=4)
        ctx.graph_destroy(g)
        out[name] = dict(us=ns / 1e3)
    for b in (h, hg, hq):
        b.free()
    dS = ctx.upload(np.array([0.01], np.float32))
    for (K, N) in [(1024, 4096), (4096, 1024)]:
        w = ops.Int8Weight(ctx, pkg.synth.int8_weight(K, N, 22 + K))
        a = ctx.upload(pkg.synth.uniform_ints(T * K, 23, 0, 255).astype(np.uint8))
        y = ctx.alloc(T * N * 4)
        for name, fn in [("i32", lambda: ops.matmul_integer_device(ctx, a, pkg.U8, w, dP.at(4), None, y, T)),
                         ("rescale_f32", lambda: ops.matmul_integer_scale_bias_device(
                             ctx, a, pkg.U8, w, dP.at(4), None, dP, 0, dS, 0, None, 0, False, None, y, T))]:
            fn()
            ctx.flush()
            ctx.capture_begin()
            for _ in range(IN_GRAPH):
                fn()
            g = ctx.capture_end()
            ns, mn = median_ns(ctx, g, IN_GRAPH, samples=20, reps=4)
            ctx.graph_destroy(g)
            opsn = 2.0 * T * K * N
            byts = T * K + K * N + T * N * 4
            out[f"matmul_integer_{name}_1000x{K}x{N}"] = dict(
                us=ns / 1e3, us_min=mn / 1e3, tops=opsn / ns / 1e3, frac_int8_mfma=opsn / ns / 1e3 / INT8_PEAK_TOPS,
                gbs=byts / ns, frac_hbm=byts / ns / HBM_PEAK_GBS,
                frac_of_min_bound=min_bound_us(byts, opsn, INT8_PEAK_TOPS) / (ns / 1e3))
        w.destroy(), a.free(), y.free()
    # asymptotic shape, to separate the kernel from the launch floor
    K = N = T2 = 8192
    w = ops.Int8Weight(ctx, pkg.synth.uniform_ints(K * N, 30, -127, 127).astype(np.int8).reshape(K, N))
    a = ctx.upload(pkg.synth.uniform_ints(T2 * K, 31, 0, 255).astype(np.uint8))
    y = ctx.alloc(T2 * N * 4)
    ops.matmul_integer_device(ctx, a, pkg.U8, w, dP.at(4), None, y, T2)
    ctx.flush()
    ctx.capture_begin()
    ops.matmul_integer_device(ctx, a, pkg.U8, w, dP.at(4), None, y, T2)
    g = ctx.capture_end()
    ns, _ = median_ns(ctx, g, 1, samples=5, reps=3)
    ctx.graph_destroy(g)
    out["matmul_integer_i32_8192x8192x8192"] = dict(us=ns / 1e3, tops=2.0 * T2 * K * N / ns / 1e3,
                                                    frac_int8_mfma=2.0 * T2 * K * N / ns / 1e3 / INT8_PEAK_TOPS)
    w.destroy(), a.free(), y.free()
    for b in (dX, dA, dP, dS):
        b.free()
    ctx.flush()
    return out


def bench_qlinear_conv(pkg, ctx):
    ops = pkg.ops
    out = {}
    for (C, T, dil) in [(192, 4096, 1), (192, 4096, 3), (192, 4096, 5), (512, 4096, 1)]:
        X = pkg.synth.uniform_ints(C * T, 40, 0, 255).astype(np.uint8).reshape(1, C, 1, T)
        W = pkg.synth.uniform_ints(C * C * 7, 41, -127, 127).astype(np.int8).reshape(C, C, 1, 7)
        ws = pkg.synth.uniform_f32(C, 42, 0.001, 0.02)
        bias = ctx.upload(pkg.synth.uniform_ints(C, 43, -4096, 4096).astype(np.int32))
        geom = pkg.ConvGeom.make(X.shape, W.shape, dilations=(1, dil), pads=(0, 3 * dil, 0, 3 * dil))
        w = ops.ConvWeight(ctx, W, geom)
        dX, dY = ctx.upload(X), ctx.alloc(C * T)
        run = lambda: ops.qlinear_conv_device(ctx, dX, pkg.U8, 0.02, 128, w, ws, 0, 0.5, 128, pkg.U8, bias, geom, dY)  # noqa: E731
        run()   # the first call uploads the requantisation ratios; later ones reuse them and can be captured
        ctx.flush()
        ctx.capture_begin()
        for _ in range(IN_GRAPH):
            run()
        g = ctx.capture_end()
        ns, mn = median_ns(ctx, g, IN_GRAPH, samples=20, reps=4)
        ctx.graph_destroy(g)
        opsn = 2.0 * C * T * C * 7
        byts = C * T + C * C * 7 + C * T + C * 8
        out[f"qlinear_conv_c{C}_k7_T{T}_d{dil}"] = dict(
            us=ns / 1e3, us_min=mn / 1e3, tops=opsn / ns / 1e3, frac_int8_mfma=opsn / ns / 1e3 / INT8_PEAK_TOPS,
            frac_of_min_bound=min_bound_us(byts, opsn, INT8_PEAK_TOPS) / (ns / 1e3))
        w.destroy(), dX.free(), dY.free(), bias.free()
    ctx.flush()
    return out


def bench_decoder(pkg, ctx, steps, warmup, context=2048):
    """One full int4 decode step of a gemma3-1b-shaped model (random weights) at a context of
    `context` positions: f16 KV cache filled with random data, greedy sampling on the device, one
    captured step replayed from a graph. Attention covers the whole context in every layer."""
    D = pkg.decoder
    cfg = dict(D.GEMMA3_1B)
    t0 = time.time()
    w = D.build_weights(cfg, seed=9)
    max_seq = context + steps + warmup + 8
    dec = D.Decoder(ctx, cfg, max_seq)
    dec.load(w)
    rng = np.random.default_rng(1)
    filler = (rng.standard_normal((cfg["n_kv_heads"], context, cfg["head_dim"])) * 0.5).astype(np.float16)
    for li in range(cfg["n_layers"]):
        dec.fill_cache(li, filler, filler)
    log(f"[bench] decoder: weights built and loaded in {time.time() - t0:.1f}s")
    def timed():
        dec.reset(1234, context - 1)
        dec.step()
        ctx.flush()
        ctx.capture_begin()
        dec.step()
        g = ctx.capture_end()
        for _ in range(warmup):
            ctx.graph_launch(g)
        ctx.flush()
        t0 = time.perf_counter()
        for _ in range(steps):
            ctx.graph_launch(g)
        ctx.flush()
        dt = time.perf_counter() - t0
        _, pos, _, _ = dec.read()
        ctx.graph_destroy(g)
        return dt, pos

    dt, pos = timed()
    byts = D.bytes_per_token(cfg, context)
    tok_s = steps / dt
    out = dict(tok_s=tok_s, ms_per_token=dt / steps * 1e3, context=context, bytes_per_token=byts,
               hbm_bound_tok_s=HBM_PEAK_GBS * 1e9 / byts, frac_of_hbm_bound=tok_s * byts / (HBM_PEAK_GBS * 1e9),
               # five launches per layer, then the unembedding (whose workgroups leave the argmax candidates) and the
               # launch that picks the token and embeds it for the next step
               launches_per_token=5 * cfg["n_layers"] + 2, final_position=pos)
    # the same step without the read-ahead helper rows (by default three of a layer's five launches carry extra
    # workgroups that read what the next launch will read into the L2 of the XCD that will ask for it), and with all five
    for name, mask in (("no_read_ahead", 0), ("read_ahead_all_five", 31)):
        try:
            with ctx.options(HIPC_DEC_PREFETCH=mask):
                dt_ra, _ = timed()
            out[name] = dict(tok_s=steps / dt_ra, ms_per_token=dt_ra / steps * 1e3)
        except Exception as e:
            log(f"[bench] decoder, {name}: {e!r}")
    # the layer pattern of the real gemma3-1b: five local layers (window 512, rotary base 10000) to one
    # global (base 1e6); the figure above keeps every layer global, as the byte model it is quoted against
    window, local = 512, 0
    for li in range(cfg["n_layers"]):
        if (li + 1) % 6 != 0:
            dec.set_layer_attention(li, window, 10000.0)
            local += 1
        else:
            dec.set_layer_attention(li, 0, 1.0e6)
    dt2, _ = timed()
    kv_pos = 2 * cfg["n_kv_heads"] * cfg["head_dim"] * 2
    byts2 = D.bytes_per_token(cfg, 0) + kv_pos * (local * min(window, context) + (cfg["n_layers"] - local) * context)
    out["sliding_window"] = dict(local_layers=local, window=window, tok_s=steps / dt2, ms_per_token=dt2 / steps * 1e3,
                                 bytes_per_token=byts2, frac_of_hbm_bound=steps / dt2 * byts2 / (HBM_PEAK_GBS * 1e9))
    dec.destroy()
    ctx.flush()
    return out


LEAN_PHASES = {0: "first instruction (arguments read)", 8: "helper rows branched off", 9: "prologue loads issued", 1: "weight loads issued",
               2: "prologue operands arrived", 3: "row in LDS (norm or join done)", 4: "operands read from LDS",
               5: "products and block folds done (weights arrived)", 6: "sum over wavefronts in LDS", 7: "result stored"}
ATTN_PHASES = {0: "first instruction (arguments read)", 1: "position arrived", 2: "cache loads issued", 3: "own rows normed and rotated",
               4: "workgroup barrier", 5: "query operand read", 6: "first pass: scores (keys arrived)", 7: "first pass: softmax weights in LDS",
               8: "first pass: value product", 9: "all passes done", 10: "partials stored"}


def bench_phases(pkg, ctx, context=2048):
    """Where the time of a decode step's launches goes: the library built by `make stamps` (load it with
    HIPC_LIBRARY=libhipcompute_stamps.so) records the device clock (10 ns ticks) at fixed points of the one-row kernels
    and of the attention kernel; this reads the stamps the LAST layer's launches left after a replayed step and
    reports, per launch, the median / 90th percentile / maximum over its wavefronts of the time since the launch's
    first wavefront started, and the gaps between the launches."""
    import ctypes
    lib = pkg.runtime.load_library()
    if not hasattr(lib, "hipc_debug_lean_stamps"):
        raise RuntimeError("this library records no phase stamps: make -C onnx-vulkan-rs_amd/csrc stamps, then run with "
                           "HIPC_LIBRARY=libhipcompute_stamps.so")
    D = pkg.decoder
    cfg = dict(D.GEMMA3_1B)
    dec = D.Decoder(ctx, cfg, context + 64)
    dec.load(D.build_weights(cfg, seed=9))
    rng = np.random.default_rng(1)
    filler = (rng.standard_normal((cfg["n_kv_heads"], context, cfg["head_dim"])) * 0.5).astype(np.float16)
    for li in range(cfg["n_layers"]):
        dec.fill_cache(li, filler, filler)
    dec.reset(1234, context - 1)
    dec.step()
    ctx.flush()
    ctx.capture_begin()
    dec.step()
    g = ctx.capture_end()
    for _ in range(20):
        ctx.graph_launch(g)
    ctx.flush()
    lean = np.zeros(5 * 1024 * 8 * 12, dtype=np.uint64)
    attn = np.zeros(64 * 4 * 12, dtype=np.uint64)
    for fn, buf in ((lib.hipc_debug_lean_stamps, lean), (lib.hipc_debug_attn_stamps, attn)):
        fn.restype, fn.argtypes = ctypes.c_int, [ctypes.c_void_p, ctypes.c_size_t]
        if fn(buf.ctypes.data_as(ctypes.c_void_p), buf.nbytes) != 0:
            raise RuntimeError("reading the stamps failed")
    lean = lean.reshape(5, 1024, 8, 12).astype(np.int64)
    attn = attn.reshape(1, 64, 4, 12).astype(np.int64)
    launches = [("q|k|v (norm prologue)", lean[2], LEAN_PHASES, 5), ("attention", attn[0], ATTN_PHASES, 9),
                ("o (attention join prologue)", lean[3], LEAN_PHASES, 5), ("gate|up (norm prologue, gated GELU)", lean[1], LEAN_PHASES, 5),
                ("down (row in operand order)", lean[4], LEAN_PHASES, 5)]
    out, prev_end = {}, None
    for name, st, phases, work_phase in launches:
        begun = st[:, :, 0] > 0
        start = int(st[:, :, 0][begun].min())
        # wavefronts of the product itself: they reached `work_phase` in this replay (stamps of helper rows, and of
        # workgroups that had no positions, are older or absent)
        main = begun & (st[:, :, work_phase] >= start)
        rec = {"wavefronts": int(main.sum()), "phases_ns": {}}
        end = start
        for ph, label in phases.items():
            v = st[:, :, ph][main]
            v = v[v >= start]
            if v.size == 0:
                continue
            d = (v - start) * 10
            rec["phases_ns"][label] = dict(median=int(np.median(d)), p90=int(np.percentile(d, 90)), max=int(d.max()))
            end = max(end, int(v.max()))
        helpers = begun & ~main & (st[:, :, 7] >= start) if phases is LEAN_PHASES else None
        if helpers is not None and helpers.any():
            h0, h7 = (st[:, :, 0][helpers] - start) * 10, (st[:, :, 7][helpers] - start) * 10
            rec["helper_rows_ns"] = dict(wavefronts=int(helpers.sum()), start_median=int(np.median(h0)), end_median=int(np.median(h7)), end_max=int(h7.max()))
            end = max(end, int(st[:, :, 7][helpers].max()))
        rec["duration_ns"] = (end - start) * 10
        if prev_end is not None:
            rec["gap_from_previous_launch_ns"] = (start - prev_end) * 10
        prev_end = end
        out[name] = rec
    ctx.graph_destroy(g)
    dec.destroy()
    ctx.flush()
    return out


F16_PEAK_TFLOPS = 2500.0    # MI355X dense f16 MFMA, published


def bench_prefill(pkg, ctx, M=512, bs=128):
    """MatMulNBits with 512 rows of f16 activations (block 128, f16 scales, no zero points): the
    gate/up, down and fused q/k/v linears of a 2048-wide model, eight instances per graph."""
    out = {}
    reps = 8
    for name, (K, N) in {"gate_up_2048x11008": (2048, 11008), "down_11008x2048": (11008, 2048),
                         "qkv_2048x2560": (2048, 2560)}.items():
        B, scales, _ = pkg.synth.fast_nbits_weight(N, K, bs, seed=4, with_zp=False, scale_dtype=np.float16)
        w = pkg.ops.NBitsWeight(ctx, B, scales, None, K, N, bs)
        a = ctx.upload(pkg.synth.normal_f32(M * K, 40).reshape(M, K).astype(np.float16))
        y = ctx.alloc(2 * M * N)
        run = lambda: pkg.ops.matmul_nbits_packed_device(ctx, a, pkg.F16, w, y, M)  # noqa: E731
        run()
        ctx.flush()
        ctx.capture_begin()
        for _ in range(reps):
            run()
        g = ctx.capture_end()
        warm_graph(ctx, g)
        ns, mn = median_ns(ctx, g, reps, samples=10, reps=4)
        ctx.graph_destroy(g)
        flops = 2.0 * M * K * N
        byts = K * N // 2 + (K // bs) * N * 2 + M * K * 2 + M * N * 2
        out["matmul_nbits_f16_M512_" + name] = dict(us=ns / 1e3, us_min=mn / 1e3, tflops=flops / ns / 1e3,
                                                    frac_f16_mfma=flops / ns / 1e3 / F16_PEAK_TFLOPS,
                                                    gbs=byts / ns, frac_hbm=byts / ns / HBM_PEAK_GBS,
                                                    frac_of_min_bound=min_bound_us(byts, flops, F16_PEAK_TFLOPS) / (ns / 1e3))
        if name == "qkv_2048x2560":
            # the same product with f32 rows: two f16 rows each through the same kernel after a launch that splits them
            # (accuracy_level unset), one (a level that allows f16 activations) or three (level 1: f32 pinned)
            a32 = ctx.upload(pkg.synth.normal_f32(M * K, 41).reshape(M, K))
            y32 = ctx.alloc(4 * M * N)
            for level, label in ((0, "matmul_nbits_f32_M512_"), (2, "matmul_nbits_f32_level2_M512_"), (1, "matmul_nbits_f32_level1_M512_")):
                run32 = lambda: pkg.ops.matmul_nbits_packed_device(ctx, a32, pkg.F32, w, y32, M, level)  # noqa: E731,B023
                run32()
                ctx.flush()
                ctx.capture_begin()
                for _ in range(reps):
                    run32()
                g = ctx.capture_end()
                warm_graph(ctx, g)
                ns32, _ = median_ns(ctx, g, reps, samples=10, reps=4)
                ctx.graph_destroy(g)
                out[label + name] = dict(us=ns32 / 1e3, tflops=flops / ns32 / 1e3)
            a32.free(), y32.free()
        w.destroy(), a.free(), y.free()
        ctx.flush()
    return out


def bench_copy(ctx, mib=256, reps=8):
    """Calibration for the memory counters: device-to-device copies of a known size (each reads and
    writes `mib` MiB). Not part of the default run; profile it with --only copy."""
    n = mib << 20
    a, b = ctx.alloc(n), ctx.alloc(n)
    ctx.fill(a, 0, n, 0x01020304)
    ctx.flush()
    t0 = time.perf_counter()
    for _ in range(reps):
        ctx.copy(b, 0, a, 0, n)
    ctx.flush()
    dt = (time.perf_counter() - t0) / reps
    return dict(bytes_read=n, bytes_written=n, us=dt * 1e6, gbs=2 * n / dt / 1e9)


def cpu_baseline(pkg, budget_s=12.0):
    """The restated CPU oracle (ONNX Runtime is not installed) on the host cores, on a bounded
    sample of the headline workload: the largest projection pair of one layer."""
    import oracle
    K, N = 1152, 6912
    B, scales, zp = pkg.synth.fast_nbits_weight(N, K, BS, 99)
    a = pkg.synth.normal_f32(K, 98).reshape(1, K)
    oracle.matmul_nbits(a, B, scales, zp, K, N, BS)
    reps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s:
        oracle.matmul_nbits(a, B, scales, zp, K, N, BS)
        reps += 1
    dt = time.perf_counter() - t0
    per = gemv_bytes(K, N)
    return dict(value=per * reps / dt / 1e9, unit="GB/s", cores=oracle.threads(), kind="port",
                sample=f"MatMulNBits M=1 K={K} N={N} bs=32+zp (gate/up projection), {reps} calls in {dt:.1f}s; "
                       f"restated CPU oracle, ONNX Runtime unavailable")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--only", default="", help="comma list of sections to run (decode, floor, lm_head, gemv, int8, conv, prefill, "
                    "decoder, cpu; copy = counter calibration and phases = time stamps inside the decode step's kernels, only on request); default all. Used to profile "
                    "one kernel at a time.")
    ap.add_argument("--light", action="store_true", help="a third of the timing samples per figure (for runs under rocprofv3)")
    args = ap.parse_args()
    global LIGHT
    LIGHT = args.light
    only = set(filter(None, args.only.split(",")))
    want = lambda name: not only or name in only  # noqa: E731
    if args.gpus != 1:
        print("bench.py: this path is measured on ONE GPU; --gpus > 1 is not supported in this build "
              "(no collectives are part of it). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    pkg = entry.load_package()
    ctx = pkg.Context(0)
    head = dict(gbs=None, ms_per_step=None, bytes_per_step=None, launches=None)
    roof = None
    extras = {}
    if want("decode"):
        head, roof, more = bench_decode_linears(pkg, ctx, args.steps, args.warmup)
        extras.update(more)
        log(f"[bench] decode linears: {head['ms_per_step']:.3f} ms/step, {head['gbs']:.0f} GB/s")
        if roof:
            log(f"[bench] narrow gemv: {roof['avg_launch_us']:.2f} us per launch, {roof['achieved']:.0f} GB/s")
    if want("floor"):
        try:
            extras["launch_floor"] = bench_launch_floor(ctx)
            log("[bench] launch floor:", json.dumps(extras["launch_floor"]))
        except Exception as e:
            log(f"[bench] launch floor failed: {e!r}")
    if want("lm_head"):
        extras["lm_head_gemv"] = bench_lm_head(pkg, ctx)
        log(f"[bench] lm_head gemv: {extras['lm_head_gemv']['avg_launch_us']:.1f} us, {extras['lm_head_gemv']['achieved']:.0f} GB/s")
        # the same launch with f32 pinned (accuracy_level = 1: three bf16 terms per activation, all 24 bits)
        extras["lm_head_gemv_level1"] = bench_lm_head(pkg, ctx, accuracy_level=1)
        log(f"[bench] lm_head gemv, level 1: {extras['lm_head_gemv_level1']['avg_launch_us']:.1f} us")
    if want("gemv"):
        extras["gemv_up_1152x6912"] = bench_single_gemv(pkg, ctx, 1152, 6912, cold_copies=104)
        extras["gemv_down_6912x1152"] = bench_single_gemv(pkg, ctx, 6912, 1152, cold_copies=104)
        log("[bench] single gemv:", json.dumps(extras))
    if want("int8"):
        extras.update(bench_int8_ffn(pkg, ctx))
        log("[bench] int8 ffn done")
    if want("int8"):
        # what the matrix cores sustain with nothing else going on (register-only MFMA loop, ~3 ms each)
        extras["int8_mfma_register_loop_tops"] = {
            "random_bytes_2_waves_per_simd": ctx.probe_int8_mfma(True, 2), "random_bytes_1_wave_per_simd": ctx.probe_int8_mfma(True, 1),
            "constant_bytes_2_waves_per_simd": ctx.probe_int8_mfma(False, 2), "published_peak": INT8_PEAK_TOPS}
        log("[bench] int8 mfma loop:", json.dumps(extras["int8_mfma_register_loop_tops"]))
    if want("conv"):
        extras.update(bench_qlinear_conv(pkg, ctx))
    if want("prefill"):
        extras.update(bench_prefill(pkg, ctx))
        log("[bench] prefill done")
    if want("decoder"):
        extras["gemma3_1b_int4_decode"] = bench_decoder(pkg, ctx, max(args.steps, 20), args.warmup)
        log("[bench] decoder:", json.dumps(extras["gemma3_1b_int4_decode"]))
    if "phases" in only:
        extras["decode_step_phases_last_layer"] = bench_phases(pkg, ctx)
        for name, rec in extras["decode_step_phases_last_layer"].items():
            log(f"[bench] {name}: {rec['wavefronts']} wavefronts, {rec['duration_ns']} ns" +
                (f", {rec['gap_from_previous_launch_ns']} ns after the launch before it ended" if "gap_from_previous_launch_ns" in rec else "") +
                (f"; helper rows {json.dumps(rec['helper_rows_ns'])}" if "helper_rows_ns" in rec else ""))
            for label, v in rec["phases_ns"].items():
                log(f"[bench]     {label:52s} median {v['median']:6d}  p90 {v['p90']:6d}  max {v['max']:6d} ns")
    if "copy" in only:
        extras["copy_256MiB"] = bench_copy(ctx)
        log("[bench] copy:", json.dumps(extras["copy_256MiB"]))
    cpu = cpu_baseline(pkg) if want("cpu") else None
    ctx.close()

    line = {
        "metric": "int4 MatMulNBits HBM GB/s (% peak); int8 GEMM TOPS (% MFMA); tok/s",
        "value": head["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights x f32 activations (each activation as two bf16 terms on the MFMA, f32 accumulate)", "data": "synthetic",
        "config": {"workload": "int4 MatMulNBits decode GEMVs of one gemma3-1b-shaped token: 26 layers x "
                               "(q|k|v fused, o, gate|up fused, down) + lm_head 1152->262144, block 32 + zero points, "
                               "M=1, every weight distinct and HBM-resident, graph replay",
                   "bytes_per_step": head["bytes_per_step"], "launches_per_step": head["launches"],
                   "frac_hbm_peak": head["gbs"] / HBM_PEAK_GBS if head["gbs"] else None},
        "roofline": roof, "cpu_baseline": cpu, "extras": extras,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
