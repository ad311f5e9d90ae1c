"""The decode step (RMS norm, rotary, f16 KV cache, grouped-query attention, gated GELU, argmax around
the int4 GEMV) against the numpy oracle, step by step with teacher forcing.

Tolerance on the logits: |got - ref| <= 2e-3 + 2e-3 * |ref| -- f32 arithmetic through two layers in a
different summation order, with an f16 cache on both sides."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SMALL = dict(n_layers=2, hidden=128, ffn=256, n_q_heads=4, n_kv_heads=2, head_dim=64, vocab=512, block_size=32,
             rms_eps=1e-6, rope_theta=10000.0, attn_scale=0.0, embed_scale=float(np.sqrt(128.0)))


def test_decode_steps_match_the_oracle(ctx, pkg, oracle):
    from oracle import decoder as od
    steps, max_seq = 70, 80          # crosses several 16-position chunks of the attention kernel
    w = pkg.decoder.build_weights(SMALL, seed=3)
    dec = pkg.decoder.Decoder(ctx, SMALL, max_seq)
    dec.load(w)
    ref = od.Decoder(w, max_seq)
    token = 17
    dec.reset(token, 0)
    agree = 0
    for pos in range(steps):
        dec.step()
        got_tok, got_pos, logits, _ = dec.read(want_logits=True)
        want_logits, want_tok = ref.step(token, pos)
        assert got_pos == pos + 1
        err = np.abs(logits - want_logits)
        assert np.all(err <= 2e-3 + 2e-3 * np.abs(want_logits)), (pos, float(err.max()))
        top2 = np.sort(want_logits)[-2:]
        if top2[1] - top2[0] > 1e-2:
            assert got_tok == want_tok, pos
            agree += 1
        token = got_tok              # teacher forcing: the oracle consumes what the device chose
    assert agree > steps // 2
    _, _, _, hist = dec.read(n_history=steps)
    assert hist[-1] == token
    dec.destroy()


@pytest.mark.parametrize("env", [{}, {"HIPC_DEC_FUSED_ARGMAX": 0}, {"HIPC_DEC_FUSED_GLUE": 0}], ids=["candidates-from-lm_head", "separate-scan", "separate-glue"])
def test_the_token_is_the_argmax_of_the_logits_on_a_wide_vocabulary(ctx, pkg, route, env):
    """A vocabulary wide enough for the unembedding to run on the kernel whose workgroups leave the argmax candidates
    themselves (ragged: 32768 + 48 columns): the token the device picks is the first largest of the logits it stores,
    step after step, and the same with a launch of its own scanning the logits."""
    route(env)
    cfg = dict(SMALL, vocab=32768 + 48)
    w = pkg.decoder.build_weights(cfg, seed=21)
    dec = pkg.decoder.Decoder(ctx, cfg, 24)
    dec.load(w)
    dec.reset(5, 0)
    seen = set()
    for pos in range(12):
        dec.step()
        tok, got_pos, logits, _ = dec.read(want_logits=True)
        assert got_pos == pos + 1 and tok == int(np.argmax(logits)), (pos, tok, int(np.argmax(logits)))
        seen.add(tok)
    assert len(seen) > 1
    dec.destroy()


DEEP = [  # (head_dim, query heads, kv heads, first position): every head_dim / group size the chunk kernel is built for
    (256, 4, 1, 2046),   # crosses from 64 to 128 positions per workgroup at 2048
    (128, 8, 1, 4290),   # three passes per workgroup, the last one ragged
    (64, 2, 2, 2300),    # one query head per kv head
    (128, 4, 2, 130),    # three live chunks only
    (192, 2, 1, 100),    # no instance for this head_dim: the three-kernel path
]
# The read-ahead route (helper workgroups of a launch that warm the L2 for the next launch): one bit per producer
# launch of a layer. By default three of the five producers carry helpers; the other cases run all five and none.
READ_AHEAD = {"HIPC_DEC_PREFETCH": 31}
NO_READ_AHEAD = {"HIPC_DEC_PREFETCH": 0}
PATHS = [{}, READ_AHEAD, {"HIPC_DEC_LEAN": 0}, {"HIPC_DEC_FUSED_GLUE": 0}, {"HIPC_DEC_FUSED_ATTN": 0}]


@pytest.fixture
def route(ctx):
    """Sets route options on the shared context for one test and restores the defaults afterwards."""
    touched = []

    def apply(options):
        for k, v in options.items():
            ctx.set_option(k, v)
            touched.append(k)
    yield apply
    for k in touched:
        ctx.set_option(k, -1)


@pytest.mark.parametrize("env", PATHS, ids=["default", "read-ahead", "streaming-gemv", "separate-glue", "three-kernel-attention"])
@pytest.mark.parametrize("hd,nq,nkv,p0", DEEP)
def test_attention_over_a_long_filled_cache(ctx, pkg, oracle, route, hd, nq, nkv, p0, env):
    """Steps taken deep into a context whose cache rows hold random f16 values on both sides: the
    chunked attention (several passes per workgroup, the join in the output projection's prologue
    or in the merge kernel) against the oracle's softmax over the whole context."""
    from oracle import decoder as od
    route(env)                     # read when the decoder is created
    cfg = dict(SMALL, n_q_heads=nq, n_kv_heads=nkv, head_dim=hd)
    steps, max_seq = 3, p0 + 8
    w = pkg.decoder.build_weights(cfg, seed=11)
    dec = pkg.decoder.Decoder(ctx, cfg, max_seq)
    dec.load(w)
    ref = od.Decoder(w, max_seq)
    rng = np.random.default_rng(hd + p0)
    for li in range(cfg["n_layers"]):
        k_rows, v_rows = ((rng.standard_normal((nkv, max_seq, hd)) * 0.7).astype(np.float16) for _ in range(2))
        ref.k[li], ref.v[li] = k_rows, v_rows
        dec.fill_cache(li, k_rows, v_rows)
    token = 23
    dec.reset(token, p0)
    for pos in range(p0, p0 + steps):
        dec.step()
        got_tok, got_pos, logits, _ = dec.read(want_logits=True)
        want_logits, _ = ref.step(token, pos)
        assert got_pos == pos + 1
        err = np.abs(logits - want_logits)
        assert np.all(err <= 2e-3 + 2e-3 * np.abs(want_logits)), (pos, float(err.max()))
        k_row = ctx.download(dec.kv_cache(1)[0], np.float16, (hd,), offset=((nkv - 1) * max_seq + pos) * hd * 2)
        assert np.allclose(k_row.astype(np.float32), ref.k[1, nkv - 1, pos].astype(np.float32), atol=2e-3, rtol=2e-3), pos
        stride = (max_seq + 63) // 64 * 64       # values are kept transposed: [kv head, channel, position]
        v_t = ctx.download(dec.kv_cache(1)[1], np.float16, (nkv, hd, stride))
        assert np.allclose(v_t[nkv - 1, :, pos].astype(np.float32), ref.v[1, nkv - 1, pos].astype(np.float32), atol=2e-3, rtol=2e-3), pos
        token = got_tok
    dec.destroy()


WINDOWS = [  # (head_dim, query heads, kv heads, first position, window of layer 0, window of layer 1)
    (256, 4, 1, 2300, 512, 0),     # gemma3's local window beside a global layer
    (128, 4, 2, 509, 512, 100),    # the window starts to mask at 512 positions, i.e. during these steps
    (64, 2, 2, 4400, 4200, 70),    # a window longer than one pass of all chunks; one shorter than a chunk
    (192, 2, 1, 100, 40, 16),      # the three-kernel path: whole 16-position chunks fall out of the window
]


@pytest.mark.parametrize("env", PATHS, ids=["default", "read-ahead", "streaming-gemv", "separate-glue", "three-kernel-attention"])
@pytest.mark.parametrize("hd,nq,nkv,p0,w0,w1", WINDOWS)
def test_sliding_windows_and_a_second_rotary_base(ctx, pkg, oracle, route, hd, nq, nkv, p0, w0, w1, env):
    """Local layers: the last `window` positions only, the step's own included (the reference's
    bound, shaders/attention.rs:202-214), rotating with their own base; against the oracle over a
    filled cache, across the step at which the window starts to cut."""
    from oracle import decoder as od
    route(env)
    cfg = dict(SMALL, n_q_heads=nq, n_kv_heads=nkv, head_dim=hd, rope_theta=1.0e6)
    steps, max_seq = 5, p0 + 8
    w = pkg.decoder.build_weights(cfg, seed=12)
    dec = pkg.decoder.Decoder(ctx, cfg, max_seq)
    dec.load(w)
    ref = od.Decoder(w, max_seq)
    for li, win in enumerate((w0, w1)):
        theta = 10000.0 if win else 0.0          # local layers use the second base
        dec.set_layer_attention(li, win, theta)
        ref.set_layer_attention(li, win, theta)
    rng = np.random.default_rng(hd + p0)
    for li in range(cfg["n_layers"]):
        k_rows, v_rows = ((rng.standard_normal((nkv, max_seq, hd)) * 0.7).astype(np.float16) for _ in range(2))
        ref.k[li], ref.v[li] = k_rows, v_rows
        dec.fill_cache(li, k_rows, v_rows)
    token = 31
    dec.reset(token, p0)
    for pos in range(p0, p0 + steps):
        dec.step()
        got_tok, got_pos, logits, _ = dec.read(want_logits=True)
        want_logits, _ = ref.step(token, pos)
        assert got_pos == pos + 1
        err = np.abs(logits - want_logits)
        assert np.all(err <= 2e-3 + 2e-3 * np.abs(want_logits)), (pos, float(err.max()))
        token = got_tok
    dec.destroy()


def test_a_third_rotary_base_is_refused(ctx, pkg):
    dec = pkg.decoder.Decoder(ctx, SMALL, 16)
    dec.set_layer_attention(0, 8, 500.0)
    dec.set_layer_attention(1, 0, 500.0)
    with pytest.raises(pkg.HipComputeError) as e:
        dec.set_layer_attention(1, 0, 700.0)
    assert "third rotary base" in e.value.message
    with pytest.raises(pkg.HipComputeError):
        dec.set_layer_attention(2, 0, 0.0)
    dec.destroy()


def test_a_captured_step_replays_without_patching(ctx, pkg):
    """Position and token live on the device: replaying one captured step N times must give the
    same tokens as N eager steps."""
    w = pkg.decoder.build_weights(SMALL, seed=4)
    runs = []
    for use_graph in (False, True):
        dec = pkg.decoder.Decoder(ctx, SMALL, 40)
        dec.load(w)
        dec.reset(5, 0)
        dec.step()                    # eager warm-up step (also sizes scratch)
        if use_graph:
            ctx.flush()
            ctx.capture_begin()
            dec.step()
            g = ctx.capture_end()     # recording does not execute: position is still 1
            for _ in range(20):
                ctx.graph_launch(g)
            tok, pos, _, hist = dec.read(n_history=21)
            ctx.graph_destroy(g)
        else:
            for _ in range(20):
                dec.step()
            tok, pos, _, hist = dec.read(n_history=21)
        assert pos == 21
        runs.append(hist.copy())
        dec.destroy()
    assert np.array_equal(runs[0], runs[1])


def test_the_embedded_row_follows_the_weights_it_is_made_of(ctx, pkg, oracle):
    """Every step leaves the embedded row of the token it picked for the next one. When the embedding table or the
    first layer's input norm is replaced between steps, the next step must embed again -- with the new weights -- and
    a decoder that was never reset steps from token 0 at position 0."""
    from oracle import decoder as od
    w = pkg.decoder.build_weights(SMALL, seed=6)
    w2 = pkg.decoder.build_weights(SMALL, seed=7)
    for env in ({}, {"HIPC_DEC_LEAN": 0}):
        with ctx.options(**env):
            dec = pkg.decoder.Decoder(ctx, SMALL, 24)
            dec.load(w)
            ref = od.Decoder(w, 24)
            token = 0                       # no reset: the state a new decoder starts from
            for pos in range(8):
                if pos == 3:                # a new embedding table and input norm, the other weights stay
                    w.embedding = w2.embedding
                    w.norms[(0, pkg.decoder.NORM_INPUT)] = w2.norms[(0, pkg.decoder.NORM_INPUT)]
                    B, scales, zp = w.embedding
                    dB, dS, dZ = ctx.upload(B), ctx.upload(scales), ctx.upload(zp)
                    ctx._check(ctx.lib.hipc_decoder_set_embedding(ctx.handle, dec.handle, dB.ptr, B.size, dS.ptr, scales.size, dZ.ptr, zp.size))
                    dV = ctx.upload(w.norms[(0, pkg.decoder.NORM_INPUT)])
                    ctx._check(ctx.lib.hipc_decoder_set_norm(ctx.handle, dec.handle, 0, pkg.decoder.NORM_INPUT, dV.ptr))
                    ctx.flush()
                    for buf in (dB, dS, dZ, dV):
                        buf.free()
                dec.step()
                got_tok, got_pos, logits, _ = dec.read(want_logits=True)
                want_logits, want_tok = ref.step(token, pos)
                assert got_pos == pos + 1
                err = np.abs(logits - want_logits)
                assert np.all(err <= 2e-3 + 2e-3 * np.abs(want_logits)), (env, pos, float(err.max()))
                token = got_tok
            dec.destroy()
        w = pkg.decoder.build_weights(SMALL, seed=6)   # the first route's replacements do not carry over


def test_refuses_incomplete_models_and_bad_shapes(ctx, pkg):
    dec = pkg.decoder.Decoder(ctx, SMALL, 16)
    with pytest.raises(pkg.HipComputeError) as e:
        dec.step()
    assert e.value.code == 1 and "not every weight" in e.value.message
    dec.destroy()
    with pytest.raises(pkg.HipComputeError):
        pkg.decoder.Decoder(ctx, dict(SMALL, head_dim=48), 16)


def test_the_cache_limit_is_kept_on_the_device(ctx, pkg, oracle):
    """max_seq steps fit after a reset to 0; one more (eager or replayed) writes nothing, leaves token
    and position alone and is reported by the next read -- the rule of oracle.decoder.advance_state."""
    from oracle.decoder import advance_state
    max_seq = 6
    w = pkg.decoder.build_weights(SMALL, seed=5)
    dec = pkg.decoder.Decoder(ctx, SMALL, max_seq)
    dec.load(w)
    dec.reset(3, 0)
    tok, pos, over = 3, 0, False
    for _ in range(max_seq):
        dec.step()
        got_tok, got_pos, logits, _ = dec.read(want_logits=True)
        tok, pos, over = advance_state(tok, pos, logits, max_seq)
        assert (got_tok, got_pos) == (tok, pos) and not over
    assert pos == max_seq
    k_before = ctx.download(dec.kv_cache(0)[0], np.float16, (SMALL["n_kv_heads"] * max_seq * SMALL["head_dim"],))
    dec.step()                                           # one step too many
    with pytest.raises(pkg.HipComputeError) as e:
        dec.read()
    assert e.value.code == 1 and "cache full" in e.value.message
    tok2, pos2 = ctypes_state(ctx, dec)
    assert (tok2, pos2) == advance_state(tok, pos, None, max_seq)[:2] == (tok, max_seq)
    assert np.array_equal(ctx.download(dec.kv_cache(0)[0], np.float16, k_before.shape), k_before)
    dec.reset(3, 0)                                      # a reset clears the flag
    dec.step()
    assert dec.read()[1] == 1
    dec.destroy()


def ctypes_state(ctx, dec):
    """token and position as hipc_decoder_read fills them, whatever status it returns"""
    import ctypes as C
    tok, pos = C.c_int32(), C.c_int32()
    ctx.lib.hipc_decoder_read(ctx.handle, dec.handle, C.byref(tok), C.byref(pos), None, None, 0)
    return tok.value, pos.value


@pytest.mark.parametrize("env", [{}, READ_AHEAD, NO_READ_AHEAD], ids=["default", "read-ahead-everywhere", "no-read-ahead"])
def test_gemma3_1b_shape_at_context_2040(ctx, pkg, oracle, route, env):
    """The decoder configuration at its real size -- 26 layers, hidden 1152, ffn 6912, 4 query heads on
    1 kv head of 256, vocabulary 262144, 22 local layers (window 512, base 10000) and 4 global ones
    (base 1e6) -- three steps from position 2040 over a cache filled with random f16 rows on both
    sides, logits against the oracle at 2e-3 + 2e-3 |ref|. These are the code paths the tokens-per-
    second figure runs: the one-item-per-thread norm prologue, the gated-GELU prologue of a
    k-split down projection, the attention join of 64 chunks."""
    from oracle import decoder as od
    route(env)
    D = pkg.decoder
    cfg = dict(D.GEMMA3_1B)
    p0, steps = 2040, 3
    max_seq = p0 + steps + 5
    w = D.build_weights(cfg, seed=9)
    dec = D.Decoder(ctx, cfg, max_seq)
    dec.load(w)
    ref = od.Decoder(w, max_seq)
    for li in range(cfg["n_layers"]):
        if (li + 1) % 6 != 0:
            dec.set_layer_attention(li, 512, 10000.0), ref.set_layer_attention(li, 512, 10000.0)
        else:
            dec.set_layer_attention(li, 0, 1.0e6), ref.set_layer_attention(li, 0, 1.0e6)
    rng = np.random.default_rng(2040)
    for li in range(cfg["n_layers"]):
        k_rows, v_rows = ((rng.standard_normal((1, max_seq, 256)) * 0.5).astype(np.float16) for _ in range(2))
        ref.k[li], ref.v[li] = k_rows, v_rows
        dec.fill_cache(li, k_rows, v_rows)
    token = 1234
    dec.reset(token, p0)
    for pos in range(p0, p0 + steps):
        dec.step()
        got_tok, got_pos, logits, _ = dec.read(want_logits=True)
        want_logits, want_tok = ref.step(token, pos)
        assert got_pos == pos + 1
        err = np.abs(logits - want_logits)
        assert np.all(err <= 2e-3 + 2e-3 * np.abs(want_logits)), (pos, float(err.max()))
        top2 = np.sort(want_logits)[-2:]
        if top2[1] - top2[0] > 1e-2:
            assert got_tok == want_tok, pos
        token = got_tok
    dec.destroy()
    ctx.flush()
