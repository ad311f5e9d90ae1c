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


def test_refuses_incomplete_models_and_bad_shapes(ctx, pkg):
    dec = pkg.decoder.Decoder(ctx, SMALL, 16)
    with pytest.raises(pkg.HipComputeError) as e:
        dec.step()
    assert e.value.code == 1 and "not every weight" in e.value.message
    dec.destroy()
    with pytest.raises(pkg.HipComputeError):
        pkg.decoder.Decoder(ctx, dict(SMALL, head_dim=48), 16)
