"""GPU parity of the inference enqueues of the dispatch-level C ABI (include/fast_hip.h) against the CPU oracle:
the matrix-vector products in the reference's weight layouts (F16 rows, Q8_0 blocks), the single-position row
ops, attention over the KV cache, and whole decode steps chained as the reference's forward_token does.
fp32 results to a stated tolerance (summation order and exp / sincos differ); stores bit for bit."""
import sys

import numpy as np
import pytest

from llm_metal_amd.configs import C1, GEMMA3, SFTConfig
from llm_metal_amd.synth import make_batch, make_model
from oracle import oracle
from oracle.oracle import op
from tests.decode_chain import device_decode, oracle_decode
from tests.gpu_util import Dev, maxrel

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def dev():
    d = Dev()
    yield d
    d.close()


def say(*a):
    print(*a, flush=True, file=sys.stderr)


def rnd(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(F)


# rows per wave grow at 8192 and 32768 rows; from 32768 rows on x is staged in LDS unless longer than 10240; cols % 8 != 0 takes the
# element-wise kernel
@pytest.mark.parametrize("rows,cols", [(4096, 2560), (1024, 2560), (8200, 1152), (33000, 256), (37, 9728), (21, 12800),
                                       (33000, 10248), (7, 100), (33, 24), (5000, 8)])
def test_f16_matvec(dev, rows, cols):
    say("f16_matvec", rows, cols)
    rng = np.random.default_rng(rows + cols)
    W = rnd(rng, rows, cols, scale=0.05).astype(np.float16)
    x = rnd(rng, cols)
    ref = np.zeros(rows, F)
    op("f32", "or_f16_batch_matvec", W.view(np.uint16), x, ref, rows, cols, 1)
    wb, xb, yb = dev.up(W), dev.up(x), dev.empty(rows * 4)
    dev.L.metal_enqueue_f16_matvec(wb.h, xb.h, yb.h, rows, cols)
    assert maxrel(yb.read(F), ref) < 2e-5


@pytest.mark.parametrize("rows,cols,B", [(4112, 1024, 2), (300, 2560, 3), (4096, 512, 4), (515, 1152, 5), (4096, 256, 8),
                                         (1000, 512, 9), (2048, 640, 32), (64, 50, 3)])
def test_f16_batch_matvec(dev, rows, cols, B):
    say("f16_batch_matvec", rows, cols, B)
    rng = np.random.default_rng(rows + cols + B)
    W = rnd(rng, rows, cols, scale=0.05).astype(np.float16)
    X = rnd(rng, B, cols)
    ref = np.zeros((B, rows), F)
    op("f32", "or_f16_batch_matvec", W.view(np.uint16), X, ref, rows, cols, B)
    wb, xb, yb = dev.up(W), dev.up(X), dev.empty(B * rows * 4)
    dev.L.metal_enqueue_f16_batch_matvec(wb.h, xb.h, yb.h, rows, cols, B)
    assert maxrel(yb.read(F, (B, rows)), ref) < 2e-5


@pytest.mark.parametrize("rows,nb", [(4096, 80), (1000, 36), (5, 1), (8195, 17), (33001, 4), (151, 304), (70, 416)])
def test_q8_matvec_and_its_cached_image(dev, rows, nb):
    say("q8_matvec", rows, nb)
    rng = np.random.default_rng(rows + nb)
    cols = nb * 32
    blocks = oracle.q8_quantize(rnd(rng, rows, cols, scale=0.05))
    x = rnd(rng, cols)
    ref = np.zeros(rows, F)
    op("f32", "or_q8_matvec", blocks, x, ref, rows, nb)
    wb, xb, yb = dev.up(blocks), dev.up(x), dev.empty(rows * 4)
    for _ in range(2):                                   # the second call runs on the image the first one built
        dev.L.metal_enqueue_q8_matvec(wb.h, xb.h, yb.h, rows, nb)
        assert maxrel(yb.read(F), ref) < 2e-5
    # a write to the weight buffer invalidates the image
    blocks2 = oracle.q8_quantize(rnd(rng, rows, cols, scale=0.05))
    wb.write(blocks2)
    op("f32", "or_q8_matvec", blocks2, x, ref, rows, nb)
    dev.L.metal_enqueue_q8_matvec(wb.h, xb.h, yb.h, rows, nb)
    assert maxrel(yb.read(F), ref) < 2e-5
    # a window of a larger buffer (no image is kept for views)
    big = dev.up(np.concatenate([np.zeros(68, np.uint8), blocks2]))
    wv = dev.view(big, 68, blocks2.nbytes)
    dev.L.metal_enqueue_q8_matvec(wv.h, xb.h, yb.h, rows, nb)
    assert maxrel(yb.read(F), ref) < 2e-5


def test_single_vector_row_ops(dev):
    rng = np.random.default_rng(3)
    # rms_norm of one vector, also in place
    for D in (2560, 1152, 100):
        x, g = rnd(rng, D), (1 + 0.2 * rng.standard_normal(D)).astype(F)
        ref = np.zeros(D, F); op("f32", "or_rms_norm", x, g, ref, D, 1e-6, 1)
        xb, gb, ob = dev.up(x), dev.up(g), dev.empty(D * 4)
        dev.L.metal_enqueue_rms_norm(xb.h, gb.h, ob.h, D, 1e-6)
        assert maxrel(ob.read(F), ref) < 1e-5
        dev.L.metal_enqueue_rms_norm(xb.h, gb.h, xb.h, D, 1e-6)
        assert maxrel(xb.read(F), ref) < 1e-5
    # per-head norm, plain and at an offset (the bytes before the offset stay untouched)
    for H, hd in ((32, 128), (4, 256), (3, 40)):
        v, g = rnd(rng, H + 2, hd), (1 + 0.2 * rng.standard_normal(hd)).astype(F)
        ref = v.copy(); r2 = np.ascontiguousarray(ref[2:]); op("f32", "or_rms_norm", r2, g, r2, hd, 1e-6, H); ref[2:] = r2
        vb, gb = dev.up(v), dev.up(g)
        dev.L.metal_enqueue_per_head_rms_norm_off(vb.h, 2 * hd * 4, gb.h, H, hd, 1e-6)
        got = vb.read(F, (H + 2, hd))
        assert np.array_equal(got[:2], v[:2]) and maxrel(got[2:], ref[2:]) < 1e-5
        vb2 = dev.up(v[2:])
        dev.L.metal_enqueue_per_head_rms_norm(vb2.h, gb.h, H, hd, 1e-6)
        assert maxrel(vb2.read(F, (H, hd)), ref[2:]) < 1e-5


@pytest.mark.parametrize("Hq,Hkv,hd,theta", [(32, 8, 128, 1e6), (4, 1, 256, 1e4), (4, 2, 64, 1e6), (3, 3, 32, 1e4)])
def test_rope_and_kv_cache_store(dev, Hq, Hkv, hd, theta):
    rng = np.random.default_rng(Hq + hd)
    max_seq = 40
    for pos in (0, 5, 39):
        q, k, v = rnd(rng, Hq, hd), rnd(rng, Hkv, hd), rnd(rng, Hkv, hd)
        rq, rk = q.copy(), k.copy()
        op("f32", "or_rope", rq, rk, Hq, Hkv, hd, pos, theta)
        qb, kb, vb = dev.up(q), dev.up(k), dev.up(v)
        dev.L.metal_enqueue_rope(qb.h, kb.h, Hq, Hkv, hd, pos, theta)
        assert maxrel(qb.read(F, (Hq, hd)), rq) < 2e-5 and maxrel(kb.read(F, (Hkv, hd)), rk) < 2e-5
        # offsets: q and k in one buffer
        arena = dev.up(np.concatenate([q.ravel(), k.ravel()]))
        dev.L.metal_enqueue_rope_off(arena.h, 0, arena.h, Hq * hd * 4, Hq, Hkv, hd, pos, theta)
        got = arena.read(F)
        assert maxrel(got[:Hq * hd], rq.ravel()) < 2e-5 and maxrel(got[Hq * hd:], rk.ravel()) < 2e-5
        kc0, vc0 = rnd(rng, Hkv, max_seq, hd), rnd(rng, Hkv, max_seq, hd)
        ek, ev = kc0.copy(), vc0.copy()
        op("f32", "or_kv_cache_store", rk, v, ek, ev, Hkv, max_seq, hd, pos)
        kcb, vcb = dev.up(kc0), dev.up(vc0)
        dev.L.metal_enqueue_kv_cache_store(kb.h, vb.h, kcb.h, vcb.h, Hkv, max_seq, hd, pos)
        ek_dev = kc0.copy(); ek_dev[:, pos] = kb.read(F, (Hkv, hd))      # the rotated k as the GPU holds it
        assert np.array_equal(kcb.read(F, ek.shape), ek_dev) and maxrel(ek_dev, ek) < 2e-5
        assert np.array_equal(vcb.read(F, ev.shape), ev)
        kv = dev.up(np.concatenate([k.ravel(), v.ravel()]))
        kcb2, vcb2 = dev.up(kc0), dev.up(vc0)
        dev.L.metal_enqueue_kv_cache_store_off(kv.h, 0, kv.h, Hkv * hd * 4, kcb2.h, vcb2.h, Hkv, max_seq, hd, pos)
        e2 = kc0.copy(); e2[:, pos] = k
        assert np.array_equal(kcb2.read(F, ek.shape), e2) and np.array_equal(vcb2.read(F, ev.shape), ev)


# up to 128 keys one query head per workgroup, beyond that the whole group; n_attend > 256 splits the keys over
# several workgroups
@pytest.mark.parametrize("Hq,ratio,hd,max_seq,n", [(32, 4, 128, 512, 1), (32, 4, 128, 512, 100), (32, 4, 128, 512, 200), (4, 4, 256, 1024, 700), (6, 2, 30, 200, 77),
                                                   (6, 3, 32, 300, 300), (2, 1, 64, 64, 64), (8, 8, 128, 2100, 2100),
                                                   (5, 5, 48, 260, 257)])
def test_attention_over_the_cache(dev, Hq, ratio, hd, max_seq, n):
    say("attention", Hq, ratio, hd, max_seq, n)
    rng = np.random.default_rng(Hq + hd + n)
    Hkv = Hq // ratio
    Q, Kc, Vc = rnd(rng, Hq, hd), rnd(rng, Hkv, max_seq, hd), rnd(rng, Hkv, max_seq, hd)
    ref = np.zeros((Hq, hd), F)
    op("f32", "or_attention", Q, Kc, Vc, ref, n, hd, max_seq, Hq, ratio)
    qb, kb, vb, ob = dev.up(Q), dev.up(Kc), dev.up(Vc), dev.empty(Hq * hd * 4)
    dev.L.metal_enqueue_attention(qb.h, kb.h, vb.h, ob.h, n, hd, max_seq, Hq, ratio)
    assert maxrel(ob.read(F, (Hq, hd)), ref) < 2e-5
    arena = dev.up(np.concatenate([np.zeros(16, F), Q.ravel(), np.zeros(Hq * hd, F)]))
    dev.L.metal_enqueue_attention_off(arena.h, 64, kb.h, vb.h, arena.h, 64 + Hq * hd * 4, n, hd, max_seq, Hq, ratio)
    assert maxrel(arena.read(F)[16 + Hq * hd:].reshape(Hq, hd), ref) < 2e-5


def test_bad_arguments_are_refused_without_a_launch(dev, capfd):
    x = dev.up(np.ones(64, F))
    y = dev.up(np.full(4, 7, F))
    dev.L.metal_enqueue_f16_matvec(x.h, x.h, y.h, 64, 64)               # weight buffer too small
    dev.L.metal_enqueue_attention(x.h, x.h, x.h, y.h, 5, 512, 4, 1, 1)  # head_dim beyond the kernel's limit
    dev.L.metal_enqueue_rope_off(x.h, 2, x.h, 0, 1, 1, 8, 0, 1e4)       # offset not a multiple of 4
    dev.L.metal_flush()
    assert np.array_equal(y.read(F), np.full(4, 7, F))
    assert "launch skipped" in capfd.readouterr().err


TINY_GEMMA = SFTConfig("tiny_gemma3", GEMMA3, NL=7, D=128, Hq=4, Hkv=1, hd=32, IS=256, V=512, seq=5, tied=True)


@pytest.mark.parametrize("cfg,fmt,use_off", [(C1.with_(seq=8), "f16", False), (C1.with_(seq=8), "q8_0", True),
                                             (TINY_GEMMA, "f16", True), (TINY_GEMMA, "q8_0", False)])
def test_decode_steps_chained_as_forward_token(dev, cfg, fmt, use_off):
    say("decode chain", cfg.name, fmt, use_off)
    c = cfg.with_(weight_format=fmt)
    model = make_model(c, seed=5, gamma_jitter=0.1)
    tok, tgt = make_batch(c, seed=6)
    toks = [int(t) for t in tok]
    ref = oracle_decode(c, model, fmt, toks, max_seq=c.seq + 3, precision="f32", lora=model["lora"])
    got = device_decode(dev, c, model, fmt, toks, max_seq=c.seq + 3, lora=model["lora"], use_off=use_off)
    assert maxrel(got, ref) < 2e-4
    assert (got.argmax(1) == ref.argmax(1)).all()
    # and against the rows of the training forward of the CPU oracle (pinned on its own)
    used = oracle.weights_as_used(model, fmt)
    _, rows = oracle.sft_loss(c, used, model["lora"], tok, tgt, precision="f32", want_logits=True)
    assert maxrel(got, rows) < 2e-4
