"""GPU parity of the dispatch-level C ABI (include/fast_hip.h) against the CPU
oracle, op by op, in the reference's buffer layouts.  Integer / F16 / Q8_0
results are compared bit for bit; fp32 results to a stated tolerance (the GEMMs
round the activation operand to fp16 with a per-row power-of-two scale, which
bounds their error at ~2^-11 per element before averaging)."""
import json
import os

import numpy as np
import pytest

from oracle import oracle
from oracle.oracle import SZ, op
from tests.gpu_util import Dev, maxrel, rel

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def dev():
    d = Dev()
    yield d
    d.close()


def rnd(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(F)


# ---------------------------------------------------------------- formats (bit exact)

def test_f16_conversion_bit_exact(dev):
    rng = np.random.default_rng(0)
    kat = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "q8_0_kat.json")))
    special = np.array([c["f32_bits"] for c in kat["f16"]], dtype=np.uint32).view(F)
    halves = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((halves[:-1] + halves[1:]) / 2).astype(F)
    x = np.concatenate([special, mids, -mids, rnd(rng, 300000, scale=0.02),
                        (rng.standard_normal(100000) * np.exp(rng.uniform(-20, 12, 100000))).astype(F)])
    src, dst = dev.up(x), dev.empty(x.size * 2)
    dev.L.hip_enqueue_f32_to_f16(src.h, dst.h, x.size)
    got = dst.read(np.uint16)
    assert np.array_equal(got, oracle.f32_to_f16_bits(x))
    assert np.array_equal(got[:special.size], np.array([c["f16_bits"] for c in kat["f16"]], dtype=np.uint16))


def test_wmat_create_f16_and_q8_bit_exact(dev):
    rng = np.random.default_rng(1)
    kat = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "q8_0_kat.json")))
    blocks = np.stack([np.array(c["x_bits"], dtype=np.uint32).view(F) for c in kat["q8_blocks"]])   # [6, 32]
    w = rnd(rng, 64, 160 + 7, scale=0.02)                   # 7 ragged columns: dropped by Q8_0, kept by F16
    w[3, 32:64] = 0
    w[:6, 64:96] = blocks
    wm = dev.L.wmat_create_q8(w.ctypes.data, w.shape[0], w.shape[1])
    assert (wm.contents.rows, wm.contents.cols, wm.contents.nb) == (64, 167, 5)
    got = np.empty(64 * 5 * 34, dtype=np.uint8)
    dev.L.metal_buf_read(wm.contents.mbuf, 0, got.ctypes.data, got.nbytes)
    assert np.array_equal(got, oracle.q8_quantize(w))
    for i, c in enumerate(kat["q8_blocks"]):
        assert got.reshape(64, 5, 34)[i, 2].tolist() == c["bytes"], c["name"]
    # dequantise on the device: float(scale) * code, bit for bit
    deq = dev.empty(64 * 167 * 4)
    dev.L.hip_enqueue_q8_dequant(wm.contents.mbuf, deq.h, 64, 167)
    d = deq.read(F, (64, 167))[:, :160]
    assert np.array_equal(d.view(np.uint32), oracle.q8_dequant(got, 64, 167)[:, :160].view(np.uint32))
    dev.L.wmat_free(wm)
    wf = dev.L.wmat_create_f16(w.ctypes.data, 64, 167)
    gh = np.empty(64 * 167, dtype=np.uint16)
    dev.L.metal_buf_read(wf.contents.mbuf, 0, gh.ctypes.data, gh.nbytes)
    assert np.array_equal(gh, oracle.f32_to_f16_bits(w).ravel())
    dev.L.wmat_free(wf)


# ---------------------------------------------------------------- GEMMs

@pytest.mark.parametrize("M,N,K", [(64, 256, 256), (64, 768, 256), (64, 4096, 256), (64, 256, 768),
                                   (64, 1024, 2560), (64, 2560, 4096), (37, 96, 136), (160, 1152, 1024),
                                   (1, 64, 64), (64, 6176, 2560), (64, 2560, 6176)])
def test_f16_matmul_and_nt(dev, M, N, K):
    rng = np.random.default_rng(M * 7 + N + K)
    A = rnd(rng, M, K)
    A[0] *= 1e-6                                          # a tiny row and a huge row: per-row scaling
    A[M - 1] *= 3e4
    W = oracle.round_f16(rnd(rng, N, K, scale=0.02))
    Wb = dev.up(oracle.f32_to_f16_bits(W))
    C = dev.empty(M * N * 4)
    dev.L.metal_enqueue_f16_matmul(dev.up(A).h, Wb.h, C.h, M, N, K)
    ref = np.zeros((M, N), F)
    op("f32", "or_wmatmul", A, W, ref, M, N, K)
    got = C.read(F, (M, N))
    for m in (0, M // 2, M - 1):
        assert rel(got[m], ref[m]) < 1.5e-3
    assert rel(got, ref) < 1e-3
    A2 = rnd(rng, M, N)
    C2 = dev.empty(M * K * 4)
    for _ in range(2):                                    # second call reuses the cached transposed copy
        dev.L.metal_enqueue_f16_matmul_nt(dev.up(A2).h, Wb.h, C2.h, M, N, K)
    ref2 = np.zeros((M, K), F)
    op("f32", "or_wmatmul_nt", A2, W, ref2, M, N, K)
    assert rel(C2.read(F, (M, K)), ref2) < 1e-3


def test_matmul_nt_sees_weight_updates(dev):
    """The transposed copy kept with a weight buffer must follow f16_sgd_apply."""
    rng = np.random.default_rng(5)
    M, N, K = 16, 64, 64
    W = oracle.f32_to_f16_bits(rnd(rng, N, K, scale=0.02))
    G = oracle.f32_to_f16_bits(rnd(rng, N, K, scale=0.01))
    Wb, Gb = dev.up(W), dev.up(G)
    A = rnd(rng, M, N)
    Ab, C = dev.up(A), dev.empty(M * K * 4)
    dev.L.metal_enqueue_f16_matmul_nt(Ab.h, Wb.h, C.h, M, N, K)
    dev.L.metal_enqueue_f16_sgd_apply(Wb.h, Gb.h, N * K, 0.5)
    dev.L.metal_enqueue_f16_matmul_nt(Ab.h, Wb.h, C.h, M, N, K)
    W2, G2 = W.copy(), G.copy()
    op("f32", "or_f16_sgd_apply", W2, G2, SZ(N * K), 0.5)
    assert np.array_equal(Wb.read(np.uint16, (N, K)), W2) and not Gb.read(np.uint16).any()
    ref = np.zeros((M, K), F)
    op("f32", "or_wmatmul_nt", A, oracle.f16_bits_to_f32(W2), ref, M, N, K)
    assert rel(C.read(F, (M, K)), ref) < 1e-3


def test_float_matmuls(dev):
    rng = np.random.default_rng(2)
    M, N, K = 64, 16, 200
    A, W = rnd(rng, M, K), rnd(rng, N, K)
    C = dev.empty(M * N * 4)
    dev.L.metal_enqueue_float_matmul(dev.up(A).h, dev.up(W).h, C.h, M, N, K)
    assert rel(C.read(F, (M, N)), A.astype(np.float64) @ W.T.astype(np.float64)) < 1e-6
    At, B = rnd(rng, K, M), rnd(rng, K, N)
    dev.L.metal_enqueue_float_matmul_tn(dev.up(At).h, dev.up(B).h, C.h, M, N, K)
    assert rel(C.read(F, (M, N)), At.T.astype(np.float64) @ B.astype(np.float64)) < 1e-6
    A2, W2 = rnd(rng, M, N), rnd(rng, N, K)
    C2 = dev.empty(M * K * 4)
    dev.L.metal_enqueue_float_matmul_nt(dev.up(A2).h, dev.up(W2).h, C2.h, M, N, K)
    assert rel(C2.read(F, (M, K)), A2.astype(np.float64) @ W2.astype(np.float64)) < 1e-6


# ---------------------------------------------------------------- row / layout / elementwise ops

@pytest.mark.parametrize("B,D", [(64, 2560), (64 * 8, 128), (5, 100), (3, 1152), (7, 64)])
def test_rms_norm_fwd_bwd_and_aliasing(dev, B, D):
    rng = np.random.default_rng(B + D)
    x, dy = rnd(rng, B, D), rnd(rng, B, D)
    g = (1 + 0.2 * rng.standard_normal(D)).astype(F)
    xb, gb, ob = dev.up(x), dev.up(g), dev.empty(B * D * 4)
    dev.L.metal_enqueue_rms_norm_batched(xb.h, gb.h, ob.h, D, 1e-6, B)
    ref = np.zeros((B, D), F)
    op("f32", "or_rms_norm", x, g, ref, D, 1e-6, B)
    assert maxrel(ob.read(F, (B, D)), ref) < 1e-5
    dev.L.metal_enqueue_rms_norm_batched(xb.h, gb.h, xb.h, D, 1e-6, B)            # in place
    assert maxrel(xb.read(F, (B, D)), ref) < 1e-5
    xb2, dyb, dxb = dev.up(x), dev.up(dy), dev.empty(B * D * 4)
    dev.L.metal_enqueue_rms_norm_backward(xb2.h, dyb.h, gb.h, dxb.h, B, D, 1e-6)
    refd = np.zeros((B, D), F)
    op("f32", "or_rms_norm_backward", x, dy, g, refd, B, D, 1e-6)
    assert maxrel(dxb.read(F, (B, D)), refd) < 2e-5
    dev.L.metal_enqueue_rms_norm_backward(xb2.h, dyb.h, gb.h, dyb.h, B, D, 1e-6)   # dx aliases dy
    assert maxrel(dyb.read(F, (B, D)), refd) < 2e-5


def test_layout_ops(dev):
    rng = np.random.default_rng(3)
    N, H, D, ratio = 13, 6, 16, 3
    src = rnd(rng, N, H * D)
    t, back = dev.empty(src.nbytes), dev.empty(src.nbytes)
    dev.L.metal_enqueue_transpose_heads_fwd(dev.up(src).h, t.h, N, H, D)
    assert np.array_equal(t.read(F, (H, N, D)), src.reshape(N, H, D).transpose(1, 0, 2))
    dev.L.metal_enqueue_transpose_heads_rev(t.h, back.h, N, H, D)
    assert np.array_equal(back.read(F, (N, H * D)), src)
    kv = rnd(rng, 2, N, D)
    ex = dev.empty(kv.nbytes * ratio)
    dev.L.metal_enqueue_repeat_kv(dev.up(kv).h, ex.h, 2, N, D, ratio)
    assert np.array_equal(ex.read(F, (2 * ratio, N, D)), np.repeat(kv, ratio, axis=0))
    d = rnd(rng, 2 * ratio, N, D)
    dk = dev.empty(kv.nbytes)
    dev.L.metal_enqueue_repeat_kv_bwd(dev.up(d).h, dk.h, 2, N, D, ratio)
    ref = np.zeros((2, N, D), F)
    op("f32", "or_repeat_kv_bwd", d, ref, 2, N, D, ratio)
    assert maxrel(dk.read(F, (2, N, D)), ref) < 1e-6


@pytest.mark.parametrize("hd,theta", [(128, 1e6), (256, 1e4), (64, 1e6), (32, 1e4)])
def test_rope_fwd_bwd(dev, hd, theta):
    rng = np.random.default_rng(hd)
    Hq, Hkv, N = 4, 2, 64
    q, k = rnd(rng, Hq, N, hd), rnd(rng, Hkv, N, hd)
    qb, kb = dev.up(q), dev.up(k)
    dev.L.metal_enqueue_rope_train(qb.h, kb.h, Hq, Hkv, hd, N, theta)
    rq, rk = q.copy(), k.copy()
    op("f32", "or_rope_train", rq, rk, Hq, Hkv, hd, N, theta)
    # angles reach pos*freq ~ 63 rad; sin/cos of a float angle agree to a few ulp of the angle
    assert maxrel(qb.read(F, q.shape), rq) < 2e-5 and maxrel(kb.read(F, k.shape), rk) < 2e-5
    dev.L.metal_enqueue_rope_train_bwd(qb.h, kb.h, Hq, Hkv, hd, N, theta)
    assert maxrel(qb.read(F, q.shape), q) < 2e-5 and maxrel(kb.read(F, k.shape), k) < 2e-5


@pytest.mark.parametrize("H,N,D", [(4, 64, 64), (3, 160, 32), (2, 17, 128), (1, 1, 16)])
def test_attention_fwd_bwd(dev, H, N, D):
    rng = np.random.default_rng(H * N + D)
    scale = float(1.0 / np.sqrt(F(D)))
    Q, K, V, dO = (rnd(rng, H, N, D) for _ in range(4))
    Qb, Kb, Vb, dOb = dev.up(Q), dev.up(K), dev.up(V), dev.up(dO)
    out, probs = dev.empty(Q.nbytes), dev.empty(H * N * N * 4)
    dev.L.metal_enqueue_attn_train_fwd(Qb.h, Kb.h, Vb.h, out.h, probs.h, H, N, D, scale)
    ro, rp = np.zeros_like(Q), np.zeros((H, N, N), F)
    op("f32", "or_attn_train_fwd", Q, K, V, ro, rp, H, N, D, scale)
    assert maxrel(out.read(F, Q.shape), ro) < 2e-5 and maxrel(probs.read(F, rp.shape), rp) < 2e-5
    got_p = probs.read(F, rp.shape)
    assert np.allclose(got_p.sum(-1), 1, atol=1e-5) and not np.triu(got_p, 1).any()   # exact sums at N = 160 too
    ds, dQ, dK, dV = dev.empty(rp.nbytes), dev.empty(Q.nbytes), dev.empty(Q.nbytes), dev.empty(Q.nbytes)
    dev.L.metal_enqueue_attn_bwd_dq(dOb.h, probs.h, Vb.h, Kb.h, ds.h, dQ.h, H, N, D, scale)
    dev.L.metal_enqueue_attn_bwd_dkv(ds.h, Qb.h, probs.h, dOb.h, dK.h, dV.h, H, N, D)
    rds, rdq, rdk, rdv = np.zeros_like(rp), np.zeros_like(Q), np.zeros_like(Q), np.zeros_like(Q)
    op("f32", "or_attn_bwd_dq", dO, rp, V, K, rds, rdq, H, N, D, scale)
    op("f32", "or_attn_bwd_dkv", rds, Q, rp, dO, rdk, rdv, H, N, D)
    assert maxrel(dQ.read(F, Q.shape), rdq) < 5e-5
    assert maxrel(dK.read(F, Q.shape), rdk) < 5e-5 and maxrel(dV.read(F, Q.shape), rdv) < 5e-5


@pytest.mark.parametrize("name", ["silu", "gelu"])
def test_glu_ops(dev, name):
    rng = np.random.default_rng(4)
    n = 64 * 768 + 3                                       # not a multiple of the workgroup size
    g, u, dy = rnd(rng, n, scale=3), rnd(rng, n), rnd(rng, n)
    gb, ub = dev.up(g), dev.up(u)
    getattr(dev.L, f"metal_enqueue_{name}_mul")(gb.h, ub.h, n)
    ref = g.copy()
    op("f32", f"or_{name}_mul", ref, u, SZ(n))
    assert maxrel(gb.read(F), ref) < 1e-5
    dyb, g2, dgb, dub = dev.up(dy), dev.up(g), dev.empty(n * 4), dev.empty(n * 4)
    getattr(dev.L, f"metal_enqueue_{name}_mul_backward")(dyb.h, g2.h, ub.h, dgb.h, dub.h, n)
    rdg, rdu = np.zeros(n, F), np.zeros(n, F)
    op("f32", f"or_{name}_mul_backward", dy, g, u, rdg, rdu, SZ(n))
    assert maxrel(dgb.read(F), rdg) < 2e-5 and maxrel(dub.read(F), rdu) < 2e-5
    getattr(dev.L, f"metal_enqueue_{name}_mul_backward")(dyb.h, g2.h, ub.h, dyb.h, dub.h, n)   # dgate aliases dout
    assert maxrel(dyb.read(F), rdg) < 2e-5


def test_elementwise_and_empty_inputs(dev):
    rng = np.random.default_rng(6)
    n = 1000
    x, y = rnd(rng, n), rnd(rng, n)
    xb, yb = dev.up(x), dev.up(y)
    dev.L.metal_enqueue_residual_add(xb.h, yb.h, n)
    assert np.array_equal(xb.read(F), x + y)
    dev.L.metal_enqueue_scale(xb.h, 0.25, n)
    assert np.array_equal(xb.read(F), (x + y) * F(0.25))
    dev.L.metal_enqueue_add_scaled(yb.h, xb.h, 2.0, n)
    assert np.allclose(yb.read(F), y + F(2.0) * ((x + y) * F(0.25)), rtol=1e-6, atol=0)
    dev.L.metal_enqueue_clamp(yb.h, 0.5, n)
    assert np.abs(yb.read(F)).max() <= 0.5
    cb = dev.empty(n * 4)
    dev.L.metal_enqueue_copy(yb.h, cb.h, n)
    assert np.array_equal(cb.read(F), yb.read(F))
    # n = 0 and undersized buffers are refused without touching memory
    dev.L.metal_enqueue_scale(xb.h, 2.0, 0)
    dev.L.metal_enqueue_scale(xb.h, 2.0, n + 1)
    dev.be.flush()
    assert np.array_equal(xb.read(F), (x + y) * F(0.25))


@pytest.mark.parametrize("B,V", [(64, 4096), (5, 333), (2, 151936)])
def test_softmax_ce_and_grpo(dev, B, V):
    rng = np.random.default_rng(V)
    lg = rnd(rng, B, V, scale=3)
    tgt = rng.integers(0, V, B).astype(np.uint32)
    losses, dl = dev.empty(B * 4), dev.empty(B * V * 4)
    lgb, tb = dev.up(lg), dev.up(tgt)
    dev.L.metal_enqueue_softmax_ce(lgb.h, tb.h, losses.h, dl.h, B, V)
    # reference in double: a sequential fp32 sum over 151936 terms is itself only good to ~2e-5
    rl, rd = np.zeros(B), np.zeros((B, V))
    op("f64", "or_softmax_ce", lg.astype(np.float64), tgt, rl, rd, B, V)
    assert maxrel(losses.read(F), rl) < 1e-5 and maxrel(dl.read(F, (B, V)), rd) < 1e-5
    assert np.abs(dl.read(F, (B, V)).sum(-1)).max() < 1e-4
    rl = rl.astype(F)
    old = (-rl + rng.uniform(-0.4, 0.4, B)).astype(F)       # ratios on both sides of the clip band
    adv = rnd(rng, B)
    new_lp = dev.empty(B * 4)
    dev.L.metal_enqueue_grpo_policy_grad(lgb.h, tb.h, dev.up(old).h, dev.up(adv).h, new_lp.h, dl.h, B, V, 0.2)
    rn, rg = np.zeros(B), np.zeros((B, V))
    op("f64", "or_grpo_policy_grad", lg.astype(np.float64), tgt, old.astype(np.float64), adv.astype(np.float64),
       rn, rg, B, V, 0.2)
    assert maxrel(new_lp.read(F), rn) < 1e-5
    got = dl.read(F, (B, V))
    same_gate = (np.abs(got).sum(-1) > 0) == (np.abs(rg).sum(-1) > 0)
    assert same_gate.all() and maxrel(got, rg) < 2e-5


def test_f16_rank_updates(dev):
    rng = np.random.default_rng(7)
    M, K, N = 100, 64, 72
    dY, X = rnd(rng, K, M, scale=0.1), rnd(rng, K, N)
    G = oracle.f32_to_f16_bits(rnd(rng, M, N, scale=0.1))
    Gb = dev.up(G)
    dev.L.metal_enqueue_f16_grad_accum(Gb.h, dev.up(dY).h, dev.up(X).h, M, K, N)
    ref = G.copy()
    op("f32", "or_f16_grad_accum", ref, dY, X, M, K, N)
    got = Gb.read(np.uint16, (M, N))
    # the fp32 sum order differs from the oracle's, so an element may land on the neighbouring half
    diff = np.abs(got.view(np.float16).astype(F) - ref.view(np.float16).astype(F))
    ulp = np.spacing(np.abs(ref.view(np.float16)).astype(np.float16)).astype(F)
    assert (diff <= ulp).all() and (got == ref).mean() > 0.98
    W = oracle.f32_to_f16_bits(rnd(rng, M, N, scale=0.02))
    Wb = dev.up(W)
    dev.L.metal_enqueue_f16_sgd_fused(Wb.h, dev.up(dY).h, dev.up(X).h, M, K, N, 0.01)
    refw = W.copy()
    op("f32", "or_f16_sgd_fused", refw, dY, X, M, K, N, 0.01)
    gw = Wb.read(np.uint16, (M, N))
    diff = np.abs(gw.view(np.float16).astype(F) - refw.view(np.float16).astype(F))
    ulp = np.spacing(np.abs(refw.view(np.float16)).astype(np.float16)).astype(F)
    assert (diff <= ulp).all() and (gw == refw).mean() > 0.98


def test_metal_buf_ptr_is_coherent_at_flush(dev):
    """The shared-memory contract of the reference's buffers: CPU writes are seen by the next
    enqueue, GPU writes by the CPU after metal_flush."""
    import ctypes as C
    n = 4096
    b = dev.empty(n * 4)
    p = dev.L.metal_buf_ptr(b.h)
    host = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float)), shape=(n,))
    host[:] = np.arange(n, dtype=F)
    dev.L.metal_enqueue_scale(b.h, 2.0, n)
    dev.be.flush()
    assert np.array_equal(host, 2 * np.arange(n, dtype=F))
    assert dev.L.metal_buf_ptr(b.h) == p                 # stable for the buffer's lifetime
    view = dev.L.metal_buf_view(b.h, 1024 * 4, 16 * 4)
    dev.L.metal_enqueue_scale(view, 0.5, 16)
    dev.be.flush()
    assert np.array_equal(host[1024:1040], np.arange(1024, 1040, dtype=F)) and host[1040] == 2080
    dev.L.metal_buf_free(view)
