"""Pins the oracle's single ops in the reference's buffer layouts ([H,N,D] heads,
[K,M] transposed operands ...) against numpy/torch fp64 library routines,
autograd and hand-derived answers.  The LoRA step as a whole is pinned in
test_oracle_step.py; the ops only the full-parameter GRPO variant uses
(grpo_policy_grad, f16_grad_accum, f16_sgd_apply, f16_sgd_fused) are pinned here."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import oracle
from oracle.oracle import SZ, op

P = "f64"
rng = np.random.default_rng(123)


def r(*shape):
    return rng.standard_normal(shape)


def rel(a, b):
    return float(np.abs(a - b).max() / (np.abs(b).max() + 1e-300))


def test_matmul_orientations():
    M, N, K = 5, 7, 9
    A, W = r(M, K), r(N, K).astype(np.float32)
    C = np.zeros((M, N)); op(P, "or_wmatmul", A, W, C, M, N, K)
    assert rel(C, A @ W.T.astype(np.float64)) < 1e-14
    A2 = r(M, N); C2 = np.zeros((M, K)); op(P, "or_wmatmul_nt", A2, W, C2, M, N, K)
    assert rel(C2, A2 @ W.astype(np.float64)) < 1e-14
    Wd = r(N, K); C3 = np.zeros((M, N)); op(P, "or_matmul", A, Wd, C3, M, N, K)
    assert rel(C3, A @ Wd.T) < 1e-14
    At, B = r(K, M), r(K, N); C4 = np.zeros((M, N)); op(P, "or_matmul_tn", At, B, C4, M, N, K)
    assert rel(C4, At.T @ B) < 1e-14
    C5 = np.zeros((M, K)); op(P, "or_matmul_nt", A2, Wd, C5, M, N, K)
    assert rel(C5, A2 @ Wd) < 1e-14


def test_rms_norm_forward_backward_vs_autograd_and_in_place():
    B, D, eps = 6, 40, 1e-6
    x, dy = r(B, D), r(B, D)
    g = (1 + 0.2 * r(D)).astype(np.float32)
    out = np.zeros((B, D)); op(P, "or_rms_norm", x, g, out, D, eps, B)
    xt = torch.tensor(x, requires_grad=True)
    yt = F.rms_norm(xt, (D,), torch.tensor(g.astype(np.float64)), float(np.float32(eps)))
    assert rel(out, yt.detach().numpy()) < 1e-13
    yt.backward(torch.tensor(dy))
    dx = np.zeros((B, D)); op(P, "or_rms_norm_backward", x, dy, g, dx, B, D, eps)
    assert rel(dx, xt.grad.numpy()) < 1e-12
    dy2 = dy.copy(); op(P, "or_rms_norm_backward", x, dy2, g, dy2, B, D, eps)     # dx aliases dy
    assert np.array_equal(dy2, dx)
    x2 = x.copy(); op(P, "or_rms_norm", x2, g, x2, D, eps, B)                    # out aliases x
    assert np.array_equal(x2, out)


def test_head_layout_ops():
    N, H, D, ratio = 5, 6, 4, 3
    src = r(N, H * D)
    t = np.zeros((H, N, D)); op(P, "or_transpose_heads_fwd", src, t, N, H, D)
    assert np.array_equal(t, src.reshape(N, H, D).transpose(1, 0, 2))
    back = np.zeros((N, H * D)); op(P, "or_transpose_heads_rev", t, back, N, H, D)
    assert np.array_equal(back, src)
    kv = r(2, N, D)
    ex = np.zeros((2 * ratio, N, D)); op(P, "or_repeat_kv", kv, ex, 2, N, D, ratio)
    assert np.array_equal(ex, np.repeat(kv, ratio, axis=0))        # q-head h reads kv-head h // ratio
    d = r(2 * ratio, N, D); dk = np.zeros((2, N, D)); op(P, "or_repeat_kv_bwd", d, dk, 2, N, D, ratio)
    assert rel(dk, d.reshape(2, ratio, N, D).sum(1)) < 1e-15


def test_rope_known_answer_orthogonality_and_inverse():
    Hq, Hkv, hd, N, theta = 2, 1, 8, 6, 10000.0
    # unit vector e_0 at position 1 rotates into (cos 1, 0.., sin 1 at index hd/2): freq(d=0) = 1
    q = np.zeros((Hq, N, hd)); k = np.zeros((Hkv, N, hd))
    q[0, 1, 0] = 1.0
    # pair d=1 uses freq = theta^(-2/hd): put e_{1+hd/2} at position 3
    k[0, 3, 1 + hd // 2] = 1.0
    op(P, "or_rope_train", q, k, Hq, Hkv, hd, N, theta)
    exp_q = np.zeros(hd); exp_q[0], exp_q[hd // 2] = np.cos(1.0), np.sin(1.0)
    assert np.allclose(q[0, 1], exp_q, atol=1e-15)
    a = 3.0 * np.float32(theta) ** (-2.0 / hd)
    exp_k = np.zeros(hd); exp_k[1], exp_k[1 + hd // 2] = -np.sin(a), np.cos(a)
    assert np.allclose(k[0, 3], exp_k, atol=1e-12)
    q, k = r(Hq, N, hd), r(Hkv, N, hd)
    q0, k0 = q.copy(), k.copy()
    op(P, "or_rope_train", q, k, Hq, Hkv, hd, N, theta)
    assert np.allclose(np.linalg.norm(q, axis=-1), np.linalg.norm(q0, axis=-1))
    assert np.array_equal(q[:, 0], q0[:, 0])                         # position 0 is the identity
    # relative-position property: <rope(a,m), rope(b,n)> depends on m-n only
    assert np.isclose(q[0, 4] @ (lambda z: z)(q[0, 4]), q0[0, 4] @ q0[0, 4])
    op(P, "or_rope_train_bwd", q, k, Hq, Hkv, hd, N, theta)
    assert np.allclose(q, q0, atol=1e-13) and np.allclose(k, k0, atol=1e-13)


def test_attention_forward_backward_vs_sdpa_autograd():
    H, N, D = 3, 7, 8
    scale = 1.0 / np.sqrt(np.float32(D))
    Q, K, V, dO = r(H, N, D), r(H, N, D), r(H, N, D), r(H, N, D)
    out, probs = np.zeros((H, N, D)), np.zeros((H, N, N))
    op(P, "or_attn_train_fwd", Q, K, V, out, probs, H, N, D, float(scale))
    qt, kt, vt = (torch.tensor(a, requires_grad=True) for a in (Q, K, V))
    ot = F.scaled_dot_product_attention(qt[None], kt[None], vt[None], is_causal=True, scale=float(scale))[0]
    assert rel(out, ot.detach().numpy()) < 1e-13
    assert np.allclose(probs.sum(-1), 1) and np.all(np.triu(probs, 1) == 0)
    ot.backward(torch.tensor(dO))
    ds, dQ = np.zeros((H, N, N)), np.zeros((H, N, D))
    op(P, "or_attn_bwd_dq", dO, probs, V, K, ds, dQ, H, N, D, float(scale))
    dK, dV = np.zeros((H, N, D)), np.zeros((H, N, D))
    op(P, "or_attn_bwd_dkv", ds, Q, probs, dO, dK, dV, H, N, D)
    assert rel(dQ, qt.grad.numpy()) < 1e-12
    assert rel(dK, kt.grad.numpy()) < 1e-12
    assert rel(dV, vt.grad.numpy()) < 1e-12
    assert np.all(np.triu(ds, 1) == 0) and np.allclose(ds.sum(-1), 0, atol=1e-14)


def test_activation_ops_vs_torch():
    n = 301
    g, u, dy = 3 * r(n), r(n), r(n)
    for name, fn in (("silu", F.silu), ("gelu", lambda t: F.gelu(t, approximate="tanh"))):
        gt, ut = torch.tensor(g, requires_grad=True), torch.tensor(u, requires_grad=True)
        y = fn(gt) * ut
        got = g.copy(); op(P, f"or_{name}_mul", got, u, SZ(n))
        assert rel(got, y.detach().numpy()) < 1e-9              # gelu constant is the 10-digit one
        y.backward(torch.tensor(dy))
        dg, du = np.zeros(n), np.zeros(n)
        op(P, f"or_{name}_mul_backward", dy, g, u, dg, du, SZ(n))
        assert rel(dg, gt.grad.numpy()) < 1e-9 and rel(du, ut.grad.numpy()) < 1e-9
        d2 = dy.copy(); op(P, f"or_{name}_mul_backward", d2, g, u, d2, du, SZ(n))   # dgate aliases dout
        assert np.array_equal(d2, dg)
    # the tanh argument clamp at +-15: tanh(15) = 1 - 1.9e-13, so the value moves by ~1e-11 at most
    big = np.array([40.0, -40.0]); one = np.ones(2)
    op(P, "or_gelu_mul", big, one, SZ(2))
    assert abs(big[0] - 40.0) < 1e-10 and abs(big[1]) < 1e-10


def test_elementwise_helpers():
    x, y = r(50), r(50)
    a = x.copy(); op(P, "or_residual_add", a, y, SZ(50)); assert np.array_equal(a, x + y)
    a = x.copy(); op(P, "or_scale", a, 0.25, SZ(50)); assert np.array_equal(a, x * 0.25)
    a = y.copy(); op(P, "or_add_scaled", a, x, 2.0, SZ(50)); assert np.array_equal(a, y + 2.0 * x)
    a = (10 * x).copy(); op(P, "or_clamp", a, 3.0, SZ(50)); assert np.array_equal(a, np.clip(10 * x, -3, 3))


def test_softmax_ce_vs_torch():
    B, V = 5, 33
    lg = 4 * r(B, V)
    tgt = rng.integers(0, V, B).astype(np.uint32)
    losses, dl = np.zeros(B), np.zeros((B, V))
    op(P, "or_softmax_ce", lg, tgt, losses, dl, B, V)
    lt = torch.tensor(lg, requires_grad=True)
    ce = F.cross_entropy(lt, torch.tensor(tgt.astype(np.int64)), reduction="none")
    assert rel(losses, ce.detach().numpy()) < 1e-13
    ce.sum().backward()
    assert rel(dl, lt.grad.numpy()) < 1e-13
    assert np.allclose(dl.sum(-1), 0, atol=1e-14)


def test_grpo_policy_grad_vs_autograd_of_the_ppo_clip_objective():
    """The kernel writes  w * r * (softmax - onehot)  with  w = -A  where the un-clipped branch is
    active and 0 where clipping binds (shaders/q8_kernels.metal:741-760).  Since
    (softmax - onehot) = -d(log p_a)/d(logits), that is the gradient of the surrogate OBJECTIVE
    A*min(r, clip(r)) and therefore MINUS the autograd gradient of the textbook PPO-clip loss:
    a sign quirk of the reference which parity reproduces."""
    N, V, e = 8, 21, 0.2
    lg = 2 * r(N, V)
    act = rng.integers(0, V, N).astype(np.uint32)
    lp_now = (torch.log_softmax(torch.tensor(lg), -1)[torch.arange(N), torch.tensor(act.astype(np.int64))]).numpy()
    # ratios 1 (inactive), inside the band, above and below it, with both advantage signs
    ratio = np.array([1.0, 1.1, 1.5, 1.5, 0.5, 0.5, 0.95, 1.0])
    adv = np.array([1.0, -2.0, 1.0, -1.0, 1.0, -1.0, 0.5, 0.0])
    old = lp_now - np.log(ratio)
    new_lp, dl = np.zeros(N), np.zeros((N, V))
    op(P, "or_grpo_policy_grad", lg, act, old, adv, new_lp, dl, N, V, e)
    assert rel(new_lp, lp_now) < 1e-13
    lt = torch.tensor(lg, requires_grad=True)
    lp = torch.log_softmax(lt, -1)[torch.arange(N), torch.tensor(act.astype(np.int64))]
    rt = torch.exp(lp - torch.tensor(old))
    advt = torch.tensor(adv)
    obj = -torch.minimum(rt * advt, torch.clamp(rt, 1 - e, 1 + e) * advt)     # textbook PPO-clip loss
    obj.sum().backward()
    assert rel(dl, -lt.grad.numpy()) < 1e-12
    assert np.all(dl[2] == 0) and np.all(dl[5] == 0) and np.any(dl[3] != 0) and np.any(dl[4] != 0)


def test_f16_grad_accum_and_sgd():
    M, K, N = 6, 5, 8
    dY, X = r(K, M), r(K, N)
    G0 = (0.1 * r(M, N)).astype(np.float16)
    G = G0.view(np.uint16).copy()
    op(P, "or_f16_grad_accum", G, dY, X, M, K, N)
    exp = (G0.astype(np.float32) + (dY.T @ X).astype(np.float32)).astype(np.float16)
    assert np.array_equal(G.view(np.float16), exp)
    W0 = (0.02 * r(M, N)).astype(np.float16)
    W = W0.view(np.uint16).copy()
    lr = 0.5
    Gc = G.copy()
    op(P, "or_f16_sgd_apply", W, Gc, SZ(M * N), lr)
    expw = (W0.astype(np.float32) - np.float32(lr) * G.view(np.float16).astype(np.float32)).astype(np.float16)
    assert np.array_equal(W.view(np.float16), expw) and not Gc.any()
    W = W0.view(np.uint16).copy()
    op(P, "or_f16_sgd_fused", W, dY, X, M, K, N, lr)
    expw = (W0.astype(np.float32) - np.float32(lr) * (dY.T @ X).astype(np.float32)).astype(np.float16)
    assert np.array_equal(W.view(np.float16), expw)


def test_adamw_vs_torch_and_clip_rule():
    n = 64
    p0, g = r(n), r(n)
    p, m, v = p0.copy(), np.zeros(n), np.zeros(n)
    tp = torch.nn.Parameter(torch.tensor(p0))
    opt = torch.optim.AdamW([tp], lr=1e-2, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    for step in (1, 2, 3):
        gs = g * step
        op(P, "or_adamw", p, gs, m, v, SZ(n), 1e-2, 0.9, 0.999, 1e-8, 0.01, step)
        tp.grad = torch.tensor(gs)
        opt.step()
        assert rel(p, tp.detach().numpy()) < 1e-6           # float hyper-parameters vs double
    big = 3 * r(n)
    nrm = np.linalg.norm(big)
    b2 = big.copy()
    ret = op(P, "or_clip_grad_norm", b2, SZ(n), 1.0)
    assert abs(ret - nrm) < 1e-12 and abs(np.linalg.norm(b2) - 1.0) < 1e-6
    small = big / (2 * nrm)
    s2 = small.copy()
    op(P, "or_clip_grad_norm", s2, SZ(n), 1.0)
    assert np.array_equal(s2, small)                        # norm <= 1: untouched


# ---------------------------------------------------------------- decode-step ops

def test_q8_matvec_known_answer_and_vs_dequantised_product():
    # one block: d = 0.5, q = 1..32, x = 1  ->  0.5 * (1 + ... + 32) = 264
    blk = np.zeros(34, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    blk[2:] = np.arange(1, 33, dtype=np.int8).view(np.uint8)
    y = np.zeros(1); op(P, "or_q8_matvec", blk, np.ones(32), y, 1, 1)
    assert y[0] == 264.0
    # negative codes and a negative scale keep their signs
    blk[0:2] = np.frombuffer(np.float16(-2.0).tobytes(), np.uint8)
    blk[2:] = np.full(32, -128, np.int8).view(np.uint8)
    x = np.zeros(32); x[5] = 1.0
    op(P, "or_q8_matvec", blk, x, y, 1, 1)
    assert y[0] == 256.0
    # random matrix: equals (dequantised weight) @ x with numpy
    rows, nb = 7, 5
    w = r(rows, nb * 32).astype(np.float32)
    q = oracle.q8_quantize(w)
    wd = oracle.q8_dequant(q, rows, nb * 32).astype(np.float64)
    x = r(nb * 32)
    y = np.zeros(rows); op(P, "or_q8_matvec", q, x, y, rows, nb)
    assert rel(y, wd @ x) < 1e-14


def test_f16_matvec_and_batch_vs_numpy():
    rows, cols, B = 9, 50, 3
    W = r(rows, cols).astype(np.float16)
    X = r(B, cols)
    Y = np.zeros((B, rows)); op(P, "or_f16_batch_matvec", W.view(np.uint16), X, Y, rows, cols, B)
    assert rel(Y, X @ W.astype(np.float64).T) < 1e-14
    y1 = np.zeros(rows); op(P, "or_f16_batch_matvec", W.view(np.uint16), X[1].copy(), y1, rows, cols, 1)
    assert np.array_equal(y1, Y[1])


def test_rope_at_one_position_is_the_training_rope_row():
    Hq, Hkv, hd, N, theta = 4, 2, 16, 9, 1e4
    q, k = r(Hq, N, hd), r(Hkv, N, hd)
    qt, kt = q.copy(), k.copy(); op(P, "or_rope_train", qt, kt, Hq, Hkv, hd, N, theta)   # pinned above
    for pos in (0, 3, 8):
        q1, k1 = np.ascontiguousarray(q[:, pos]), np.ascontiguousarray(k[:, pos])
        op(P, "or_rope", q1, k1, Hq, Hkv, hd, pos, theta)
        assert np.array_equal(q1, qt[:, pos]) and np.array_equal(k1, kt[:, pos])
    q0 = np.ascontiguousarray(q[:, 0]); k0 = np.ascontiguousarray(k[:, 0])
    assert np.array_equal(q0, qt[:, 0])                                                # position 0: identity


def test_kv_cache_store_writes_one_row_per_head():
    Hkv, max_seq, hd, pos = 3, 6, 4, 4
    k, v = r(Hkv, hd), r(Hkv, hd)
    kc, vc = r(Hkv, max_seq, hd), r(Hkv, max_seq, hd)
    ek, ev = kc.copy(), vc.copy(); ek[:, pos] = k; ev[:, pos] = v
    op(P, "or_kv_cache_store", k, v, kc, vc, Hkv, max_seq, hd, pos)
    assert np.array_equal(kc, ek) and np.array_equal(vc, ev)


def test_decode_attention_vs_sdpa_and_the_training_kernel_row():
    Hq, ratio, hd, max_seq, n = 6, 3, 16, 12, 7          # 1/sqrt(16) is exact in the dispatch's float
    Hkv = Hq // ratio
    Q, Kc, Vc = r(Hq, hd), r(Hkv, max_seq, hd), r(Hkv, max_seq, hd)
    out = np.zeros((Hq, hd)); op(P, "or_attention", Q, Kc, Vc, out, n, hd, max_seq, Hq, ratio)
    Kx = np.repeat(Kc[:, :n], ratio, axis=0); Vx = np.repeat(Vc[:, :n], ratio, axis=0)        # [Hq, n, hd]
    ref = F.scaled_dot_product_attention(torch.tensor(Q)[:, None], torch.tensor(Kx), torch.tensor(Vx)).numpy()[:, 0]
    assert rel(out, ref) < 1e-13
    # the last query of the causal training kernel attends the same n keys
    Qn = r(Hq, n, hd); Qn[:, n - 1] = Q
    o2, probs = np.zeros((Hq, n, hd)), np.zeros((Hq, n, n))
    op(P, "or_attn_train_fwd", Qn, np.ascontiguousarray(Kx), np.ascontiguousarray(Vx), o2, probs, Hq, n, hd, float(1 / np.sqrt(hd)))
    assert rel(out, o2[:, n - 1]) < 1e-13
    # one key: the output is that key's value
    op(P, "or_attention", Q, Kc, Vc, out, 1, hd, max_seq, Hq, ratio)
    assert rel(out, np.repeat(Vc[:, 0], ratio, axis=0)) < 1e-15
