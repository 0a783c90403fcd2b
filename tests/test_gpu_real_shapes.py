"""GPU parity at the shapes the benchmark launches (through the C ABI).

Three layers of checks:
  * the step at the real widths of configs 2-5 with one or two layers and a truncated vocabulary, against the CPU
    oracle: live for the 64-row cases, against committed oracle outputs (tests/golden/real_width_*.npz, written by
    tests/golden/make_real_width.py) for the 2048-row Q8_0 case and the 160-row full-parameter GRPO case;
  * the dispatch-level GEMMs at the three matrix shapes of config 3 that no layer-level case reaches
    (gate|up 19456 x 2560, down 2560 x 9728, LM head 151936 x 2560);
  * the configurations exactly as they are benchmarked (all layers, real vocabulary), through properties that hold
    at any size: loss of a random-init model at its closed-form value (ln V + D * 0.02^2 / 2), a zero B gives dA == 0
    and dB != 0, everything finite,
    the loss of a repeated batch falls, and the two GEMM families agree.

Tolerances as everywhere: loss 1e-3 relative, gradients and adapters 1e-2 relative per tensor."""
import os

import numpy as np
import pytest

from llm_metal_amd import lib
from llm_metal_amd.configs import C2, C3, C4, C5
from llm_metal_amd.sft import SFTState
from llm_metal_amd.synth import lora_views, make_batch, make_model
from oracle import oracle
from oracle.oracle import op
from tests import real_width_cases as rw
from tests.gpu_util import Dev, rel

pytestmark = pytest.mark.gpu
F = np.float32
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
MATS = ("wq", "wk", "wv", "wo", "wg", "wu", "wd")


def f16(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)


# ---------------------------------------------------------------- real widths, few layers, against the oracle

@pytest.mark.parametrize("cfg", [rw.C3_WIDTHS, rw.C2_WIDTHS, rw.C3Q_WIDTHS], ids=lambda c: c.name)
def test_step_at_real_widths_matches_oracle(cfg):
    model = make_model(cfg, seed=rw.MODEL_SEED, gamma_jitter=rw.GAMMA_JITTER)
    used = oracle.weights_as_used(model, "f16" if cfg.weight_format == "f16" else "q8")
    lora = model["lora"].copy()
    m, v, step = np.zeros_like(lora), np.zeros_like(lora), 0
    lr = 1e-4
    with SFTState(cfg, model) as st:
        for i in range(2):
            tok, tgt = make_batch(cfg, seed=rw.BATCH_SEED + i)
            r = oracle.sft_train_step(cfg, used, lora, m, v, step, tok, tgt, lr, want_logits=True)
            step = r["step"]
            loss = st.train_step(tok, tgt, lr)
            assert abs(loss - r["loss"]) <= 1e-3 * abs(r["loss"]), (i, loss, r["loss"])
            assert rel(st.logits(), r["logits"]) < 1e-2
            assert abs(st.grad_norm() - r["grad_norm"]) <= 1e-2 * r["grad_norm"]
            for L, (gv, rv) in enumerate(zip(lora_views(cfg, st.lora_grads()), lora_views(cfg, r["grad"]))):
                for k in ("A_q", "B_q", "A_v", "B_v"):
                    assert rel(gv[k], rv[k]) < 1e-2, (i, L, k, rel(gv[k], rv[k]))
            for L, (wv, rv) in enumerate(zip(lora_views(cfg, st.lora()), lora_views(cfg, lora))):
                for k in ("A_q", "B_q", "A_v", "B_v"):
                    assert rel(wv[k], rv[k]) < 1e-2, (i, L, k)
        d_gpu, d_ref = st.lora() - model["lora"], lora - model["lora"]
        assert rel(d_gpu, d_ref) < 0.1 and (np.sign(d_gpu) == np.sign(d_ref)).mean() > 0.97


def _golden(name, model):
    g = np.load(os.path.join(GOLDEN, name))
    fp = rw.weights_fingerprint(model)
    assert abs(fp - float(g["fingerprint"])) <= 1e-9 * abs(fp), \
        "the synthetic model differs from the one the fixture was made from: run tests/golden/make_real_width.py"
    return g


def _check_sampled(g, key, tensor, tol):
    tensor = np.asarray(tensor, dtype=np.float64).ravel()
    want_norm = float(g[key + "_norm"])
    got_norm = float(np.sqrt((tensor ** 2).sum()))
    assert abs(got_norm - want_norm) <= tol * want_norm, (key, got_norm, want_norm)
    idx = rw.sample_idx(key, tensor.size)
    assert rel(tensor[idx], g[key + "_sample"]) < tol, (key, rel(tensor[idx], g[key + "_sample"]))


@pytest.mark.parametrize("policy,attention", [(0, -1), (2, -1), (0, 0)],
                         ids=["measured_rule", "q8_unpacked_in_lds", "attention_with_saved_probabilities"])
def test_q8_step_at_2048_rows_matches_oracle_fixture(policy, attention):
    """Config 4's shape on one layer: Q8_0 weights, 4 x 512 rows.  Policy 0 is what the benchmark runs (every product
    on the large-M kernel over an F16 image of the operand, attention without saved probabilities); policy 2 keeps the
    operand quantised and unpacks the Q8_0 tiles into LDS inside the large-M kernel; the third case pins the attention
    kernels that save the probabilities, which the rule leaves at this shape."""
    cfg = rw.C4_WIDTHS
    model = make_model(cfg, seed=rw.MODEL_SEED, gamma_jitter=rw.GAMMA_JITTER)
    g = _golden("real_width_c4.npz", model)
    tok, tgt = make_batch(cfg, seed=rw.BATCH_SEED)
    L = lib.load()
    L.hip_gemm_force_large_m(policy)
    L.hip_attention_flash(attention)
    try:
        with SFTState(cfg, model) as st:
            loss = st.train_step(tok, tgt, 1e-4)
            assert abs(loss - float(g["loss"])) <= 1e-3 * float(g["loss"]), (loss, float(g["loss"]))
            assert abs(st.grad_norm() - float(g["grad_norm"])) <= 1e-2 * float(g["grad_norm"])
            _check_sampled(g, "logits", st.logits(), 1e-2)
            # the update leaves the clipped gradients in place: undo the clip
            grads = lora_views(cfg, st.lora_grads() * max(1.0, float(g["grad_norm"])))[0]
            for k in ("A_q", "B_q", "A_v", "B_v"):
                _check_sampled(g, "grad_" + k, grads[k], 1e-2)
            after, before = lora_views(cfg, st.lora())[0], lora_views(cfg, model["lora"])[0]
            for k in ("A_q", "B_q", "A_v", "B_v"):
                _check_sampled(g, "delta_" + k, after[k] - before[k], 0.1)
    finally:
        L.hip_gemm_force_large_m(0)
        L.hip_attention_flash(-1)


@pytest.mark.parametrize("batch", [1, 2], ids=["one_completion_per_pass", "group_in_one_pass"])
def test_grpo_full_parameter_at_real_widths_matches_oracle_fixture(batch):
    """Config 5's shape on two layers: Gemma3-1B widths, full-parameter, 160 rows per completion, F16 accumulation
    over the group and one apply (grpo_apply_completions, src/nn/fast_grpo.c:376-495); the fixture's two completions
    one per pass (as the reference runs them) and both in one pass (as the benchmark runs its group of four)."""
    cfg = rw.C5_WIDTHS.with_(batch=batch)
    model = make_model(cfg, seed=rw.MODEL_SEED, gamma_jitter=rw.GAMMA_JITTER)
    g = _golden("real_width_c5.npz", model)
    used = oracle.weights_as_used(model)
    prompt, toks, adv, _ = rw.c5_completions(cfg)
    old = [g[f"old_lp_{i}"] for i in range(len(toks))]
    with SFTState(cfg, model) as st:
        got_lp = st.grpo_apply_completions(prompt, toks, old, adv, rw.C5_CLIP, rw.C5_LR, accurate=True)
        for i, t in enumerate(toks):
            _, use, comp = rw.c5_sequence(cfg, used, prompt, t)
            assert np.allclose(got_lp[i, use:use + comp], g["new_lp"][i, use:use + comp], atol=2e-3), i
        for L, k in [(L, k) for L in range(cfg.NL) for k in MATS] + [(0, "lm_head")]:
            got = st.matrix_f16(L, k, 0)
            assert np.array_equal(st.matrix_f16(L, k, 1), got), (L, k)        # the transposed image follows
            assert not st.matrix_f16(L, k, 2).any()                           # accumulators zeroed by the apply
            w0 = used["lm_head"] if k == "lm_head" else used[k][L]
            _check_sampled(g, f"delta_{L}_{k}", f16(got) - w0, 3e-2)


# ---------------------------------------------------------------- GEMM shapes of config 3 at the dispatch level

@pytest.mark.parametrize("M,N,K", [(64, 19456, 2560), (64, 2560, 9728), (64, 151936, 2560)],
                         ids=["gate_up", "down", "lm_head"])
def test_f16_matmul_and_nt_at_config3_shapes(M, N, K):
    dev = Dev()
    try:
        rng = np.random.default_rng(N + K)
        A = rng.standard_normal((M, K)).astype(F)
        A[0] *= 1e-6
        A[M - 1] *= 3e4
        Wbits = oracle.f32_to_f16_bits((rng.standard_normal((N, K), dtype=F) * F(0.02)))
        W = oracle.f16_bits_to_f32(Wbits)
        Wb = dev.up(Wbits)
        C = dev.empty(M * N * 4)
        dev.L.metal_enqueue_f16_matmul(dev.up(A).h, Wb.h, C.h, M, N, K)
        got = C.read(F, (M, N))
        rows = (0, 17, M - 1)                                  # the oracle follows three rows; all rows against fp64 BLAS
        ref = np.zeros((len(rows), N), F)
        op("f32", "or_wmatmul", np.ascontiguousarray(A[list(rows)]), W, ref, len(rows), N, K)
        for j, m in enumerate(rows):
            assert rel(got[m], ref[j]) < 1.5e-3, (m, rel(got[m], ref[j]))
        assert rel(got, A.astype(np.float64) @ W.T.astype(np.float64)) < 1e-3
        A2 = rng.standard_normal((M, N)).astype(F)
        C2 = dev.empty(M * K * 4)
        dev.L.metal_enqueue_f16_matmul_nt(dev.up(A2).h, Wb.h, C2.h, M, N, K)
        got2 = C2.read(F, (M, K))
        ref2 = np.zeros((len(rows), K), F)
        op("f32", "or_wmatmul_nt", np.ascontiguousarray(A2[list(rows)]), W, ref2, len(rows), N, K)
        for j, m in enumerate(rows):
            assert rel(got2[m], ref2[j]) < 1.5e-3, (m, rel(got2[m], ref2[j]))
        assert rel(got2, A2.astype(np.float64) @ W.astype(np.float64)) < 1e-3
    finally:
        dev.close()


# ---------------------------------------------------------------- the benchmarked configurations, full size

def expected_initial_loss(cfg):
    """Cross-entropy of a random-init model, in closed form: the final RMSNorm (gamma 1) leaves every row with mean
    square 1, so a logit is a sum of D terms x_k w_k with w ~ N(0, 0.02^2): N(0, s2) with s2 = D * 0.02^2, independent of
    the target.  log sum exp over V such logits is ln V + s2 / 2 (mean of a log-normal), the target's logit has mean 0."""
    return float(np.log(cfg.V) + cfg.D * 0.02 ** 2 / 2)


def _zero_b_properties(cfg, st, model, steps=3, lr=1e-4):
    """Step properties that need no oracle: see the module docstring."""
    tok, tgt = make_batch(cfg, seed=100)
    losses = []
    for i in range(steps):
        losses.append(st.train_step(tok, tgt, lr))
        if i == 0:
            assert abs(losses[0] - expected_initial_loss(cfg)) < 0.2, (losses[0], expected_initial_loss(cfg))
            assert np.isfinite(st.grad_norm()) and st.grad_norm() > 0
            for L, gv in enumerate(lora_views(cfg, st.lora_grads())):
                # B = 0: the adapters add nothing to the forward and dA = dh^T x with dh = sc * dY B is exactly zero
                assert not gv["A_q"].any() and not gv["A_v"].any(), L
                assert np.isfinite(gv["B_q"]).all() and np.isfinite(gv["B_v"]).all(), L
                assert np.abs(gv["B_q"]).max() > 0 and np.abs(gv["B_v"]).max() > 0, L
    assert np.isfinite(losses).all()
    assert np.isfinite(st.lora()).all()
    assert losses[-1] < losses[0], losses                  # the same batch again: AdamW on B alone already lowers it
    return losses


@pytest.fixture(scope="module")
def qwen3_4b_model():
    return make_model(C3, seed=0, lora_b_std=0.0)


def test_config3_as_benchmarked(qwen3_4b_model):
    with SFTState(C3, qwen3_4b_model) as st:
        _zero_b_properties(C3, st, qwen3_4b_model)


def test_config3_as_benchmarked_on_both_workgroup_shapes_of_the_ring_kernel(qwen3_4b_model):
    """1 x 64 rows on F16 weights, all layers: with gemm_ring_wide on five product shapes (the default) and with gemm_ring
    alone the step gives the same loss and gradient norm; so does the register-staged kernel."""
    L = lib.load()
    with SFTState(C3, qwen3_4b_model) as st:
        tok, tgt = make_batch(C3, seed=100)
        out = {}
        for ring, wide in ((1, 1), (1, 0), (0, 0)):
            L.hip_gemm_ring(ring)
            L.hip_gemm_ring_wide(wide)
            st.set_lora(qwen3_4b_model["lora"])
            out[ring, wide] = (st.train_step(tok, tgt, 0.0), st.grad_norm())   # lr 0: the adapters stay put
        L.hip_gemm_ring(1)
        L.hip_gemm_ring_wide(1)
        for other in ((1, 0), (0, 0)):
            assert abs(out[other][0] - out[1, 1][0]) <= 1e-3 * out[1, 1][0], out
            assert abs(out[other][1] - out[1, 1][1]) <= 1e-2 * out[1, 1][1], out


def test_config3_with_q8_weights_as_benchmarked_and_the_two_streaming_kernels_agree(qwen3_4b_model):
    """1 x 64 rows on Q8_0 weights, all layers: the products take gemm_ring and gemm_ring_wide with the tiles quantised up to
    LDS (and planes of halves); on gemm_ring alone, and on the register-staged kernel, the step must give the same loss and
    gradient norm."""
    from llm_metal_amd.configs import C3Q
    L = lib.load()
    with SFTState(C3Q, qwen3_4b_model) as st:
        tok, tgt = make_batch(C3Q, seed=100)
        out = {}
        for ring, wide in ((1, 1), (1, 0), (0, 0)):
            L.hip_gemm_ring(ring)
            L.hip_gemm_ring_wide(wide)
            st.set_lora(qwen3_4b_model["lora"])
            out[ring, wide] = (st.train_step(tok, tgt, 0.0), st.grad_norm())   # lr 0: the adapters stay put
        L.hip_gemm_ring(1)
        L.hip_gemm_ring_wide(1)
        for other in ((1, 0), (0, 0)):
            assert abs(out[other][0] - out[1, 1][0]) <= 1e-3 * out[1, 1][0], out
            assert abs(out[other][1] - out[1, 1][1]) <= 1e-2 * out[1, 1][1], out
        _zero_b_properties(C3Q, st, qwen3_4b_model)


def test_config4_as_benchmarked_and_gemm_families_agree(qwen3_4b_model):
    """4 x 512 rows on Q8_0 weights: the measured rule sends every product to the large-M kernel; forced onto the
    weight-streaming kernel (policy -1) the step must give the same loss and gradient norm."""
    L = lib.load()
    with SFTState(C4, qwen3_4b_model) as st:
        tok, tgt = make_batch(C4, seed=100)
        out = {}
        for policy in (1, -1, 2):
            L.hip_gemm_force_large_m(policy)
            st.set_lora(qwen3_4b_model["lora"])
            out[policy] = (st.train_step(tok, tgt, 0.0), st.grad_norm())       # lr 0: the adapters stay put
        L.hip_gemm_force_large_m(0)
        for policy in (-1, 2):
            assert abs(out[policy][0] - out[1][0]) <= 1e-3 * out[1][0], out
            assert abs(out[policy][1] - out[1][1]) <= 1e-3 * out[1][1], out
        _zero_b_properties(C4, st, qwen3_4b_model, steps=2)


def test_config2_as_benchmarked():
    model = make_model(C2, seed=0, lora_b_std=0.0)
    with SFTState(C2, model) as st:
        _zero_b_properties(C2, st, model)


def test_config5_as_benchmarked():
    """Four completions of 128 tokens after a 32-token prompt through Gemma3-1B, full-parameter, accumulate + apply:
    log-probabilities near -ln V for a random-init model, finite, every weight image moved, accumulators zero,
    transposed images equal to the forward ones."""
    cfg = C5
    model = make_model(cfg, seed=0)
    rng = np.random.default_rng(7)
    G, p_len = 4, 32
    prompt = rng.integers(0, cfg.V, p_len).astype(np.uint32)
    comps = [rng.integers(0, cfg.V, cfg.seq - p_len).astype(np.uint32) for _ in range(G)]
    r = rng.standard_normal(G).astype(np.float32)
    adv = (r - r.mean()) / (r.std() + 1e-8)
    zeros = [np.zeros(cfg.seq - p_len, dtype=np.float32) for _ in range(G)]
    with SFTState(cfg, model) as st:
        lp0 = st.grpo_apply_completions(prompt, comps, zeros, np.zeros(G, dtype=np.float32), 0.2, 0.0)
        assert np.isfinite(lp0).all()
        # an action is the token fed in at its own position (src/nn/fast_grpo.c:430-443) and the head is tied to the
        # embedding table, so its logit carries the residual stream's own embedding component: the log-probabilities sit
        # a little above the closed form for independent targets, never below it
        mean_lp = float(lp0[:, p_len:].mean())
        assert -expected_initial_loss(cfg) - 0.2 < mean_lp < -expected_initial_loss(cfg) + 3.0, mean_lp
        # prompt rows carry action id 0 and advantage 0: a token independent of the inputs, so there the closed form holds
        assert abs(float(lp0[:, :p_len].mean()) + expected_initial_loss(cfg)) < 0.3, float(lp0[:, :p_len].mean())
        before = {k: st.matrix_f16(cfg.NL - 1, k, 0) for k in ("wq", "wd")}
        old = [lp0[i, p_len:].copy() for i in range(G)]
        lp1 = st.grpo_apply_completions(prompt, comps, old, adv, 0.2, 1.0)
        assert np.allclose(lp1, lp0, atol=1e-3)                # same policy as the pass that produced `old`
        for k in ("wq", "wd"):
            now = st.matrix_f16(cfg.NL - 1, k, 0)
            assert np.isfinite(f16(now)).all()
            assert (now != before[k]).any(), k
            assert np.array_equal(st.matrix_f16(cfg.NL - 1, k, 1), now), k
            assert not st.matrix_f16(cfg.NL - 1, k, 2).any(), k
