"""Pins the oracle's full-parameter mode (weight gradients into F16 accumulators,
fused SGD, apply) and its GRPO pass.

Pins: torch autograd for every dW = dY^T X (a transposed operand, a wrong saved
activation or a wrong dY fails here); a custom autograd function for the
reference's order "update W_q/k/v, then propagate through the new W" in SGD mode;
numpy float16 arithmetic for the apply rule; the sign/gate of the policy gradient
against autograd of the clipped surrogate."""
import numpy as np
import pytest
import torch

from llm_metal_amd.configs import C1, TINY_GEMMA3
from llm_metal_amd.synth import make_batch, make_model
from oracle import oracle
from tests import torch_ref

SMALL_Q = C1.with_(name="small_q_full", NL=2, D=64, Hq=4, Hkv=2, hd=16, IS=96, V=160, seq=12, batch=2, R=0)
SMALL_G = TINY_GEMMA3.with_(name="small_g_full", NL=3, D=48, Hq=4, Hkv=1, hd=16, IS=80, V=128, seq=10, batch=1, R=0)
MATS = torch_ref.MATS
GA = {"wq": "gq", "wk": "gk", "wv": "gv", "wo": "go", "wg": "gg", "wu": "gu", "wd": "gd"}


def _rel(a, b):
    return float(np.linalg.norm(np.asarray(a, dtype=np.float64) - b) / (np.linalg.norm(b) + 1e-300))


def _pairs(c, got, want):
    for k in MATS:
        for L in range(c.NL):
            yield f"{k}[{L}]", got[k][L], want[k][L]
    yield "lm_head", got["lm_head"], want["lm_head"]


@pytest.mark.parametrize("cfg", [SMALL_Q, SMALL_G], ids=lambda c: c.name)
def test_accumulated_gradients_match_autograd(cfg):
    model = make_model(cfg, seed=7, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    before = {k: [w.copy() for w in used[k]] for k in MATS}
    tok, tgt = make_batch(cfg, seed=8)
    want, loss, logits = torch_ref.full_param_grads(cfg, used, tok, tgt)
    ga = oracle.new_grad_accum(used)
    out = oracle.full_param_pass(cfg, used, ga, tok=tok, tgt=tgt, precision="f64", want_logits=True)
    assert abs(out["loss"] - loss) < 1e-8 * abs(loss)
    assert _rel(out["logits"], logits) < 1e-8
    got = {k: [oracle.f16_bits_to_f32(ga[GA[k]][L]) for L in range(cfg.NL)] for k in MATS}
    got["lm_head"] = oracle.f16_bits_to_f32(ga["glm"])
    for name, g, w in _pairs(cfg, got, want):
        # one F16 rounding of an fp64-accurate sum: half an ulp of 2^-10 relative, or the subnormal step
        tol = np.maximum(np.abs(w) * 2.0 ** -11, 2.0 ** -25) * 1.0001 + 1e-12
        assert np.all(np.abs(g - w) <= tol), name
        assert np.abs(w).max() > 0, name
    for k in MATS:                                       # accumulation leaves the weights alone
        for L in range(cfg.NL):
            assert np.array_equal(used[k][L], before[k][L])
    # a second pass adds: G2 = half(G1 + dW)
    g1 = got
    oracle.full_param_pass(cfg, used, ga, tok=tok, tgt=tgt, precision="f64")
    g2 = oracle.f16_bits_to_f32(ga["gd"][0])
    want2 = (g1["wd"][0].astype(np.float32) + want["wd"][0].astype(np.float32)).astype(np.float16).astype(np.float32)
    assert np.mean(g2 == want2) > 0.999 and _rel(g2, 2 * want["wd"][0]) < 1e-3
    # apply: W = half(W - lr G), G = 0, checked with numpy's float16
    lr = np.float32(0.05)
    Gd = oracle.f16_bits_to_f32(ga["gd"][0])
    Wd = used["wd"][0].copy()
    oracle.apply_grad_sgd(cfg, used, ga, float(lr))
    expect = (Wd - lr * Gd).astype(np.float16).astype(np.float32)
    assert np.array_equal(used["wd"][0], expect)
    assert not np.array_equal(used["wd"][0], Wd)
    assert all(not a.any() for k in GA.values() for a in ga[k]) and not ga["glm"].any()


@pytest.mark.parametrize("cfg", [SMALL_Q, SMALL_G], ids=lambda c: c.name)
def test_fused_sgd_updates_qkv_before_propagating(cfg):
    model = make_model(cfg, seed=9, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    before = {k: [w.copy() for w in used[k]] for k in MATS}
    before["lm_head"] = used["lm_head"].copy()
    tok, tgt = make_batch(cfg, seed=10)
    lr = 0.5                                             # large, so that the order of update and use is visible
    quirk, _, _ = torch_ref.full_param_grads(cfg, used, tok, tgt, qkv_lr=lr)
    plain, _, _ = torch_ref.full_param_grads(cfg, used, tok, tgt)
    oracle.full_param_pass(cfg, used, None, lr=lr, tok=tok, tgt=tgt, precision="f64")
    delta = {k: [used[k][L].astype(np.float64) - before[k][L] for L in range(cfg.NL)] for k in MATS}
    delta["lm_head"] = used["lm_head"].astype(np.float64) - before["lm_head"]
    worst_plain = 0.0
    for (name, d, gq), (_, _, gp) in zip(_pairs(cfg, delta, quirk), _pairs(cfg, delta, plain)):
        W = before[name[:2]][int(name[3])] if name != "lm_head" else before["lm_head"]
        ulp = np.maximum(np.maximum(np.abs(W), np.abs(W - lr * gq)), 2.0 ** -14) * 2.0 ** -10   # F16 spacing (upper bound)
        assert np.all(np.abs(d + lr * gq) <= 0.51 * ulp + 1e-12), name
        worst_plain = max(worst_plain, float(np.max(np.abs(d + lr * gp) / ulp)))
    # the plain gradient (propagating through the OLD Q/K/V weights) is measurably different in the lower layers
    assert worst_plain > 2.0


def test_grpo_pass_matches_autograd_of_clipped_surrogate():
    cfg = SMALL_Q.with_(batch=1, seq=12)
    model = make_model(cfg, seed=11, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    tok, _ = make_batch(cfg, seed=12)
    rng = np.random.default_rng(0)
    actions = rng.integers(0, cfg.V, cfg.BN).astype(np.uint32)
    advs = rng.standard_normal(cfg.BN)
    advs[:4] = 0.0                                       # prompt positions carry no advantage
    first = oracle.full_param_pass(cfg, used, oracle.new_grad_accum(used), tok=tok, precision="f64",
                                   grpo=dict(actions=actions, old_lp=np.zeros(cfg.BN), advs=np.zeros(cfg.BN),
                                             clip_eps=0.2, dl_scale=1.0))
    old_lp = first["new_lp"] + rng.uniform(-0.5, 0.5, cfg.BN)          # ratios on both sides of the clip range
    G = 4
    ga = oracle.new_grad_accum(used)
    oracle.full_param_pass(cfg, used, ga, tok=tok, precision="f64",
                           grpo=dict(actions=actions, old_lp=old_lp, advs=advs, clip_eps=0.2, dl_scale=1.0 / G))
    # autograd of the surrogate objective sum_p min(r A, clip(r) A) / G itself: the kernel's dlogits equal
    # +d(surrogate)/d(logits), i.e. minus the gradient of the textbook PPO-clip loss (the reference's sign)
    params = {k: [torch_ref._t(w).requires_grad_(True) for w in used[k]] for k in MATS}
    params["lm_head"] = torch_ref._t(used["lm_head"]).requires_grad_(True)
    _, logits = torch_ref.forward_loss(cfg, used, None, tok, np.zeros(cfg.BN, dtype=np.uint32), params=params)
    lp = torch.log_softmax(logits, -1)[torch.arange(cfg.BN), torch.as_tensor(actions.astype(np.int64))]
    ratio = torch.exp(lp - torch.as_tensor(old_lp))
    A = torch.as_tensor(advs)
    sur = torch.minimum(ratio * A, torch.clamp(ratio, 0.8, 1.2) * A).sum() / G
    sur.backward()
    assert _rel(first["new_lp"], lp.detach().numpy()) < 1e-9
    for k in ("wd", "wq", "wo"):
        for L in range(cfg.NL):
            got = oracle.f16_bits_to_f32(ga[GA[k]][L])
            assert _rel(got, params[k][L].grad.numpy()) < 1e-3, (k, L)
    assert _rel(oracle.f16_bits_to_f32(ga["glm"]), params["lm_head"].grad.numpy()) < 1e-3


def test_lora_mode_pass_equals_the_training_step_gradient():
    cfg = C1.with_(name="small_q_lora", NL=2, D=64, Hq=4, Hkv=2, hd=16, IS=96, V=160, seq=12, batch=1, R=4, alpha=8.0)
    model = make_model(cfg, seed=13, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    tok, tgt = make_batch(cfg, seed=14)
    lora = model["lora"].astype(np.float64)
    z = np.zeros_like(lora)
    step = oracle.sft_train_step(cfg, used, lora.copy(), z.copy(), z.copy(), 0, tok, tgt, 1e-3, do_update=False,
                                 precision="f64")
    one = oracle.full_param_pass(cfg, used, None, tok=tok, tgt=tgt, precision="f64", lora=lora)
    assert np.array_equal(one["grad"], step["grad"]) and one["loss"] == step["loss"]
