"""Pins the oracle's whole-step functions (forward, CE, backward, clip, AdamW).

The reference holds no golden vectors for this path, so the pins are:
  * a torch fp64 model assembled from library routines whose backward is
    autograd (catches a dropped term, wrong sign/index or transposed operand in
    any hand-written backward op, and a wrong op order in the Gemma3 block);
  * torch.optim.AdamW for the update rule;
  * central finite differences of the oracle's own loss;
  * structural properties (causality, zero-B equivalence).
"""
import numpy as np
import pytest

from llm_metal_amd.configs import C1, TINY_GEMMA3
from llm_metal_amd.synth import make_batch, make_model
from oracle import oracle
from tests import torch_ref

SMALL_Q = C1.with_(name="small_q", NL=2, D=64, Hq=4, Hkv=2, hd=16, IS=96, V=160, seq=12, batch=2, R=4, alpha=8.0)
SMALL_G = TINY_GEMMA3.with_(name="small_g", NL=7, D=48, Hq=4, Hkv=1, hd=16, IS=80, V=128, seq=10, batch=2, R=4,
                            alpha=8.0)


def _rel(a, b):
    return float(np.linalg.norm(np.asarray(a, dtype=np.float64) - b) / (np.linalg.norm(b) + 1e-300))


# sliding-window attention (an option the reference stores and never applies): the torch model masks with
# F.scaled_dot_product_attention(attn_mask=...), windows shorter than the sequence, local and global Gemma3 layers
WINDOW_Q = SMALL_Q.with_(name="small_q_window5", window=5)
WINDOW_G = SMALL_G.with_(name="small_g_window4", window=4)


@pytest.mark.parametrize("cfg", [SMALL_Q, SMALL_G, WINDOW_Q, WINDOW_G], ids=lambda c: c.name)
def test_f64_step_matches_torch_autograd_and_adamw(cfg):
    model = make_model(cfg, seed=3, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    batches = [make_batch(cfg, seed=10 + i) for i in range(3)]
    lr = 1e-2
    ref = torch_ref.train_steps(cfg, used, model["lora"], batches, lr)
    lora = model["lora"].astype(np.float64)
    m, v, step = np.zeros_like(lora), np.zeros_like(lora), 0
    for i, (tok, tgt) in enumerate(batches):
        raw = oracle.sft_train_step(cfg, used, lora.copy(), m.copy(), v.copy(), step, tok, tgt, lr,
                                    do_update=False, precision="f64", want_logits=True)
        tol = 1e-8 if i == 0 else 1e-7       # float eps constant; later steps inherit the float-constant AdamW difference
        assert abs(raw["loss"] - ref[i]["loss"]) < tol * abs(ref[i]["loss"])
        assert _rel(raw["logits"], ref[i]["logits"]) < tol
        # the oracle keeps the reference's float constants (1/BN, eps, 1/sqrt(hd)): 2^-24 relative
        assert _rel(raw["grad"], ref[i]["grad"]) < 2e-7
        assert abs(raw["grad_norm"] - ref[i]["grad_norm"]) < 2e-7 * ref[i]["grad_norm"]
        out = oracle.sft_train_step(cfg, used, lora, m, v, step, tok, tgt, lr, precision="f64")
        step = out["step"]
        assert step == i + 1
        # powf/float constants in the oracle vs double in torch: agreement to ~1e-7 relative
        assert _rel(lora, ref[i]["lora"]) < 1e-6
    # every LoRA tensor must have moved (non-zero B makes dA non-zero)
    assert np.all(np.abs(lora - model["lora"]) > 0)


@pytest.mark.parametrize("cfg", [SMALL_Q, SMALL_G], ids=lambda c: c.name)
def test_f32_build_tracks_f64(cfg):
    model = make_model(cfg, seed=4, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    tok, tgt = make_batch(cfg, seed=5)
    out = {}
    for prec in ("f32", "f64"):
        dt = oracle.real_dtype(prec)
        lora = model["lora"].astype(dt)
        m, v = np.zeros_like(lora), np.zeros_like(lora)
        out[prec] = oracle.sft_train_step(cfg, used, lora, m, v, 0, tok, tgt, 1e-3, precision=prec)
        out[prec]["lora"] = lora
    assert abs(out["f32"]["loss"] - out["f64"]["loss"]) < 1e-5 * out["f64"]["loss"]
    assert _rel(out["f32"]["grad"], out["f64"]["grad"]) < 1e-4
    assert _rel(out["f32"]["lora"], out["f64"]["lora"]) < 1e-5


def test_finite_differences_of_oracle_loss():
    cfg = SMALL_Q
    model = make_model(cfg, seed=6, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    tok, tgt = make_batch(cfg, seed=7)
    lora = model["lora"].astype(np.float64)
    z = np.zeros_like(lora)
    g = oracle.sft_train_step(cfg, used, lora.copy(), z.copy(), z.copy(), 0, tok, tgt, 0.0,
                              do_update=False, precision="f64")["grad"]
    rng = np.random.default_rng(0)
    for _ in range(4):
        u = rng.standard_normal(lora.size)
        u /= np.linalg.norm(u)
        h = 1e-5
        fd = (oracle.sft_loss(cfg, used, lora + h * u, tok, tgt, "f64")
              - oracle.sft_loss(cfg, used, lora - h * u, tok, tgt, "f64")) / (2 * h)
        assert abs(fd - g @ u) < 1e-6 * max(1e-3, abs(fd))


def test_zero_b_is_base_model_and_da_is_zero():
    cfg = SMALL_Q
    model = make_model(cfg, seed=8, lora_b_std=0.0)
    used = oracle.weights_as_used(model)
    tok, tgt = make_batch(cfg, seed=9)
    lora = model["lora"].astype(np.float64)
    z = np.zeros_like(lora)
    out = oracle.sft_train_step(cfg, used, lora.copy(), z.copy(), z.copy(), 0, tok, tgt, 0.0,
                                do_update=False, precision="f64")
    base = oracle.sft_loss(cfg.with_(R=0), used, np.zeros(0), tok, tgt, "f64")
    assert abs(out["loss"] - base) < 1e-13
    from llm_metal_amd.synth import lora_views
    for lv in lora_views(cfg, out["grad"]):
        assert np.all(lv["A_q"] == 0) and np.all(lv["A_v"] == 0)
        assert np.any(lv["B_q"] != 0) and np.any(lv["B_v"] != 0)


def test_causality_and_per_sequence_positions():
    cfg = SMALL_Q
    model = make_model(cfg, seed=11)
    used = oracle.weights_as_used(model)
    tok, tgt = make_batch(cfg, seed=12)
    _, lg = oracle.sft_loss(cfg, used, model["lora"].astype(np.float64), tok, tgt, "f64", want_logits=True)
    # changing the last token of each sequence leaves all earlier rows untouched
    tok2 = tok.copy().reshape(cfg.batch, cfg.seq)
    tok2[:, -1] = (tok2[:, -1] + 1) % cfg.V
    _, lg2 = oracle.sft_loss(cfg, used, model["lora"].astype(np.float64), tok2.reshape(-1), tgt, "f64",
                             want_logits=True)
    lg, lg2 = lg.reshape(cfg.batch, cfg.seq, -1), lg2.reshape(cfg.batch, cfg.seq, -1)
    assert np.array_equal(lg[:, :-1], lg2[:, :-1]) and not np.allclose(lg[:, -1], lg2[:, -1])
    # a batch of two equal sequences gives two equal row blocks (positions restart per sequence)
    tok3 = np.concatenate([tok[:cfg.seq], tok[:cfg.seq]])
    _, lg3 = oracle.sft_loss(cfg, used, model["lora"].astype(np.float64), tok3, tgt, "f64", want_logits=True)
    assert np.array_equal(lg3[:cfg.seq], lg3[cfg.seq:])


def test_c1_f32_step_runs_in_seconds():
    model = make_model(C1, seed=0)
    used = oracle.weights_as_used(model)
    tok, tgt = make_batch(C1, seed=1)
    lora = model["lora"].copy()
    m, v = np.zeros_like(lora), np.zeros_like(lora)
    out = oracle.sft_train_step(C1, used, lora, m, v, 0, tok, tgt, 1e-4)
    assert abs(out["loss"] - np.log(C1.V)) < 0.2      # random init: loss ~ ln V
    assert out["step"] == 1 and np.isfinite(out["grad"]).all()


def test_window_changes_the_result_and_a_long_window_does_not():
    """The option is live (a short window moves loss and gradients) and a window that covers the whole sequence is the
    unwindowed step bit for bit."""
    cfg = SMALL_Q
    model = make_model(cfg, seed=8, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    tok, tgt = make_batch(cfg, seed=9)

    def run(c):
        lora = model["lora"].copy()
        z = np.zeros_like(lora)
        return oracle.sft_train_step(c, used, lora, z, z.copy(), 0, tok, tgt, 1e-3, do_update=False)
    base, wide, short = run(cfg), run(cfg.with_(window=cfg.seq)), run(cfg.with_(window=3))
    assert base["loss"] == wide["loss"] and np.array_equal(base["grad"], wide["grad"])
    assert abs(short["loss"] - base["loss"]) > 1e-6 and _rel(short["grad"], base["grad"]) > 1e-3
