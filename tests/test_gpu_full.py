"""GPU parity of the full-parameter mode (F16 gradient accumulation, fused SGD,
apply) and of the GRPO accumulation pass, through the C ABI, against the CPU
oracle on the same seeded inputs.

Bars: F16 byte work (apply rule, both weight images, zeroed accumulators,
checkpoint file) bit-exact; accumulated gradients and weight updates within 1e-2
relative per matrix (the GEMM operands are F16 on the device, fp32 in the
oracle); loss within 1e-3."""
import os
import struct
import tempfile

import numpy as np
import pytest

from llm_metal_amd.configs import C1, TINY_GEMMA3
from llm_metal_amd.sft import SFTState
from llm_metal_amd.synth import make_batch, make_model
from oracle import oracle
from tests.gpu_util import rel

pytestmark = pytest.mark.gpu

FULL_Q = C1.with_(name="c1_full", R=0)
FULL_G = TINY_GEMMA3.with_(name="tiny_gemma3_full", NL=3, R=0, seq=40)       # ragged: 40 rows, not a tile multiple
FULL_Q3 = C1.with_(name="c1_full_batch3", R=0, batch=3, seq=32, V=1000, D=192, Hq=3, Hkv=1, IS=416)   # odd tile counts
MATS = ("wq", "wk", "wv", "wo", "wg", "wu", "wd")
GA = {"wq": "gq", "wk": "gk", "wv": "gv", "wo": "go", "wg": "gg", "wu": "gu", "wd": "gd"}


def f16(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)


def all_matrices(cfg):
    for L in range(cfg.NL):
        for k in MATS:
            yield L, k
    yield 0, "lm_head"


def oracle_matrix(cfg, used, L, k):
    return used["lm_head"] if k == "lm_head" else used[k][L]


def oracle_accum(cfg, ga, L, k):
    return f16(ga["glm"] if k == "lm_head" else ga[GA[k]][L])


@pytest.mark.parametrize("cfg", [FULL_Q, FULL_G, FULL_Q3], ids=lambda c: c.name)
def test_accumulate_then_apply(cfg):
    model = make_model(cfg, seed=41, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    ga = oracle.new_grad_accum(used)
    batches = [make_batch(cfg, seed=50 + i) for i in range(2)]
    lr = 0.05
    with SFTState(cfg, model) as st:
        assert st.is_full_param()
        st.alloc_grad_accum()
        for i, (tok, tgt) in enumerate(batches):
            want = oracle.full_param_pass(cfg, used, ga, tok=tok, tgt=tgt)
            loss = st.train_step(tok, tgt, lr)            # accumulators allocated: accumulates, no update
            assert abs(loss - want["loss"]) <= 1e-3 * abs(want["loss"])
            for L, k in all_matrices(cfg):
                g = f16(st.matrix_f16(L, k, 2))
                w = oracle_accum(cfg, ga, L, k)
                assert np.abs(w).max() > 0
                assert rel(g, w) < 1e-2, (i, L, k, rel(g, w))
                # accumulation leaves both weight images alone, bit for bit
                bits = oracle.f32_to_f16_bits(oracle_matrix(cfg, used, L, k))
                assert np.array_equal(st.matrix_f16(L, k, 0), bits), (L, k)
                assert np.array_equal(st.matrix_f16(L, k, 1), bits), (L, k)
        # the apply rule is F16 arithmetic: bit-exact from the device's own G and W
        before = {(L, k): (st.matrix_f16(L, k, 0), st.matrix_f16(L, k, 2)) for L, k in all_matrices(cfg)}
        st.apply_grad_sgd(lr)
        oracle.apply_grad_sgd(cfg, used, ga, lr)
        for L, k in all_matrices(cfg):
            Wb, Gb = before[(L, k)]
            expect = (f16(Wb) - np.float32(lr) * f16(Gb)).astype(np.float16).view(np.uint16)
            got = st.matrix_f16(L, k, 0)
            assert np.array_equal(got, expect), (L, k)
            assert np.array_equal(st.matrix_f16(L, k, 1), expect), (L, k)        # transposed image follows
            assert not st.matrix_f16(L, k, 2).any()                              # G = 0
            d_gpu, d_ref = f16(got) - f16(Wb), oracle_matrix(cfg, used, L, k) - f16(Wb)
            assert rel(d_gpu, d_ref) < 2e-2, (L, k, rel(d_gpu, d_ref))
        # the updated weights are what the next forward multiplies with
        tok, tgt = batches[0]
        want = oracle.full_param_pass(cfg, used, ga, tok=tok, tgt=tgt)
        assert abs(st.train_step(tok, tgt, lr) - want["loss"]) <= 1e-3 * abs(want["loss"])


@pytest.mark.parametrize("cfg", [FULL_Q, FULL_G], ids=lambda c: c.name)
def test_fused_sgd_step_updates_qkv_before_propagating(cfg):
    model = make_model(cfg, seed=43, gamma_jitter=0.1)
    tok, tgt = make_batch(cfg, seed=44)
    lr = 0.2                                              # large, so that the reference's update order is visible
    used0 = oracle.weights_as_used(model)
    ga = oracle.new_grad_accum(used0)
    oracle.full_param_pass(cfg, used0, ga, tok=tok, tgt=tgt)                  # plain gradients (no update in flight)
    used = oracle.weights_as_used(model)
    want = oracle.full_param_pass(cfg, used, None, lr=lr, tok=tok, tgt=tgt)   # fused SGD, updates `used`
    with SFTState(cfg, model) as st:
        loss = st.train_step(tok, tgt, lr)                # no accumulators: sft_backward_sgd(lr)
        assert abs(loss - want["loss"]) <= 1e-3 * abs(want["loss"])
        assert st.step_count() == 0                       # no AdamW step in this mode
        order_seen = 0.0
        for L, k in all_matrices(cfg):
            W0 = oracle_matrix(cfg, used0, L, k)
            d_ref = oracle_matrix(cfg, used, L, k) - W0
            got = st.matrix_f16(L, k, 0)
            assert np.array_equal(st.matrix_f16(L, k, 1), got), (L, k)
            d_gpu = f16(got) - W0
            assert rel(d_gpu, d_ref) < 3e-2, (L, k, rel(d_gpu, d_ref))
            if L == 0 and k != "lm_head":
                order_seen = max(order_seen, rel(-lr * oracle_accum(cfg, ga, L, k), d_ref))
        assert order_seen > 0.2                           # propagating through the OLD W_q/k/v would miss by this much


def _completions(cfg, rng, G, prompt_len, lens):
    prompt = rng.integers(0, cfg.V, prompt_len).astype(np.uint32)
    toks = [rng.integers(0, cfg.V, n).astype(np.uint32) for n in lens]
    rewards = rng.standard_normal(G).astype(np.float32)
    adv = (rewards - rewards.mean()) / (rewards.std() + 1e-8)                  # src/nn/fast_grpo.c:350-365
    return prompt, toks, adv.astype(np.float32)


def _oracle_sequence(cfg, used, prompt, toks_i):
    """[prompt tail | completion | zero rows] as grpo_train_step builds it (src/nn/fast_grpo.c:388-422)."""
    seq = cfg.seq
    comp = min(len(toks_i), seq)
    use = max(0, min(seq - comp, len(prompt)))
    ids = np.concatenate([prompt[len(prompt) - use:], toks_i[:comp]]).astype(np.int64)
    x = np.zeros((seq, cfg.D), dtype=np.float32)
    x[: len(ids)] = used["token_emb"][ids] * np.float32(cfg.emb_scale)
    return x, use, comp


# the last two run the whole group (4 completions) and three of the four per pass: a state built with batch B takes B
# completions per forward / backward, the oracle stays sequential (one F16 rounding of G per completion instead of per pass)
@pytest.mark.parametrize("cfg", [FULL_G.with_(name="grpo_full_gemma", seq=48), FULL_Q.with_(name="grpo_full_qwen", seq=32),
                                 FULL_G.with_(name="grpo_full_gemma_batch4", seq=48, batch=4),
                                 FULL_Q.with_(name="grpo_full_qwen_batch3", seq=32, batch=3)],
                         ids=lambda c: c.name)
def test_grpo_accumulate_and_apply(cfg):
    gpu_cfg, cfg = cfg, cfg.with_(batch=1)                 # the oracle follows one completion at a time
    rng = np.random.default_rng(5)
    G = 4
    prompt, toks, adv = _completions(cfg, rng, G, 12, [cfg.seq - 12, cfg.seq - 20, 5, cfg.seq + 7])   # exact, short, tiny, too long
    model = make_model(cfg, seed=45, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    W0 = {(L, k): oracle_matrix(cfg, used, L, k).copy() for L, k in all_matrices(cfg)}
    # sampling-time log-probabilities: the current policy's, shifted so that some ratios leave the clip band
    old = []
    for t in toks:
        x, use, comp = _oracle_sequence(cfg, used, prompt, t)
        act = np.zeros(cfg.seq, dtype=np.uint32)
        act[use:use + comp] = t[:comp]
        r = oracle.full_param_pass(cfg, used, oracle.new_grad_accum(used), x_rows=x,
                                   grpo=dict(actions=act, old_lp=np.zeros(cfg.seq), advs=np.zeros(cfg.seq), clip_eps=0.2, dl_scale=0.0))
        old.append((r["new_lp"][use:use + comp] + rng.uniform(-0.3, 0.3, comp)).astype(np.float32))
        if len(t) > comp:
            old[-1] = np.concatenate([old[-1], np.zeros(len(t) - comp, dtype=np.float32)])
    lr, clip = 0.05, 0.2
    ga = oracle.new_grad_accum(used)
    want_lp = np.zeros((G, cfg.seq), dtype=np.float32)
    for i, t in enumerate(toks):
        x, use, comp = _oracle_sequence(cfg, used, prompt, t)
        act, olp, advs = np.zeros(cfg.seq, dtype=np.uint32), np.zeros(cfg.seq, dtype=np.float32), np.zeros(cfg.seq, dtype=np.float32)
        act[use:use + comp] = t[:comp]
        olp[use:use + comp] = old[i][:comp]
        advs[use:use + comp] = adv[i]
        r = oracle.full_param_pass(cfg, used, ga, x_rows=x, grpo=dict(actions=act, old_lp=olp, advs=advs, clip_eps=clip, dl_scale=1.0 / G))
        want_lp[i] = r["new_lp"]
    oracle.apply_grad_sgd(cfg, used, ga, lr)
    with SFTState(gpu_cfg, model) as st:
        got_lp = st.grpo_apply_completions(prompt, toks, old, adv, clip, lr, accurate=True)
        for i, t in enumerate(toks):
            _, use, comp = _oracle_sequence(cfg, used, prompt, t)
            assert np.allclose(got_lp[i, use:use + comp], want_lp[i, use:use + comp], atol=2e-3), i
        for L, k in all_matrices(cfg):
            got = st.matrix_f16(L, k, 0)
            assert np.array_equal(st.matrix_f16(L, k, 1), got)
            assert not st.matrix_f16(L, k, 2).any()
            d_gpu, d_ref = f16(got) - W0[(L, k)], oracle_matrix(cfg, used, L, k) - W0[(L, k)]
            assert np.abs(d_ref).max() > 0
            assert rel(d_gpu, d_ref) < 3e-2, (L, k, rel(d_gpu, d_ref))


@pytest.mark.parametrize("batch", [1, 2], ids=["one_per_pass", "two_per_pass"])
def test_grpo_lora_mode_sums_adapter_gradients_then_adamw(batch):
    cfg = C1.with_(name="grpo_lora", seq=32)
    rng = np.random.default_rng(6)
    G = 3
    prompt, toks, adv = _completions(cfg, rng, G, 10, [22, 9, 30])
    model = make_model(cfg, seed=46, gamma_jitter=0.1)
    used = oracle.weights_as_used(model)
    lora = model["lora"].copy()
    old = [rng.uniform(-9.0, -7.0, len(t)).astype(np.float32) for t in toks]          # ~log(1/V): ratios near the band
    lr, clip = 1e-3, 0.2
    acc = np.zeros_like(lora)
    for i, t in enumerate(toks):
        x, use, comp = _oracle_sequence(cfg, used, prompt, t)
        act, olp, advs = np.zeros(cfg.seq, dtype=np.uint32), np.zeros(cfg.seq, dtype=np.float32), np.zeros(cfg.seq, dtype=np.float32)
        act[use:use + comp] = t[:comp]
        olp[use:use + comp] = old[i][:comp]
        advs[use:use + comp] = adv[i]
        r = oracle.full_param_pass(cfg, used, None, x_rows=x, lora=lora,
                                   grpo=dict(actions=act, old_lp=olp, advs=advs, clip_eps=clip, dl_scale=1.0 / G))
        acc += r["grad"]
    with SFTState(cfg.with_(batch=batch), model) as st:
        st.grpo_apply_completions(prompt, toks, old, adv, clip, lr)
        assert st.step_count() == 1
        gn = float(np.sqrt((acc.astype(np.float64) ** 2).sum()))
        assert gn > 0 and abs(st.grad_norm() - gn) <= 1e-2 * gn
        g = st.lora_grads() * max(1.0, gn)                # the update leaves the clipped gradients in place
        assert rel(g, acc) < 1e-2
        m, v = np.zeros_like(lora), np.zeros_like(lora)
        gc = acc.copy()
        oracle.op("f32", "or_clip_grad_norm", gc, oracle.SZ(gc.size), 1.0)
        oracle.op("f32", "or_adamw", lora, gc, m, v, oracle.SZ(lora.size), lr, 0.9, 0.999, 1e-8, 0.01, 1)
        d_gpu, d_ref = st.lora() - model["lora"], lora - model["lora"]
        assert rel(d_gpu, d_ref) < 0.1 and (np.sign(d_gpu) == np.sign(d_ref)).mean() > 0.97


def test_full_checkpoint_file_and_layer_accessors():
    cfg = FULL_Q
    model = make_model(cfg, seed=47)
    used = oracle.weights_as_used(model)
    with SFTState(cfg, model) as st:
        path = os.path.join(tempfile.mkdtemp(), "full.bin")
        st.save_full_checkpoint(path)
        raw = open(path, "rb").read()
        hdr = struct.unpack("<9I", raw[:36])
        assert hdr == (0x46554C4C, cfg.model_type, cfg.NL, cfg.D, cfg.Hq, cfg.Hkv, cfg.hd, cfg.IS, cfg.V)   # src/nn/fast_sft.c:1292-1309
        body = np.frombuffer(raw[36:], dtype=np.uint16)
        off = 0
        for L, k in all_matrices(cfg):
            w = oracle.f32_to_f16_bits(oracle_matrix(cfg, used, L, k)).ravel()
            assert np.array_equal(body[off:off + w.size], w), (L, k)
            off += w.size
        assert off == body.size
        # sft_get_layers / sft_get_lm_head: row-major F16 WMats with the reference's shapes
        from llm_metal_amd.sft import Buf
        layers = st.L.sft_get_layers(st.h)
        lw = layers[1]
        for field, key in (("q_proj", "wq"), ("down_proj", "wd"), ("up_proj", "wu")):
            wm = getattr(lw, field).contents
            assert (wm.rows, wm.cols) == used[key][1].shape and wm.nb == wm.cols // 32
            got = Buf(st.L, wm.mbuf, wm.rows * wm.cols * 2, owned=False).read(np.uint16, (wm.rows, wm.cols))
            assert np.array_equal(got, oracle.f32_to_f16_bits(used[key][1]))
        g = Buf(st.L, lw.q_norm_g, cfg.hd * 4, owned=False).read(np.float32)
        assert np.array_equal(g, model["g_q"][1])
        lm = st.L.sft_get_lm_head(st.h).contents
        got = Buf(st.L, lm.mbuf, lm.rows * lm.cols * 2, owned=False).read(np.uint16, (lm.rows, lm.cols))
        assert np.array_equal(got, oracle.f32_to_f16_bits(used["lm_head"]))
