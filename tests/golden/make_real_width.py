#!/usr/bin/env python3
"""Writes tests/golden/real_width_c4.npz and real_width_c5.npz: what the CPU oracle computes for the two
real-width parity cases it needs minutes for (2048 rows through Qwen3-4B widths on Q8_0 weights; four
full-parameter passes of 160 rows through Gemma3-1B widths).  Imports only the oracle and the seeded synthetic
model generator; run from the repository root:

    python tests/golden/make_real_width.py [c4] [c5]

Every tensor is stored as its norm plus its values at seeded positions (tests/real_width_cases.py: sample_idx).
"""
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from llm_metal_amd.synth import lora_views, make_batch, make_model  # noqa: E402
from oracle import oracle  # noqa: E402
from tests import real_width_cases as rw  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
MATS = ("wq", "wk", "wv", "wo", "wg", "wu", "wd")


def norm(a):
    return float(np.sqrt((np.asarray(a, dtype=np.float64) ** 2).sum()))


def make_c4():
    cfg = rw.C4_WIDTHS
    model = make_model(cfg, seed=rw.MODEL_SEED, gamma_jitter=rw.GAMMA_JITTER)
    used = oracle.weights_as_used(model, "q8")
    tok, tgt = make_batch(cfg, seed=rw.BATCH_SEED)
    lora = model["lora"].copy()
    m, v = np.zeros_like(lora), np.zeros_like(lora)
    t0 = time.time()
    r = oracle.sft_train_step(cfg, used, lora, m, v, 0, tok, tgt, 1e-4, want_logits=True)
    print(f"c4: oracle step {time.time() - t0:.0f} s, loss {r['loss']:.6f}, grad norm {r['grad_norm']:.6f}")
    out = {"fingerprint": rw.weights_fingerprint(model), "loss": r["loss"], "grad_norm": r["grad_norm"],
           "logits_norm": norm(r["logits"]),
           "logits_sample": r["logits"].ravel()[rw.sample_idx("logits", r["logits"].size)].astype(np.float32)}
    for k, g in lora_views(cfg, r["grad"])[0].items():
        out[f"grad_{k}_norm"] = norm(g)
        out[f"grad_{k}_sample"] = g.ravel()[rw.sample_idx("grad_" + k, g.size)]
    after, before = lora_views(cfg, lora)[0], lora_views(cfg, model["lora"])[0]
    for k in after:                                       # what one AdamW step moved
        d = after[k] - before[k]
        out[f"delta_{k}_norm"] = norm(d)
        out[f"delta_{k}_sample"] = d.ravel()[rw.sample_idx("delta_" + k, d.size)]
    np.savez_compressed(os.path.join(HERE, "real_width_c4.npz"), **out)


def make_c5():
    cfg = rw.C5_WIDTHS
    model = make_model(cfg, seed=rw.MODEL_SEED, gamma_jitter=rw.GAMMA_JITTER)
    used = oracle.weights_as_used(model)
    W0 = {(L, k): used[k][L].copy() for L in range(cfg.NL) for k in MATS}
    W0[(0, "lm_head")] = used["lm_head"].copy()
    prompt, toks, adv, shift = rw.c5_completions(cfg)
    G = len(toks)
    t0 = time.time()
    old = []
    for t, sh in zip(toks, shift):                        # sampling-time log-probabilities: the policy's own, shifted
        x, use, comp = rw.c5_sequence(cfg, used, prompt, t)
        act = np.zeros(cfg.seq, dtype=np.uint32)
        act[use:use + comp] = t[:comp]
        r = oracle.full_param_pass(cfg, used, oracle.new_grad_accum(used), x_rows=x,
                                   grpo=dict(actions=act, old_lp=np.zeros(cfg.seq), advs=np.zeros(cfg.seq), clip_eps=rw.C5_CLIP, dl_scale=0.0))
        old.append((r["new_lp"][use:use + comp] + sh[:comp]).astype(np.float32))
    ga = oracle.new_grad_accum(used)
    new_lp = np.zeros((G, cfg.seq), dtype=np.float32)
    for i, t in enumerate(toks):
        x, use, comp = rw.c5_sequence(cfg, used, prompt, t)
        act, olp, advs = np.zeros(cfg.seq, dtype=np.uint32), np.zeros(cfg.seq, dtype=np.float32), np.zeros(cfg.seq, dtype=np.float32)
        act[use:use + comp] = t[:comp]
        olp[use:use + comp] = old[i][:comp]
        advs[use:use + comp] = adv[i]
        r = oracle.full_param_pass(cfg, used, ga, x_rows=x,
                                   grpo=dict(actions=act, old_lp=olp, advs=advs, clip_eps=rw.C5_CLIP, dl_scale=1.0 / G))
        new_lp[i] = r["new_lp"]
    oracle.apply_grad_sgd(cfg, used, ga, rw.C5_LR)
    print(f"c5: oracle passes {time.time() - t0:.0f} s")
    out = {"fingerprint": rw.weights_fingerprint(model), "new_lp": new_lp}
    for i in range(G):
        out[f"old_lp_{i}"] = old[i]
    for (L, k), w0 in W0.items():
        d = (used["lm_head"] if k == "lm_head" else used[k][L]) - w0
        out[f"delta_{L}_{k}_norm"] = norm(d)
        out[f"delta_{L}_{k}_sample"] = d.ravel()[rw.sample_idx(f"delta_{L}_{k}", d.size)]
    np.savez_compressed(os.path.join(HERE, "real_width_c5.npz"), **out)


if __name__ == "__main__":
    which = sys.argv[1:] or ["c4", "c5"]
    oracle.build()
    if "c5" in which:
        make_c5()
    if "c4" in which:
        make_c4()
