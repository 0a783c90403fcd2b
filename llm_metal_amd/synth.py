"""Seeded synthetic models and batches for the SFT step.

Weights ~ N(0, 0.02), norm gammas = 1 (rms_norm_create, src/nn/layers.c:336-344),
LoRA A ~ U(-1, 1)/sqrt(D) (src/nn/fast_sft.c:100-104), B = 0 for timing runs or
N(0, 0.01) for parity runs (a zero B makes the first-step dA exactly zero),
tokens uniform on [0, V), target = next token with the last wrapping to the
first (main.c:471-477).
"""
import os

import numpy as np
from .configs import SFTConfig, GEMMA3

MATS = ("wq", "wk", "wv", "wo", "wg", "wu", "wd")


def mat_shapes(c: SFTConfig):
    qd, kd = c.Hq * c.hd, c.Hkv * c.hd
    return {"wq": (qd, c.D), "wk": (kd, c.D), "wv": (kd, c.D), "wo": (c.D, qd),
            "wg": (c.IS, c.D), "wu": (c.IS, c.D), "wd": (c.D, c.IS)}


def _normal(rng, shape, std):
    a = rng.standard_normal(shape, dtype=np.float32)
    a *= np.float32(std)
    return a


def make_model(c: SFTConfig, seed=0, gamma_jitter=0.0, lora_b_std=0.01, threads=None):
    """Returns a dict of fp32 numpy arrays: per-layer lists for the 7 matrices and
    the norm gammas, token_emb, lm_head (same object when tied), g_final, lora
    (flat [NL * lora_layer_size]: A_q | B_q | A_v | B_v per layer).  Every array has
    its own generator derived from (seed, index), so the result does not depend on
    how many threads filled it."""
    from concurrent.futures import ThreadPoolExecutor
    shp = mat_shapes(c)
    m = {k: [None] * c.NL for k in MATS}
    jobs = []                                              # (dict, key/index, shape)
    for L in range(c.NL):
        for k in MATS:
            jobs.append((m[k], L, shp[k]))
    m["token_emb"] = None
    jobs.append((m, "token_emb", (c.V, c.D)))
    if not c.tied:
        jobs.append((m, "lm_head", (c.V, c.D)))
    seqs = np.random.SeedSequence(seed).spawn(len(jobs) + 2)

    def fill(i):
        dst, key, shape = jobs[i]
        dst[key] = _normal(np.random.default_rng(seqs[i]), shape, 0.02)

    big = sum(int(np.prod(j[2])) for j in jobs) > 50_000_000
    if big:
        with ThreadPoolExecutor(threads or min(16, (os.cpu_count() or 8))) as ex:
            list(ex.map(fill, range(len(jobs))))
    else:
        for i in range(len(jobs)):
            fill(i)
    if c.tied:
        m["lm_head"] = m["token_emb"]

    rng = np.random.default_rng(seqs[-2])

    def gamma(n):
        g = np.ones(n, dtype=np.float32)
        if gamma_jitter:
            g += _normal(rng, n, gamma_jitter)
        return g

    for k in ("g_in", "g_post_attn", "g_pre_ff", "g_post_ff", "g_q", "g_k"):
        m[k] = []
    for _ in range(c.NL):
        m["g_in"].append(gamma(c.D))
        m["g_post_attn"].append(gamma(c.D))
        m["g_pre_ff"].append(gamma(c.D) if c.model_type == GEMMA3 else None)
        m["g_post_ff"].append(gamma(c.D) if c.model_type == GEMMA3 else None)
        m["g_q"].append(gamma(c.hd))
        m["g_k"].append(gamma(c.hd))
    m["g_final"] = gamma(c.D)
    m["lora"] = make_lora(c, np.random.default_rng(seqs[-1]), lora_b_std)
    return m


def make_lora(c: SFTConfig, rng, lora_b_std):
    if c.R == 0:
        return np.zeros(0, dtype=np.float32)
    qd, kd = c.Hq * c.hd, c.Hkv * c.hd
    parts = []
    for _ in range(c.NL):
        for rows, cols, is_a in ((c.R, c.D, True), (qd, c.R, False), (c.R, c.D, True), (kd, c.R, False)):
            if is_a:
                a = (rng.random((rows, cols), dtype=np.float32) * 2 - 1) / np.float32(np.sqrt(c.D))
            elif lora_b_std:
                a = _normal(rng, (rows, cols), lora_b_std)
            else:
                a = np.zeros((rows, cols), dtype=np.float32)
            parts.append(a.astype(np.float32).ravel())
    return np.concatenate(parts)


def lora_views(c: SFTConfig, flat):
    """Split a flat LoRA arena into per-layer dicts of (A_q, B_q, A_v, B_v) views."""
    qd, kd = c.Hq * c.hd, c.Hkv * c.hd
    out, o = [], 0
    for _ in range(c.NL):
        d = {}
        for name, (r, k) in (("A_q", (c.R, c.D)), ("B_q", (qd, c.R)), ("A_v", (c.R, c.D)), ("B_v", (kd, c.R))):
            d[name] = flat[o:o + r * k].reshape(r, k)
            o += r * k
        out.append(d)
    return out


def make_batch(c: SFTConfig, seed=1):
    rng = np.random.default_rng(seed)
    tok = rng.integers(0, c.V, size=(c.batch, c.seq), dtype=np.uint32)
    tgt = np.roll(tok, -1, axis=1)
    return tok.reshape(-1).copy(), tgt.reshape(-1).copy()
