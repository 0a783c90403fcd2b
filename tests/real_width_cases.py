"""Parity cases at the widths of the benchmarked configurations (few layers, truncated vocabulary), shared by
the GPU tests and by tests/golden/make_real_width.py, which writes the expected values of the two cases that are
too slow for the CPU oracle to follow inside a GPU test run.

Config 3's widths (hidden 2560, 32 / 8 heads of 128, FFN 9728) and config 2's (hidden 1152, 4 / 1 heads of 256,
FFN 6912) are the ones the benchmark launches: the GEMM grids, the row kernels' register widths, the attention
tile shapes and the GLU column groups depend on them and on nothing that the layer count or the vocabulary changes.
"""
import numpy as np

from llm_metal_amd.configs import C2, C3

V_CUT = 8192

# Qwen3-4B widths, one layer, 64 rows, F16 (config 3)
C3_WIDTHS = C3.with_(name="c3_widths", NL=1, V=V_CUT)
# the same with Q8_0 weights (config 3's Q8_0 variant): the tiles stay quantised up to LDS in every product
C3Q_WIDTHS = C3.with_(name="c3q_widths", NL=1, V=V_CUT, weight_format="q8_0")
# Gemma3-1B widths, two layers (layer 0 global theta, layer 1 local), 64 rows, tied head (config 2)
C2_WIDTHS = C2.with_(name="c2_widths", NL=2, V=V_CUT)
# Qwen3-4B widths, Q8_0 weights, 4 x 512 rows (config 4): every product takes the large-M path
C4_WIDTHS = C3.with_(name="c4_widths", NL=1, V=V_CUT, batch=4, seq=512, weight_format="q8_0")
# Gemma3-1B widths, full-parameter, 160 rows, through the GRPO accumulate-and-apply entry point (config 5)
C5_WIDTHS = C2.with_(name="c5_widths", NL=2, V=V_CUT, R=0, seq=160)

MODEL_SEED, BATCH_SEED, GAMMA_JITTER = 21, 30, 0.1
C5_LR, C5_CLIP, C5_PROMPT = 0.05, 0.2, 32
C5_LENGTHS = (128, 100)                                   # one completion fills the sequence, one leaves zero rows
SAMPLE = 4096


def sample_idx(name, n, k=SAMPLE):
    """Seeded positions at which a tensor of n elements is compared (all of them when it is small)."""
    if n <= k:
        return np.arange(n)
    seed = int.from_bytes(name.encode()[:8].ljust(8, b"\0"), "little") % (2 ** 32)
    return np.sort(np.random.default_rng(seed).choice(n, size=k, replace=False))


def weights_fingerprint(model):
    """Detects a synthetic model that differs from the one the fixture was made from."""
    parts = [model["wq"][0].ravel()[:1024], model["wd"][-1].ravel()[-1024:], model["token_emb"].ravel()[:1024],
             model["lora"][:1024] if model["lora"].size else np.zeros(1, np.float32)]
    return np.concatenate(parts).astype(np.float64).sum()


def c5_completions(cfg):
    rng = np.random.default_rng(5)
    G = len(C5_LENGTHS)
    prompt = rng.integers(0, cfg.V, C5_PROMPT).astype(np.uint32)
    toks = [rng.integers(0, cfg.V, n).astype(np.uint32) for n in C5_LENGTHS]
    rewards = rng.standard_normal(G).astype(np.float32)
    adv = ((rewards - rewards.mean()) / (rewards.std() + 1e-8)).astype(np.float32)     # src/nn/fast_grpo.c:350-365
    shift = [rng.uniform(-0.3, 0.3, n).astype(np.float32) for n in C5_LENGTHS]         # moves some ratios out of the clip band
    return prompt, toks, adv, shift


def c5_sequence(cfg, used, prompt, toks_i):
    """[prompt tail | completion | zero rows] as grpo_train_step builds it (src/nn/fast_grpo.c:388-422)."""
    seq = cfg.seq
    comp = min(len(toks_i), seq)
    use = max(0, min(seq - comp, len(prompt)))
    ids = np.concatenate([prompt[len(prompt) - use:], toks_i[:comp]]).astype(np.int64)
    x = np.zeros((seq, cfg.D), dtype=np.float32)
    x[: len(ids)] = used["token_emb"][ids] * np.float32(cfg.emb_scale)
    return x, use, comp
