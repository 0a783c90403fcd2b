"""Workload shapes of the fused LoRA SFT step (the five benchmark configurations).

Field names follow the reference's SFTState dims (src/nn/fast_sft.c:33-44):
NL layers, D hidden, Hq/Hkv heads, hd head dim, IS FFN width, V vocab.
"""
from dataclasses import dataclass, replace

QWEN3, GEMMA3 = 0, 1


@dataclass(frozen=True)
class SFTConfig:
    name: str
    model_type: int          # QWEN3 | GEMMA3
    NL: int
    D: int
    Hq: int
    Hkv: int
    hd: int
    IS: int
    V: int
    batch: int = 1
    seq: int = 64
    R: int = 16              # LoRA rank
    alpha: float = 32.0
    eps: float = 1e-6        # src/nn/fast_sft.c:190
    rope_theta: float = 1e6  # Qwen3: every layer; Gemma3: global layers (L % 6 == 0)
    local_rope_theta: float = 1e4   # Gemma3 local layers (src/nn/fast_sft.c:310-313)
    tied: bool = False       # lm_head shares the embedding table
    weight_format: str = "f16"      # "f16" | "q8_0"
    window: int = 0          # sliding-window attention on the local layers (0 = off: the reference never applies it)

    @property
    def BN(self):
        return self.batch * self.seq

    @property
    def lora_scaling(self):
        return self.alpha / self.R

    @property
    def emb_scale(self):
        import numpy as np
        return float(np.sqrt(np.float32(self.D))) if self.model_type == GEMMA3 else 1.0

    def rope_thetas(self):
        if self.model_type == GEMMA3:
            return [self.rope_theta if (L % 6) == 0 else self.local_rope_theta for L in range(self.NL)]
        return [self.rope_theta] * self.NL

    def local_layers(self):
        """Layers the sliding window applies to: Gemma3's pattern (src/nn/gemma3.c:49-57), every layer otherwise."""
        return [(L % 6) != 0 if self.model_type == GEMMA3 else True for L in range(self.NL)]

    @property
    def lora_layer_size(self):
        return 2 * self.R * self.D + self.Hq * self.hd * self.R + self.Hkv * self.hd * self.R

    @property
    def frozen_params(self):
        per = (self.Hq * self.hd + 2 * self.Hkv * self.hd) * self.D + self.D * self.Hq * self.hd + 3 * self.IS * self.D
        return per * self.NL + self.V * self.D

    def with_(self, **kw):
        return replace(self, **kw)


C1 = SFTConfig("c1_tiny_qwen3", QWEN3, NL=2, D=256, Hq=4, Hkv=2, hd=64, IS=768, V=4096, tied=True)
C2 = SFTConfig("c2_gemma3_1b", GEMMA3, NL=26, D=1152, Hq=4, Hkv=1, hd=256, IS=6912, V=262144, tied=True)
C3 = SFTConfig("c3_qwen3_4b_f16", QWEN3, NL=36, D=2560, Hq=32, Hkv=8, hd=128, IS=9728, V=151936)
C4 = C3.with_(name="c4_qwen3_4b_q8", batch=4, seq=512, weight_format="q8_0")
# the group of four 160-token sequences is one batch: a pass streams every weight once for the whole group
C5 = C2.with_(name="c5_gemma3_1b_grpo", batch=4, seq=160, R=0)
# config 3's step on Q8_0 weights: the dequant-fused weight-streaming GEMM at M = 64
C3Q = C3.with_(name="c3_qwen3_4b_q8_seq64", weight_format="q8_0")

# small Gemma3-shaped case for parity tests (4-norm ordering, GeGLU, tied head, mixed thetas)
TINY_GEMMA3 = SFTConfig("tiny_gemma3", GEMMA3, NL=7, D=128, Hq=4, Hkv=1, hd=32, IS=384, V=2048, tied=True, seq=32)

CONFIGS = {c.name: c for c in (C1, C2, C3, C4, C5, C3Q, TINY_GEMMA3)}
