"""MI355X-native fused LoRA SFT step of llm.metal (HIP kernels behind a C ABI).

Python here is only a thin ctypes mirror of the C host API (include/sft_hip.h,
include/fast_hip.h) for tests and benchmarks; all compute is in
libllm_metal_hip.so.  Importing the package does not load the library;
`lib.load()` does and raises if it has not been built.
"""
from .configs import CONFIGS, SFTConfig  # noqa: F401
