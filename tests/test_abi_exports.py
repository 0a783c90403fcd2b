"""CPU-side checks of the C-ABI library: it loads, exports every function that
include/*.h declares, and refuses to start without a GPU (no compute calls here)."""
import os

import pytest

from llm_metal_amd import lib


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(lib.LIB_PATH):
        lib.build()
    return lib.load()


def test_every_declared_symbol_is_exported(L):
    decl = lib.declared_symbols()
    assert len(decl) >= 90
    missing = [n for n in decl if not hasattr(L, n)]
    assert not missing, missing


def test_reference_abi_names_present(L):
    # all 49 symbols of src/nn/fast_metal.h: the 33 the LoRA SFT step uses, the 4 of the full-parameter / GRPO
    # path, and the 12 inference enqueues (+ 4 offset variants counted among them)
    names = """fast_metal_init fast_metal_shutdown metal_buf_create metal_buf_from_data metal_buf_free metal_buf_ptr
    metal_flush metal_enqueue_rms_norm_batched metal_enqueue_silu_mul metal_enqueue_gelu_mul metal_enqueue_residual_add
    metal_enqueue_f16_matmul metal_enqueue_f16_matmul_nt metal_enqueue_transpose_heads_fwd
    metal_enqueue_transpose_heads_rev metal_enqueue_repeat_kv metal_enqueue_rope_train metal_enqueue_silu_mul_backward
    metal_enqueue_gelu_mul_backward metal_enqueue_rms_norm_backward metal_enqueue_scale metal_enqueue_add_scaled
    metal_enqueue_softmax_ce metal_enqueue_attn_train_fwd metal_enqueue_attn_bwd_dq metal_enqueue_attn_bwd_dkv
    metal_enqueue_repeat_kv_bwd metal_enqueue_rope_train_bwd metal_enqueue_float_matmul metal_enqueue_float_matmul_tn
    metal_enqueue_float_matmul_nt metal_enqueue_copy metal_enqueue_clamp metal_enqueue_f16_sgd_fused
    metal_enqueue_grpo_policy_grad metal_enqueue_f16_grad_accum metal_enqueue_f16_sgd_apply
    metal_enqueue_q8_matvec metal_enqueue_f16_matvec metal_enqueue_f16_batch_matvec metal_enqueue_rms_norm
    metal_enqueue_per_head_rms_norm metal_enqueue_rope metal_enqueue_kv_cache_store metal_enqueue_attention
    metal_enqueue_per_head_rms_norm_off metal_enqueue_rope_off metal_enqueue_kv_cache_store_off
    metal_enqueue_attention_off""".split()
    assert len(names) == 49
    for n in names:
        assert hasattr(L, n), n


def test_init_fails_loudly_without_a_gpu(L):
    import torch
    if torch.cuda.device_count() > 0:
        pytest.skip("a GPU is present")
    assert L.fast_metal_init() == -1
    assert not L.metal_buf_create(16)          # refused before init, returns NULL
