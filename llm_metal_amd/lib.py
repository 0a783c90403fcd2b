"""ctypes binding of libllm_metal_hip.so (the C ABI of include/fast_hip.h and
include/sft_hip.h).  There is no fallback: a missing library or a failed
fast_metal_init raises."""
import ctypes as C
import os
import re
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libllm_metal_hip.so")
_lib = None


def build(jobs=8):
    """Compile every HIP source for gfx950 into libllm_metal_hip.so (always recompiles)."""
    csrc = os.path.join(_HERE, "csrc")
    subprocess.check_call(["make", "-C", csrc, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", csrc, f"-j{jobs}"], stdout=subprocess.DEVNULL)
    return LIB_PATH


def declared_symbols():
    """Function names declared in include/*.h (used to check the exports)."""
    names = []
    inc = os.path.join(os.path.dirname(_HERE), "include")
    for fn in sorted(os.listdir(inc)):
        if not fn.endswith(".h"):
            continue
        text = open(os.path.join(inc, fn)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        for m in re.finditer(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{]*\)\s*;", text):
            names.append(m.group(1))
    return sorted(set(names))


class WeightRef(C.Structure):
    _fields_ = [("data", C.c_void_p), ("rows", C.c_int), ("cols", C.c_int)]


class LayerWeightRef(C.Structure):
    _fields_ = [(k, WeightRef) for k in ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")] + \
               [(k, C.c_void_p) for k in ("input_norm_g", "post_attn_norm_g", "pre_ff_norm_g", "post_ff_norm_g",
                                          "q_norm_g", "k_norm_g")] + \
               [("d_model", C.c_int), ("head_dim", C.c_int)]


class SFTModelRef(C.Structure):
    _fields_ = [("model_type", C.c_int)] + \
               [(k, C.c_int) for k in ("n_layers", "d_model", "n_q_heads", "n_kv_heads", "head_dim",
                                       "intermediate_size", "vocab_size")] + \
               [("rope_thetas", C.c_void_p), ("layers", C.POINTER(LayerWeightRef)), ("token_emb", C.c_void_p),
                ("lm_head", C.c_void_p), ("final_norm_g", C.c_void_p), ("lora_init", C.c_void_p)]


class WMat(C.Structure):
    _fields_ = [("mbuf", C.c_void_p), ("rows", C.c_int), ("cols", C.c_int), ("nb", C.c_int)]


class LayerW(C.Structure):
    _fields_ = [(k, C.POINTER(WMat)) for k in ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")] + \
               [(k, C.c_void_p) for k in ("input_norm_g", "post_attn_norm_g", "pre_ff_norm_g", "post_ff_norm_g",
                                          "q_norm_g", "k_norm_g")]


class GRPOCompletions(C.Structure):
    _fields_ = [("prompt", C.c_void_p), ("prompt_len", C.c_int), ("group_size", C.c_int),
                ("gen_tokens", C.POINTER(C.c_void_p)), ("gen_lengths", C.c_void_p),
                ("gen_logprobs", C.POINTER(C.c_void_p)), ("advantages", C.c_void_p),
                ("clip_eps", C.c_float), ("accurate", C.c_int)]


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is not built: run `python -c 'import __graft_entry__ as g; g.build()'`")
    L = C.CDLL(LIB_PATH)
    vp, i, f, sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t
    sig = {
        "fast_metal_init": (i, []), "fast_metal_shutdown": (None, []), "metal_flush": (None, []),
        "metal_buf_create": (vp, [sz]), "metal_buf_from_data": (vp, [vp, sz]), "metal_buf_free": (None, [vp]),
        "metal_buf_ptr": (vp, [vp]), "metal_buf_read": (None, [vp, sz, vp, sz]), "metal_buf_write": (None, [vp, sz, vp, sz]),
        "metal_buf_size": (sz, [vp]), "metal_buf_view": (vp, [vp, sz, sz]), "hip_buf_device_ptr": (vp, [vp]),
        "hip_attention_noalloc": (i, [vp, vp, vp, vp, i, i, i, i, i]),
        "metal_enqueue_rms_norm_batched": (None, [vp, vp, vp, i, f, i]),
        "metal_enqueue_silu_mul": (None, [vp, vp, i]), "metal_enqueue_gelu_mul": (None, [vp, vp, i]),
        "metal_enqueue_residual_add": (None, [vp, vp, i]),
        "metal_enqueue_q8_matvec": (None, [vp, vp, vp, i, i]), "metal_enqueue_f16_matvec": (None, [vp, vp, vp, i, i]),
        "metal_enqueue_f16_batch_matvec": (None, [vp, vp, vp, i, i, i]), "metal_enqueue_rms_norm": (None, [vp, vp, vp, i, f]),
        "metal_enqueue_per_head_rms_norm": (None, [vp, vp, i, i, f]), "metal_enqueue_rope": (None, [vp, vp, i, i, i, i, f]),
        "metal_enqueue_kv_cache_store": (None, [vp, vp, vp, vp, i, i, i, i]),
        "metal_enqueue_attention": (None, [vp, vp, vp, vp, i, i, i, i, i]),
        "metal_enqueue_per_head_rms_norm_off": (None, [vp, sz, vp, i, i, f]),
        "metal_enqueue_rope_off": (None, [vp, sz, vp, sz, i, i, i, i, f]),
        "metal_enqueue_kv_cache_store_off": (None, [vp, sz, vp, sz, vp, vp, i, i, i, i]),
        "metal_enqueue_attention_off": (None, [vp, sz, vp, vp, vp, sz, i, i, i, i, i]),
        "metal_enqueue_f16_matmul": (None, [vp, vp, vp, i, i, i]), "metal_enqueue_f16_matmul_nt": (None, [vp, vp, vp, i, i, i]),
        "metal_enqueue_transpose_heads_fwd": (None, [vp, vp, i, i, i]), "metal_enqueue_transpose_heads_rev": (None, [vp, vp, i, i, i]),
        "metal_enqueue_repeat_kv": (None, [vp, vp, i, i, i, i]), "metal_enqueue_repeat_kv_bwd": (None, [vp, vp, i, i, i, i]),
        "metal_enqueue_rope_train": (None, [vp, vp, i, i, i, i, f]), "metal_enqueue_rope_train_bwd": (None, [vp, vp, i, i, i, i, f]),
        "metal_enqueue_silu_mul_backward": (None, [vp, vp, vp, vp, vp, i]),
        "metal_enqueue_gelu_mul_backward": (None, [vp, vp, vp, vp, vp, i]),
        "metal_enqueue_rms_norm_backward": (None, [vp, vp, vp, vp, i, i, f]),
        "metal_enqueue_scale": (None, [vp, f, i]), "metal_enqueue_add_scaled": (None, [vp, vp, f, i]),
        "metal_enqueue_softmax_ce": (None, [vp, vp, vp, vp, i, i]),
        "metal_enqueue_attn_train_fwd": (None, [vp, vp, vp, vp, vp, i, i, i, f]),
        "metal_enqueue_attn_bwd_dq": (None, [vp, vp, vp, vp, vp, vp, i, i, i, f]),
        "metal_enqueue_attn_bwd_dkv": (None, [vp, vp, vp, vp, vp, vp, i, i, i]),
        "metal_enqueue_float_matmul": (None, [vp, vp, vp, i, i, i]), "metal_enqueue_float_matmul_tn": (None, [vp, vp, vp, i, i, i]),
        "metal_enqueue_float_matmul_nt": (None, [vp, vp, vp, i, i, i]),
        "metal_enqueue_copy": (None, [vp, vp, i]), "metal_enqueue_clamp": (None, [vp, f, i]),
        "metal_enqueue_f16_sgd_fused": (None, [vp, vp, vp, i, i, i, f]),
        "metal_enqueue_grpo_policy_grad": (None, [vp, vp, vp, vp, vp, vp, i, i, f]),
        "metal_enqueue_f16_grad_accum": (None, [vp, vp, vp, i, i, i]), "metal_enqueue_f16_sgd_apply": (None, [vp, vp, i, f]),
        "hip_enqueue_f32_to_f16": (None, [vp, vp, sz]), "hip_enqueue_q8_quantize": (None, [vp, vp, i, i]),
        "hip_enqueue_q8_dequant": (None, [vp, vp, i, i]), "hip_enqueue_q8_to_f16": (None, [vp, vp, i, i]),
        "hip_gemm_time_shape": (C.c_double, [i, i, i, i, i, i, i, C.POINTER(i), C.POINTER(i)]),
        "hip_matvec_time_shape": (C.c_double, [i, i, i, i, i]),
        "hip_gemm_profile_enable": (None, [i]), "hip_gemm_force_large_m": (None, [i]), "hip_gemm_ring": (None, [i]), "hip_gemm_ring_wide": (None, [i]), "hip_gemm_half_planes": (None, [i]), "hip_mem_info": (None, [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]), "hip_gemm_large_m_split": (None, [i]), "hip_gemm_large_m_block": (None, [i]), "hip_attention_flash": (None, [i]), "hip_attention_backward_one_launch": (None, [i]), "hip_gemm_image_budget_mb": (None, [i]), "hip_gemm_profile_read": (i, [C.POINTER(C.c_double), C.POINTER(C.c_double)]),
        "hip_gemm_profile_read2": (i, [C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
        "wmat_create_f16": (C.POINTER(WMat), [vp, i, i]), "wmat_create_q8": (C.POINTER(WMat), [vp, i, i]),
        "wmat_convert": (C.POINTER(WMat), [vp, i, i, i]), "wmat_free": (None, [C.POINTER(WMat)]),
        "norm_upload": (vp, [vp, i]),
        "sft_state_create_from_ref": (vp, [C.POINTER(SFTModelRef), i, i, i, f, i]), "sft_state_free": (None, [vp]),
        "sft_train_step": (f, [vp, vp, vp, f]), "sft_enqueue_train_step": (None, [vp, vp, vp, f]),
        "sft_finish_train_step": (f, [vp]),
        "forward_to_logits": (None, [vp]), "sft_backward": (None, [vp]), "sft_lora_update": (None, [vp, f]),
        "sft_get_logits": (vp, [vp]), "sft_get_dlogits": (vp, [vp]), "sft_get_x_cpu": (vp, [vp]),
        "sft_get_losses_cpu": (vp, [vp]), "sft_get_seq_len": (i, [vp]), "sft_get_vocab_size": (i, [vp]),
        "sft_get_d_model": (i, [vp]), "sft_get_lora_rank": (i, [vp]), "sft_get_n_layers": (i, [vp]),
        "sft_get_emb_scale": (f, [vp]), "sft_get_step_count": (i, [vp]), "sft_set_step_count": (None, [vp, i]),
        "sft_get_n_lora_grad_bufs": (i, [vp]), "sft_get_lora_grad_ptr": (vp, [vp, i, C.POINTER(i)]),
        "sft_set_lora_grad": (None, [vp, i, vp, i]), "sft_get_lora_weight_buf": (vp, [vp, i, i]),
        "sft_get_lora_scaling": (f, [vp]), "sft_set_sliding_window": (None, [vp, i, vp]), "sft_get_model_type": (i, [vp]), "sft_get_n_q_heads": (i, [vp]),
        "sft_get_n_kv_heads": (i, [vp]), "sft_get_head_dim": (i, [vp]), "sft_get_intermediate_size": (i, [vp]),
        "sft_get_rope_thetas": (vp, [vp]), "sft_is_full_param": (i, [vp]), "sft_save_lora": (None, [vp, C.c_char_p]), "sft_load_lora": (i, [vp, C.c_char_p]),
        "sft_lora_numel": (sz, [vp]), "sft_copy_lora": (None, [vp, vp]), "sft_copy_lora_grads": (None, [vp, vp]),
        "sft_set_lora": (None, [vp, vp]), "sft_get_last_grad_norm": (f, [vp]),
        "sft_get_token_emb": (vp, [vp]), "sft_get_token_emb_buf": (vp, [vp]),
        "inference_state_create_from_ref": (vp, [C.POINTER(SFTModelRef), i, i]),
        "inference_state_create_from_sft": (vp, [vp, i]), "inference_state_refresh_from_sft": (None, [vp]),
        "inference_state_free": (None, [vp]), "inference_generate": (i, [vp, vp, i, vp, i]), "inference_generate_batch": (i, [vp, vp, i, vp, i, i]),
        "inference_step_batch": (i, [vp, vp, i, i, vp]),
        "inference_state_model_type": (i, [vp]), "inference_state_vocab_size": (i, [vp]),
        "inference_state_reset": (None, [vp]), "inference_forward_token": (C.POINTER(C.c_float), [vp, i]),
        "inference_forward_token_argmax": (i, [vp, i]), "inference_state_set_lora": (None, [vp, vp]),
        "inference_state_set_eos": (None, [vp, vp, i]), "inference_state_load_eos": (None, [vp, C.c_char_p]),
        "inference_state_position": (i, [vp]),
        "inference_state_create_from_file": (vp, [C.c_char_p, i, i, i]),
        "model_file_open": (vp, [C.c_char_p]), "model_file_close": (None, [vp]), "model_file_is_gguf": (i, [vp]),
        "model_file_count": (i, [vp]), "model_file_name": (C.c_char_p, [vp, i]),
        "model_file_find": (i, [vp, C.c_char_p, C.POINTER(i), C.POINTER(i), C.POINTER(C.c_uint64)]),
        "model_file_matrix_shape": (i, [vp, C.c_char_p, C.POINTER(i), C.POINTER(i)]),
        "model_file_data": (vp, [vp, C.c_char_p, C.POINTER(sz)]),
        "model_file_load_f32": (vp, [vp, C.c_char_p, C.POINTER(sz)]),
        "model_file_load_wmat": (C.POINTER(WMat), [vp, C.c_char_p, i]),
        "token_loader_open": (vp, [C.c_char_p, i, i]), "token_loader_free": (None, [vp]),
        "token_loader_next": (i, [vp, vp, vp]), "token_loader_reset": (None, [vp]), "token_loader_shuffle": (None, [vp]),
        "token_loader_n_batches": (sz, [vp]), "token_loader_n_tokens": (sz, [vp]), "token_loader_position": (sz, [vp]),
        "model_ref_load": (C.POINTER(SFTModelRef), [C.c_char_p, i]), "model_ref_free": (None, [C.POINTER(SFTModelRef)]), "sft_get_final_norm_g": (vp, [vp]),
        "sft_get_layers": (C.POINTER(LayerW), [vp]), "sft_get_lm_head": (C.POINTER(WMat), [vp]),
        "sft_backward_sgd": (None, [vp, f]), "sft_alloc_grad_accum": (None, [vp]), "sft_backward_accum": (None, [vp]),
        "sft_apply_grad_sgd": (None, [vp, f]), "sft_save_full_checkpoint": (None, [vp, C.c_char_p]),
        "sft_copy_matrix_f16": (None, [vp, i, i, i, vp]),
        "grpo_apply_completions": (None, [vp, C.POINTER(GRPOCompletions), f, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L
