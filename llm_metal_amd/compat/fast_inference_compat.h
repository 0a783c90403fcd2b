/*
 * fast_inference_compat.h -- the entry points of src/nn/fast_inference.h that take the reference's model structs,
 * with the reference's signatures:
 *
 *   inference_state_create, inference_state_create_gemma3     src/nn/fast_inference.h:15, 18
 *   qwen3_generate_fast                                        src/nn/fast_inference.h:63-65
 *   qwen3_generate_fast_batch                                  src/nn/fast_inference.h:70-72
 *
 * Everything else that header declares (inference_state_free, inference_generate, inference_forward_token,
 * inference_state_reset, _vocab_size, _model_type, _set_lora, _create_from_sft, _load_eos) is exported by the library
 * under the same name and signature (inference_hip.h).  Compiled inside the reference tree like fast_sft_compat.h,
 * in place of fast_inference.h and fast_inference.c: a caller that includes both gets this one.
 */
#ifndef FAST_INFERENCE_COMPAT_H
#define FAST_INFERENCE_COMPAT_H
#define FAST_INFERENCE_H        /* shadows src/nn/fast_inference.h */

#include "fast_sft_compat.h"
#include "inference_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* use_fp16 != 0: F16 weights, else Q8_0 (quantised on the device, bit-identical to wmat_create_q8) */
InferenceState *inference_state_create(Qwen3Model *model, int max_seq_len, int use_fp16);
InferenceState *inference_state_create_gemma3(Gemma3Model *model, int max_seq_len, int use_fp16);
/* create, inference_generate, free (src/nn/fast_inference.c:681-692); returns the number of generated tokens */
int qwen3_generate_fast(Qwen3Model *model, const uint32_t *prompt_tokens, int prompt_len, uint32_t *output_tokens,
                        int max_gen_len, int max_seq_len, int use_fp16);
/* batch_size (<= 32) copies of one prompt decoded greedily in lock step over F16 weights, output_tokens
 * [batch_size][max_gen_len] (src/nn/fast_inference.c:895-1000); returns the tokens generated per sequence */
int qwen3_generate_fast_batch(Qwen3Model *model, const uint32_t *prompt_tokens, int prompt_len, uint32_t *output_tokens,
                              int max_gen_len, int max_seq_len, int batch_size);

#ifdef __cplusplus
}
#endif
#endif /* FAST_INFERENCE_COMPAT_H */
