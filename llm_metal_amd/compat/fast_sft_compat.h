/*
 * fast_sft_compat.h — the entry points of src/nn/fast_sft.h that take the
 * reference's model structs, with the reference's signatures:
 *
 *   sft_state_create, sft_state_create_gemma3            src/nn/fast_sft.h:14-19
 *   sft_state_create_full, sft_state_create_gemma3_full  src/nn/fast_sft.h:22-23
 *   sft_sync_lora_to_model, sft_sync_lora_to_gemma3      src/nn/fast_sft.h:54-55
 *
 * Qwen3Model and Gemma3Model belong to the reference's CPU tensor runtime, so
 * this header (and fast_sft_compat.c next to it, which implements it over
 * sft_state_create_from_ref and sft_copy_lora of the library) is compiled
 * inside the reference tree, with src/nn and this repository's include/ on the
 * include path and -DFAST_METAL_H (fast_hip.h stands in for fast_metal.h).
 * It replaces fast_sft.h: a caller that includes both gets this one.
 */
#ifndef FAST_SFT_COMPAT_H
#define FAST_SFT_COMPAT_H
#define FAST_SFT_H              /* shadows src/nn/fast_sft.h */

#include "qwen3.h"              /* src/nn/qwen3.h: Qwen3Model */
#include "gemma3.h"             /* src/nn/gemma3.h: Gemma3Model */
#include "sft_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* F16 frozen weights, batch 1, adapters taken from model->q_loras / v_loras when attached
 * (src/nn/fast_sft.c:96-98), else A ~ U(-1,1)/sqrt(d_model), B = 0. */
SFTState *sft_state_create(Qwen3Model *model, int seq_len, int lora_rank, float lora_alpha);
SFTState *sft_state_create_gemma3(Gemma3Model *model, int seq_len, int lora_rank, float lora_alpha);
/* full-parameter mode: every matrix trainable, no adapters (src/nn/fast_sft.c:402-610) */
SFTState *sft_state_create_full(Qwen3Model *model, int seq_len);
SFTState *sft_state_create_gemma3_full(Gemma3Model *model, int seq_len);
/* adapters back into the model's LoRALinear tensors, attaching them first when the model has none
 * (src/nn/fast_sft.c:1163-1195) */
void sft_sync_lora_to_model(SFTState *state, Qwen3Model *model);
void sft_sync_lora_to_gemma3(SFTState *state, Gemma3Model *model);

#ifdef __cplusplus
}
#endif
#endif /* FAST_SFT_COMPAT_H */
