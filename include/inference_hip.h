/*
 * inference_hip.h — pipeline-level C ABI of the HIP backend for token-by-token generation: the replacement for the
 * reference's src/nn/fast_inference.h.  One decode step is the sequence of src/nn/fast_inference.c:376-467 (embedding
 * row, per layer RMSNorm -> Q/K/V products (+ LoRA on Q and V) -> per-head RMSNorm -> RoPE -> KV-cache store ->
 * attention over the cache -> O product -> residual -> RMSNorm -> gated FFN -> residual, final RMSNorm, LM head),
 * enqueued on the library's stream through the inference enqueues of fast_hip.h.  Weights are the reference's WMat
 * containers (F16 rows or Q8_0 blocks).
 *
 * The reference takes its Qwen3Model / Gemma3Model structs; this library takes the same plain description of the
 * model that the SFT state takes (SFTModelRef, sft_hip.h), which a caller fills from those structs as the
 * reference's build_refs does (src/nn/fast_sft.c:171-225).
 */
#ifndef INFERENCE_HIP_H
#define INFERENCE_HIP_H

#include "sft_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct InferenceState InferenceState;

/* inference_state_create / inference_state_create_gemma3 (src/nn/fast_inference.h:17-20; impl
 * src/nn/fast_inference.c:262-316): converts and uploads every matrix (use_fp16 != 0: F16, else Q8_0), allocates the
 * KV caches [n_kv_heads, max_seq_len, head_dim] per layer.  max_seq_len is not clamped to 4096 (the reference's
 * attention kernel holds 4096 scores; this one has no such limit).  NULL when no GPU is present. */
InferenceState *inference_state_create_from_ref(const SFTModelRef *model, int max_seq_len, int use_fp16);

/* The same from a checkpoint file (loader_hip.h: safetensors file / shard directory or GGUF): the reference's
 * qwen3_load_safetensors / qwen3_load_gguf / gemma3_load_safetensors followed by inference_state_create, without the
 * fp32 copy of the model in host memory: tensor bytes are uploaded as stored and converted on the GPU, and F16 / Q8_0
 * tensors that already have the wanted format are used bit for bit (no dequantise -> requantise). */
InferenceState *inference_state_create_from_file(const char *path, ModelType model_type, int max_seq_len, int use_fp16);

/* src/nn/fast_inference.h:49 (impl src/nn/fast_inference.c:527-610, owns_weights = 0 at :596-603): the state owns no
 * weights.  It reads the SFT state's own operands in place -- the F16 or Q8_0 tiles of its forward products, embedding
 * table, norm gammas and LoRA adapter buffers -- so it allocates only caches and scratch, and whatever training writes
 * (adapters, or every matrix in full-parameter mode) is what the next token is computed with.  The SFT state must
 * outlive it.  There are no row-major matrices for the matrix-vector kernels in such a state: every step, also of a
 * single sequence, runs the products of the lock-step batch path on the matrix cores (22 bits of the activations kept;
 * Q8_0 tiles enter as half(d * q), as in training), at about 1.6x the time per token of a state with its own weights.
 * A caller that wants the fastest single-sequence decode with a training state's adapters builds a state of its own
 * (inference_state_create_from_ref) and attaches them with inference_state_set_lora.  Hidden size <= 8192. */
InferenceState *inference_state_create_from_sft(SFTState *sft, int max_seq_len);
/* does nothing (kept for callers written against weight copies): the shared buffers are the training weights themselves */
void inference_state_refresh_from_sft(InferenceState *state);

void inference_state_free(InferenceState *state);                    /* src/nn/fast_inference.h:21 */

/* src/nn/fast_inference.h:26-28 (impl :612-675): greedy decoding.  Prefills the prompt token by token, then emits
 * argmax tokens until an EOS token has been emitted, max_gen_len tokens are out or the cache is full.  Returns the
 * number of tokens written (the EOS token included, as in the reference). */
int inference_generate(InferenceState *state, const uint32_t *prompt_tokens, int prompt_len,
                       uint32_t *output_tokens, int max_gen_len);

/* qwen3_generate_fast_batch (src/nn/fast_inference.h:70-72; impl src/nn/fast_inference.c:895-1000) on the weights of a
 * state: batch_size copies of one prompt, prefilled and decoded greedily in lock step, every weight read once per step
 * for all of them.  Runs with its own KV caches (the state's position and cache are left alone); F16 weights only and
 * batch_size <= 32, as in the reference, but for either model type and with the state's adapters.  A sequence ends at
 * one of the state's EOS ids or at token 0 (:944-947); the loop ends when all have.  output_tokens: [batch_size][max_gen_len].
 * Returns the number of tokens written per sequence (0: arguments refused).  The batch's caches and scratch stay with
 * the state until inference_state_free or a call with another batch_size, so repeated calls allocate nothing. */
int inference_generate_batch(InferenceState *state, const uint32_t *prompt_tokens, int prompt_len, uint32_t *output_tokens,
                             int max_gen_len, int batch_size);

/* One lock-step step of the same batch path with a token of its own per sequence -- the call a sampling caller makes
 * where the reference's forward_token_batch (src/nn/fast_inference.c:808-893, static there) takes tokens_b[b]; no
 * public counterpart in the reference.  tokens[b] enters sequence b at position pos; logits ([batch_size][vocab], host)
 * may be NULL.  pos = 0 starts new sequences; otherwise pos must follow the step before on the same batch_size (a step
 * of this call or the end of inference_generate_batch).  Returns 0, -1 when the arguments do not fit. */
int inference_step_batch(InferenceState *state, const int *tokens, int batch_size, int pos, float *logits);

ModelType inference_state_model_type(InferenceState *state);         /* src/nn/fast_inference.h:31 */
int  inference_state_vocab_size(InferenceState *state);              /* src/nn/fast_inference.h:34 */
void inference_state_reset(InferenceState *state);                   /* src/nn/fast_inference.h:37: position := 0 */
/* src/nn/fast_inference.h:41: one step at the current position, which it advances; returns the logits [vocab] in
 * host memory, valid until the next call.  NULL when the cache is full. */
const float *inference_forward_token(InferenceState *state, int token);
/* the same without the copy of the logits to the host: returns their argmax (computed on the GPU) */
int  inference_forward_token_argmax(InferenceState *state, int token);

void inference_state_set_lora(InferenceState *state, SFTState *sft); /* src/nn/fast_inference.h:46 */
/* src/nn/fast_inference.h:52 reads eos_token_id from <model_path>/generation_config.json or config.json; here the
 * caller passes the ids (at most 4); the defaults are the reference's (Qwen3: 151645, 151643; Gemma3: 1, 106). */
void inference_state_set_eos(InferenceState *state, const int *eos_tokens, int n_eos);
void inference_state_load_eos(InferenceState *state, const char *model_path);
int  inference_state_position(InferenceState *state);

#ifdef __cplusplus
}
#endif
#endif /* INFERENCE_HIP_H */
