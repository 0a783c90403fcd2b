/*
 * sft_hip.h — host API of the fused LoRA SFT step on MI355X.
 *
 * Keeps the reference's C host API for this path: the weight container of
 * src/nn/wmat.h and the SFTState functions of src/nn/fast_sft.h, with the same
 * names, argument meaning and error behaviour (constructors return NULL when
 * the backend cannot start; everything else is silent).  What differs:
 *
 *  - State is built from the reference's own model-independent description
 *    (LayerWeightRef, src/nn/wmat.h:39-56) wrapped in SFTModelRef, not from
 *    Qwen3Model / Gemma3Model: those structs belong to the reference's CPU
 *    tensor runtime.  The constructors and the adapter sync with the
 *    reference's signatures (src/nn/fast_sft.h:14-23, 54-55) are declared and
 *    implemented, over the functions below, in llm_metal_amd/compat/
 *    fast_sft_compat.{h,c}, which are compiled inside the reference tree.
 *  - `batch` sequences per step (the reference has batch 1): RoPE positions and
 *    causal attention restart at every sequence.
 *  - Embedding gather, loss scaling, global-norm clipping and AdamW run on the
 *    device; the host touches only tokens, targets and the per-row losses.
 *
 * Limits (sft_state_create_from_ref checks all of them before it uploads anything,
 * prints the reason and returns NULL):
 *  - d_model, FFN width, vocabulary and head_dim multiples of 4; n_q_heads a
 *    multiple of n_kv_heads; Q8_0 additionally needs d_model, FFN width and
 *    n_q_heads * head_dim to be multiples of 32;
 *  - LoRA rank even and at most 16 (0 selects full-parameter mode);
 *  - d_model and FFN width at most 12 288 (one workgroup keeps a row in
 *    registers); (n_q_heads + 2 n_kv_heads) * head_dim + 2 rank at most 15 872
 *    (a row of dq | dk | dv | dh is staged in 64 KB of LDS); head_dim at most 512;
 *    seq_len at most 4096.  head_dim 32, 64, 128 or 256 with seq_len <= 1024
 *    takes the matrix-core attention, other shapes a slower kernel.
 */
#ifndef SFT_HIP_H
#define SFT_HIP_H

#include "fast_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- src/nn/wmat.h:10-78, under that header's own include guard: whichever of the two comes first in a
 *      translation unit of the reference declares these types and functions ---- */
#ifndef WMAT_H
#define WMAT_H
typedef enum { MODEL_QWEN3, MODEL_GEMMA3 } ModelType;

typedef struct WMat {
    MetalBuf *mbuf;
    int rows, cols, nb;            /* nb = cols/32, Q8_0 only */
} WMat;

typedef struct {
    WMat *q_proj, *k_proj, *v_proj, *o_proj;
    WMat *gate_proj, *up_proj, *down_proj;
    MetalBuf *input_norm_g, *post_attn_norm_g;
    MetalBuf *pre_ff_norm_g, *post_ff_norm_g;   /* Gemma3 only */
    MetalBuf *q_norm_g, *k_norm_g;
} LayerW;

typedef struct { const float *data; int rows, cols; } WeightRef;

typedef struct {
    WeightRef q_proj, k_proj, v_proj, o_proj;
    WeightRef gate_proj, up_proj, down_proj;
    const float *input_norm_g;
    const float *post_attn_norm_g;
    const float *pre_ff_norm_g;    /* Gemma3 only */
    const float *post_ff_norm_g;   /* Gemma3 only */
    const float *q_norm_g;
    const float *k_norm_g;
    int d_model;
    int head_dim;
} LayerWeightRef;

WMat *wmat_create_f16(const float *src, int rows, int cols);   /* src/nn/wmat.c:63-75, bit-identical */
WMat *wmat_create_q8(const float *src, int rows, int cols);    /* src/nn/wmat.c:46-61, bit-identical */
void  wmat_free(WMat *w);
LayerW *layers_convert_upload(const LayerWeightRef *refs, int n_layers, int use_fp16);
void  layers_free(LayerW *layers, int n_layers);
WMat *wmat_convert(const float *data, int rows, int cols, int use_fp16);
MetalBuf *norm_upload(const float *gamma, int dim);
#endif /* WMAT_H */

/* ---- model description (replaces the Qwen3Model / Gemma3Model arguments of
 *      sft_state_create*, src/nn/fast_sft.c:171-396) ---- */
typedef struct {
    ModelType model_type;
    int n_layers, d_model, n_q_heads, n_kv_heads, head_dim, intermediate_size, vocab_size;
    const float *rope_thetas;          /* [n_layers]; Gemma3: global on layers with L % 6 == 0 */
    const LayerWeightRef *layers;      /* [n_layers], fp32 host arrays */
    const float *token_emb;            /* [vocab, d_model] fp32 */
    const float *lm_head;              /* [vocab, d_model] fp32; Gemma3 passes token_emb (tied) */
    const float *final_norm_g;         /* [d_model] */
    /* optional initial adapters, flat per layer A_q[R,D] | B_q[Hq*hd,R] | A_v[R,D] | B_v[Hkv*hd,R];
     * NULL: A ~ U(-1,1)/sqrt(D) from rand(), B = 0 (src/nn/fast_sft.c:89-131) */
    const float *lora_init;
} SFTModelRef;

typedef struct SFTState SFTState;

/* weight_format: 1 = F16 frozen weights, 0 = Q8_0 (quantised with the reference's
 * algorithm; the GEMMs multiply with the dequantised values). */
SFTState *sft_state_create_from_ref(const SFTModelRef *model, int batch, int seq_len,
                                    int lora_rank, float lora_alpha, int weight_format);
void sft_state_free(SFTState *state);

/* src/nn/fast_sft.h:43-49; tokens are [batch*seq_len] */
float sft_train_step(SFTState *state, const uint32_t *input_tokens, const uint32_t *target_tokens, float lr);

/* src/nn/fast_sft.h:57-63: embeddings must be in sft_get_x_cpu's buffer */
void forward_to_logits(SFTState *state);
void sft_backward(SFTState *state);            /* consumes sft_get_dlogits (fp32 [BN, V]) */
void sft_lora_update(SFTState *state, float lr);

MetalBuf *sft_get_logits(SFTState *state);
MetalBuf *sft_get_dlogits(SFTState *state);
float *sft_get_x_cpu(SFTState *state);
float *sft_get_losses_cpu(SFTState *state);
int sft_get_seq_len(SFTState *state);          /* rows per step = batch * seq_len, as callers size by it */
int sft_get_vocab_size(SFTState *state);
int sft_get_d_model(SFTState *state);
int sft_get_lora_rank(SFTState *state);
int sft_get_n_layers(SFTState *state);
float sft_get_emb_scale(SFTState *state);
int sft_get_step_count(SFTState *state);
void sft_set_step_count(SFTState *state, int step);
int sft_get_n_lora_grad_bufs(SFTState *state);
float *sft_get_lora_grad_ptr(SFTState *state, int idx, int *out_size);
void sft_set_lora_grad(SFTState *state, int idx, const float *data, int size);
MetalBuf *sft_get_lora_weight_buf(SFTState *state, int layer, int sub);
float sft_get_lora_scaling(SFTState *state);
/* Extension: sliding-window attention.  window > 0: on the local layers query i attends keys i - window + 1 .. i
 * (forward and, through the saved probabilities, backward); 0 (the state's default) = every earlier key on every
 * layer, which is what the reference computes: it stores Gemma3's window (src/nn/gemma3.c:20, 99) and never reads it.
 * layer_is_local: [n_layers] flags, or NULL for Gemma3's pattern (src/nn/gemma3.c:49-57: all layers but L % 6 == 0;
 * every layer of a Qwen3 model). */
void sft_set_sliding_window(SFTState *state, int window, const int *layer_is_local);
ModelType sft_get_model_type(SFTState *state);
int sft_get_n_q_heads(SFTState *state);
int sft_get_n_kv_heads(SFTState *state);
int sft_get_head_dim(SFTState *state);
int sft_get_intermediate_size(SFTState *state);
const float *sft_get_rope_thetas(SFTState *state);
int sft_is_full_param(SFTState *state);          /* 1 when the state was created with lora_rank 0 (sft_state_create_full) */
const float *sft_get_token_emb(SFTState *state);  /* the caller's fp32 table, borrowed: it must outlive the state */
MetalBuf *sft_get_final_norm_g(SFTState *state);
/* the device copy of the embedding table, fp32 [vocab, d_model], unscaled (no counterpart in the reference, whose
 * shared-memory table is the host pointer above); borrowed by inference_state_create_from_sft */
MetalBuf *sft_get_token_emb_buf(SFTState *state);
/* Weight sharing accessors (src/nn/fast_sft.h:98-101).  The state keeps its matrices in the GEMM's own
 * operand layout, so these hand out row-major F16 COPIES, refreshed on every call. */
LayerW *sft_get_layers(SFTState *state);
WMat *sft_get_lm_head(SFTState *state);

/* ---- full-parameter mode (src/nn/fast_sft.h:20-39).  sft_train_step then runs forward, loss and
 *      sft_backward_sgd(lr) (or accumulates, once sft_alloc_grad_accum was called); no AdamW. ---- */
void sft_backward_sgd(SFTState *state, float lr);   /* W = half(W - lr dY^T X) per matrix, inside the backward */
void sft_alloc_grad_accum(SFTState *state);         /* zeroed F16 accumulators mirroring every weight */
void sft_backward_accum(SFTState *state);           /* G = half(G + dY^T X), weights untouched */
void sft_apply_grad_sgd(SFTState *state, float lr); /* W = half(W - lr G), G = 0; flushes */
void sft_save_full_checkpoint(SFTState *state, const char *path);   /* "FULL" file, src/nn/fast_sft.c:1286-1340 */
/* Extension: row-major F16 bits of one matrix.  which: 0..6 = q, k, v, o, gate, up, down of `layer`,
 * 7 = lm_head.  source: 0 = the weight, 1 = its transposed image (same values), 2 = the accumulator. */
void sft_copy_matrix_f16(SFTState *state, int layer, int which, int source, uint16_t *dst);

/* ---- GRPO phases 3-4 (src/nn/fast_grpo.c:376-495) over completions sampled elsewhere ---- */
typedef struct {
    const uint32_t *prompt; int prompt_len;
    int group_size;                       /* G */
    const uint32_t *const *gen_tokens;    /* [G] arrays of gen_lengths[i] sampled tokens */
    const int *gen_lengths;
    const float *const *gen_logprobs;     /* log-probabilities at sampling time */
    const float *advantages;              /* [G], group-normalised */
    float clip_eps;
    int accurate;                         /* full-parameter only: 1 = accumulate, apply once; 0 = SGD per completion with lr/G */
} GRPOCompletions;
/* new_logprobs: optional, [G][seq_len].  A state built with batch B takes B completions per forward / backward pass
 * (every weight is streamed once per pass, not once per completion); the F16 accumulators are then rounded once per
 * pass instead of once per completion.  Full-parameter SGD after every completion (accurate == 0) needs batch 1. */
void grpo_apply_completions(SFTState *state, const GRPOCompletions *c, float lr, float *new_logprobs);
/* "LORA" adapter file, src/nn/fast_sft.c:1255-1285 */
void sft_save_lora(SFTState *state, const char *path);
/* the reverse (qwen3_load_lora, src/nn/qwen3.c:558-602, applied to the state): 0, or -1 with a message when the file is
 * unreadable, has another magic, layer count or rank, or is truncated (the state is then unchanged) */
int sft_load_lora(SFTState *state, const char *path);

/* Extensions: bulk copies that leave the adapters in HBM (flat layout as lora_init). */
size_t sft_lora_numel(SFTState *state);
void sft_copy_lora(SFTState *state, float *dst);
void sft_copy_lora_grads(SFTState *state, float *dst);
void sft_set_lora(SFTState *state, const float *src);
float sft_get_last_grad_norm(SFTState *state);
/* Enqueue forward + loss + backward + update without waiting (sft_train_step = this + flush + mean).
 * One step is in flight at a time: the kernels read tokens, targets and optimiser parameters from pinned buffers of
 * the state, so a second enqueue before sft_finish_train_step first waits for the outstanding step.
 * Token and target ids are checked against the vocabulary on the host; with an id outside it nothing is launched, a
 * message goes to stderr and sft_finish_train_step / sft_train_step return NaN (grpo_apply_completions returns
 * without touching the state). */
void sft_enqueue_train_step(SFTState *state, const uint32_t *input_tokens, const uint32_t *target_tokens, float lr);
float sft_finish_train_step(SFTState *state);

#ifdef __cplusplus
}
#endif
#endif /* SFT_HIP_H */
