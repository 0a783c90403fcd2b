/*
 * model_ref_compat.h -- the reference's model structs read into the model description the HIP pipeline takes
 * (SFTModelRef, sft_hip.h).  Shared by fast_sft_compat.c and fast_inference_compat.c; compiled inside the reference
 * tree (src/nn on the include path).  Only field reads: the seven matrices and the norm vectors of every block (what
 * src/nn/fast_sft.c:212-239, :327-356 and src/nn/fast_inference.c:277-316 hand to layers_convert_upload), the
 * per-layer RoPE base (src/nn/fast_sft.c:310-313) and, when the model carries attached adapters, their A and B tensors
 * (:96-98, 110-112).
 */
#ifndef MODEL_REF_COMPAT_H
#define MODEL_REF_COMPAT_H

#include "qwen3.h"
#include "gemma3.h"
#include "sft_hip.h"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    ModelType type;
    int NL, D, Hq, Hkv, hd, IS, V;
    LoRALinear **q_loras, **v_loras;
    Embedding *token_emb;
    const float *lm_head, *final_norm_g;
} Dims;

static inline void fill_layer(LayerWeightRef *r, const Dims *d, GroupedQueryAttention *attn,
                       Linear *gate, Linear *up, Linear *down,
                       RMSNorm *in, RMSNorm *post_attn, RMSNorm *pre_ff, RMSNorm *post_ff)
{
    const int qd = d->Hq * d->hd, kd = d->Hkv * d->hd;
    r->q_proj = (WeightRef){ attn->q_proj->weight->data, qd, d->D };
    r->k_proj = (WeightRef){ attn->k_proj->weight->data, kd, d->D };
    r->v_proj = (WeightRef){ attn->v_proj->weight->data, kd, d->D };
    r->o_proj = (WeightRef){ attn->o_proj->weight->data, d->D, qd };
    r->gate_proj = (WeightRef){ gate->weight->data, d->IS, d->D };
    r->up_proj = (WeightRef){ up->weight->data, d->IS, d->D };
    r->down_proj = (WeightRef){ down->weight->data, d->D, d->IS };
    r->input_norm_g = in->gamma->data;
    r->post_attn_norm_g = post_attn->gamma->data;
    r->pre_ff_norm_g = pre_ff ? pre_ff->gamma->data : NULL;
    r->post_ff_norm_g = post_ff ? post_ff->gamma->data : NULL;
    r->q_norm_g = attn->q_norm->gamma->data;
    r->k_norm_g = attn->k_norm->gamma->data;
    r->d_model = d->D;
    r->head_dim = d->hd;
}

/* A_q | B_q | A_v | B_v per layer from the model's attached adapters, or NULL when it has none
 * (or their rank differs from the one asked for). */
static inline float *pack_attached_lora(const Dims *d, int rank)
{
    if (rank <= 0 || !d->q_loras || !d->v_loras) return NULL;
    const size_t a = (size_t)rank * d->D, bq = (size_t)d->Hq * d->hd * rank, bv = (size_t)d->Hkv * d->hd * rank;
    for (int L = 0; L < d->NL; L++)
        if (!d->q_loras[L] || !d->v_loras[L] || d->q_loras[L]->rank != rank || d->v_loras[L]->rank != rank) return NULL;
    float *flat = malloc((2 * a + bq + bv) * d->NL * sizeof(float)), *p = flat;
    if (!flat) return NULL;
    for (int L = 0; L < d->NL; L++) {
        memcpy(p, d->q_loras[L]->lora_A->data, a * sizeof(float));  p += a;
        memcpy(p, d->q_loras[L]->lora_B->data, bq * sizeof(float)); p += bq;
        memcpy(p, d->v_loras[L]->lora_A->data, a * sizeof(float));  p += a;
        memcpy(p, d->v_loras[L]->lora_B->data, bv * sizeof(float)); p += bv;
    }
    return flat;
}


/* The description of a whole model: `refs` and `thetas` are malloc'ed here and freed by model_desc_free. */
typedef struct { Dims d; LayerWeightRef *refs; float *thetas; } ModelDesc;

static inline void model_desc_free(ModelDesc *m) { free(m->refs); free(m->thetas); m->refs = NULL; m->thetas = NULL; }

static inline int model_desc_qwen3(ModelDesc *out, Qwen3Model *m)
{
    const Dims d = { MODEL_QWEN3, m->n_layers, m->d_model, m->n_q_heads, m->n_kv_heads, m->head_dim,
                     m->intermediate_size, m->vocab_size, m->q_loras, m->v_loras, m->token_emb,
                     m->lm_head->weight->data, m->final_norm->gamma->data };
    out->d = d;
    out->refs = calloc((size_t)d.NL, sizeof *out->refs);
    out->thetas = malloc((size_t)d.NL * sizeof *out->thetas);
    if (!out->refs || !out->thetas) { model_desc_free(out); return -1; }
    for (int i = 0; i < d.NL; i++) {
        Qwen3Block *b = m->blocks[i];
        fill_layer(&out->refs[i], &d, b->attn, b->gate_proj, b->up_proj, b->down_proj, b->input_norm, b->post_attn_norm, NULL, NULL);
        out->thetas[i] = m->rope_theta;
    }
    return 0;
}

static inline int model_desc_gemma3(ModelDesc *out, Gemma3Model *m)
{
    /* the head is tied to the embedding table (src/nn/fast_sft.c:351) */
    const Dims d = { MODEL_GEMMA3, m->n_layers, m->d_model, m->n_q_heads, m->n_kv_heads, m->head_dim,
                     m->intermediate_size, m->vocab_size, m->q_loras, m->v_loras, m->token_emb,
                     m->token_emb->weight->data, m->final_norm->gamma->data };
    out->d = d;
    out->refs = calloc((size_t)d.NL, sizeof *out->refs);
    out->thetas = malloc((size_t)d.NL * sizeof *out->thetas);
    if (!out->refs || !out->thetas) { model_desc_free(out); return -1; }
    for (int i = 0; i < d.NL; i++) {
        Gemma3Block *b = m->blocks[i];
        fill_layer(&out->refs[i], &d, b->attn, b->gate_proj, b->up_proj, b->down_proj, b->input_norm, b->post_attn_norm,
                   b->pre_ff_norm, b->post_ff_norm);
        out->thetas[i] = (i % 6) != 0 ? m->local_rope_theta : m->global_rope_theta;      /* src/nn/fast_sft.c:310-313 */
    }
    return 0;
}

/* `lora`: flat adapters (pack_attached_lora) or NULL */
static inline SFTModelRef model_desc_ref(const ModelDesc *m, const float *lora)
{
    const Dims *d = &m->d;
    SFTModelRef ref = { d->type, d->NL, d->D, d->Hq, d->Hkv, d->hd, d->IS, d->V, m->thetas, m->refs,
                        d->token_emb->weight->data, d->lm_head, d->final_norm_g, lora };
    return ref;
}

#endif /* MODEL_REF_COMPAT_H */
