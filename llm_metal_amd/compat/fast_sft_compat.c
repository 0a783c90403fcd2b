/*
 * Adapters from the reference's model structs to the model description the
 * HIP pipeline takes (fast_sft_compat.h, next to this file).  Compiled inside the
 * reference tree:
 *
 *   cc -DFAST_METAL_H -I<reference>/src/nn -I<this repo>/include -c fast_sft_compat.c
 *
 * Only field reads: the seven matrices and the norm vectors of every block
 * (what src/nn/fast_sft.c:212-239 and :327-356 hand to layers_convert_upload),
 * the per-layer RoPE base (:310-313) and, when the model carries attached
 * adapters, their A and B tensors (:96-98, 110-112).
 */
#include "fast_sft_compat.h"
#include <stdlib.h>
#include <string.h>

typedef struct {
    ModelType type;
    int NL, D, Hq, Hkv, hd, IS, V;
    LoRALinear **q_loras, **v_loras;
    Embedding *token_emb;
    const float *lm_head, *final_norm_g;
} Dims;

static void fill_layer(LayerWeightRef *r, const Dims *d, GroupedQueryAttention *attn,
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
static float *pack_attached_lora(const Dims *d, int rank)
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

static SFTState *create(const Dims *d, LayerWeightRef *refs, float *thetas, int seq_len, int rank, float alpha)
{
    SFTState *s = NULL;
    if (refs && thetas) {
        float *lora = pack_attached_lora(d, rank);
        SFTModelRef ref = { d->type, d->NL, d->D, d->Hq, d->Hkv, d->hd, d->IS, d->V, thetas, refs,
                            d->token_emb->weight->data, d->lm_head, d->final_norm_g, lora };
        s = sft_state_create_from_ref(&ref, /* batch */ 1, seq_len, rank, alpha, /* F16 weights */ 1);
        free(lora);
    }
    free(refs);
    free(thetas);
    return s;
}

static SFTState *create_qwen3(Qwen3Model *m, int seq_len, int rank, float alpha)
{
    const Dims d = { MODEL_QWEN3, m->n_layers, m->d_model, m->n_q_heads, m->n_kv_heads, m->head_dim,
                     m->intermediate_size, m->vocab_size, m->q_loras, m->v_loras, m->token_emb,
                     m->lm_head->weight->data, m->final_norm->gamma->data };
    LayerWeightRef *refs = calloc((size_t)d.NL, sizeof *refs);
    float *thetas = malloc((size_t)d.NL * sizeof *thetas);
    for (int i = 0; refs && thetas && i < d.NL; i++) {
        Qwen3Block *b = m->blocks[i];
        fill_layer(&refs[i], &d, b->attn, b->gate_proj, b->up_proj, b->down_proj, b->input_norm, b->post_attn_norm, NULL, NULL);
        thetas[i] = m->rope_theta;
    }
    return create(&d, refs, thetas, seq_len, rank, alpha);
}

static SFTState *create_gemma3(Gemma3Model *m, int seq_len, int rank, float alpha)
{
    /* the head is tied to the embedding table (src/nn/fast_sft.c:351) */
    const Dims d = { MODEL_GEMMA3, m->n_layers, m->d_model, m->n_q_heads, m->n_kv_heads, m->head_dim,
                     m->intermediate_size, m->vocab_size, m->q_loras, m->v_loras, m->token_emb,
                     m->token_emb->weight->data, m->final_norm->gamma->data };
    LayerWeightRef *refs = calloc((size_t)d.NL, sizeof *refs);
    float *thetas = malloc((size_t)d.NL * sizeof *thetas);
    for (int i = 0; refs && thetas && i < d.NL; i++) {
        Gemma3Block *b = m->blocks[i];
        fill_layer(&refs[i], &d, b->attn, b->gate_proj, b->up_proj, b->down_proj, b->input_norm, b->post_attn_norm,
                   b->pre_ff_norm, b->post_ff_norm);
        thetas[i] = (i % 6) != 0 ? m->local_rope_theta : m->global_rope_theta;      /* src/nn/fast_sft.c:310-313 */
    }
    return create(&d, refs, thetas, seq_len, rank, alpha);
}

SFTState *sft_state_create(Qwen3Model *model, int seq_len, int lora_rank, float lora_alpha)
{
    return create_qwen3(model, seq_len, lora_rank, lora_alpha);
}

SFTState *sft_state_create_gemma3(Gemma3Model *model, int seq_len, int lora_rank, float lora_alpha)
{
    return create_gemma3(model, seq_len, lora_rank, lora_alpha);
}

SFTState *sft_state_create_full(Qwen3Model *model, int seq_len) { return create_qwen3(model, seq_len, 0, 0.0f); }

SFTState *sft_state_create_gemma3_full(Gemma3Model *model, int seq_len) { return create_gemma3(model, seq_len, 0, 0.0f); }

static void scatter_lora(SFTState *s, LoRALinear **q, LoRALinear **v, int NL, int D, int qd, int kd)
{
    const int R = sft_get_lora_rank(s);
    const size_t a = (size_t)R * D, bq = (size_t)qd * R, bv = (size_t)kd * R;
    float *flat = malloc(sft_lora_numel(s) * sizeof(float)), *p = flat;
    if (!flat) return;
    sft_copy_lora(s, flat);
    for (int L = 0; L < NL; L++) {
        memcpy(q[L]->lora_A->data, p, a * sizeof(float));  p += a;
        memcpy(q[L]->lora_B->data, p, bq * sizeof(float)); p += bq;
        memcpy(v[L]->lora_A->data, p, a * sizeof(float));  p += a;
        memcpy(v[L]->lora_B->data, p, bv * sizeof(float)); p += bv;
    }
    free(flat);
}

void sft_sync_lora_to_model(SFTState *s, Qwen3Model *model)
{
    if (sft_is_full_param(s)) return;
    if (!model->q_loras) qwen3_attach_lora(model, sft_get_lora_rank(s), sft_get_lora_scaling(s) * (float)sft_get_lora_rank(s));
    scatter_lora(s, model->q_loras, model->v_loras, sft_get_n_layers(s), sft_get_d_model(s),
                 sft_get_n_q_heads(s) * sft_get_head_dim(s), sft_get_n_kv_heads(s) * sft_get_head_dim(s));
}

void sft_sync_lora_to_gemma3(SFTState *s, Gemma3Model *model)
{
    if (sft_is_full_param(s)) return;
    if (!model->q_loras) gemma3_attach_lora(model, sft_get_lora_rank(s), sft_get_lora_scaling(s) * (float)sft_get_lora_rank(s));
    scatter_lora(s, model->q_loras, model->v_loras, sft_get_n_layers(s), sft_get_d_model(s),
                 sft_get_n_q_heads(s) * sft_get_head_dim(s), sft_get_n_kv_heads(s) * sft_get_head_dim(s));
}
