/*
 * Adapters from the reference's model structs to the model description the
 * HIP pipeline takes (fast_sft_compat.h, next to this file).  Compiled inside the
 * reference tree:
 *
 *   cc -DFAST_METAL_H -I<reference>/src/nn -I<this repo>/include -c fast_sft_compat.c
 *
 * The struct reads themselves are in model_ref_compat.h, shared with
 * fast_inference_compat.c.
 */
#include "fast_sft_compat.h"
#include "model_ref_compat.h"

/* Attached adapters of another rank, or attached to some layers only, are not used: say so (the reference takes the
 * attached adapters of every layer that has them, src/nn/fast_sft.c:96-112; this pipeline keeps all layers at one rank). */
static float *attached_or_warn(const Dims *d, int rank)
{
    float *lora = pack_attached_lora(d, rank);
    if (!lora && rank > 0 && d->q_loras && d->v_loras)
        fprintf(stderr, "[FastSFT] the model's attached adapters are ignored (a layer without them, or a rank other than %d): "
                        "starting from A ~ U(-1,1)/sqrt(d_model), B = 0\n", rank);
    return lora;
}

static SFTState *create(ModelDesc *m, int have, int seq_len, int rank, float alpha)
{
    SFTState *s = NULL;
    if (have == 0) {
        float *lora = attached_or_warn(&m->d, rank);
        const SFTModelRef ref = model_desc_ref(m, lora);
        s = sft_state_create_from_ref(&ref, /* batch */ 1, seq_len, rank, alpha, /* F16 weights */ 1);
        free(lora);
        model_desc_free(m);
    }
    return s;
}

static SFTState *create_qwen3(Qwen3Model *model, int seq_len, int rank, float alpha)
{
    ModelDesc m;
    return create(&m, model_desc_qwen3(&m, model), seq_len, rank, alpha);
}

static SFTState *create_gemma3(Gemma3Model *model, int seq_len, int rank, float alpha)
{
    ModelDesc m;
    return create(&m, model_desc_gemma3(&m, model), seq_len, rank, alpha);
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
