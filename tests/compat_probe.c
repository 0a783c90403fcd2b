/*
 * Host-only check of llm_metal_amd/compat/fast_sft_compat.c and fast_inference_compat.c (test infrastructure; built and
 * run by tests/test_reference_boundary.py inside the reference tree, never shipped).
 *
 * The reference's own constructors (qwen3_create, gemma3_create, *_attach_lora) build small models; the library entry
 * points that the compat units call are replaced here by test doubles that compare the model description they are
 * handed with the model it was made from, field by field, and by a fake adapter arena for the sync direction.
 * Prints one "ok <what>" or "FAIL <what>" line per check and exits non-zero on the first failure.
 */
#include "fast_inference_compat.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static int failures = 0;
#define CHECK(cond, ...) do { if (cond) { printf("ok "); } else { printf("FAIL "); failures++; } printf(__VA_ARGS__); printf("\n"); } while (0)

/* what the doubles compare against */
static Qwen3Model *g_q;
static Gemma3Model *g_g;
static int g_expect_rank, g_expect_seq, g_expect_fp16, g_expect_max_seq, g_calls_sft, g_calls_inf;
static int g_expect_lora;          /* 1: lora_init must hold the attached adapters, 0: must be NULL */

static void check_layer(const LayerWeightRef *r, GroupedQueryAttention *a, Linear *gate, Linear *up, Linear *down,
                        RMSNorm *in, RMSNorm *post_attn, RMSNorm *pre_ff, RMSNorm *post_ff, int D, int qd, int kd, int IS, int hd, int L)
{
    CHECK(r->q_proj.data == a->q_proj->weight->data && r->q_proj.rows == qd && r->q_proj.cols == D, "layer %d q_proj", L);
    CHECK(r->k_proj.data == a->k_proj->weight->data && r->k_proj.rows == kd && r->k_proj.cols == D, "layer %d k_proj", L);
    CHECK(r->v_proj.data == a->v_proj->weight->data && r->v_proj.rows == kd && r->v_proj.cols == D, "layer %d v_proj", L);
    CHECK(r->o_proj.data == a->o_proj->weight->data && r->o_proj.rows == D && r->o_proj.cols == qd, "layer %d o_proj", L);
    CHECK(r->gate_proj.data == gate->weight->data && r->gate_proj.rows == IS && r->gate_proj.cols == D, "layer %d gate_proj", L);
    CHECK(r->up_proj.data == up->weight->data && r->up_proj.rows == IS && r->up_proj.cols == D, "layer %d up_proj", L);
    CHECK(r->down_proj.data == down->weight->data && r->down_proj.rows == D && r->down_proj.cols == IS, "layer %d down_proj", L);
    CHECK(r->input_norm_g == in->gamma->data && r->post_attn_norm_g == post_attn->gamma->data, "layer %d block norms", L);
    CHECK(r->pre_ff_norm_g == (pre_ff ? pre_ff->gamma->data : NULL) && r->post_ff_norm_g == (post_ff ? post_ff->gamma->data : NULL),
          "layer %d feed-forward norms", L);
    CHECK(r->q_norm_g == a->q_norm->gamma->data && r->k_norm_g == a->k_norm->gamma->data, "layer %d head norms", L);
    CHECK(r->d_model == D && r->head_dim == hd, "layer %d dims", L);
}

static void check_lora(const SFTModelRef *m, LoRALinear **ql, LoRALinear **vl)
{
    if (!g_expect_lora) { CHECK(m->lora_init == NULL, "no initial adapters handed over"); return; }
    CHECK(m->lora_init != NULL, "attached adapters handed over");
    if (!m->lora_init) return;
    const int R = g_expect_rank, D = m->d_model, qd = m->n_q_heads * m->head_dim, kd = m->n_kv_heads * m->head_dim;
    const float *p = m->lora_init;
    int same = 1;
    for (int L = 0; L < m->n_layers; L++) {
        same &= !memcmp(p, ql[L]->lora_A->data, sizeof(float) * R * D); p += (size_t)R * D;
        same &= !memcmp(p, ql[L]->lora_B->data, sizeof(float) * qd * R); p += (size_t)qd * R;
        same &= !memcmp(p, vl[L]->lora_A->data, sizeof(float) * R * D); p += (size_t)R * D;
        same &= !memcmp(p, vl[L]->lora_B->data, sizeof(float) * kd * R); p += (size_t)kd * R;
    }
    CHECK(same, "adapter arena order A_q | B_q | A_v | B_v per layer");
}

static void check_ref(const SFTModelRef *m)
{
    if (m->model_type == MODEL_QWEN3) {
        Qwen3Model *q = g_q;
        CHECK(m->n_layers == q->n_layers && m->d_model == q->d_model && m->n_q_heads == q->n_q_heads && m->n_kv_heads == q->n_kv_heads &&
              m->head_dim == q->head_dim && m->intermediate_size == q->intermediate_size && m->vocab_size == q->vocab_size, "qwen3 dims");
        CHECK(m->token_emb == q->token_emb->weight->data && m->lm_head == q->lm_head->weight->data && m->final_norm_g == q->final_norm->gamma->data,
              "qwen3 embedding, head, final norm");
        for (int L = 0; L < q->n_layers; L++) {
            Qwen3Block *b = q->blocks[L];
            check_layer(&m->layers[L], b->attn, b->gate_proj, b->up_proj, b->down_proj, b->input_norm, b->post_attn_norm, NULL, NULL,
                        q->d_model, q->n_q_heads * q->head_dim, q->n_kv_heads * q->head_dim, q->intermediate_size, q->head_dim, L);
            CHECK(m->rope_thetas[L] == q->rope_theta, "layer %d theta %.0f", L, m->rope_thetas[L]);
        }
        check_lora(m, q->q_loras, q->v_loras);
    } else {
        Gemma3Model *g = g_g;
        CHECK(m->n_layers == g->n_layers && m->d_model == g->d_model && m->n_q_heads == g->n_q_heads && m->n_kv_heads == g->n_kv_heads &&
              m->head_dim == g->head_dim && m->intermediate_size == g->intermediate_size && m->vocab_size == g->vocab_size, "gemma3 dims");
        CHECK(m->token_emb == g->token_emb->weight->data && m->lm_head == g->token_emb->weight->data && m->final_norm_g == g->final_norm->gamma->data,
              "gemma3 embedding, tied head, final norm");
        for (int L = 0; L < g->n_layers; L++) {
            Gemma3Block *b = g->blocks[L];
            check_layer(&m->layers[L], b->attn, b->gate_proj, b->up_proj, b->down_proj, b->input_norm, b->post_attn_norm, b->pre_ff_norm,
                        b->post_ff_norm, g->d_model, g->n_q_heads * g->head_dim, g->n_kv_heads * g->head_dim, g->intermediate_size, g->head_dim, L);
            const float want = (L % 6) != 0 ? g->local_rope_theta : g->global_rope_theta;   /* src/nn/gemma3.c:49-57 */
            CHECK(m->rope_thetas[L] == want, "layer %d theta %.0f (%s)", L, m->rope_thetas[L], (L % 6) ? "local" : "global");
        }
        check_lora(m, g->q_loras, g->v_loras);
    }
}

/* ---- test doubles for the library entry points the compat units call ---- */
struct SFTState { int NL, D, Hq, Hkv, hd, R; float scaling; };
static struct SFTState g_fake_state;

SFTState *sft_state_create_from_ref(const SFTModelRef *m, int batch, int seq_len, int lora_rank, float lora_alpha, int weight_format)
{
    g_calls_sft++;
    CHECK(batch == 1 && seq_len == g_expect_seq && lora_rank == g_expect_rank && weight_format == 1, "sft_state_create_from_ref arguments (rank %d, alpha %.1f)", lora_rank, lora_alpha);
    check_ref(m);
    return &g_fake_state;
}

InferenceState *inference_state_create_from_ref(const SFTModelRef *m, int max_seq_len, int use_fp16)
{
    g_calls_inf++;
    CHECK(max_seq_len == g_expect_max_seq && use_fp16 == g_expect_fp16, "inference_state_create_from_ref arguments");
    check_ref(m);
    return (InferenceState *)&g_fake_state;
}

int inference_generate(InferenceState *s, const uint32_t *p, int n, uint32_t *out, int max_gen)
{
    for (int i = 0; i < max_gen; i++) out[i] = p[0] + (uint32_t)i;
    return max_gen;
}
int inference_generate_batch(InferenceState *s, const uint32_t *p, int n, uint32_t *out, int max_gen, int B)
{
    for (int i = 0; i < B * max_gen; i++) out[i] = (uint32_t)i;
    return max_gen;
}
static int g_freed;
void inference_state_free(InferenceState *s) { g_freed++; }

int sft_is_full_param(SFTState *s) { return s->R == 0; }
int sft_get_lora_rank(SFTState *s) { return s->R; }
float sft_get_lora_scaling(SFTState *s) { return s->scaling; }
int sft_get_n_layers(SFTState *s) { return s->NL; }
int sft_get_d_model(SFTState *s) { return s->D; }
int sft_get_n_q_heads(SFTState *s) { return s->Hq; }
int sft_get_n_kv_heads(SFTState *s) { return s->Hkv; }
int sft_get_head_dim(SFTState *s) { return s->hd; }
size_t sft_lora_numel(SFTState *s) { return (size_t)s->NL * (2 * (size_t)s->R * s->D + (size_t)(s->Hq + s->Hkv) * s->hd * s->R); }
void sft_copy_lora(SFTState *s, float *dst) { const size_t n = sft_lora_numel(s); for (size_t i = 0; i < n; i++) dst[i] = (float)i; }

static void check_sync(LoRALinear **ql, LoRALinear **vl, const struct SFTState *s)
{
    const size_t a = (size_t)s->R * s->D, bq = (size_t)s->Hq * s->hd * s->R, bv = (size_t)s->Hkv * s->hd * s->R;
    size_t off = 0;
    int good = 1;
    for (int L = 0; L < s->NL; L++) {
        good &= ql[L]->lora_A->data[0] == (float)off && ql[L]->lora_A->data[a - 1] == (float)(off + a - 1); off += a;
        good &= ql[L]->lora_B->data[0] == (float)off && ql[L]->lora_B->data[bq - 1] == (float)(off + bq - 1); off += bq;
        good &= vl[L]->lora_A->data[0] == (float)off && vl[L]->lora_A->data[a - 1] == (float)(off + a - 1); off += a;
        good &= vl[L]->lora_B->data[0] == (float)off && vl[L]->lora_B->data[bv - 1] == (float)(off + bv - 1); off += bv;
    }
    CHECK(good, "sync scatters A_q | B_q | A_v | B_v of every layer into the model's adapters");
}

int main(void)
{
    /* ---- Qwen3: 3 layers, attached adapters of the rank asked for ---- */
    Qwen3Config qc = { .n_layers = 3, .d_model = 64, .n_q_heads = 4, .n_kv_heads = 2, .head_dim = 16, .intermediate_size = 96,
                       .vocab_size = 50, .rope_theta = 1000000.0f, .rms_norm_eps = 1e-6f };
    g_q = qwen3_create(qc);
    qwen3_attach_lora(g_q, 8, 16.0f);
    for (int L = 0; L < 3; L++)           /* B is zero after attach: make every tensor distinguishable */
        for (int i = 0; i < 4 * 16 * 8; i++) g_q->q_loras[L]->lora_B->data[i] = (float)(L * 1000 + i);
    g_expect_rank = 8; g_expect_seq = 32; g_expect_lora = 1;
    SFTState *s = sft_state_create(g_q, 32, 8, 16.0f);
    CHECK(s == &g_fake_state && g_calls_sft == 1, "sft_state_create reaches the library once");

    /* another rank than the attached one: adapters not handed over (a warning goes to stderr) */
    g_expect_rank = 4; g_expect_lora = 0;
    sft_state_create(g_q, 32, 4, 8.0f);
    /* full-parameter constructor: rank 0 */
    g_expect_rank = 0;
    sft_state_create_full(g_q, 32);
    CHECK(g_calls_sft == 3, "three constructor calls");

    /* sync back into the model (rank 8 adapters attached) */
    g_fake_state = (struct SFTState){ 3, 64, 4, 2, 16, 8, 2.0f };
    sft_sync_lora_to_model(&g_fake_state, g_q);
    check_sync(g_q->q_loras, g_q->v_loras, &g_fake_state);

    /* generation entry points */
    g_expect_max_seq = 40; g_expect_fp16 = 0; g_expect_lora = 0;
    InferenceState *is = inference_state_create(g_q, 40, 0);
    CHECK(is == (InferenceState *)&g_fake_state && g_calls_inf == 1, "inference_state_create reaches the library once");
    uint32_t prompt[3] = { 7, 8, 9 }, out[2 * 5];
    g_expect_max_seq = 64; g_expect_fp16 = 1;
    CHECK(qwen3_generate_fast(g_q, prompt, 3, out, 5, 64, 1) == 5 && out[4] == 11 && g_freed == 1, "qwen3_generate_fast: create, generate, free");
    g_expect_max_seq = 3 + 5 + 1; g_expect_fp16 = 1;
    CHECK(qwen3_generate_fast_batch(g_q, prompt, 3, out, 5, 64, 2) == 5 && out[9] == 9 && g_freed == 2, "qwen3_generate_fast_batch: create, generate, free");

    /* ---- Gemma3: 7 layers (global layers 0 and 6), no adapters attached; sync attaches them ---- */
    Gemma3Config gc = gemma3_1b_config();
    gc.n_layers = 7; gc.d_model = 48; gc.n_q_heads = 2; gc.n_kv_heads = 1; gc.head_dim = 16; gc.intermediate_size = 64; gc.vocab_size = 40;
    g_g = gemma3_create(gc);
    g_expect_rank = 2; g_expect_seq = 16; g_expect_lora = 0;
    sft_state_create_gemma3(g_g, 16, 2, 4.0f);
    g_expect_rank = 0;
    sft_state_create_gemma3_full(g_g, 16);
    g_fake_state = (struct SFTState){ 7, 48, 2, 1, 16, 2, 2.0f };
    sft_sync_lora_to_gemma3(&g_fake_state, g_g);
    CHECK(g_g->q_loras && g_g->v_loras && g_g->q_loras[6]->rank == 2, "sync attaches adapters of the state's rank to a model without them");
    if (g_g->q_loras) check_sync(g_g->q_loras, g_g->v_loras, &g_fake_state);
    g_expect_max_seq = 24; g_expect_fp16 = 1;
    inference_state_create_gemma3(g_g, 24, 1);

    printf("%s: %d failure(s)\n", failures ? "FAILED" : "PASSED", failures);
    return failures ? 1 : 0;
}
