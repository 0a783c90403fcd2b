// Token-by-token generation on top of the inference enqueues: the host pipeline of the reference's
// src/nn/fast_inference.c (state, forward_token, generate, sharing with the SFT state) for the HIP backend.
// Every step is enqueued on the library's one stream; the host waits once per token, for the logits or for
// the argmax computed on the GPU.
#include "backend.h"
#include "devutil.h"
#include "../../include/inference_hip.h"

#include <fstream>
#include <math.h>
#include <sstream>
#include <string.h>
#include <string>
#include <sys/stat.h>
#include <vector>

using namespace lmhip;

extern "C" MetalBuf *sft_get_token_emb_buf(SFTState *s);

struct InferenceState {
    int D, Hq, Hkv, hd, IS, V, NL, max_seq, cur_len, use_fp16;
    ModelType model_type;
    float emb_scale, eps;
    int eos[4], n_eos;
    std::vector<float> thetas;
    MetalBuf *x, *x2, *ln, *q, *k, *v, *att, *gate, *up, *ff, *logits, *best;
    float *logits_host;
    int *best_host;
    std::vector<MetalBuf *> kc, vc;
    LayerW *layers;
    WMat *lm_head;
    MetalBuf *g_final, *emb;
    int owns_weights;
    SFTState *sft;                       // source of borrowed weights, or NULL
    struct Lora { MetalBuf *Aq, *Bq, *Av, *Bv; };
    std::vector<Lora> lora;
    int R;
    float scaling;
    MetalBuf *lora_tmp, *lora_out;
};

namespace {

constexpr int TB = 256;

// x = emb[token] * scale: the embedding row, scaled by sqrt(D) for Gemma3 (src/nn/fast_inference.c:385-391)
__global__ __launch_bounds__(TB) void k_embed_row(const float *__restrict__ emb, int token, float scale, float *__restrict__ x, int D)
{
    const int i = blockIdx.x * TB + threadIdx.x;
    if (i < D) x[i] = emb[(size_t)token * D + i] * scale;
}

// index of the first maximum of v[0..n) (src/nn/fast_inference.c:469-476), one workgroup of 1024 threads
__global__ __launch_bounds__(1024) void k_argmax(const float *__restrict__ v, int n, int *__restrict__ out)
{
    __shared__ float bv[16];
    __shared__ int bi[16];
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < n; i += 1024) {
        const float a = v[i];
        if (a > best || (a == best && i < idx)) { best = a; idx = i; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(idx, o, 64);
        if (ob > best || (ob == best && oi < idx)) { best = ob; idx = oi; }
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) { bv[w] = best; bi[w] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 16; i++)
            if (bv[i] > best || (bv[i] == best && bi[i] < idx)) { best = bv[i]; idx = bi[i]; }
        *out = idx == 0x7fffffff ? 0 : idx;
    }
}

MetalBuf *fbuf(size_t n) { return metal_buf_create(n * sizeof(float)); }

void matvec(InferenceState *s, WMat *w, MetalBuf *x, MetalBuf *y)
{
    if (s->use_fp16) metal_enqueue_f16_matvec(w->mbuf, x, y, w->rows, w->cols);
    else metal_enqueue_q8_matvec(w->mbuf, x, y, w->rows, w->nb);
}

// src/nn/fast_inference.c:376-467
void forward_token(InferenceState *s, int token, int pos)
{
    const int D = s->D, Hq = s->Hq, Hkv = s->Hkv, hd = s->hd, qd = Hq * hd, kd = Hkv * hd;
    const bool gemma = s->model_type == MODEL_GEMMA3;
    hipLaunchKernelGGL(k_embed_row, dim3((D + TB - 1) / TB), dim3(TB), 0, stream(), dptr_as<float>(s->emb), token, s->emb_scale,
                       dptr_as<float>(s->x), D);
    for (int L = 0; L < s->NL; L++) {
        LayerW *lw = &s->layers[L];
        metal_enqueue_rms_norm(s->x, lw->input_norm_g, s->ln, D, s->eps);
        matvec(s, lw->q_proj, s->ln, s->q);
        matvec(s, lw->k_proj, s->ln, s->k);
        matvec(s, lw->v_proj, s->ln, s->v);
        if (!s->lora.empty()) {
            const InferenceState::Lora &lr = s->lora[L];
            metal_enqueue_float_matmul(s->ln, lr.Aq, s->lora_tmp, 1, s->R, D);
            metal_enqueue_float_matmul(s->lora_tmp, lr.Bq, s->lora_out, 1, qd, s->R);
            metal_enqueue_add_scaled(s->q, s->lora_out, s->scaling, qd);
            metal_enqueue_float_matmul(s->ln, lr.Av, s->lora_tmp, 1, s->R, D);
            metal_enqueue_float_matmul(s->lora_tmp, lr.Bv, s->lora_out, 1, kd, s->R);
            metal_enqueue_add_scaled(s->v, s->lora_out, s->scaling, kd);
        }
        if (lw->q_norm_g) metal_enqueue_per_head_rms_norm(s->q, lw->q_norm_g, Hq, hd, s->eps);
        if (lw->k_norm_g) metal_enqueue_per_head_rms_norm(s->k, lw->k_norm_g, Hkv, hd, s->eps);
        metal_enqueue_rope(s->q, s->k, Hq, Hkv, hd, pos, s->thetas[L]);
        metal_enqueue_kv_cache_store(s->k, s->v, s->kc[L], s->vc[L], Hkv, s->max_seq, hd, pos);
        metal_enqueue_attention(s->q, s->kc[L], s->vc[L], s->att, pos + 1, hd, s->max_seq, Hq, Hq / Hkv);
        matvec(s, lw->o_proj, s->att, s->x2);
        if (lw->post_attn_norm_g && lw->pre_ff_norm_g) {         // Gemma3: norm of the branch before the residual add
            metal_enqueue_rms_norm(s->x2, lw->post_attn_norm_g, s->ln, D, s->eps);
            metal_enqueue_residual_add(s->x, s->ln, D);
        } else {
            metal_enqueue_residual_add(s->x, s->x2, D);
        }
        MetalBuf *ff_norm = lw->pre_ff_norm_g ? lw->pre_ff_norm_g : lw->post_attn_norm_g;
        metal_enqueue_rms_norm(s->x, ff_norm, s->ln, D, s->eps);
        matvec(s, lw->gate_proj, s->ln, s->gate);
        matvec(s, lw->up_proj, s->ln, s->up);
        if (gemma) metal_enqueue_gelu_mul(s->gate, s->up, s->IS);
        else metal_enqueue_silu_mul(s->gate, s->up, s->IS);
        matvec(s, lw->down_proj, s->gate, s->ff);
        if (lw->post_ff_norm_g) {
            metal_enqueue_rms_norm(s->ff, lw->post_ff_norm_g, s->x2, D, s->eps);
            metal_enqueue_residual_add(s->x, s->x2, D);
        } else {
            metal_enqueue_residual_add(s->x, s->ff, D);
        }
    }
    metal_enqueue_rms_norm(s->x, s->g_final, s->ln, D, s->eps);
    matvec(s, s->lm_head, s->ln, s->logits);
}

const float *logits_to_host(InferenceState *s)
{
    HIP_CHECK(hipMemcpyAsync(s->logits_host, dptr(s->logits), (size_t)s->V * 4, hipMemcpyDeviceToHost, stream()));
    HIP_CHECK(hipStreamSynchronize(stream()));
    return s->logits_host;
}

int argmax_to_host(InferenceState *s)
{
    hipLaunchKernelGGL(k_argmax, dim3(1), dim3(1024), 0, stream(), dptr_as<float>(s->logits), s->V, dptr_as<int>(s->best));
    HIP_CHECK(hipMemcpyAsync(s->best_host, dptr(s->best), sizeof(int), hipMemcpyDeviceToHost, stream()));
    HIP_CHECK(hipStreamSynchronize(stream()));
    return *s->best_host;
}

void default_eos(InferenceState *s)
{
    if (s->model_type == MODEL_GEMMA3) { s->eos[0] = 1; s->eos[1] = 106; }            // <eos>, <end_of_turn>
    else { s->eos[0] = 151645; s->eos[1] = 151643; }
    s->n_eos = 2;
}

InferenceState *new_state(ModelType mt, int D, int Hq, int Hkv, int hd, int IS, int V, int NL, int max_seq, int use_fp16,
                          const float *thetas)
{
    if (fast_metal_init() != 0) { fprintf(stderr, "[FastGen] no GPU: fast_metal_init failed\n"); return nullptr; }
    if (Hkv <= 0 || Hq % Hkv || hd > 256 || Hq / Hkv > 16 || max_seq <= 0) {
        fprintf(stderr, "[FastGen] unsupported shape: %d / %d heads of %d (head_dim <= 256, group ratio <= 16)\n", Hq, Hkv, hd);
        fast_metal_shutdown();
        return nullptr;
    }
    InferenceState *s = new InferenceState();
    s->D = D; s->Hq = Hq; s->Hkv = Hkv; s->hd = hd; s->IS = IS; s->V = V; s->NL = NL;
    s->max_seq = max_seq; s->cur_len = 0; s->use_fp16 = use_fp16; s->model_type = mt;
    s->emb_scale = mt == MODEL_GEMMA3 ? sqrtf((float)D) : 1.0f;
    s->eps = 1e-6f;                                                       // src/nn/fast_inference.c:383
    s->thetas.assign(thetas, thetas + NL);
    default_eos(s);
    const int qd = Hq * hd, kd = Hkv * hd;
    s->x = fbuf(D); s->x2 = fbuf(D); s->ln = fbuf(D);
    s->q = fbuf(qd); s->k = fbuf(kd); s->v = fbuf(kd); s->att = fbuf(qd);
    s->gate = fbuf(IS); s->up = fbuf(IS); s->ff = fbuf(D);
    s->logits = fbuf(V); s->best = metal_buf_create(sizeof(int));
    HIP_CHECK(hipHostMalloc((void **)&s->logits_host, (size_t)V * 4, hipHostMallocDefault));
    HIP_CHECK(hipHostMalloc((void **)&s->best_host, sizeof(int), hipHostMallocDefault));
    const size_t cache_bytes = (size_t)Hkv * max_seq * hd * sizeof(float);
    for (int L = 0; L < NL; L++) { s->kc.push_back(metal_buf_create(cache_bytes)); s->vc.push_back(metal_buf_create(cache_bytes)); }
    s->R = 0; s->scaling = 0.f; s->lora_tmp = s->lora_out = nullptr;
    s->sft = nullptr; s->owns_weights = 0;
    s->layers = nullptr; s->lm_head = nullptr; s->g_final = s->emb = nullptr;
    return s;
}

// "eos_token_id": 7  or  "eos_token_id": [1, 106]  in the text of a config.json
int eos_ids_in(const std::string &text, int *out, int max_out)
{
    const std::string key = "\"eos_token_id\"";
    size_t p = text.find(key);
    if (p == std::string::npos) return 0;
    p = text.find(':', p + key.size());
    if (p == std::string::npos) return 0;
    p = text.find_first_not_of(" \t\r\n", p + 1);
    if (p == std::string::npos) return 0;
    int n = 0;
    const bool list = text[p] == '[';
    if (list) p++;
    while (p < text.size() && n < max_out) {
        p = text.find_first_not_of(" \t\r\n,", p);
        if (p == std::string::npos || text[p] == ']') break;
        char *end = nullptr;
        const long id = strtol(text.c_str() + p, &end, 10);
        if (end == text.c_str() + p) break;
        out[n++] = (int)id;
        p = (size_t)(end - text.c_str());
        if (!list) break;
    }
    return n;
}

}  // namespace

extern "C" {

InferenceState *inference_state_create_from_ref(const SFTModelRef *m, int max_seq_len, int use_fp16)
{
    InferenceState *s = new_state(m->model_type, m->d_model, m->n_q_heads, m->n_kv_heads, m->head_dim, m->intermediate_size,
                                  m->vocab_size, m->n_layers, max_seq_len, use_fp16, m->rope_thetas);
    if (!s) return nullptr;
    s->layers = layers_convert_upload(m->layers, m->n_layers, use_fp16);
    s->lm_head = wmat_convert(m->lm_head, m->vocab_size, m->d_model, use_fp16);
    s->g_final = norm_upload(m->final_norm_g, m->d_model);
    s->emb = metal_buf_from_data(m->token_emb, (size_t)m->vocab_size * m->d_model * sizeof(float));
    s->owns_weights = 1;
    return s;
}

InferenceState *inference_state_create_from_sft(SFTState *sft, int max_seq_len)
{
    InferenceState *s = new_state(sft_get_model_type(sft), sft_get_d_model(sft), sft_get_n_q_heads(sft), sft_get_n_kv_heads(sft),
                                  sft_get_head_dim(sft), sft_get_intermediate_size(sft), sft_get_vocab_size(sft),
                                  sft_get_n_layers(sft), max_seq_len, 1, sft_get_rope_thetas(sft));
    if (!s) return nullptr;
    s->sft = sft;
    s->g_final = sft_get_final_norm_g(sft);
    s->emb = sft_get_token_emb_buf(sft);
    inference_state_refresh_from_sft(s);
    inference_state_set_lora(s, sft);
    return s;
}

void inference_state_refresh_from_sft(InferenceState *s)
{
    if (!s || !s->sft) return;
    s->layers = sft_get_layers(s->sft);
    s->lm_head = sft_get_lm_head(s->sft);
}

void inference_state_set_lora(InferenceState *s, SFTState *sft)
{
    const int R = sft_get_lora_rank(sft);
    if (R == 0) return;                                                   // full-parameter state: no adapters
    const int qd = s->Hq * s->hd, kd = s->Hkv * s->hd;
    if (s->lora.empty()) {
        s->lora_tmp = fbuf(R);
        s->lora_out = fbuf(qd > kd ? qd : kd);
    }
    s->lora.resize(s->NL);
    for (int L = 0; L < s->NL; L++)
        s->lora[L] = InferenceState::Lora{sft_get_lora_weight_buf(sft, L, 0), sft_get_lora_weight_buf(sft, L, 1),
                                          sft_get_lora_weight_buf(sft, L, 2), sft_get_lora_weight_buf(sft, L, 3)};
    s->R = R;
    s->scaling = sft_get_lora_scaling(sft);
}

void inference_state_free(InferenceState *s)
{
    if (!s) return;
    metal_flush();
    for (MetalBuf *b : {s->x, s->x2, s->ln, s->q, s->k, s->v, s->att, s->gate, s->up, s->ff, s->logits, s->best, s->lora_tmp, s->lora_out})
        metal_buf_free(b);
    for (MetalBuf *b : s->kc) metal_buf_free(b);
    for (MetalBuf *b : s->vc) metal_buf_free(b);
    hipHostFree(s->logits_host);
    hipHostFree(s->best_host);
    if (s->owns_weights) {
        layers_free(s->layers, s->NL);
        wmat_free(s->lm_head);
        metal_buf_free(s->g_final);
        metal_buf_free(s->emb);
    }
    delete s;
    fast_metal_shutdown();
}

ModelType inference_state_model_type(InferenceState *s) { return s->model_type; }
int inference_state_vocab_size(InferenceState *s) { return s->V; }
void inference_state_reset(InferenceState *s) { s->cur_len = 0; }
int inference_state_position(InferenceState *s) { return s->cur_len; }

static bool token_ok(InferenceState *s, int token)
{
    if (token < 0 || token >= s->V) { fprintf(stderr, "[FastGen] token %d outside the vocabulary (%d)\n", token, s->V); return false; }
    if (s->cur_len >= s->max_seq) { fprintf(stderr, "[FastGen] KV cache full (%d positions)\n", s->max_seq); return false; }
    return true;
}

const float *inference_forward_token(InferenceState *s, int token)
{
    if (!token_ok(s, token)) return nullptr;
    forward_token(s, token, s->cur_len);
    s->cur_len++;
    return logits_to_host(s);
}

int inference_forward_token_argmax(InferenceState *s, int token)
{
    if (!token_ok(s, token)) return -1;
    forward_token(s, token, s->cur_len);
    s->cur_len++;
    return argmax_to_host(s);
}

int inference_generate(InferenceState *s, const uint32_t *prompt_tokens, int prompt_len, uint32_t *output_tokens, int max_gen_len)
{
    s->cur_len = 0;
    if (prompt_len <= 0 || max_gen_len <= 0 || prompt_len > s->max_seq) return 0;
    for (int i = 0; i < prompt_len; i++) {
        if (!token_ok(s, (int)prompt_tokens[i])) return 0;
        forward_token(s, (int)prompt_tokens[i], i);                      // prefill: only the last logits are looked at
        s->cur_len = i + 1;
    }
    int next = argmax_to_host(s);
    output_tokens[0] = (uint32_t)next;
    int n_gen = 1;
    for (int gen = 1; gen < max_gen_len && s->cur_len < s->max_seq; gen++) {
        bool is_eos = false;
        for (int e = 0; e < s->n_eos; e++) is_eos |= next == s->eos[e];
        if (is_eos) break;
        forward_token(s, next, s->cur_len);
        s->cur_len++;
        next = argmax_to_host(s);
        output_tokens[n_gen++] = (uint32_t)next;
    }
    return n_gen;
}

void inference_state_set_eos(InferenceState *s, const int *eos_tokens, int n_eos)
{
    if (n_eos <= 0 || !eos_tokens) { default_eos(s); return; }
    s->n_eos = n_eos > 4 ? 4 : n_eos;
    for (int i = 0; i < s->n_eos; i++) s->eos[i] = eos_tokens[i];
}

// src/nn/fast_inference.c:13-49, 324-342: config.json inside model_path when that is a directory, else next to it
void inference_state_load_eos(InferenceState *s, const char *model_path)
{
    std::string path = model_path ? model_path : "";
    struct stat st;
    if (stat(path.c_str(), &st) == 0 && S_ISDIR(st.st_mode)) path += "/config.json";
    else {
        const size_t sl = path.rfind('/');
        path = sl == std::string::npos ? "config.json" : path.substr(0, sl) + "/config.json";
    }
    int ids[4], n = 0;
    std::ifstream f(path);
    if (f) {
        std::stringstream ss;
        ss << f.rdbuf();
        n = eos_ids_in(ss.str(), ids, 4);
    }
    inference_state_set_eos(s, ids, n);
    fprintf(stderr, "[FastGen] EOS tokens (%d):", s->n_eos);
    for (int i = 0; i < s->n_eos; i++) fprintf(stderr, " %d", s->eos[i]);
    fprintf(stderr, "\n");
}

}  // extern "C"
