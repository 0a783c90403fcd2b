// Token-by-token generation on top of the inference enqueues: the host pipeline of the reference's
// src/nn/fast_inference.c (state, forward_token, generate, sharing with the SFT state) for the HIP backend.
// Every step is enqueued on the library's one stream; the host waits once per token, for the logits or for
// the argmax computed on the GPU.
//
// One decode step computes what src/nn/fast_inference.c:376-467 computes, in 9 launches per layer instead of 17
// (10 instead of 23 with adapters): Q|K|V and gate|up are one matrix each (row concatenation, built when the state is
// created), the residual add travels with the RMSNorm that follows it, and one kernel does LoRA up-projection,
// per-head RMSNorm, RoPE and the KV-cache store for all heads.
#include "backend.h"
#include "devutil.h"
#include "fused.h"
#include "../../include/inference_hip.h"
#include "../../include/loader_hip.h"

#include <fstream>
#include <math.h>
#include <sstream>
#include <string.h>
#include <string>
#include <sys/stat.h>
#include <vector>

using namespace lmhip;

extern "C" MetalBuf *sft_get_token_emb_buf(SFTState *s);

namespace {
struct BatchRun;
void batch_release(BatchRun *r);
// a state on a training state's tiles: one token through the lock-step path with a run of one sequence
void step_on_tiles(InferenceState *s, int token, int pos);
const float *logits_on_tiles(InferenceState *s);
int argmax_on_tiles(InferenceState *s);
}

struct InferenceState {
    int D, Hq, Hkv, hd, IS, V, NL, max_seq, cur_len, use_fp16;
    ModelType model_type;
    float emb_scale, eps;
    int eos[4], n_eos;
    std::vector<float> thetas;
    MetalBuf *rope_tabs;                 // (cos, sin) [distinct thetas][max_seq][hd/2], as rope forms them
    std::vector<int> theta_slot;         // table of each layer
    MetalBuf *x, *x2, *branch, *ln, *qkv, *att, *gu, *gate_v, *up_v, *logits, *best;   // gate_v / up_v: the halves of gu
    float *logits_host;
    int *best_host;
    std::vector<MetalBuf *> kc, vc;
    // per layer: fused [Wq; Wk; Wv] and [Wgate; Wup] (owned), Wo and Wdown and the norm gammas (owned, or the SFT state's)
    struct Layer { WMat qkv, gu; WMat *o, *down; MetalBuf *g_in, *g_post_attn, *g_pre_ff, *g_post_ff, *g_q, *g_k; };
    // A state made from a training state owns no weights at all: `borrowed` holds the training state's tiled images
    // (F16 or Q8_0 tiles, the operands of its own forward), read in place, so whatever training writes there is what the
    // next token sees.  Such a state has no row-major matrices for the matrix-vector kernels; every step, also of a
    // single sequence, goes through the matrix-core products of the lock-step batch path (`single`: its run of one).
    int borrows_tiles;
    std::vector<BorrowedLayer> borrowed;
    WeightOp borrowed_lm;
    BatchRun *single;
    std::vector<Layer> layers;
    WMat *lm_head;
    MetalBuf *g_final, *emb;
    int owns_weights;
    SFTState *sft;                       // source of borrowed weights, or NULL
    struct Lora { MetalBuf *Aq, *Bq, *Av, *Bv; };
    std::vector<Lora> lora;
    int R;
    float scaling;
    MetalBuf *lora_t;                    // [2R]: A_q ln | A_v ln
    BatchRun *batch;                     // scratch and caches of the lock-step batch path, kept from call to call (NULL until used)
};

namespace {

constexpr int TB = 256;

// x = emb[token] * scale: the embedding row, scaled by sqrt(D) for Gemma3 (src/nn/fast_inference.c:385-391)
__global__ __launch_bounds__(TB) void k_embed_row(const float *__restrict__ emb, int token, float scale, float *__restrict__ x, int D)
{
    const int i = blockIdx.x * TB + threadIdx.x;
    if (i < D) x[i] = emb[(size_t)token * D + i] * scale;
}

// index of the first maximum of v[0..n) (src/nn/fast_inference.c:469-476) in two launches: AM_WGS workgroups leave
// (value, index) of their slice, one workgroup picks among them
constexpr int AM_WGS = 128;

__device__ __forceinline__ void am_pick(float &best, int &idx, float ob, int oi)
{
    if (ob > best || (ob == best && oi < idx)) { best = ob; idx = oi; }
}

__device__ __forceinline__ void am_block(float &best, int &idx, float *bv, int *bi)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) am_pick(best, idx, __shfl_xor(best, o, 64), __shfl_xor(idx, o, 64));
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) { bv[w] = best; bi[w] = idx; }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int i = 1; i < (int)(blockDim.x >> 6); i++) am_pick(best, idx, bv[i], bi[i]);
}

__global__ __launch_bounds__(TB) void k_argmax_part(const float *__restrict__ v, int n, float *__restrict__ pv, int *__restrict__ pi)
{
    __shared__ float bv[4];
    __shared__ int bi[4];
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = blockIdx.x * TB + threadIdx.x; i < n; i += AM_WGS * TB) am_pick(best, idx, v[i], i);
    am_block(best, idx, bv, bi);
    if (threadIdx.x == 0) { pv[blockIdx.x] = best; pi[blockIdx.x] = idx; }
}

__global__ __launch_bounds__(AM_WGS) void k_argmax_final(const float *__restrict__ pv, const int *__restrict__ pi, int *__restrict__ out)
{
    __shared__ float bv[AM_WGS / 64];
    __shared__ int bi[AM_WGS / 64];
    float best = pv[threadIdx.x];
    int idx = pi[threadIdx.x];
    am_block(best, idx, bv, bi);
    if (threadIdx.x == 0) *out = idx == 0x7fffffff ? 0 : idx;
}

// x += b (b = branch, or RMSNorm(branch; g_branch) where Gemma3 norms the branch output first); ln = RMSNorm(x; g).
// branch == NULL: only the norm.  One workgroup of 1024 threads: the vector is a few thousand floats.
__global__ __launch_bounds__(1024) void k_add_norm(float *__restrict__ x, const float *__restrict__ branch,
                                                   const float *__restrict__ g_branch, const float *__restrict__ g,
                                                   float *__restrict__ ln, int D, float eps)
{
    __shared__ float sm[16];
    x += (size_t)blockIdx.x * D; ln += (size_t)blockIdx.x * D;           // one workgroup per vector of a batch
    if (branch) branch += (size_t)blockIdx.x * D;
    float inv_b = 1.f;
    if (branch && g_branch) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < D; i += 1024) { const float v = branch[i]; ss += v * v; }
        inv_b = rsqrtf(block_sum(ss, sm) / (float)D + eps);
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < D; i += 1024) {
        float v = x[i];
        if (branch) { v += g_branch ? branch[i] * inv_b * g_branch[i] : branch[i]; x[i] = v; }
        ss += v * v;
    }
    const float inv = rsqrtf(block_sum(ss, sm) / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += 1024) ln[i] = x[i] * inv * g[i];       // own elements only: no barrier needed
}

// t[r] = A_q[r] . ln for r < R, t[R + r] = A_v[r] . ln: one wave per adapter row
__global__ __launch_bounds__(64) void k_lora_down(const float *__restrict__ ln, const float *__restrict__ Aq,
                                                  const float *__restrict__ Av, float *__restrict__ t, int R, int D)
{
    const int r = blockIdx.x;
    ln += (size_t)blockIdx.y * D; t += (size_t)blockIdx.y * 2 * R;       // one vector of a batch per blockIdx.y
    const float *a = r < R ? Aq + (size_t)r * D : Av + (size_t)(r - R) * D;
    float s = 0.f;
    if ((D & 3) == 0) {                                                   // 16-byte loads, eight pairs of them in flight per lane
        const float4 *a4 = reinterpret_cast<const float4 *>(a), *l4 = reinterpret_cast<const float4 *>(ln);
        const int n4 = D >> 2;
        for (int i0 = threadIdx.x; i0 < n4; i0 += 64 * 8) {
            float4 av[8], lv[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int i = i0 + 64 * u;
                av[u] = lv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (i < n4) { av[u] = a4[i]; lv[u] = l4[i]; }
            }
#pragma unroll
            for (int u = 0; u < 8; u++) s += av[u].x * lv[u].x + av[u].y * lv[u].y + av[u].z * lv[u].z + av[u].w * lv[u].w;
        }
    } else {
        for (int i = threadIdx.x; i < D; i += 64) s = fmaf(a[i], ln[i], s);
    }
    s = wave_sum(s);
    if (threadIdx.x == 0) t[r] = s;
}

// A product of the batched step as the GEMM leaves it (gemm_f32a_exact without its last part): S planes of [2B, N], rows
// b and B + b the value and residual images of sequence b, inv their factors.
struct SplitPlanes {
    const float *P, *inv;
    size_t plane;
    int S, N;
};
__device__ __forceinline__ float planes_at(const SplitPlanes &p, int B, int b, int n)
{
    return split_planes_value(p.P, p.S, p.plane, p.N, p.inv, B, b, n);
}

// act[b][i] = silu | gelu (gate) * up from the planes of the [gate | up] product of a batch
__global__ __launch_bounds__(TB) void k_glu_planes(SplitPlanes gu, float *__restrict__ act, int B, int IS, int gelu)
{
    const int b = blockIdx.y, i = blockIdx.x * TB + threadIdx.x;
    if (i >= IS) return;
    const float g = planes_at(gu, B, b, i), u = planes_at(gu, B, b, IS + i);
    float a;
    if (gelu) {                                                           // shaders/q8_kernels.metal:349-362
        float t = 0.7978845608f * (g + 0.044715f * g * g * g);
        t = fminf(fmaxf(t, -15.f), 15.f);
        a = 0.5f * g * (1.0f + tanhf(t));
    } else a = g / (1.0f + expf(-g));                                     // :337-347
    act[(size_t)b * IS + i] = a * u;
}

// k_add_norm for row blockIdx.x of a batch, with the branch taken from a product's planes (br.P) or absent, and with
// ln also written as the next product's operand: rows b and B + b of the tiled fp16 image a16 [2B, D] and their factors
// (what rows_to_f16_split makes of ln, element for element).  A thread holds elements tid + 1024 u, u < EPT, so
// 1024 EPT >= the padded row; the sums run in k_add_norm's order.
template <int EPT>
__global__ __launch_bounds__(1024) void k_add_norm_split(float *__restrict__ x, SplitPlanes br, const float *__restrict__ g_branch,
                                                         const float *__restrict__ g, float *__restrict__ ln,
                                                         half_t *__restrict__ a16, float *__restrict__ inv_out, int B, int D, float eps)
{
    __shared__ float sm[32];
    const int b = blockIdx.x, Kb = tiled_kb(D);
    x += (size_t)b * D;
    float bv[EPT], v[EPT], xv[EPT], gv[EPT], gbv[EPT];
    float inv_b = 1.f;
    // the row, the norm weights and the branch norm's weights are requested with the planes, not after the reductions
    // (a round trip each)
#pragma unroll
    for (int u = 0; u < EPT; u++) {
        const int i = threadIdx.x + 1024 * u;
        xv[u] = gv[u] = gbv[u] = 0.f;
        if (i < D) { xv[u] = x[i]; gv[u] = g[i]; if (br.P && g_branch) gbv[u] = g_branch[i]; }
    }
    if (br.P) {
#pragma unroll
        for (int u = 0; u < EPT; u++) { const int i = threadIdx.x + 1024 * u; bv[u] = i < D ? planes_at(br, B, b, i) : 0.f; }
        if (g_branch) {
            float ss = 0.f;
#pragma unroll
            for (int u = 0; u < EPT; u++) ss += bv[u] * bv[u];
            inv_b = rsqrtf(block_sum(ss, sm) / (float)D + eps);
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < EPT; u++) {
        const int i = threadIdx.x + 1024 * u;
        v[u] = 0.f;
        if (i < D) {
            v[u] = xv[u];
            if (br.P) { v[u] += g_branch ? bv[u] * inv_b * gbv[u] : bv[u]; x[i] = v[u]; }
        }
        ss += v[u] * v[u];
    }
    // the row maximum of v g, which the factor 1 / rms scales like every entry, goes through the same pair of barriers
    // as the sum of squares
    float mxg = 0.f;
#pragma unroll
    for (int u = 0; u < EPT; u++) mxg = fmaxf(mxg, fabsf(v[u] * gv[u]));
    block_sum_max(ss, mxg, sm);
    const float inv = rsqrtf(ss / (float)D + eps);
#pragma unroll
    for (int u = 0; u < EPT; u++) {
        const int i = threadIdx.x + 1024 * u;
        v[u] = i < D ? v[u] * inv * gv[u] : 0.f;
        if (ln && i < D) ln[(size_t)b * D + i] = v[u];
    }
    const float s = row_scale_for(mxg * inv), is = 1.0f / s;
    float lmax = 0.f;
#pragma unroll
    for (int u = 0; u < EPT; u++) {
        const int i = threadIdx.x + 1024 * u;
        const half_t h = f2h(v[u] * s);
        if (i < Kb * 64) a16[tiled_a_index(b, i, Kb)] = h;
        v[u] = v[u] - h2f(h) * is;
        lmax = fmaxf(lmax, fabsf(v[u]));
    }
    lmax = block_max(lmax, sm);
    const float s2 = row_scale_for(lmax);
#pragma unroll
    for (int u = 0; u < EPT; u++) {
        const int i = threadIdx.x + 1024 * u;
        if (i < Kb * 64) a16[tiled_a_index(B + b, i, Kb)] = f2h(v[u] * s2);
    }
    if (threadIdx.x == 0) { inv_out[b] = is; inv_out[B + b] = 1.0f / s2; }
}

MetalBuf *fbuf(size_t n) { return metal_buf_create(n * sizeof(float)); }

void matvec(InferenceState *s, const WMat *w, MetalBuf *x, MetalBuf *y)
{
    if (s->use_fp16) metal_enqueue_f16_matvec(w->mbuf, x, y, w->rows, w->cols);
    else metal_enqueue_q8_matvec(w->mbuf, x, y, w->rows, w->nb);
}

void add_norm(InferenceState *s, MetalBuf *x, MetalBuf *branch, MetalBuf *g_branch, MetalBuf *g)
{
    hipLaunchKernelGGL(k_add_norm, dim3(1), dim3(1024), 0, stream(), dptr_as<float>(x), branch ? dptr_as<float>(branch) : nullptr,
                       g_branch ? dptr_as<float>(g_branch) : nullptr, dptr_as<float>(g), dptr_as<float>(s->ln), s->D, s->eps);
}

// src/nn/fast_inference.c:376-467
void forward_token(InferenceState *s, int token, int pos)
{
    const int D = s->D, Hq = s->Hq, Hkv = s->Hkv, hd = s->hd;
    const bool gemma = s->model_type == MODEL_GEMMA3;
    hipLaunchKernelGGL(k_embed_row, dim3((D + TB - 1) / TB), dim3(TB), 0, stream(), dptr_as<float>(s->emb), token, s->emb_scale,
                       dptr_as<float>(s->x), D);
    MetalBuf *pending = nullptr, *pending_g = nullptr;           // FFN branch of the previous layer, added by the next norm kernel
    // Where the branch enters the sum as it is (Qwen3), the product after a norm forms sum and norm itself
    // (matvec_norm) and the sum goes to the other of two residual buffers; the Q|K|V product only without adapters,
    // whose down-projection reads the normed vector too.
    MetalBuf *x = s->x, *x_other = s->x2;
    const bool fuse_ffn = !gemma && D <= 12288, fuse_qkv = fuse_ffn && s->lora.empty();
    const int q8 = s->use_fp16 ? 0 : 1;
    auto normed_product = [&](MetalBuf *W, MetalBuf *branch, MetalBuf *g, MetalBuf *y, int rows, int glu) {
        NormIn n{dptr_as<float>(x), branch ? dptr_as<float>(branch) : nullptr, dptr_as<float>(g), branch ? dptr_as<float>(x_other) : nullptr,
                 s->eps};
        matvec_norm(W, n, y, rows, D, q8, glu);
        if (branch) std::swap(x, x_other);
    };
    for (int L = 0; L < s->NL; L++) {
        const InferenceState::Layer &lw = s->layers[L];
        if (fuse_qkv) normed_product(lw.qkv.mbuf, pending, lw.g_in, s->qkv, lw.qkv.rows, 0);
        else {
            add_norm(s, x, pending, pending_g, lw.g_in);
            matvec(s, &lw.qkv, s->ln, s->qkv);
        }
        // LoRA on q and v, per-head RMSNorm and RoPE on q and k, k and v into the caches, and the attention over the
        // cache: one launch (infer_kernels.hip: k_attn_decode<.., FUSED>)
        HeadPost a{};
        a.qkv = dptr_as<float>(s->qkv);
        a.g_q = lw.g_q ? dptr_as<float>(lw.g_q) : nullptr; a.g_k = lw.g_k ? dptr_as<float>(lw.g_k) : nullptr;
        a.kc = dptr_as<float>(s->kc[L]); a.vc = dptr_as<float>(s->vc[L]);
        a.Hq = Hq; a.Hkv = Hkv; a.pos = pos;
        a.rope = dptr_as<float2>(s->rope_tabs) + ((size_t)s->theta_slot[L] * s->max_seq + pos) * (hd / 2); a.eps = s->eps;
        if (!s->lora.empty()) {
            const InferenceState::Lora &lr = s->lora[L];
            hipLaunchKernelGGL(k_lora_down, dim3(2 * s->R), dim3(64), 0, stream(), dptr_as<float>(s->ln), dptr_as<float>(lr.Aq),
                               dptr_as<float>(lr.Av), dptr_as<float>(s->lora_t), s->R, D);
            a.t = dptr_as<float>(s->lora_t); a.Bq = dptr_as<float>(lr.Bq); a.Bv = dptr_as<float>(lr.Bv);
            a.R = s->R; a.sc = s->scaling;
        }
        // the O weights (F16 rows; up to 24 MB) travel while the attention's few workgroups run: 128 more workgroups ask
        // for them, 2.324 -> 2.290 ms per token (64: 2.305, 192: 2.305; 48 MB, i.e. part of the gate|up rows as well: no change)
        if (!q8) { a.pf_base = (const char *)dptr(lw.o->mbuf); a.pf_bytes = std::min<size_t>(lw.o->mbuf->size, (size_t)24 << 20) & ~(size_t)15; a.pf_wgs = 128; }
        attention_decode_fused(a, s->kc[L], s->vc[L], dptr_as<float>(s->att), hd, s->max_seq);
        mark_written(s->att);
        matvec(s, lw.o, s->att, s->branch);
        // x += o (Gemma3: RMSNorm(o; g_post_attn)); ln = RMSNorm(x; g_pre_ff | g_post_attn);
        // act = silu | gelu (gate) * up, formed in the epilogue of the [gate; up] product
        if (fuse_ffn) normed_product(lw.gu.mbuf, s->branch, lw.g_post_attn, s->gate_v, s->IS, 1);
        else {
            add_norm(s, x, s->branch, gemma ? lw.g_post_attn : nullptr, gemma ? lw.g_pre_ff : lw.g_post_attn);
            matvec_glu(lw.gu.mbuf, s->ln, s->gate_v, s->IS, D, q8, gemma ? 1 : 0);
        }
        matvec(s, lw.down, s->gate_v, s->branch);
        pending = s->branch;
        pending_g = gemma ? lw.g_post_ff : nullptr;
    }
    add_norm(s, x, pending, pending_g, s->g_final);
    HIP_CHECK(hipGetLastError());
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
    float *pv = dptr_as<float>(s->best) + 4;
    int *pi = dptr_as<int>(s->best) + 4 + AM_WGS;
    hipLaunchKernelGGL(k_argmax_part, dim3(AM_WGS), dim3(TB), 0, stream(), dptr_as<float>(s->logits), s->V, pv, pi);
    hipLaunchKernelGGL(k_argmax_final, dim3(1), dim3(AM_WGS), 0, stream(), pv, pi, dptr_as<int>(s->best));
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
                          const float *thetas, bool matvec_path = true)
{
    if (fast_metal_init() != 0) { fprintf(stderr, "[FastGen] no GPU: fast_metal_init failed\n"); return nullptr; }
    if (Hkv <= 0 || Hq % Hkv || hd > 256 || (hd & 1) || Hq / Hkv > 16 || max_seq <= 0 || (IS & 3)) {
        fprintf(stderr, "[FastGen] unsupported shape: %d / %d heads of %d (head_dim even and <= 256, group ratio <= 16, FFN width a multiple of 4)\n", Hq, Hkv, hd);
        fast_metal_shutdown();
        return nullptr;
    }
    InferenceState *s = new InferenceState();
    s->D = D; s->Hq = Hq; s->Hkv = Hkv; s->hd = hd; s->IS = IS; s->V = V; s->NL = NL;
    s->max_seq = max_seq; s->cur_len = 0; s->use_fp16 = use_fp16; s->model_type = mt;
    s->emb_scale = mt == MODEL_GEMMA3 ? sqrtf((float)D) : 1.0f;
    s->eps = 1e-6f;                                                       // src/nn/fast_inference.c:383
    s->thetas.assign(thetas, thetas + NL);
    {                                                                     // one table per distinct RoPE base
        std::vector<float> distinct;
        for (int L = 0; L < NL; L++) {
            size_t k = 0;
            while (k < distinct.size() && distinct[k] != thetas[L]) k++;
            if (k == distinct.size()) distinct.push_back(thetas[L]);
            s->theta_slot.push_back((int)k);
        }
        const size_t per = (size_t)max_seq * (hd / 2);
        s->rope_tabs = metal_buf_create(distinct.size() * per * sizeof(float2));
        for (size_t k = 0; k < distinct.size(); k++) launch_rope_table(dptr_as<float2>(s->rope_tabs) + k * per, max_seq, hd, distinct[k]);
    }
    default_eos(s);
    const int qd = Hq * hd, kd = Hkv * hd;
    HIP_CHECK(hipHostMalloc((void **)&s->logits_host, (size_t)V * 4, hipHostMallocDefault));
    HIP_CHECK(hipHostMalloc((void **)&s->best_host, sizeof(int), hipHostMallocDefault));
    if (matvec_path) {                                                    // scratch and caches of the matrix-vector pipeline
        s->x = fbuf(D); s->x2 = fbuf(D); s->branch = fbuf(D); s->ln = fbuf(D);
        s->qkv = fbuf(qd + 2 * kd); s->att = fbuf(qd);
        s->gu = fbuf(2 * (size_t)IS);
        s->gate_v = metal_buf_view(s->gu, 0, (size_t)IS * 4); s->up_v = metal_buf_view(s->gu, (size_t)IS * 4, (size_t)IS * 4);
        s->logits = fbuf(V); s->best = metal_buf_create((4 + 2 * AM_WGS) * sizeof(int));   // result, then the per-workgroup (value, index) pairs
        const size_t cache_bytes = (size_t)Hkv * max_seq * hd * sizeof(float);
        for (int L = 0; L < NL; L++) { s->kc.push_back(metal_buf_create(cache_bytes)); s->vc.push_back(metal_buf_create(cache_bytes)); }
    }
    s->R = 0; s->scaling = 0.f; s->lora_t = nullptr;
    s->sft = nullptr; s->owns_weights = 0;
    s->layers.resize(NL);
    s->lm_head = nullptr; s->g_final = s->emb = nullptr;
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
    // [Wq; Wk; Wv] and [Wgate; Wup] are converted as one matrix each: F16 rounding and Q8_0 blocks are per row, so
    // the rows of the fused matrix are bit for bit those of wmat_create_f16 / wmat_create_q8 on the parts
    std::vector<float> cat;
    auto fused = [&](std::initializer_list<const WeightRef *> parts) {
        int rows = 0;
        const int cols = (*parts.begin())->cols;
        for (const WeightRef *w : parts) rows += w->rows;
        cat.resize((size_t)rows * cols);
        size_t o = 0;
        for (const WeightRef *w : parts) { memcpy(cat.data() + o, w->data, (size_t)w->rows * cols * sizeof(float)); o += (size_t)w->rows * cols; }
        WMat *t = wmat_convert(cat.data(), rows, cols, use_fp16);
        WMat out = *t;
        free(t);                                                          // the handle only; the buffer lives on in `out`
        return out;
    };
    for (int L = 0; L < m->n_layers; L++) {
        const LayerWeightRef *r = &m->layers[L];
        InferenceState::Layer &lw = s->layers[L];
        lw.qkv = fused({&r->q_proj, &r->k_proj, &r->v_proj});
        lw.gu = fused({&r->gate_proj, &r->up_proj});
        lw.o = wmat_convert(r->o_proj.data, r->o_proj.rows, r->o_proj.cols, use_fp16);
        lw.down = wmat_convert(r->down_proj.data, r->down_proj.rows, r->down_proj.cols, use_fp16);
        lw.g_in = norm_upload(r->input_norm_g, r->d_model);
        lw.g_post_attn = norm_upload(r->post_attn_norm_g, r->d_model);
        lw.g_pre_ff = r->pre_ff_norm_g ? norm_upload(r->pre_ff_norm_g, r->d_model) : nullptr;
        lw.g_post_ff = r->post_ff_norm_g ? norm_upload(r->post_ff_norm_g, r->d_model) : nullptr;
        lw.g_q = r->q_norm_g ? norm_upload(r->q_norm_g, r->head_dim) : nullptr;
        lw.g_k = r->k_norm_g ? norm_upload(r->k_norm_g, r->head_dim) : nullptr;
    }
    s->lm_head = wmat_convert(m->lm_head, m->vocab_size, m->d_model, use_fp16);
    s->g_final = norm_upload(m->final_norm_g, m->d_model);
    s->emb = metal_buf_from_data(m->token_emb, (size_t)m->vocab_size * m->d_model * sizeof(float));
    s->owns_weights = 1;
    return s;
}

// Straight from the file to HBM: every matrix is uploaded as stored and converted on the GPU (F16 and Q8_0 tensors that
// already have the wanted format are used bit for bit); Q|K|V and gate|up are joined by device copies of whole rows.
InferenceState *inference_state_create_from_file(const char *path, ModelType model_type, int max_seq_len, int use_fp16)
{
    ModelFile *f = model_file_open(path);
    if (!f) return nullptr;
    const bool gg = model_file_is_gguf(f);
    if (gg && model_type == MODEL_GEMMA3) { fprintf(stderr, "[FastGen] Gemma3 is read from safetensors only\n"); model_file_close(f); return nullptr; }
    auto lname = [&](int L, const char *hf, const char *g) {
        char buf[256];
        if (gg) snprintf(buf, sizeof buf, "blk.%d.%s.weight", L, g); else snprintf(buf, sizeof buf, "model.layers.%d.%s.weight", L, hf);
        return std::string(buf);
    };
    const char *emb_name = gg ? "token_embd.weight" : "model.embed_tokens.weight";
    int V = 0, D = 0, NL = 0, qd = 0, kd = 0, IS = 0, hd = 0, one = 0, c = 0;
    bool ok = model_file_matrix_shape(f, emb_name, &V, &D) != 0;
    while (ok && model_file_find(f, lname(NL, "self_attn.q_proj", "attn_q").c_str(), nullptr, nullptr, nullptr)) NL++;
    ok = ok && NL > 0 && model_file_matrix_shape(f, lname(0, "self_attn.q_proj", "attn_q").c_str(), &qd, &c) && c == D &&
         model_file_matrix_shape(f, lname(0, "self_attn.k_proj", "attn_k").c_str(), &kd, &c) && c == D &&
         model_file_matrix_shape(f, lname(0, "mlp.gate_proj", "ffn_gate").c_str(), &IS, &c) && c == D &&
         model_file_matrix_shape(f, lname(0, "self_attn.q_norm", "attn_q_norm").c_str(), &one, &hd) && hd > 0 && qd % hd == 0 && kd % hd == 0;
    if (!ok) { fprintf(stderr, "[FastGen] %s: embedding or layer 0 tensors missing or inconsistent\n", path); model_file_close(f); return nullptr; }
    const bool gemma = model_type == MODEL_GEMMA3;
    std::vector<float> thetas(NL);
    for (int L = 0; L < NL; L++) thetas[L] = gemma ? ((L % 6) != 0 ? 1e4f : 1e6f) : 1e6f;   // src/nn/fast_sft.c:308-313
    InferenceState *s = new_state(model_type, D, qd / hd, kd / hd, hd, IS, V, NL, max_seq_len, use_fp16, thetas.data());
    if (!s) { model_file_close(f); return nullptr; }
    s->owns_weights = 1;
    auto gamma = [&](const std::string &name, int dim) -> MetalBuf * {
        size_t n = 0;
        float *g = model_file_load_f32(f, name.c_str(), &n);
        if (!g || (int)n != dim) { free(g); ok = false; return nullptr; }
        if (gemma) for (size_t i = 0; i < n; i++) g[i] += 1.0f;                            // src/nn/gemma3.c:259-278
        MetalBuf *b = norm_upload(g, dim);
        free(g);
        return b;
    };
    auto matrix = [&](const std::string &name, int rows, int cols) -> WMat * {
        WMat *w = model_file_load_wmat(f, name.c_str(), use_fp16);
        if (!w || w->rows != rows || w->cols != cols) { fprintf(stderr, "[FastGen] %s: expected %d x %d\n", name.c_str(), rows, cols); wmat_free(w); ok = false; return nullptr; }
        return w;
    };
    auto fuse = [&](std::initializer_list<WMat *> parts, int cols) {
        int rows = 0;
        for (WMat *w : parts) { if (!w) return WMat{nullptr, 0, 0, 0}; rows += w->rows; }
        const size_t row_bytes = use_fp16 ? (size_t)cols * 2 : (size_t)(cols / 32) * 34;
        WMat out{metal_buf_create((size_t)rows * row_bytes), rows, cols, use_fp16 ? 0 : cols / 32};
        size_t o = 0;
        for (WMat *w : parts) {
            HIP_CHECK(hipMemcpyAsync((char *)dptr(out.mbuf) + o, dptr(w->mbuf), (size_t)w->rows * row_bytes, hipMemcpyDeviceToDevice, stream()));
            o += (size_t)w->rows * row_bytes;
        }
        mark_written(out.mbuf);
        for (WMat *w : parts) wmat_free(w);                                                // synchronises the stream first
        return out;
    };
    for (int L = 0; L < NL && ok; L++) {
        InferenceState::Layer &lw = s->layers[L];
        lw.g_in = gamma(lname(L, "input_layernorm", "attn_norm"), D);
        lw.qkv = fuse({matrix(lname(L, "self_attn.q_proj", "attn_q"), qd, D), matrix(lname(L, "self_attn.k_proj", "attn_k"), kd, D),
                       matrix(lname(L, "self_attn.v_proj", "attn_v"), kd, D)}, D);
        lw.g_q = gamma(lname(L, "self_attn.q_norm", "attn_q_norm"), hd);
        lw.g_k = gamma(lname(L, "self_attn.k_norm", "attn_k_norm"), hd);
        lw.o = matrix(lname(L, "self_attn.o_proj", "attn_output"), D, qd);
        lw.g_post_attn = gamma(lname(L, "post_attention_layernorm", "ffn_norm"), D);
        if (gemma) lw.g_pre_ff = gamma(lname(L, "pre_feedforward_layernorm", ""), D);
        lw.gu = fuse({matrix(lname(L, "mlp.gate_proj", "ffn_gate"), IS, D), matrix(lname(L, "mlp.up_proj", "ffn_up"), IS, D)}, D);
        lw.down = matrix(lname(L, "mlp.down_proj", "ffn_down"), D, IS);
        if (gemma) lw.g_post_ff = gamma(lname(L, "post_feedforward_layernorm", ""), D);
    }
    if (ok) {
        s->g_final = gamma(gg ? "output_norm.weight" : "model.norm.weight", D);
        const char *head = gg ? "output.weight" : "lm_head.weight";
        const bool tied = gemma || !model_file_find(f, head, nullptr, nullptr, nullptr);   // src/nn/qwen3.c:264-270, 363-367
        s->lm_head = matrix(tied ? emb_name : head, V, D);
        size_t n = 0;
        float *emb = model_file_load_f32(f, emb_name, &n);
        if (emb && n == (size_t)V * D) s->emb = metal_buf_from_data(emb, n * sizeof(float)); else ok = false;
        free(emb);
    }
    model_file_close(f);
    if (!ok) { fprintf(stderr, "[FastGen] %s: a tensor is missing or mis-shaped\n", path); inference_state_free(s); return nullptr; }
    return s;
}

InferenceState *inference_state_create_from_sft(SFTState *sft, int max_seq_len)
{
    InferenceState *s = new_state(sft_get_model_type(sft), sft_get_d_model(sft), sft_get_n_q_heads(sft), sft_get_n_kv_heads(sft),
                                  sft_get_head_dim(sft), sft_get_intermediate_size(sft), sft_get_vocab_size(sft),
                                  sft_get_n_layers(sft), max_seq_len, 1, sft_get_rope_thetas(sft), false);
    if (!s) return nullptr;
    if (s->D > 8192) { fprintf(stderr, "[FastGen] hidden size %d not supported for a state on a training state's weights (<= 8192)\n", s->D); inference_state_free(s); return nullptr; }
    s->sft = sft;
    s->g_final = sft_get_final_norm_g(sft);
    s->emb = sft_get_token_emb_buf(sft);
    s->borrows_tiles = 1;
    s->borrowed.resize(s->NL);
    for (int L = 0; L < s->NL; L++) {
        sft_borrow_layer(sft, L, &s->borrowed[L]);
        const BorrowedLayer &b = s->borrowed[L];
        InferenceState::Layer &lw = s->layers[L];
        lw.g_in = b.g_in; lw.g_post_attn = b.g_post_attn; lw.g_pre_ff = b.g_pre_ff; lw.g_post_ff = b.g_post_ff; lw.g_q = b.g_q; lw.g_k = b.g_k;
    }
    s->borrowed_lm = sft_borrow_lm_head(sft);
    s->use_fp16 = s->borrowed_lm.fmt == 0;
    inference_state_set_lora(s, sft);
    return s;
}

// Kept for callers written against copies: a state made from a training state reads that state's weights in place, so
// there is nothing to refresh after a full-parameter update.
void inference_state_refresh_from_sft(InferenceState *s) { (void)s; }

void inference_state_set_lora(InferenceState *s, SFTState *sft)
{
    const int R = sft_get_lora_rank(sft);
    if (R == 0) return;                                                   // full-parameter state: no adapters
    if (!s->lora_t && !s->borrows_tiles) s->lora_t = fbuf(2 * (size_t)R);
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
    batch_release(s->batch);
    batch_release(s->single);
    for (MetalBuf *b : {s->gate_v, s->up_v, s->x, s->x2, s->branch, s->ln, s->qkv, s->att, s->gu, s->logits, s->best, s->lora_t, s->rope_tabs})
        metal_buf_free(b);
    for (MetalBuf *b : s->kc) metal_buf_free(b);
    for (MetalBuf *b : s->vc) metal_buf_free(b);
    hipHostFree(s->logits_host);
    hipHostFree(s->best_host);
    for (InferenceState::Layer &lw : s->layers) {
        metal_buf_free(lw.qkv.mbuf);
        metal_buf_free(lw.gu.mbuf);
        if (s->owns_weights) {
            wmat_free(lw.o); wmat_free(lw.down);
            for (MetalBuf *b : {lw.g_in, lw.g_post_attn, lw.g_pre_ff, lw.g_post_ff, lw.g_q, lw.g_k}) metal_buf_free(b);
        }
    }
    if (s->owns_weights) {
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

static void step_token(InferenceState *s, int token, int pos)
{
    if (s->borrows_tiles) step_on_tiles(s, token, pos);
    else forward_token(s, token, pos);
}
static int argmax_host(InferenceState *s) { return s->borrows_tiles ? argmax_on_tiles(s) : argmax_to_host(s); }

const float *inference_forward_token(InferenceState *s, int token)
{
    if (!token_ok(s, token)) return nullptr;
    step_token(s, token, s->cur_len);
    s->cur_len++;
    return s->borrows_tiles ? logits_on_tiles(s) : logits_to_host(s);
}

int inference_forward_token_argmax(InferenceState *s, int token)
{
    if (!token_ok(s, token)) return -1;
    step_token(s, token, s->cur_len);
    s->cur_len++;
    return argmax_host(s);
}

int inference_generate(InferenceState *s, const uint32_t *prompt_tokens, int prompt_len, uint32_t *output_tokens, int max_gen_len)
{
    s->cur_len = 0;
    if (prompt_len <= 0 || max_gen_len <= 0 || prompt_len > s->max_seq) return 0;
    for (int i = 0; i < prompt_len; i++) {
        if (!token_ok(s, (int)prompt_tokens[i])) return 0;
        step_token(s, (int)prompt_tokens[i], i);                      // prefill: only the last logits are looked at
        s->cur_len = i + 1;
    }
    int next = argmax_host(s);
    output_tokens[0] = (uint32_t)next;
    int n_gen = 1;
    for (int gen = 1; gen < max_gen_len && s->cur_len < s->max_seq; gen++) {
        bool is_eos = false;
        for (int e = 0; e < s->n_eos; e++) is_eos |= next == s->eos[e];
        if (is_eos) break;
        step_token(s, next, s->cur_len);
        s->cur_len++;
        next = argmax_host(s);
        output_tokens[n_gen++] = (uint32_t)next;
    }
    return n_gen;
}

namespace {

// the embedding rows of a batch of tokens, scaled: x[b] = emb[tokens.id[b]] * scale
struct TokenIds { int id[32]; };
__global__ __launch_bounds__(TB) void k_embed_rows(const float *__restrict__ emb, TokenIds tokens, float scale, float *__restrict__ x, int D)
{
    const int i = blockIdx.x * TB + threadIdx.x, b = blockIdx.y;
    if (i < D) x[(size_t)b * D + i] = emb[(size_t)tokens.id[b] * D + i] * scale;
}

// k_argmax_part and k_argmax_final for every vector of a batch at once (blockIdx.y: the vector)
__global__ __launch_bounds__(TB) void k_argmax_part_batch(const float *__restrict__ v, int n, float *__restrict__ pv, int *__restrict__ pi)
{
    __shared__ float bv[4];
    __shared__ int bi[4];
    v += (size_t)blockIdx.y * n; pv += (size_t)blockIdx.y * AM_WGS; pi += (size_t)blockIdx.y * AM_WGS;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = blockIdx.x * TB + threadIdx.x; i < n; i += AM_WGS * TB) am_pick(best, idx, v[i], i);
    am_block(best, idx, bv, bi);
    if (threadIdx.x == 0) { pv[blockIdx.x] = best; pi[blockIdx.x] = idx; }
}

__global__ __launch_bounds__(AM_WGS) void k_argmax_final_batch(const float *__restrict__ pv, const int *__restrict__ pi, int *__restrict__ out)
{
    __shared__ float bv[AM_WGS / 64];
    __shared__ int bi[AM_WGS / 64];
    float best = pv[(size_t)blockIdx.x * AM_WGS + threadIdx.x];
    int idx = pi[(size_t)blockIdx.x * AM_WGS + threadIdx.x];
    am_block(best, idx, bv, bi);
    if (threadIdx.x == 0) out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
}

// Scratch and KV caches of a batch of B sequences decoded in lock step (BatchState of src/nn/fast_inference.c:699-776).
struct BatchRun {
    int B, R, len;                                                       // sequences; adapter rank the scratch was sized for; positions held by the caches
    MetalBuf *x, *ln, *qkv, *att, *act, *logits, *best, *lora_t;
    MetalBuf *a16, *inv_ln, *inv_br, *planes;                            // a product's operand, its factors (of ln | of att and act), its planes
    std::vector<MetalBuf *> kc, vc;                                      // per layer: [B][Hkv, max_seq, hd]
    int *best_host;
};

void batch_release(BatchRun *r)
{
    if (!r) return;
    for (MetalBuf *b : {r->x, r->ln, r->qkv, r->att, r->act, r->logits, r->best, r->lora_t, r->a16, r->inv_ln, r->inv_br, r->planes}) metal_buf_free(b);
    for (MetalBuf *b : r->kc) metal_buf_free(b);
    for (MetalBuf *b : r->vc) metal_buf_free(b);
    if (r->best_host) hipHostFree(r->best_host);
    delete r;
}

// One step for B tokens at the same position: forward_token_batch, src/nn/fast_inference.c:808-893.  Every product
// reads its weight once for all B vectors (matrix cores over the tiled image, the arithmetic of gemm_f32a_exact); what
// is per sequence -- adapter terms, per-head RMSNorm, RoPE, cache store, attention -- has the sequence as a grid
// dimension, so a layer is the same 11 launches (12 with adapters) for any B.  A product's planes are summed by the kernel
// that consumes them and the norm kernel writes the next product's operand itself, where a row is one workgroup's.
void forward_token_batch(InferenceState *s, BatchRun &r, const int *tokens, int pos)
{
    const int D = s->D, Hq = s->Hq, Hkv = s->Hkv, hd = s->hd, IS = s->IS, B = r.B;
    const int qd = Hq * hd, kd = Hkv * hd, nqkv = qd + 2 * kd;
    const bool gemma = s->model_type == MODEL_GEMMA3;
    TokenIds ids{};
    for (int b = 0; b < B; b++) ids.id[b] = tokens[b];
    hipLaunchKernelGGL(k_embed_rows, dim3((D + TB - 1) / TB, B), dim3(TB), 0, stream(), dptr_as<float>(s->emb), ids, s->emb_scale,
                       dptr_as<float>(r.x), D);
    half_t *a16 = dptr_as<half_t>(r.a16);
    float *inv_ln = dptr_as<float>(r.inv_ln), *inv_br = dptr_as<float>(r.inv_br), *P = dptr_as<float>(r.planes);
    // x += branch (the planes `br` of the product before, none at the start); ln = RMSNorm(x) as fp32 (only the adapters
    // read it) and as the operand of the next product
    auto add_norm_b = [&](const SplitPlanes &br, MetalBuf *g_branch, MetalBuf *g) {
        float *ln = (s->lora.empty() || s->borrows_tiles) ? nullptr : dptr_as<float>(r.ln);      // fp32 copy: only k_lora_down reads it
        const float *gb = g_branch ? dptr_as<float>(g_branch) : nullptr;
        if (tiled_kb(D) * 64 <= 4096)
            hipLaunchKernelGGL(k_add_norm_split<4>, dim3(B), dim3(1024), 0, stream(), dptr_as<float>(r.x), br, gb, dptr_as<float>(g), ln,
                               a16, inv_ln, B, D, s->eps);
        else
            hipLaunchKernelGGL(k_add_norm_split<8>, dim3(B), dim3(1024), 0, stream(), dptr_as<float>(r.x), br, gb, dptr_as<float>(g), ln,
                               a16, inv_ln, B, D, s->eps);
    };
    // planes of (the operand in a16) x w^T; `inv`: the factors that operand's rows were split with.  The weight: the
    // tiled image of the state's own row-major matrix (made on first use), or the training state's tiles
    auto product = [&](const WMat *w, const WeightOp *tiles, int rows, int cols, const float *inv) {
        const WeightOp op = tiles ? *tiles : weight_f16(tiled_weight_of(w->mbuf, rows, cols));
        const GemmPlan p = plan_gemm(2 * B, rows, cols, op.fmt ? op.nbq : 0, op.fmt);
        const size_t plane = (size_t)2 * B * rows;
        launch_gemm(a16, nullptr, op, P, rows, plane, 2 * B, rows, cols, p);
        return SplitPlanes{P, inv, plane, p.S, rows};
    };
    const bool bt = s->borrows_tiles;
    auto split = [&](MetalBuf *in, int K) { launch_rows_to_f16_split(dptr_as<float>(in), a16, inv_br, B, K); };
    SplitPlanes pending{};                                               // FFN branch of the layer before, added by the next norm kernel
    MetalBuf *pending_g = nullptr;
    for (int L = 0; L < s->NL; L++) {
        const InferenceState::Layer &lw = s->layers[L];
        const BorrowedLayer *bl = bt ? &s->borrowed[L] : nullptr;
        add_norm_b(pending, pending_g, lw.g_in);
        // a training state's fused matrix continues with the rows of A_q and A_v (their fp16 images, as its own forward
        // reads them): the product then yields the adapters' down-projections as well, and no launch forms them
        const bool t_in_product = bt && !s->lora.empty();
        const int nq_rows = nqkv + (t_in_product ? 2 * s->R : 0);
        const SplitPlanes qkv = product(&lw.qkv, bt ? &bl->qkv : nullptr, nq_rows, D, inv_ln);
        launch_reduce_planes_split(qkv.P, qkv.S, qkv.plane, qkv.N, qkv.inv, dptr_as<float>(r.qkv), B, qkv.N);
        HeadPost a{};
        a.qkv = dptr_as<float>(r.qkv); a.qkv_step = (size_t)nq_rows;
        a.g_q = lw.g_q ? dptr_as<float>(lw.g_q) : nullptr; a.g_k = lw.g_k ? dptr_as<float>(lw.g_k) : nullptr;
        a.kc = dptr_as<float>(r.kc[L]); a.vc = dptr_as<float>(r.vc[L]); a.cache_step = (size_t)Hkv * s->max_seq * hd;
        a.Hq = Hq; a.Hkv = Hkv; a.pos = pos;
        a.rope = dptr_as<float2>(s->rope_tabs) + ((size_t)s->theta_slot[L] * s->max_seq + pos) * (hd / 2); a.eps = s->eps;
        if (!s->lora.empty()) {
            const InferenceState::Lora &lr = s->lora[L];
            if (t_in_product) { a.t = dptr_as<float>(r.qkv) + nqkv; a.t_step = (size_t)nq_rows; }
            else {
                hipLaunchKernelGGL(k_lora_down, dim3(2 * s->R, B), dim3(64), 0, stream(), dptr_as<float>(r.ln), dptr_as<float>(lr.Aq),
                                   dptr_as<float>(lr.Av), dptr_as<float>(r.lora_t), s->R, D);
                a.t = dptr_as<float>(r.lora_t); a.t_step = (size_t)2 * s->R;
            }
            a.Bq = dptr_as<float>(lr.Bq); a.Bv = dptr_as<float>(lr.Bv); a.R = s->R; a.sc = s->scaling;
        }
        attention_decode_fused(a, r.kc[L], r.vc[L], dptr_as<float>(r.att), hd, s->max_seq, B);
        split(r.att, qd);
        const SplitPlanes o = product(lw.o, bt ? &bl->o : nullptr, D, qd, inv_br);
        add_norm_b(o, gemma ? lw.g_post_attn : nullptr, gemma ? lw.g_pre_ff : lw.g_post_attn);
        const SplitPlanes gu = product(&lw.gu, bt ? &bl->gu : nullptr, 2 * IS, D, inv_ln);
        hipLaunchKernelGGL(k_glu_planes, dim3((IS + TB - 1) / TB, B), dim3(TB), 0, stream(), gu, dptr_as<float>(r.act), B, IS, gemma ? 1 : 0);
        split(r.act, IS);
        pending = product(lw.down, bt ? &bl->down : nullptr, D, IS, inv_br);
        pending_g = gemma ? lw.g_post_ff : nullptr;
    }
    add_norm_b(pending, pending_g, s->g_final);
    const SplitPlanes lg = product(s->lm_head, bt ? &s->borrowed_lm : nullptr, s->V, D, inv_ln);
    launch_reduce_planes_split(lg.P, lg.S, lg.plane, lg.N, lg.inv, dptr_as<float>(r.logits), B, lg.N);
    HIP_CHECK(hipGetLastError());
}

// argmax of every sequence's logits, computed on the GPU; one wait for all of them
void argmax_batch(InferenceState *s, BatchRun &r, int *out)
{
    float *pv = dptr_as<float>(r.best) + r.B;                            // [B][AM_WGS] values, then as many indices
    int *pi = reinterpret_cast<int *>(pv) + (size_t)r.B * AM_WGS;
    hipLaunchKernelGGL(k_argmax_part_batch, dim3(AM_WGS, r.B), dim3(TB), 0, stream(), dptr_as<float>(r.logits), s->V, pv, pi);
    hipLaunchKernelGGL(k_argmax_final_batch, dim3(r.B), dim3(AM_WGS), 0, stream(), pv, pi, dptr_as<int>(r.best));
    HIP_CHECK(hipMemcpyAsync(r.best_host, dptr(r.best), (size_t)r.B * sizeof(int), hipMemcpyDeviceToHost, stream()));
    HIP_CHECK(hipStreamSynchronize(stream()));
    for (int b = 0; b < r.B; b++) out[b] = r.best_host[b];
}

// The state's batch run for B sequences: the one kept from the call before when that had the same B and rank (its buffers
// are strided by B), else a new one in its place.  Caches are not cleared: a step at position pos reads what steps
// 0..pos-1 of the same run wrote.
BatchRun &batch_acquire(InferenceState *s, BatchRun *&slot, int B)
{
    const int R = s->lora.empty() ? 0 : s->R;
    if (slot && slot->B == B && slot->R == R) return *slot;
    metal_flush();
    batch_release(slot);
    slot = new BatchRun{};
    BatchRun &r = *slot;
    const int D = s->D, qd = s->Hq * s->hd, kd = s->Hkv * s->hd, IS = s->IS, V = s->V;
    r.B = B; r.R = R; r.len = 0;
    r.x = fbuf((size_t)B * D); r.ln = fbuf((size_t)B * D);
    r.qkv = fbuf((size_t)B * (qd + 2 * kd + 2 * R)); r.att = fbuf((size_t)B * qd);
    r.act = fbuf((size_t)B * IS); r.logits = fbuf((size_t)B * V);
    size_t a16_elems = 0, plane_floats = 0;                              // the largest operand and planes of the step's products
    const int shapes[5][2] = {{qd + 2 * kd + (s->borrows_tiles ? 2 * R : 0), D}, {D, qd}, {2 * IS, D}, {D, IS}, {V, D}};
    const int fmt = s->borrows_tiles ? s->borrowed_lm.fmt : 0;
    for (const auto &nk : shapes) {
        a16_elems = std::max(a16_elems, tiled_elems(2 * B, nk[1]));
        for (int ring = 0; ring < 2; ring++)                             // either kernel policy may be switched in later
            for (int wide = 0; wide <= ring; wide++) {                   // (the wide workgroups of the ring kernel may take twice the K chunks)
                const int was = gemm_ring_enabled(), wide_was = gemm_ring_wide_mode();
                set_gemm_ring(ring);
                set_gemm_ring_wide(wide);
                const int nbq = !fmt ? 0 : &nk == &shapes[0] ? tiled_rb(qd + 2 * kd) : tiled_rb(nk[0]);   // the adapter rows are F16 tiles
                plane_floats = std::max(plane_floats, (size_t)plan_gemm(2 * B, nk[0], nk[1], nbq, fmt).S * 2 * B * nk[0]);
                set_gemm_ring(was);
                set_gemm_ring_wide(wide_was);
            }
    }
    r.a16 = metal_buf_create(a16_elems * sizeof(half_t)); r.planes = fbuf(plane_floats);
    r.inv_ln = fbuf((size_t)2 * B); r.inv_br = fbuf((size_t)2 * B);
    r.best = metal_buf_create(((size_t)B + (size_t)B * 2 * AM_WGS) * sizeof(int));
    r.lora_t = R ? fbuf((size_t)B * 2 * R) : nullptr;
    HIP_CHECK(hipHostMalloc((void **)&r.best_host, (size_t)B * sizeof(int), hipHostMallocDefault));
    const size_t cache_bytes = (size_t)s->Hkv * s->max_seq * s->hd * sizeof(float);
    for (int L = 0; L < s->NL; L++) { r.kc.push_back(metal_buf_create(cache_bytes * B)); r.vc.push_back(metal_buf_create(cache_bytes * B)); }
    return r;
}

void step_on_tiles(InferenceState *s, int token, int pos)
{
    BatchRun &r = batch_acquire(s, s->single, 1);
    forward_token_batch(s, r, &token, pos);
    r.len = pos + 1;
}
const float *logits_on_tiles(InferenceState *s)
{
    HIP_CHECK(hipMemcpyAsync(s->logits_host, dptr(s->single->logits), (size_t)s->V * 4, hipMemcpyDeviceToHost, stream()));
    HIP_CHECK(hipStreamSynchronize(stream()));
    return s->logits_host;
}
int argmax_on_tiles(InferenceState *s)
{
    int best = 0;
    argmax_batch(s, *s->single, &best);
    return best;
}

bool batch_args_ok(InferenceState *s, int B)
{
    if (!s->use_fp16 && !s->borrows_tiles) { fprintf(stderr, "[BatchGen] F16 weights only\n"); return false; }
    if (B < 1 || B > 32) return false;
    if (s->D > 8192) { fprintf(stderr, "[BatchGen] hidden size %d not supported (<= 8192)\n", s->D); return false; }
    return true;
}

}  // namespace

// qwen3_generate_fast_batch, src/nn/fast_inference.c:895-1000, on a state's weights: batch_size copies of one prompt are
// prefilled and then decoded greedily in lock step, so that a step reads every weight once for all of them.  The loop
// ends when every sequence has emitted an end token (the state's EOS ids, or token 0 as in the reference, :944-947),
// after max_gen_len tokens or when the cache is full; sequences that have ended keep being stepped and written, as in
// the reference.  output_tokens: [batch_size][max_gen_len].  Returns the tokens written per sequence, 0 when the
// arguments do not fit (F16 weights only, 1 <= batch_size <= 32, prompt within the cache).
int inference_generate_batch(InferenceState *s, const uint32_t *prompt_tokens, int prompt_len, uint32_t *output_tokens,
                             int max_gen_len, int batch_size)
{
    const int B = batch_size;
    if (!batch_args_ok(s, B) || prompt_len <= 0 || max_gen_len <= 0 || prompt_len > s->max_seq) return 0;
    for (int i = 0; i < prompt_len; i++)
        if (prompt_tokens[i] >= (uint32_t)s->V) { fprintf(stderr, "[BatchGen] token %u outside the vocabulary (%d)\n", prompt_tokens[i], s->V); return 0; }
    BatchRun &r = batch_acquire(s, s->batch, B);
    int tokens[32], next[32], active[32];
    for (int i = 0; i < prompt_len; i++) {                               // prefill: the same token for every sequence (:910-916)
        for (int b = 0; b < B; b++) tokens[b] = (int)prompt_tokens[i];
        forward_token_batch(s, r, tokens, i);
    }
    int cur_len = prompt_len;
    argmax_batch(s, r, next);
    for (int b = 0; b < B; b++) { output_tokens[(size_t)b * max_gen_len] = (uint32_t)next[b]; active[b] = 1; }
    int n_gen = 1;
    for (int gen = 1; gen < max_gen_len && cur_len < s->max_seq; gen++) {
        int any_active = 0;
        for (int b = 0; b < B; b++) {
            bool ended = next[b] == 0;
            for (int e = 0; e < s->n_eos; e++) ended |= next[b] == s->eos[e];
            if (active[b] && ended) active[b] = 0;
            any_active |= active[b];
        }
        if (!any_active) break;
        forward_token_batch(s, r, next, cur_len);
        cur_len++;
        argmax_batch(s, r, next);
        for (int b = 0; b < B; b++) output_tokens[(size_t)b * max_gen_len + n_gen] = (uint32_t)next[b];
        n_gen++;
    }
    r.len = cur_len;
    return n_gen;
}

// One lock-step step with a token of its own for every sequence (what forward_token_batch, src/nn/fast_inference.c:808-893,
// is given by a sampling caller): tokens[b] enters sequence b at position pos, logits [batch_size][vocab] come back when
// `logits` is not NULL.  Positions run 0, 1, 2, ... on the state's kept batch caches; pos = 0 starts new sequences, any
// other pos must be the one after the step before (of this call or of inference_generate_batch with the same batch_size).
// Returns 0, or -1 when the arguments do not fit.
int inference_step_batch(InferenceState *s, const int *tokens, int batch_size, int pos, float *logits)
{
    const int B = batch_size;
    if (!s || !tokens || !batch_args_ok(s, B) || pos < 0 || pos >= s->max_seq) return -1;
    for (int b = 0; b < B; b++)
        if (tokens[b] < 0 || tokens[b] >= s->V) { fprintf(stderr, "[BatchGen] token %d outside the vocabulary (%d)\n", tokens[b], s->V); return -1; }
    BatchRun &r = batch_acquire(s, s->batch, B);
    if (pos != 0 && pos != r.len) { fprintf(stderr, "[BatchGen] step at position %d, but the batch's caches hold %d\n", pos, r.len); return -1; }
    forward_token_batch(s, r, tokens, pos);
    r.len = pos + 1;
    if (logits) {
        HIP_CHECK(hipMemcpyAsync(logits, dptr(r.logits), (size_t)B * s->V * sizeof(float), hipMemcpyDeviceToHost, stream()));
        HIP_CHECK(hipStreamSynchronize(stream()));
    }
    return 0;
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
