// Host pipeline of the fused LoRA SFT step: state, forward, loss, backward,
// update.  Restates the sequencing of the reference's src/nn/fast_sft.c
// (forward_to_logits :616-752, sft_apply_ce_loss :754-760, sft_backward_ex
// :766-982, lora_update :1090-1107, sft_train_step :1113-1157) as ~20 launches
// per layer on one stream instead of ~82:
//   * Q, K, V and the two LoRA down-projections are ONE GEMM against the fused
//     weight [Wq; Wk; Wv; A_q; A_v]; gate and up are one GEMM against [Wg; Wu];
//   * every dX product of the backward uses a transposed copy of the weight made
//     at start-up, so it runs through the same weight-streaming kernel; the QKV
//     backward is one GEMM whose operand row is [dq | dk | dv | dh_q | dh_v];
//   * GEMM outputs stay as K-split partial planes that the next row kernel sums;
//   * saved activations are simply where the forward wrote them (no copies).
#include "backend.h"
#include "devutil.h"
#include "gemm.h"
#include "fused.h"
#include "../../include/sft_hip.h"
#include <math.h>
#include <string.h>
#include <vector>
#include <algorithm>
#include <unordered_map>

using namespace lmhip;

struct SFTState {
    int D, Hq, Hkv, hd, IS, V, NL, N, B, BN;
    int qd, kd, R, nq_ext;               // nq_ext = qd + 2kd + 2R rows of the fused QKV weight
    size_t st_qkv, st_qkvT, st_o, st_oT, st_gu, st_guT, st_d, st_dT, st_ln1;   // layer strides (elements) of the tiled weight arenas
    float eps, lora_scaling, emb_scale;
    ModelType model_type;
    int step_count, weight_format;
    std::vector<float> rope_thetas;
    int window;                          // sliding-window attention (sft_set_sliding_window): 0 = off, the reference's behaviour
    std::vector<int> layer_local;        // layers the window applies to
    MetalBuf *rope_tabs;                 // one (cos, sin) table [seq][hd/2] per distinct theta
    std::vector<int> rope_slot;          // layer -> table index

    // frozen weights, F16 in the GEMM's tiled layout, one arena per matrix kind with a fixed layer stride;
    // the ...T arenas hold the transposed matrices for the dX products
    MetalBuf *wqkv, *wqkvT, *wo, *woT, *wgu, *wguT, *wd, *wdT, *wlm, *wlmT;
    // Q8_0-native mode: the frozen matrices stay quantised in HBM (int8 tiles + fp16 scales, both orientations,
    // 1.0625 bytes per weight and image) and the GEMM dequantises on the fly; wqkv / wqkvT then hold only the F16
    // tiles of the LoRA A rows.  Layer strides are in tiles (32 x 64 weights).
    int q8_native;
    struct Q8Arena { MetalBuf *q, *d, *qT, *dT; size_t st, stT; } zqkv, zo, zgu, zd, zlm;
    MetalBuf *g_in, *g_post_attn, *g_pre_ff, *g_post_ff, *g_q, *g_k, *g_final;
    MetalBuf *emb;                       // fp32 [V, D]
    std::vector<LayerW> layer_views;     // WMat/MetalBuf windows handed out by sft_get_layers-style accessors

    // LoRA arena and optimiser state (fp32, device)
    size_t lsz, lora_n;
    MetalBuf *lora, *lora_grad, *adam_m, *adam_v, *sq_slots, *grad_norm;
    MetalBuf *lora16;                    // fp16 copy of `lora`, refreshed wherever the adapters are written (B_q, B_v for the QKV backward rows)
    int slots_per_layer;
    std::vector<MetalBuf *> lora_views, grad_views;

    // host-visible small buffers
    MetalBuf *tokens, *targets, *losses, *hyper, *x_in_host;
    uint32_t *tokens_cpu, *targets_cpu;
    float *losses_cpu, *hyper_cpu, *x_cpu;

    // saved activations (layer-strided arenas)
    MetalBuf *xs;                        // [2*NL + 1][BN*D]: x_in[L] = 2L, x_mid[L] = 2L+1, x_final = 2NL
    MetalBuf *ln1_16, *ln1_inv;          // [NL][BN*D] f16, [NL][BN]
    MetalBuf *q_pre, *k_pre, *q_fin, *k_fin, *v_sav, *probs, *gu_sav, *tq, *tv, *o_raw, *ff_raw;   // gu_sav: [NL][BN][gate (IS) | up (IS)]
    MetalBuf *kT, *vT;                   // k_fin / v_sav once more, per head and transposed, for the matrix-core attention
    // attention without saved probabilities (attn_flash.hip; probs, kT, vT, dO_red, dscore are then not allocated):
    // per layer the bf16-pair fragments of q, k, v ([RT | PT] each), the output and the row statistics
    int use_flash;
    MetalBuf *fa_q, *fa_k, *fa_v, *fa_O, *fa_lse, *fa_do, *fa_D, *fa_dkp, *fa_dvp;
    // transients
    MetalBuf *a16, *a16_inv;             // largest fp16 operand (BN x max K) and its row factors
    MetalBuf *group_inv;                 // row factors per column group [BN][MAX_SCALE_GROUPS]: never the buffer the
                                         // kernel that writes them reads its own input factors from
    MetalBuf *ones;                      // [BN] of 1.0f
    MetalBuf *planes;
    MetalBuf *logits, *dlogits, *dl16, *dl_inv;
    MetalBuf *dkp, *dvp;                 // dk / dv as shares per (query block, query head) where one launch forms dq and them (at most 64 keys)
    MetalBuf *dx[2], *dO_red, *dscore, *dq, *dk, *dv, *dq_f, *dh;   // LoRA mode: dv, dq_f, dh are kept per layer until the
                                                                   // adapter gradients of all layers are formed in one launch
    MetalBuf *ce_part;
    size_t planes_cap;

    // full-parameter mode (lora_rank == 0): the GEMM operands of the forward are kept per layer, because
    // every one of them is the X of a weight gradient dW = dY^T X
    int full_param;
    const float *token_emb_host;         // the caller's table, borrowed (src/nn/fast_sft.c:239)
    MetalBuf *ln2_16, *ln2_inv, *act16, *act_inv, *attn16, *lnf16, *lnf_inv;
    size_t st_act, st_attn;
    MetalBuf *xT, *xT_inv, *yT, *yT_inv; // transposed operands of the weight gradient being formed
    // accumulate mode: the loss-gradient operands of a layer's four products (down, gate|up, o, qkv) stay until its
    // backward has run, and all eight operands of its weight gradients are transposed in one launch
    MetalBuf *dy16[4], *dy_inv[4], *lyT[4], *lyT_inv[4], *lxT[4], *lxT_inv[4];
    MetalBuf *gqkv, *go, *ggu, *gd, *glm;   // F16 gradient accumulators, tiled like the weights (sft_alloc_grad_accum)
    MetalBuf *grpo_old_lp, *grpo_advs, *grpo_new_lp;   // host-visible [BN] inputs/outputs of the policy gradient
    float *grpo_old_lp_cpu, *grpo_advs_cpu, *grpo_new_lp_cpu;
    MetalBuf *lora_acc;                  // LoRA gradients summed over the completions of a GRPO group
    // Q8_0 states whose products run on the large-M kernel keep the F16 image of every frozen weight they have used
    // (dequantised once, not once per product), as long as all of them fit the budget
    std::unordered_map<const void *, MetalBuf *> img_slots;
    size_t img_bytes;
    int step_in_flight, step_rejected;   // sft_enqueue_train_step without its sft_finish_train_step yet; ids refused
    std::vector<LayerW> layers_out;      // row-major F16 copies handed out by sft_get_layers
    std::vector<WMat> wmats_out;
    std::vector<MetalBuf *> views_out;
    std::vector<MetalBuf *> gamma_views; // [NL][6] windows on the norm gammas for a generation state that borrows them
    // LoRA states of at most 64 rows on F16 weights: per frozen matrix (kind, as stored / transposed, layer) the power of
    // two with which the chunk sums of its products leave as halves (half_plane_scale of the matrix's largest row sum of
    // |w|); empty when the state's products do not take that path
    std::vector<float> half_scale[5][2];
    WMat lm_head_out;
};

enum { BWD_LORA = 0, BWD_ACCUM = 1, BWD_SGD = 2 };

namespace {

inline MetalBuf *fbuf(size_t n) { return metal_buf_create(n * sizeof(float)); }
inline MetalBuf *hbuf(size_t n) { return metal_buf_create(n * sizeof(half_t)); }
template <typename T> inline T *at(MetalBuf *b, size_t elem_off = 0) { return dptr_as<T>(b) + elem_off; }

struct Dest { MetalBuf *arena; size_t elem_off; int Kb; int row_off, k_off, transpose; };

// Upload one fp32 matrix [rows, cols], round it to F16 (Q8_0 mode: quantise, then take the
// dequantised values) and scatter it into tiled weight arenas: `a` as is, `b` transposed.
void put_matrix(SFTState *s, const float *src, int rows, int cols, const Dest &a, const Dest &b)
{
    const size_t n = (size_t)rows * cols;
    MetalBuf *stage = metal_buf_from_data(src, n * sizeof(float));
    MetalBuf *rm = metal_buf_create(n * sizeof(half_t));
    MetalBuf *q8 = nullptr;
    if (s->weight_format) {
        hip_enqueue_f32_to_f16(stage, rm, n);
    } else {
        q8 = metal_buf_create((size_t)rows * (cols / 32) * 34);
        hip_enqueue_q8_quantize(stage, q8, rows, cols);
        hip_enqueue_q8_to_f16(q8, rm, rows, cols);
    }
    for (const Dest *d : {&a, &b})
        launch_tile_f16(at<half_t>(rm), rows, cols, at<half_t>(d->arena, d->elem_off), d->Kb, d->row_off, d->k_off, d->transpose);
    metal_buf_free(rm);                                   // synchronises the stream first
    metal_buf_free(q8);
    metal_buf_free(stage);
}

struct QDest { MetalBuf *q, *d; size_t tile_off; int Kb; int row_off, k_off, transpose; };

// Q8_0-native upload: quantise (bit-exact GGML blocks) and scatter the blocks into the GEMM's int8 tiles,
// `a` with row scales, `b` (the transposed image) with column scales.
void put_matrix_q8(const float *src, int rows, int cols, const QDest &a, const QDest &b)
{
    const size_t n = (size_t)rows * cols;
    MetalBuf *stage = metal_buf_from_data(src, n * sizeof(float));
    MetalBuf *q8 = metal_buf_create((size_t)rows * (cols / 32) * 34);
    hip_enqueue_q8_quantize(stage, q8, rows, cols);
    for (const QDest *d : {&a, &b})
        launch_tile_q8(at<uint8_t>(q8), rows, cols, at<uint8_t>(d->q, d->tile_off * 2048), at<half_t>(d->d, d->tile_off * 64),
                       d->Kb, d->row_off, d->k_off, d->transpose);
    metal_buf_free(q8);                                   // synchronises the stream first
    metal_buf_free(stage);
}

enum { W_QKV = 0, W_O, W_GU, W_D, W_LM };

// The weight operand of one GEMM: matrix kind of layer L, as stored (T = false) or transposed.
WeightOp wop(SFTState *s, int kind, int L, bool T)
{
    MetalBuf *w16[5][2] = {{s->wqkv, s->wqkvT}, {s->wo, s->woT}, {s->wgu, s->wguT}, {s->wd, s->wdT}, {s->wlm, s->wlmT}};
    const size_t st16[5][2] = {{s->st_qkv, s->st_qkvT}, {s->st_o, s->st_oT}, {s->st_gu, s->st_guT}, {s->st_d, s->st_dT}, {0, 0}};
    if (!s->q8_native) return weight_f16(at<half_t>(w16[kind][T], (size_t)L * st16[kind][T]));
    SFTState::Q8Arena *z[5] = {&s->zqkv, &s->zo, &s->zgu, &s->zd, &s->zlm};
    const int qcols = s->qd + 2 * s->kd;                  // quantised part of the fused QKV matrix
    const int Nfwd[5] = {qcols, s->D, 2 * s->IS, s->D, s->V}, Kfwd[5] = {s->D, s->qd, s->D, s->IS, s->D};
    WeightOp w{};
    w.fmt = T ? 2 : 1;
    const size_t off = (size_t)L * (T ? z[kind]->stT : z[kind]->st);
    w.q = at<uint8_t>(T ? z[kind]->qT : z[kind]->q, off * 2048);
    w.d = at<half_t>(T ? z[kind]->dT : z[kind]->d, off * 64);
    w.nbq = tiled_rb(Nfwd[kind]);                         // forward image: every row block up to the LoRA rows
    w.kbq = T ? tiled_kb(Nfwd[kind]) : 0;                 // transposed image: the K steps that hold quantised columns
    (void)Kfwd;
    if (kind == W_QKV && s->R > 0) w.w16 = at<half_t>(T ? s->wqkvT : s->wqkv, (size_t)L * (T ? s->st_qkvT : s->st_qkv));
    return w;
}

size_t max_planes_elems(SFTState *s)
{
    struct Sh { int N, K; };
    const Sh shapes[] = {{s->nq_ext, s->D}, {s->D, s->qd}, {2 * s->IS, s->D}, {s->D, s->IS}, {s->V, s->D},
                         {s->D, s->V}, {s->IS, s->D}, {s->D, 2 * s->IS}, {s->qd, s->D}, {s->D, s->nq_ext}};
    size_t mx = 0;
    const int ring_was = gemm_ring_enabled(), wide_was = gemm_ring_wide_mode();   // the kernel family can be switched at run time: room for either
    for (int ring = 0; ring < 2; ring++)
    for (int wide = 0; wide <= ring; wide++)              // (the wide workgroups may take twice the K chunks)
    for (const Sh &sh : shapes) {
        set_gemm_ring(ring);
        set_gemm_ring_wide(wide);
        GemmPlan p = plan_gemm(s->BN, sh.N, sh.K, (s->q8_native && s->R > 0 && sh.N == s->nq_ext && sh.K == s->D) ? (s->qd + 2 * s->kd) / 32 : 0, s->q8_native ? 1 : 0);
        // whichever kernel the product takes (the choice can be forced at run time): the planes of the streaming kernel, or
        // up to four K chunks of the large-M one; the LM head writes the logits directly unless the streaming kernel splits K
        const bool head = sh.N == s->V && sh.K == s->D;
        const size_t e = (size_t)(head ? (p.S > 1 ? p.S : 0) : std::max({p.S, 4, big_gemm_chunks(s->BN, sh.N, sh.K, 0)})) * s->BN * sh.N;
        if (e > mx) mx = e;
    }
    set_gemm_ring(ring_was);
    set_gemm_ring_wide(wide_was);
    return mx;
}

constexpr int MAX_SCALE_GROUPS = 64;                      // group_inv holds this many factors per row

// Column groups for the row kernel that writes the operand [BN, K] of the product with W [N, K]: as many groups as it
// takes to put about two workgroups on every CU, each a power-of-two number of the GEMM's K chunks and at most 2048
// columns wide (a single chunk: up to 4096).  None (cols = 0) when the product does not leave planes (large M, S == 1) or the rows alone fill the GPU.
ScaleGroups scale_groups_for(SFTState *s, const WeightOp &W, int N, int K)
{
    ScaleGroups none{0, 1, 0};
    if (s->full_param || use_big_gemm(s->BN, N, K, W.fmt)) return none;      // weight gradients take one factor per row
    const GemmPlan p = plan_gemm(s->BN, N, K, (W.fmt == 1 && W.nbq < tiled_rb(N)) ? W.nbq : 0, W.fmt);
    const int plane_cols = p.steps * 64, cus = num_cus() > 0 ? num_cus() : 256;
    const int want = (2 * cus + s->BN - 1) / s->BN;
    if (p.S <= 1 || want <= 1 || plane_cols > 4096) return none;
    int shift = 0;
    while ((plane_cols << (shift + 1)) <= 2048 && ((p.S + (2 << shift) - 1) >> (shift + 1)) >= want) shift++;
    ScaleGroups g{plane_cols << shift, (p.S + (1 << shift) - 1) >> shift, shift};
    return g.groups <= MAX_SCALE_GROUPS ? g : none;
}

// What the workgroups a row kernel starts beyond its own request ahead for the product with W [N, K] that follows it.
// `threads`: block size of that kernel; `unit`: its prefetching workgroups come in multiples of this many (1 for a
// one-dimensional grid, else the size of a grid slice).  About 16 MB, the first K steps of as many of the product's
// workgroups as that covers: what fits beside the row kernel's own work in time.
WeightPrefetch prefetch_for(SFTState *s, const WeightOp &W, int N, int K, int threads, int unit = 1)
{
    // measured on config 3 (MI355X): 16 MB by 160 workgroups of 1024 threads shortens the product by 3 us and lengthens
    // the row kernel by 1.5; less fetches too little, more (or fewer, longer-running workgroups) holds the row kernel up
    constexpr int mb = 16, depth = 4, wgs1024 = 160;
    WeightPrefetch pf{};
    const bool q8 = W.fmt != 0;
    if (s->full_param || (!q8 && !W.w16) || use_big_gemm(s->BN, N, K, W.fmt)) return pf;
    const GemmPlan p = plan_gemm(s->BN, N, K, 0, W.fmt);
    if (p.m_tiles != 1 || unit <= 0) return pf;
    // Q8_0: the int8 tiles of the quantised part, two K steps per 4 KB load (an even number of K steps per row block)
    const int kbq = !q8 ? tiled_kb(K) : W.fmt == 1 ? tiled_kb(K) : W.kbq;
    const int nbq = W.fmt == 1 ? W.nbq : tiled_rb(N);
    if (q8 && (!p.ring || !W.q || kbq <= 0 || (kbq & 1) || nbq <= 0)) return pf;
    const long tile_bytes = q8 ? 2048 : 4096;
    int wgs = wgs1024 * (1024 / threads);
    wgs = (wgs + unit - 1) / unit * unit;
    pf.base = q8 ? reinterpret_cast<const char *>(W.q) : reinterpret_cast<const char *>(W.w16);
    pf.Kb = kbq; pf.Nb = nbq;
    pf.nb = p.nb; pf.steps = p.steps; pf.S = p.S; pf.n_tiles = p.n_tiles; pf.rotate = (p.rotate ? 1 : 0) | (q8 ? 2 : 0);
    // few workgroups with long chunks (gemm_ring): the same bytes reach further into each chunk
    const long total = (long)p.n_tiles * p.S;
    const int depth_q = q8 ? 2 * depth : depth;              // K steps: the same bytes
    int d = depth_q;
    if (total * p.nb * depth_q * tile_bytes < (long)mb * 1024 * 1024) d = (int)std::min<long>(p.steps, (long)mb * 1024 * 1024 / (total * p.nb * tile_bytes));
    if (d < depth_q) d = std::min(depth_q, p.steps);
    if (q8) d = (d + 1) & ~1;
    pf.wgs = wgs; pf.depth = q8 ? d / 2 : d;                 // loads per row block of a product workgroup
    const long covered = std::min<long>((long)mb * 1024 * 1024 / ((long)p.nb * d * tile_bytes), total);
    pf.per_wg = (int)((covered + wgs - 1) / wgs);
    return pf;
}

// The flash attention's buffers of layer L
AttnFlashArgs flash_args(SFTState *s, int L)
{
    AttnFlashArgs f{};
    const size_t eq = attn_flash_tile_elems(s->hd, s->N, s->Hq, s->B), ek = attn_flash_tile_elems(s->hd, s->N, s->Hkv, s->B);
    const size_t stat = (size_t)s->B * s->Hq * ((s->N + 31) / 32) * 32;
    f.Hq = s->Hq; f.Hkv = s->Hkv; f.hd = s->hd; f.seq = s->N; f.batch = s->B;
    f.window = (s->window > 0 && s->layer_local[L]) ? s->window : 0;
    f.scale = 1.0f / sqrtf((float)s->hd);
    f.q_rt = at<uint4>(s->fa_q, (size_t)L * 2 * eq); f.q_pt = f.q_rt + eq;
    f.k_rt = at<uint4>(s->fa_k, (size_t)L * 2 * ek); f.k_pt = f.k_rt + ek;
    f.v_rt = at<uint4>(s->fa_v, (size_t)L * 2 * ek); f.v_pt = f.v_rt + ek;
    f.do_rt = at<uint4>(s->fa_do); f.do_pt = f.do_rt + eq;
    f.O = at<float>(s->fa_O, (size_t)L * s->BN * s->qd); f.lse = at<float>(s->fa_lse, (size_t)L * stat); f.D = at<float>(s->fa_D);
    f.dkp = at<float>(s->fa_dkp); f.dvp = at<float>(s->fa_dvp);
    return f;
}

// F16 tiles of a weight for the large-M kernel.  A Q8_0 weight of a LoRA state is frozen, so its image is made once
// and kept (16 GB for the 4B model's two orientations; MI355X has the room, and the product then reads what it would
// read anyway); only the adapter rows of the fused QKV matrix, which every step changes, are copied again.  A weight
// whose image no longer fits the budget gets one per product in the scratch arena.
size_t g_image_budget = (size_t)64 << 30;
WeightOp resident_image(SFTState *s, const WeightOp &W, int N, int K)
{
    if (W.fmt == 0 || s->full_param || large_m_unpacks_q8() || !g_image_budget) return f16_image_of(W, N, K);
    auto it = s->img_slots.find(W.q);
    if (it != s->img_slots.end()) return f16_image_of(W, N, K, at<half_t>(it->second), true);
    const size_t bytes = tiled_elems(N, K) * sizeof(half_t);
    // no room in the budget, or on the device (2 GB kept free for everything allocated later): this weight's image is
    // made per product in the scratch arena instead
    size_t free_b = 0, total_b = 0;
    HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
    if (s->img_bytes + bytes > g_image_budget || free_b < bytes + ((size_t)2 << 30)) return f16_image_of(W, N, K);
    MetalBuf *slot = metal_buf_create(bytes);
    s->img_bytes += bytes;
    s->img_slots.emplace(W.q, slot);
    return f16_image_of(W, N, K, at<half_t>(slot), false);
}

// P = A16 * W^T as K-split planes in the state's plane buffer (operands tiled)
// The factor for the half planes of a product with matrix `kind` of layer L (0: fp32 planes).  Only where the consumer of
// the planes reads them through planes_at4_multi and the operand rows are scaled below 8192: gate|up and down forward,
// and the three frozen backward products.  (The O forward takes the attention output at unit scale, the Q|K|V products
// contain the adapter rows, which change.)
float half_scale_for(SFTState *s, int kind, int L, bool T)
{
    if (!gemm_half_planes_enabled() || kind < 0 || kind >= 5) return 0.f;
    const std::vector<float> &v = s->half_scale[kind][T ? 1 : 0];
    return (size_t)L < v.size() ? v[L] : 0.f;
}

// hscale != 0 (see half_scale_for): the planes of a ring product are written as halves
Planes gemm(SFTState *s, const half_t *A, const float *inv, const WeightOp &W, int N, int K, float *out = nullptr,
            const ScaleGroups *sg = nullptr, float hscale = 0.f)
{
    if (use_big_gemm(s->BN, N, K, W.fmt)) {                 // one launch; final output, or a few K chunks as planes
        float *C = out ? out : at<float>(s->planes);
        const WeightOp Wf = resident_image(s, W, N, K);
        const int chunks = out ? 1 : big_gemm_chunks_for(s->BN, N, K, Wf);
        const size_t stride = (size_t)s->BN * N;
        if (!out && chunks * stride > s->planes_cap) { fprintf(stderr, "[fast_sft] plane buffer too small\n"); abort(); }
        const int planes = launch_gemm_big(A, inv, Wf, C, N, s->BN, N, K, chunks, stride);
        return make_planes(C, planes, stride, N, nullptr);
    }
    GemmPlan p = plan_gemm(s->BN, N, K, (W.fmt == 1 && W.nbq < tiled_rb(N)) ? W.nbq : 0, W.fmt);
    float *P = out ? out : at<float>(s->planes);
    const size_t stride = (size_t)s->BN * N;
    if (!out && (size_t)p.S * stride > s->planes_cap) { fprintf(stderr, "[fast_sft] plane buffer too small\n"); abort(); }
    if (out && p.S != 1) { fprintf(stderr, "[fast_sft] direct GEMM output needs S == 1\n"); abort(); }
    // a direct (final) output gets its row factors in the GEMM epilogue; planes leave them to the consumer
    if (out || !p.ring) hscale = 0.f;
    launch_gemm(A, out ? inv : nullptr, W, P, N, stride, s->BN, N, K, p, hscale);
    const float unscale = hscale != 0.f ? 1.0f / hscale : 0.f;
    if (sg && sg->cols) {
        if (out || sg->cols != (p.steps * 64) << sg->shift || sg->groups != (p.S + (1 << sg->shift) - 1) >> sg->shift) {
            fprintf(stderr, "[fast_sft] column groups of the operand do not match the K chunks of the product\n"); abort();
        }
        return make_planes(P, p.S, stride, N, inv, sg->shift, sg->groups, unscale);
    }
    return make_planes(P, p.S, stride, N, out ? nullptr : inv, 0, 0, unscale);
}

void forward_impl(SFTState *s, bool gather, bool zero_rows = false)
{
    const int BN = s->BN, D = s->D, IS = s->IS, qd = s->qd, kd = s->kd, R = s->R;
    const size_t xsz = (size_t)BN * D;
    half_t *a16 = at<half_t>(s->a16);
    float *ainv = at<float>(s->a16_inv);
    const bool gemma = s->model_type == MODEL_GEMMA3;
    Planes pending = make_planes(nullptr, 0, 0, 0, nullptr);                    // FFN output of the previous layer, not yet added

    for (int L = 0; L < s->NL; L++) {
        float *x_in = at<float>(s->xs, (size_t)(2 * L) * xsz), *x_mid = at<float>(s->xs, (size_t)(2 * L + 1) * xsz);
        half_t *ln1 = at<half_t>(s->ln1_16, (size_t)L * s->st_ln1);
        float *ln1inv = at<float>(s->ln1_inv, (size_t)L * BN);

        // x_in = x (+ previous FFN branch); ln1 = RN(x_in; g_in)        [src/nn/fast_sft.c:631-635, 732-740]
        NormRowsArgs n1{};
        if (L == 0) {
            if (gather) { n1.emb = at<float>(s->emb); n1.tokens = at<uint32_t>(s->tokens); n1.emb_scale = s->emb_scale; n1.zero_rows = zero_rows; }
            else n1.x_prev = at<float>(s->x_in_host);
        } else {
            n1.x_prev = at<float>(s->xs, (size_t)(2 * L - 1) * xsz);
            n1.branch = pending;
            if (gemma) { n1.g_branch = at<float>(s->g_post_ff, (size_t)(L - 1) * D); n1.branch_raw_out = at<float>(s->ff_raw, (size_t)(L - 1) * xsz); }
        }
        n1.x_out = x_in;
        n1.g_norm = at<float>(s->g_in, (size_t)L * D);
        n1.ln16 = ln1; n1.inv_scale = ln1inv; n1.D = D; n1.eps = s->eps;
        n1.pf = prefetch_for(s, wop(s, W_QKV, L, false), s->nq_ext, D, 1024);
        launch_norm_rows(n1, BN);

        // [q | k | v | tq | tv] = ln1 [Wq; Wk; Wv; A_q; A_v]^T                 [:638-656]
        Planes pq = gemm(s, ln1, ln1inv, wop(s, W_QKV, L, false), s->nq_ext, D);
        QkvPostArgs qa{};
        qa.qkv = pq;
        qa.Bq = at<float>(s->lora, L * s->lsz + (size_t)R * D);
        qa.Bv = at<float>(s->lora, L * s->lsz + (size_t)2 * R * D + (size_t)qd * R);
        qa.R = R; qa.sc = s->lora_scaling;
        qa.g_q = at<float>(s->g_q, (size_t)L * s->hd); qa.g_k = at<float>(s->g_k, (size_t)L * s->hd);
        qa.eps = s->eps; qa.rope = at<float2>(s->rope_tabs, (size_t)s->rope_slot[L] * s->N * (s->hd / 2));
        qa.Hq = s->Hq; qa.Hkv = s->Hkv; qa.hd = s->hd; qa.seq = s->N;
        qa.q_pre = at<float>(s->q_pre, (size_t)L * BN * qd); qa.k_pre = at<float>(s->k_pre, (size_t)L * BN * kd);
        if (s->q_fin) {                                       // not kept by the attention that works on fragments
            qa.q_fin = at<float>(s->q_fin, (size_t)L * BN * qd); qa.k_fin = at<float>(s->k_fin, (size_t)L * BN * kd);
            qa.v_out = at<float>(s->v_sav, (size_t)L * BN * kd);
        }
        qa.tq = at<float>(s->tq, (size_t)L * BN * (R ? R : 1)); qa.tv = at<float>(s->tv, (size_t)L * BN * (R ? R : 1));
        const size_t st_kt = (size_t)s->B * kd * attn_ldt(s->N);
        if (s->kT) { qa.kT = at<float>(s->kT, (size_t)L * st_kt); qa.vT = at<float>(s->vT, (size_t)L * st_kt); }
        // causal GQA attention                                               [:678-689]
        half_t *attn16 = s->full_param ? at<half_t>(s->attn16, L * s->st_attn) : a16;
        float *probs = s->probs ? at<float>(s->probs, (size_t)L * s->B * s->Hq * s->N * s->N) : nullptr;
        const float attn_scale = 1.0f / sqrtf((float)s->hd);
        if (s->use_flash) {                                  // epilogue and attention on bf16-pair fragments, no fp32 q / k / v
            AttnFlashArgs f = flash_args(s, L);
            f.out16 = attn16;
            launch_qkv_post_flash(qa, f);
            launch_attn_fwd_flash(f);
        } else launch_qkv_post(qa, BN);
        AttnFwdArgs aa{};
        aa.q = qa.q_fin; aa.k = qa.k_fin; aa.v = qa.v_out;
        aa.Hq = s->Hq; aa.Hkv = s->Hkv; aa.hd = s->hd; aa.seq = s->N; aa.batch = s->B;
        aa.scale = attn_scale; aa.probs = probs; aa.out16 = attn16; aa.kT = qa.kT;
        aa.window = (s->window > 0 && s->layer_local[L]) ? s->window : 0;
        if (s->use_flash) {
        } else if (attn_mfma_supported(s->hd, s->N)) {
            aa.pf = prefetch_for(s, wop(s, W_O, L, false), D, qd, 256, ((s->N + 31) / 32) * s->Hq);
            launch_attn_fwd_mfma(aa);
        } else launch_attn_fwd(aa);
        // full-parameter mode keeps the FFN GEMM operands of every layer as well
        half_t *ln2 = s->full_param ? at<half_t>(s->ln2_16, L * s->st_ln1) : a16;
        float *ln2inv = s->full_param ? at<float>(s->ln2_inv, (size_t)L * BN) : ainv;
        half_t *act16 = s->full_param ? at<half_t>(s->act16, L * s->st_act) : a16;
        float *actinv = s->full_param ? at<float>(s->act_inv, (size_t)L * BN) : ainv;

        // o = attn Wo^T; x_mid = x_in + o (Qwen3) | x_in + RN(o; g_post_attn) (Gemma3); ln2 = RN(x_mid; g_ffn_in)   [:696-711]
        Planes po = gemm(s, attn16, at<float>(s->ones), wop(s, W_O, L, false), D, qd);
        NormRowsArgs n2{};
        n2.x_prev = x_in; n2.branch = po;
        if (gemma) { n2.g_branch = at<float>(s->g_post_attn, (size_t)L * D); n2.branch_raw_out = at<float>(s->o_raw, (size_t)L * xsz); }
        n2.x_out = x_mid;
        n2.g_norm = gemma ? at<float>(s->g_pre_ff, (size_t)L * D) : at<float>(s->g_post_attn, (size_t)L * D);
        n2.ln16 = ln2; n2.inv_scale = ln2inv; n2.D = D; n2.eps = s->eps;
        n2.pf = prefetch_for(s, wop(s, W_GU, L, false), 2 * IS, D, 1024);
        launch_norm_rows(n2, BN);

        // [gate | up] = ln2 [Wg; Wu]^T; act = silu|gelu(gate) * up              [:715-725]
        // [gate | up] of the layer are kept for the backward as one [BN][2 IS] array, which is the product's own output
        // layout: the large-M kernel writes it there, the streaming kernel's planes are summed into it by the GLU kernel
        float *gu_keep = at<float>(s->gu_sav, (size_t)L * BN * 2 * IS);
        const WeightOp wgu = wop(s, W_GU, L, false);
        const bool direct = use_big_gemm(BN, 2 * IS, D, wgu.fmt);
        Planes pg = gemm(s, ln2, ln2inv, wgu, 2 * IS, D, direct ? gu_keep : nullptr, nullptr, half_scale_for(s, W_GU, L, false));
        GluArgs ga{};
        ga.in = pg; ga.IS = IS; ga.gelu = gemma;
        ga.gate_pre = gu_keep; ga.up_val = gu_keep + IS; ga.ld_gu = (size_t)2 * IS; ga.in_place = direct;
        ga.sg = scale_groups_for(s, wop(s, W_D, L, false), D, IS);
        ga.out16 = act16; ga.inv_scale = ga.sg.cols ? at<float>(s->group_inv) : actinv;
        launch_glu_fwd(ga, BN);

        // ff = act Wd^T, added by the next row kernel                          [:730-740]
        pending = gemm(s, act16, ga.inv_scale, wop(s, W_D, L, false), D, IS, nullptr, &ga.sg, half_scale_for(s, W_D, L, false));
    }

    // x_final = x_mid + ff; ln = RN(x_final; g_final); logits = ln Wlm^T        [:744-751]
    NormRowsArgs nf{};
    const int L = s->NL;
    nf.x_prev = at<float>(s->xs, (size_t)(2 * L - 1) * xsz);
    nf.branch = pending;
    if (gemma) { nf.g_branch = at<float>(s->g_post_ff, (size_t)(L - 1) * D); nf.branch_raw_out = at<float>(s->ff_raw, (size_t)(L - 1) * xsz); }
    nf.x_out = at<float>(s->xs, (size_t)(2 * L) * xsz);
    nf.g_norm = at<float>(s->g_final);
    half_t *lnf = s->full_param ? at<half_t>(s->lnf16) : a16;
    float *lnfinv = s->full_param ? at<float>(s->lnf_inv) : ainv;
    nf.ln16 = lnf; nf.inv_scale = lnfinv; nf.D = D; nf.eps = s->eps;
    nf.pf = prefetch_for(s, wop(s, W_LM, 0, false), s->V, D, 1024);
    launch_norm_rows(nf, BN);
    GemmPlan pl = plan_gemm(BN, s->V, D, 0, s->q8_native ? 1 : 0);
    if (pl.S == 1 || use_big_gemm(BN, s->V, D, s->q8_native ? 1 : 0)) {
        gemm(s, lnf, lnfinv, wop(s, W_LM, 0, false), s->V, D, at<float>(s->logits));
    } else {
        Planes p = gemm(s, lnf, lnfinv, wop(s, W_LM, 0, false), s->V, D);
        launch_reduce_planes(p.p, p.S, p.stride, p.ld, p.row_scale, at<float>(s->logits), BN, s->V);
    }
}

// dW = dY^T X for one (fused) matrix [M_out, N_in] at element offsets w_off / wt_off of its arenas:
// added into the accumulator (BWD_ACCUM) or applied at once to both weight images (BWD_SGD).
void weight_grad(SFTState *s, int mode, float lr, const half_t *dY16, const float *dy_inv, int M_out,
                 const half_t *X16, const float *x_inv, int N_in,
                 MetalBuf *W, MetalBuf *WT, MetalBuf *G, size_t w_off, size_t wt_off)
{
    if (mode == BWD_ACCUM && !G) { fprintf(stderr, "[fast_sft] gradient accumulators are not allocated\n"); abort(); }
    launch_transpose_scaled_pair(dY16, dy_inv, M_out, at<half_t>(s->yT), at<float>(s->yT_inv),
                                 X16, x_inv, N_in, at<half_t>(s->xT), at<float>(s->xT_inv), s->BN);
    if (mode == BWD_ACCUM) {
        launch_wgrad(at<half_t>(s->xT), at<float>(s->xT_inv), at<half_t>(s->yT), at<float>(s->yT_inv),
                     at<half_t>(G, w_off), M_out, N_in, s->BN, 0, 0.f);
    } else {
        launch_wgrad(at<half_t>(s->xT), at<float>(s->xT_inv), at<half_t>(s->yT), at<float>(s->yT_inv),
                     at<half_t>(W, w_off), M_out, N_in, s->BN, 1, lr);
        launch_apply_retile(at<half_t>(W, w_off), nullptr, at<half_t>(WT, wt_off), M_out, N_in, 0.f);
    }
}

// Backward from the fp16 loss gradient in dl16 / dl_inv.  mode: BWD_LORA (adapter gradients),
// BWD_ACCUM / BWD_SGD (full-parameter: sft_backward_accum / sft_backward_sgd, src/nn/fast_sft.c:984-986).
void backward_impl(SFTState *s, int mode = BWD_LORA, float lr = 0.f)
{
    const int BN = s->BN, D = s->D, IS = s->IS, qd = s->qd, kd = s->kd, R = s->R, NL = s->NL;
    const size_t xsz = (size_t)BN * D;
    half_t *a16 = at<half_t>(s->a16);
    float *ainv = at<float>(s->a16_inv);
    const bool gemma = s->model_type == MODEL_GEMMA3;
    int cur = 0;                                          // dx ping-pong
    // Accumulate mode: each of a layer's four loss-gradient operands (of down, gate|up, o, qkv) has a buffer of its own,
    // so that all four weight gradients can be formed after the layer's last row kernel: one launch transposes their
    // eight operands instead of four launches of two (the weights do not change before the apply, so the order of the
    // reference's f16_grad_accum calls, src/nn/fast_sft.c:804-946, does not matter).  Otherwise one buffer serves all.
    const bool defer = mode == BWD_ACCUM && s->dy16[0];
    half_t *d16[4];
    float *dinv[4];
    for (int i = 0; i < 4; i++) { d16[i] = defer ? at<half_t>(s->dy16[i]) : a16; dinv[i] = defer ? at<float>(s->dy_inv[i]) : ainv; }

    // dx = RNB(x_final, dlogits Wlm; g_final)                                [:777-790]
    Planes p = gemm(s, at<half_t>(s->dl16), at<float>(s->dl_inv), wop(s, W_LM, 0, true), D, s->V);
    if (mode != BWD_LORA)                                                     // [:778-786]
        weight_grad(s, mode, lr, at<half_t>(s->dl16), at<float>(s->dl_inv), s->V, at<half_t>(s->lnf16), at<float>(s->lnf_inv), D,
                    s->wlm, s->wlmT, s->glm, 0, 0);
    NormBwdArgs nb{};
    nb.dy = p; nb.x_saved = at<float>(s->xs, (size_t)(2 * NL) * xsz); nb.g = at<float>(s->g_final);
    nb.eps = s->eps; nb.D = D; nb.dx_prev = nullptr; nb.dx_out = at<float>(s->dx[cur]); nb.clamp = 0.f;
    if (gemma) { nb.branch_raw = at<float>(s->ff_raw, (size_t)(NL - 1) * xsz); nb.g_branch = at<float>(s->g_post_ff, (size_t)(NL - 1) * D); }
    nb.d16 = d16[0]; nb.inv_scale = dinv[0];
    if (mode == BWD_LORA) nb.pf = prefetch_for(s, wop(s, W_D, NL - 1, true), IS, D, 1024);
    launch_norm_bwd_rows(nb, BN);

    for (int L = NL - 1; L >= 0; L--) {
        // FFN: d act = d Wd; (dgate, dup); dln2 = dgate Wg + dup Wu; dx += RNB(x_mid, dln2)   [:798-874]
        Planes pd = gemm(s, d16[0], dinv[0], wop(s, W_D, L, true), IS, D, nullptr, nullptr, half_scale_for(s, W_D, L, true));
        if (mode != BWD_LORA && !defer)                                       // [:804-811, 842-849]
            weight_grad(s, mode, lr, a16, ainv, D, at<half_t>(s->act16, L * s->st_act), at<float>(s->act_inv, (size_t)L * BN), IS,
                        s->wd, s->wdT, s->gd, L * s->st_d, L * s->st_dT);
        GluArgs gb{};
        gb.in = pd; gb.IS = IS; gb.gelu = gemma;
        gb.gate_pre = at<float>(s->gu_sav, (size_t)L * BN * 2 * IS); gb.up_val = gb.gate_pre + IS; gb.ld_gu = (size_t)2 * IS;
        if (mode == BWD_LORA) gb.sg = scale_groups_for(s, wop(s, W_GU, L, true), D, 2 * IS);
        gb.out16 = d16[1]; gb.inv_scale = gb.sg.cols ? at<float>(s->group_inv) : dinv[1];
        launch_glu_bwd(gb, BN);
        Planes pgu = gemm(s, d16[1], gb.inv_scale, wop(s, W_GU, L, true), D, 2 * IS, nullptr, &gb.sg, half_scale_for(s, W_GU, L, true));
        if (mode != BWD_LORA && !defer)                                       // gate and up as one matrix [:817-833, 853-869]
            weight_grad(s, mode, lr, a16, ainv, 2 * IS, at<half_t>(s->ln2_16, L * s->st_ln1), at<float>(s->ln2_inv, (size_t)L * BN), D,
                        s->wgu, s->wguT, s->ggu, L * s->st_gu, L * s->st_guT);
        NormBwdArgs n2{};
        n2.dy = pgu; n2.x_saved = at<float>(s->xs, (size_t)(2 * L + 1) * xsz);
        n2.g = gemma ? at<float>(s->g_pre_ff, (size_t)L * D) : at<float>(s->g_post_attn, (size_t)L * D);
        n2.eps = s->eps; n2.D = D; n2.dx_prev = at<float>(s->dx[cur]); n2.dx_out = at<float>(s->dx[cur ^ 1]); n2.clamp = 0.f;
        if (gemma) { n2.branch_raw = at<float>(s->o_raw, (size_t)L * xsz); n2.g_branch = at<float>(s->g_post_attn, (size_t)L * D); }
        n2.d16 = d16[2]; n2.inv_scale = dinv[2];
        if (mode == BWD_LORA) n2.pf = prefetch_for(s, wop(s, W_O, L, true), qd, D, 1024);
        launch_norm_bwd_rows(n2, BN);
        cur ^= 1;

        // attention: dO = d Wo; dq, dk, dv                                    [:877-911]
        // (the wave-per-query attention kernels read their planes element by element: fp32 planes for them)
        const bool dO_by4 = s->use_flash || attn_mfma_supported(s->hd, s->N);
        Planes pdo = gemm(s, d16[2], dinv[2], wop(s, W_O, L, true), qd, D, nullptr, nullptr, dO_by4 ? half_scale_for(s, W_O, L, true) : 0.f);
        if (mode != BWD_LORA && !defer)                                       // [:883-901]
            weight_grad(s, mode, lr, a16, ainv, D, at<half_t>(s->attn16, L * s->st_attn), at<float>(s->ones), qd,
                        s->wo, s->woT, s->go, L * s->st_o, L * s->st_oT);
        AttnBwdArgs ab{};
        ab.dO = pdo;
        ab.probs = s->probs ? at<float>(s->probs, (size_t)L * s->B * s->Hq * s->N * s->N) : nullptr;
        if (s->q_fin) {
            ab.q = at<float>(s->q_fin, (size_t)L * BN * qd); ab.k = at<float>(s->k_fin, (size_t)L * BN * kd);
            ab.v = at<float>(s->v_sav, (size_t)L * BN * kd);
        }
        ab.Hq = s->Hq; ab.Hkv = s->Hkv; ab.hd = s->hd; ab.seq = s->N; ab.batch = s->B;
        ab.scale = 1.0f / sqrtf((float)s->hd);
        ab.vT = s->vT ? at<float>(s->vT, (size_t)L * s->B * kd * attn_ldt(s->N)) : nullptr;
        if (!s->use_flash) { ab.dO_red = at<float>(s->dO_red); ab.dscore = at<float>(s->dscore); }
        const size_t keepL = R ? (size_t)L : 0;                 // LoRA mode keeps dv, dq_f and dh of every layer
        ab.dq = at<float>(s->dq); ab.dk = at<float>(s->dk); ab.dv = at<float>(s->dv, keepL * BN * kd);
        const bool kv_shares = !s->use_flash && s->dkp && attn_bwd_one_launch(s->hd, s->N);
        if (kv_shares) { ab.dkp = at<float>(s->dkp); ab.dvp = at<float>(s->dvp); }
        if (s->use_flash) {
            AttnFlashArgs f = flash_args(s, L);
            f.dO = pdo; f.dq = ab.dq; f.dk = ab.dk; f.dv = ab.dv;
            launch_attn_bwd_flash(f);
        } else if (attn_mfma_supported(s->hd, s->N)) launch_attn_bwd_mfma(ab);
        else launch_attn_bwd(ab);

        // inverse RoPE, QK-norm backward, dh; LoRA gradients                  [:912-966]
        QkvBwdArgs qb{};
        qb.dq = ab.dq; qb.dk = ab.dk; qb.dv = ab.dv;
        qb.q_pre = at<float>(s->q_pre, (size_t)L * BN * qd); qb.k_pre = at<float>(s->k_pre, (size_t)L * BN * kd);
        qb.g_q = at<float>(s->g_q, (size_t)L * s->hd); qb.g_k = at<float>(s->g_k, (size_t)L * s->hd);
        qb.eps = s->eps; qb.rope = at<float2>(s->rope_tabs, (size_t)s->rope_slot[L] * s->N * (s->hd / 2));
        qb.Bq = at<float>(s->lora, L * s->lsz + (size_t)R * D);
        qb.Bv = at<float>(s->lora, L * s->lsz + (size_t)2 * R * D + (size_t)qd * R);
        qb.R = R; qb.sc = s->lora_scaling;
        if (R == 16) {
            qb.Bq16 = at<half_t>(s->lora16, L * s->lsz + (size_t)R * D);
            qb.Bv16 = at<half_t>(s->lora16, L * s->lsz + (size_t)2 * R * D + (size_t)qd * R);
        }
        qb.Hq = s->Hq; qb.Hkv = s->Hkv; qb.hd = s->hd; qb.seq = s->N;
        qb.dq_f = at<float>(s->dq_f, keepL * BN * qd); qb.dv_f = nullptr; qb.dh = at<float>(s->dh, keepL * BN * (R ? 2 * R : 1));
        if (kv_shares) { qb.dkp = ab.dkp; qb.dvp = ab.dvp; qb.rows_total = BN; qb.dv_f = ab.dv; }
        qb.out16 = d16[3]; qb.inv_scale = dinv[3];
        // (adapters only: the gradient of the first layer's input has no consumer, so its product and norm backward are not run)
        const bool input_grad = mode != BWD_LORA || L > 0;
        if (mode == BWD_LORA && input_grad) qb.pf = prefetch_for(s, wop(s, W_QKV, L, true), D, s->nq_ext, 1024);
        launch_qkv_bwd(qb, BN);
        if (defer) {
            // the layer's four weight gradients: eight transposes in one launch, then G += dY^T X for the four matrices in one
            const int m_out[4] = {D, 2 * IS, D, s->nq_ext}, n_in[4] = {IS, D, qd, D};
            const half_t *x16[4] = {at<half_t>(s->act16, L * s->st_act), at<half_t>(s->ln2_16, L * s->st_ln1),
                                    at<half_t>(s->attn16, L * s->st_attn), at<half_t>(s->ln1_16, (size_t)L * s->st_ln1)};
            const float *xinv[4] = {at<float>(s->act_inv, (size_t)L * BN), at<float>(s->ln2_inv, (size_t)L * BN), at<float>(s->ones),
                                    at<float>(s->ln1_inv, (size_t)L * BN)};
            MetalBuf *G[4] = {s->gd, s->ggu, s->go, s->gqkv};
            const size_t goff[4] = {L * s->st_d, L * s->st_gu, L * s->st_o, L * s->st_qkv};
            TransposeOperand ops[8];
            for (int i = 0; i < 4; i++) {
                ops[2 * i] = TransposeOperand{d16[i], dinv[i], m_out[i], at<half_t>(s->lyT[i]), at<float>(s->lyT_inv[i])};
                ops[2 * i + 1] = TransposeOperand{x16[i], xinv[i], n_in[i], at<half_t>(s->lxT[i]), at<float>(s->lxT_inv[i])};
            }
            launch_transpose_scaled_jobs(ops, 8, BN);
            WgradOperands wg[4];
            for (int i = 0; i < 4; i++)
                wg[i] = WgradOperands{at<half_t>(s->lxT[i]), at<float>(s->lxT_inv[i]), at<half_t>(s->lyT[i]), at<float>(s->lyT_inv[i]),
                                      at<half_t>(G[i], goff[i]), m_out[i], n_in[i]};
            launch_wgrads(wg, 4, BN, 0, 0.f);
        }
        // full-parameter: W_q, W_k, W_v are updated BEFORE the dX product, which then multiplies with the
        // new weights in SGD mode, as the reference does                       [:922-946]
        if (mode != BWD_LORA && !defer)
            weight_grad(s, mode, lr, a16, ainv, s->nq_ext, at<half_t>(s->ln1_16, (size_t)L * s->st_ln1), at<float>(s->ln1_inv, (size_t)L * BN), D,
                        s->wqkv, s->wqkvT, s->gqkv, L * s->st_qkv, L * s->st_qkvT);

        // dln1 = [dq|dk|dv|dh] [Wq;Wk;Wv;A_q;A_v]; dx += RNB(x_in, dln1; g_in); clamp     [:956-980]
        if (!input_grad) break;
        Planes pl = gemm(s, d16[3], dinv[3], wop(s, W_QKV, L, true), D, s->nq_ext);
        NormBwdArgs n1{};
        n1.dy = pl; n1.x_saved = at<float>(s->xs, (size_t)(2 * L) * xsz); n1.g = at<float>(s->g_in, (size_t)L * D);
        n1.eps = s->eps; n1.D = D; n1.dx_prev = at<float>(s->dx[cur]); n1.dx_out = at<float>(s->dx[cur ^ 1]); n1.clamp = 1e6f;
        if (L > 0) {
            if (gemma) { n1.branch_raw = at<float>(s->ff_raw, (size_t)(L - 1) * xsz); n1.g_branch = at<float>(s->g_post_ff, (size_t)(L - 1) * D); }
            n1.d16 = d16[0]; n1.inv_scale = dinv[0];
        }
        if (mode == BWD_LORA && L > 0) n1.pf = prefetch_for(s, wop(s, W_D, L - 1, true), IS, D, 1024);
        launch_norm_bwd_rows(n1, BN);
        cur ^= 1;
    }

    // LoRA gradients of all layers in one launch: dB = sc * dY^T t, dA = dh^T ln1     [:948-952, 962-966]
    if (R > 0) {
        LoraGradArgs lg{};
        lg.dq_f = at<float>(s->dq_f); lg.dv_f = at<float>(s->dv); lg.tq = at<float>(s->tq); lg.tv = at<float>(s->tv); lg.dh = at<float>(s->dh);
        lg.ln16 = at<half_t>(s->ln1_16); lg.ln_inv_scale = at<float>(s->ln1_inv);
        lg.rows = BN; lg.D = D; lg.qd = qd; lg.kd = kd; lg.R = R; lg.sc = s->lora_scaling;
        lg.grad = at<float>(s->lora_grad); lg.sq_slots = at<float>(s->sq_slots);
        lg.layers = NL;
        lg.st_dq = (size_t)BN * qd; lg.st_dv = (size_t)BN * kd; lg.st_t = (size_t)BN * R; lg.st_dh = (size_t)BN * 2 * R;
        lg.st_ln16 = s->st_ln1; lg.st_lninv = BN; lg.st_grad = s->lsz; lg.st_slots = s->slots_per_layer;
        launch_lora_grads(lg);
    }
}

void write_hyper(SFTState *s, float lr, int step)
{
    s->hyper_cpu[0] = lr;
    s->hyper_cpu[1] = 1.0f - powf(0.9f, (float)step);     // bias corrections as adamw_update forms them, src/nn/fast_sft.c:1048-1049
    s->hyper_cpu[2] = 1.0f - powf(0.999f, (float)step);
}

void enqueue_update(SFTState *s)
{
    if (!s->R) return;
    AdamArgs a{};
    a.p = at<float>(s->lora); a.g = at<float>(s->lora_grad); a.m = at<float>(s->adam_m); a.v = at<float>(s->adam_v);
    a.n = s->lora_n;
    a.sq_slots = at<float>(s->sq_slots); a.n_slots = s->slots_per_layer * s->NL;
    a.hyper = at<float>(s->hyper);
    a.b1 = 0.9f; a.b2 = 0.999f; a.eps = 1e-8f; a.wd = 0.01f; a.max_norm = 1.0f;      // src/nn/fast_sft.c:1091-1094
    a.wqkv = at<half_t>(s->wqkv); a.wqkv_layer_stride = s->st_qkv;
    a.wqkvT = at<half_t>(s->wqkvT); a.wqkvT_layer_stride = s->st_qkvT;
    a.NL = s->NL; a.D = s->D; a.qd = s->qd; a.kd = s->kd; a.R = s->R; a.layer_size = s->lsz;
    a.a_row0 = s->q8_native ? 0 : s->qd + 2 * s->kd;
    a.kbT = s->q8_native ? tiled_kb(2 * s->R) : tiled_kb(s->nq_ext);
    a.grad_norm_out = at<float>(s->grad_norm);
    a.p16 = at<half_t>(s->lora16);
    launch_adamw(a);
}

void refresh_shadow(SFTState *s)
{
    if (!s->R) return;
    launch_lora_shadow(at<float>(s->lora), s->lora_n, at<half_t>(s->wqkv), s->st_qkv,
                       at<half_t>(s->wqkvT), s->st_qkvT, s->D, s->qd, s->kd, s->R, s->lsz,
                       s->q8_native ? 0 : s->qd + 2 * s->kd, s->q8_native ? tiled_kb(2 * s->R) : tiled_kb(s->nq_ext),
                       at<half_t>(s->lora16));
}

MetalBuf *host_buf(size_t bytes, void **cpu)
{
    MetalBuf *b = metal_buf_create(bytes);
    *cpu = metal_buf_ptr(b);
    memset(*cpu, 0, bytes);
    return b;
}

}  // namespace

extern "C" {

SFTState *sft_state_create_from_ref(const SFTModelRef *m, int batch, int seq_len, int lora_rank, float lora_alpha,
                                    int weight_format)
{
    if (fast_metal_init() != 0) {
        fprintf(stderr, "[FastSFT] HIP backend init failed\n");
        return nullptr;
    }
    SFTState *s = new SFTState();
    s->model_type = m->model_type;
    s->D = m->d_model; s->Hq = m->n_q_heads; s->Hkv = m->n_kv_heads; s->hd = m->head_dim;
    s->IS = m->intermediate_size; s->V = m->vocab_size; s->NL = m->n_layers;
    s->N = seq_len; s->B = batch; s->BN = batch * seq_len;
    s->qd = s->Hq * s->hd; s->kd = s->Hkv * s->hd; s->R = lora_rank;
    s->nq_ext = s->qd + 2 * s->kd + 2 * s->R;
    s->eps = 1e-6f;                                        // src/nn/fast_sft.c:190
    s->lora_scaling = lora_rank > 0 ? lora_alpha / (float)lora_rank : 0.f;
    s->emb_scale = m->model_type == MODEL_GEMMA3 ? sqrtf((float)m->d_model) : 1.0f;   // :302
    s->step_count = 0;
    s->weight_format = weight_format;
    s->full_param = lora_rank == 0;                        // sft_state_create_full, src/nn/fast_sft.c:402-410
    s->token_emb_host = m->token_emb;
    s->rope_thetas.assign(m->rope_thetas, m->rope_thetas + s->NL);
    s->window = 0;
    s->layer_local.assign(s->NL, 0);
    const int D = s->D, IS = s->IS, qd = s->qd, kd = s->kd, R = s->R, NL = s->NL, BN = s->BN, V = s->V;
    if ((s->hd & 3) || (s->Hq % s->Hkv) || (D & 3) || (IS & 3) || (V & 3) || (lora_rank & 1) || lora_rank > 16 || (!weight_format && ((D & 31) || (IS & 31) || (qd & 31)))) {
        fprintf(stderr, "[FastSFT] unsupported dims: d_model, FFN width, vocab, head_dim must be multiples of 4, Hq of Hkv, rank even and <= 16 "
                        "(and every matrix width a multiple of 32 for Q8_0)\n");
        delete s;
        fast_metal_shutdown();
        return nullptr;
    }

    // upper limits of the row kernels (each would stop the process at its first launch, after all weights are uploaded)
    {
        const char *why = nullptr;
        if (D > 12288 || IS > 12288) why = "d_model and the FFN width must be at most 12288 (a workgroup keeps a row in registers)";
        else if (s->hd > 512) why = "head_dim must be at most 512";
        else if ((long)(qd + 2 * kd + 2 * R + 16 * 32) * 4 > 64 * 1024) why = "(n_q_heads + 2 n_kv_heads) * head_dim + 2 rank must be at most 15872 (a row of dq | dk | dv | dh is staged in 64 KB of LDS)";
        else if (seq_len > 4096) why = "seq_len must be at most 4096";
        else if (batch < 1 || seq_len < 1 || NL < 1) why = "batch, seq_len and the number of layers must be positive";
        if (why) {
            fprintf(stderr, "[FastSFT] unsupported dims: %s\n", why);
            delete s;
            fast_metal_shutdown();
            return nullptr;
        }
    }

    // ---- frozen weights: tiled arenas plus transposed images for the dX products ----
    // Q8_0 weights stay quantised when the fused QKV matrix splits into quantised and LoRA parts on tile
    // boundaries; otherwise (and in full-parameter mode, which rewrites the weights) they are stored as the
    // F16 image of their dequantised values.
    s->q8_native = !weight_format && !s->full_param && (qd % 32) == 0 && (kd % 32) == 0 && ((qd + 2 * kd) % 64) == 0;
    const int kbD = tiled_kb(D), kbQ = tiled_kb(qd), kbI = tiled_kb(IS), kb2I = tiled_kb(2 * IS), kbX = tiled_kb(s->nq_ext);
    s->st_ln1 = tiled_elems(BN, D);
    if (!s->q8_native) {
        s->st_qkv = tiled_elems(s->nq_ext, D); s->st_qkvT = tiled_elems(D, s->nq_ext);
        s->st_o = tiled_elems(D, qd);          s->st_oT = tiled_elems(qd, D);
        s->st_gu = tiled_elems(2 * IS, D);     s->st_guT = tiled_elems(D, 2 * IS);
        s->st_d = tiled_elems(D, IS);          s->st_dT = tiled_elems(IS, D);
        s->wqkv = hbuf(NL * s->st_qkv); s->wqkvT = hbuf(NL * s->st_qkvT);
        s->wo = hbuf(NL * s->st_o);     s->woT = hbuf(NL * s->st_oT);
        s->wgu = hbuf(NL * s->st_gu);   s->wguT = hbuf(NL * s->st_guT);
        s->wd = hbuf(NL * s->st_d);     s->wdT = hbuf(NL * s->st_dT);
        s->wlm = hbuf(tiled_elems(V, D)); s->wlmT = hbuf(tiled_elems(D, V));
    } else {
        const int qc = qd + 2 * kd;
        auto arena = [&](SFTState::Q8Arena &z, int Nw, int Kw, int layers, int kq_T) {
            z.st = (size_t)tiled_rb(Nw) * tiled_kb(Kw);       // forward image [Nw, Kw]
            z.stT = (size_t)tiled_rb(Kw) * kq_T;              // transposed image [Kw, Nw]: kq_T quantised K steps
            z.q = metal_buf_create(layers * z.st * 2048);   z.d = hbuf(layers * z.st * 64);
            z.qT = metal_buf_create(layers * z.stT * 2048); z.dT = hbuf(layers * z.stT * 64);
        };
        arena(s->zqkv, qc, D, NL, qc / 64);
        arena(s->zo, D, qd, NL, kbD);
        arena(s->zgu, 2 * IS, D, NL, kb2I);
        arena(s->zd, D, IS, NL, kbD);
        arena(s->zlm, V, D, 1, tiled_kb(V));
        // F16 tiles of the LoRA A rows: [2R, D] next to the forward image, [D, 2R] next to the transposed one
        s->st_qkv = R ? tiled_elems(2 * R, D) : 0; s->st_qkvT = R ? tiled_elems(D, 2 * R) : 0;
        s->wqkv = hbuf(R ? NL * s->st_qkv : 1); s->wqkvT = hbuf(R ? NL * s->st_qkvT : 1);
    }
    for (MetalBuf *b : {s->wqkv, s->wqkvT, s->wo, s->woT, s->wgu, s->wguT, s->wd, s->wdT, s->wlm, s->wlmT,
                        s->zqkv.q, s->zqkv.d, s->zqkv.qT, s->zqkv.dT, s->zo.q, s->zo.d, s->zo.qT, s->zo.dT,
                        s->zgu.q, s->zgu.d, s->zgu.qT, s->zgu.dT, s->zd.q, s->zd.d, s->zd.qT, s->zd.dT,
                        s->zlm.q, s->zlm.d, s->zlm.qT, s->zlm.dT})
        if (b) HIP_CHECK(hipMemsetAsync(dptr(b), 0, b->size, stream()));     // row and K padding must read as zero
    s->g_in = fbuf((size_t)NL * D); s->g_post_attn = fbuf((size_t)NL * D);
    s->g_pre_ff = fbuf((size_t)NL * D); s->g_post_ff = fbuf((size_t)NL * D);
    s->g_q = fbuf((size_t)NL * s->hd); s->g_k = fbuf((size_t)NL * s->hd);
    for (int L = 0; L < NL; L++) {
        const LayerWeightRef *r = &m->layers[L];
        if (!s->q8_native) {
            put_matrix(s, r->q_proj.data, qd, D, {s->wqkv, L * s->st_qkv, kbD, 0, 0, 0}, {s->wqkvT, L * s->st_qkvT, kbX, 0, 0, 1});
            put_matrix(s, r->k_proj.data, kd, D, {s->wqkv, L * s->st_qkv, kbD, qd, 0, 0}, {s->wqkvT, L * s->st_qkvT, kbX, 0, qd, 1});
            put_matrix(s, r->v_proj.data, kd, D, {s->wqkv, L * s->st_qkv, kbD, qd + kd, 0, 0}, {s->wqkvT, L * s->st_qkvT, kbX, 0, qd + kd, 1});
            put_matrix(s, r->o_proj.data, D, qd, {s->wo, L * s->st_o, kbQ, 0, 0, 0}, {s->woT, L * s->st_oT, kbD, 0, 0, 1});
            put_matrix(s, r->gate_proj.data, IS, D, {s->wgu, L * s->st_gu, kbD, 0, 0, 0}, {s->wguT, L * s->st_guT, kb2I, 0, 0, 1});
            put_matrix(s, r->up_proj.data, IS, D, {s->wgu, L * s->st_gu, kbD, IS, 0, 0}, {s->wguT, L * s->st_guT, kb2I, 0, IS, 1});
            put_matrix(s, r->down_proj.data, D, IS, {s->wd, L * s->st_d, kbI, 0, 0, 0}, {s->wdT, L * s->st_dT, kbD, 0, 0, 1});
        } else {
            const int kqT = (qd + 2 * kd) / 64;
            SFTState::Q8Arena &zq = s->zqkv, &zo = s->zo, &zg = s->zgu, &zd = s->zd;
            put_matrix_q8(r->q_proj.data, qd, D, {zq.q, zq.d, L * zq.st, kbD, 0, 0, 0}, {zq.qT, zq.dT, L * zq.stT, kqT, 0, 0, 1});
            put_matrix_q8(r->k_proj.data, kd, D, {zq.q, zq.d, L * zq.st, kbD, qd, 0, 0}, {zq.qT, zq.dT, L * zq.stT, kqT, 0, qd, 1});
            put_matrix_q8(r->v_proj.data, kd, D, {zq.q, zq.d, L * zq.st, kbD, qd + kd, 0, 0}, {zq.qT, zq.dT, L * zq.stT, kqT, 0, qd + kd, 1});
            put_matrix_q8(r->o_proj.data, D, qd, {zo.q, zo.d, L * zo.st, kbQ, 0, 0, 0}, {zo.qT, zo.dT, L * zo.stT, kbD, 0, 0, 1});
            put_matrix_q8(r->gate_proj.data, IS, D, {zg.q, zg.d, L * zg.st, kbD, 0, 0, 0}, {zg.qT, zg.dT, L * zg.stT, kb2I, 0, 0, 1});
            put_matrix_q8(r->up_proj.data, IS, D, {zg.q, zg.d, L * zg.st, kbD, IS, 0, 0}, {zg.qT, zg.dT, L * zg.stT, kb2I, 0, IS, 1});
            put_matrix_q8(r->down_proj.data, D, IS, {zd.q, zd.d, L * zd.st, kbI, 0, 0, 0}, {zd.qT, zd.dT, L * zd.stT, kbD, 0, 0, 1});
        }
        metal_buf_write(s->g_in, (size_t)L * D * 4, r->input_norm_g, (size_t)D * 4);
        metal_buf_write(s->g_post_attn, (size_t)L * D * 4, r->post_attn_norm_g, (size_t)D * 4);
        if (r->pre_ff_norm_g) metal_buf_write(s->g_pre_ff, (size_t)L * D * 4, r->pre_ff_norm_g, (size_t)D * 4);
        if (r->post_ff_norm_g) metal_buf_write(s->g_post_ff, (size_t)L * D * 4, r->post_ff_norm_g, (size_t)D * 4);
        metal_buf_write(s->g_q, (size_t)L * s->hd * 4, r->q_norm_g, (size_t)s->hd * 4);
        metal_buf_write(s->g_k, (size_t)L * s->hd * 4, r->k_norm_g, (size_t)s->hd * 4);
    }
    if (!s->q8_native) put_matrix(s, m->lm_head, V, D, {s->wlm, 0, kbD, 0, 0, 0}, {s->wlmT, 0, tiled_kb(V), 0, 0, 1});
    else put_matrix_q8(m->lm_head, V, D, {s->zlm.q, s->zlm.d, 0, kbD, 0, 0, 0}, {s->zlm.qT, s->zlm.dT, 0, tiled_kb(V), 0, 0, 1});
    s->g_final = metal_buf_from_data(m->final_norm_g, (size_t)D * 4);
    s->emb = metal_buf_from_data(m->token_emb, (size_t)V * D * 4);

    // ---- RoPE tables: one per distinct theta (Gemma3 has two) ----
    {
        std::vector<float> distinct;
        for (int L = 0; L < NL; L++) {
            int slot = -1;
            for (size_t k = 0; k < distinct.size(); k++) if (distinct[k] == s->rope_thetas[L]) slot = (int)k;
            if (slot < 0) { slot = (int)distinct.size(); distinct.push_back(s->rope_thetas[L]); }
            s->rope_slot.push_back(slot);
        }
        const size_t per = (size_t)s->N * (s->hd / 2);
        s->rope_tabs = metal_buf_create(distinct.size() * per * sizeof(float2));
        for (size_t k = 0; k < distinct.size(); k++)
            launch_rope_table(at<float2>(s->rope_tabs, k * per), s->N, s->hd, distinct[k]);
    }

    // ---- LoRA arena, gradients, optimiser state ----
    s->lsz = (size_t)2 * R * D + (size_t)qd * R + (size_t)kd * R;
    s->lora_n = s->lsz * NL;
    s->slots_per_layer = R ? lora_grad_blocks(D, qd, kd, R) : 1;
    s->lora = fbuf(s->lora_n ? s->lora_n : 1); s->lora_grad = fbuf(s->lora_n ? s->lora_n : 1);
    s->lora16 = hbuf(s->lora_n ? s->lora_n : 1);
    s->adam_m = fbuf(s->lora_n ? s->lora_n : 1); s->adam_v = fbuf(s->lora_n ? s->lora_n : 1);
    s->sq_slots = fbuf((size_t)s->slots_per_layer * NL); s->grad_norm = fbuf(4);
    HIP_CHECK(hipMemsetAsync(dptr(s->lora_grad), 0, s->lora_grad->size, stream()));
    HIP_CHECK(hipMemsetAsync(dptr(s->adam_m), 0, s->adam_m->size, stream()));
    HIP_CHECK(hipMemsetAsync(dptr(s->adam_v), 0, s->adam_v->size, stream()));
    HIP_CHECK(hipMemsetAsync(dptr(s->sq_slots), 0, s->sq_slots->size, stream()));
    HIP_CHECK(hipMemsetAsync(dptr(s->grad_norm), 0, s->grad_norm->size, stream()));
    if (s->lora_n) {
        if (m->lora_init) {
            metal_buf_write(s->lora, 0, m->lora_init, s->lora_n * 4);
        } else {                                           // init_lora_layer, src/nn/fast_sft.c:100-123
            std::vector<float> tmp(s->lora_n, 0.f);
            const float std_a = 1.0f / sqrtf((float)D);
            for (int L = 0; L < NL; L++) {
                float *aq = tmp.data() + L * s->lsz, *av = aq + (size_t)R * D + (size_t)qd * R;
                for (size_t j = 0; j < (size_t)R * D; j++) aq[j] = ((float)rand() / (float)RAND_MAX - 0.5f) * 2.0f * std_a;
                for (size_t j = 0; j < (size_t)R * D; j++) av[j] = ((float)rand() / (float)RAND_MAX - 0.5f) * 2.0f * std_a;
            }
            metal_buf_write(s->lora, 0, tmp.data(), s->lora_n * 4);
        }
    }
    for (int L = 0; L < NL && R; L++) {
        const size_t o = L * s->lsz * 4;
        const size_t sz[4] = {(size_t)R * D * 4, (size_t)qd * R * 4, (size_t)R * D * 4, (size_t)kd * R * 4};
        size_t off = o;
        for (int k = 0; k < 4; k++) {
            s->lora_views.push_back(metal_buf_view(s->lora, off, sz[k]));
            s->grad_views.push_back(metal_buf_view(s->lora_grad, off, sz[k]));
            off += sz[k];
        }
    }

    // ---- host-visible small buffers ----
    s->tokens = host_buf((size_t)BN * 4, (void **)&s->tokens_cpu);
    s->targets = host_buf((size_t)BN * 4, (void **)&s->targets_cpu);
    s->losses = host_buf((size_t)BN * 4, (void **)&s->losses_cpu);
    s->hyper = host_buf(64, (void **)&s->hyper_cpu);
    s->x_in_host = nullptr; s->x_cpu = nullptr;

    // ---- saved activations and transients ----
    const size_t xsz = (size_t)BN * D;
    s->xs = fbuf((size_t)(2 * NL + 1) * xsz);
    s->ln1_16 = hbuf((size_t)NL * s->st_ln1); s->ln1_inv = fbuf((size_t)NL * BN);
    s->q_pre = fbuf((size_t)NL * BN * qd); s->k_pre = fbuf((size_t)NL * BN * kd);
    s->use_flash = attn_flash_supported(s->hd, s->N, s->Hq, s->Hkv, s->B);
    if (s->use_flash) {
        const size_t eq = attn_flash_tile_elems(s->hd, s->N, s->Hq, s->B), ek = attn_flash_tile_elems(s->hd, s->N, s->Hkv, s->B);
        const size_t stat = (size_t)s->B * s->Hq * ((s->N + 31) / 32) * 32;
        s->fa_q = metal_buf_create((size_t)NL * 2 * eq * 16); s->fa_k = metal_buf_create((size_t)NL * 2 * ek * 16);
        s->fa_v = metal_buf_create((size_t)NL * 2 * ek * 16); s->fa_do = metal_buf_create(2 * eq * 16);
        s->fa_O = fbuf((size_t)NL * BN * qd); s->fa_lse = fbuf((size_t)NL * stat); s->fa_D = fbuf(stat);
        s->fa_dkp = fbuf((size_t)(s->Hq / s->Hkv) * BN * kd); s->fa_dvp = fbuf((size_t)(s->Hq / s->Hkv) * BN * kd);
    } else {
        s->probs = fbuf((size_t)NL * s->B * s->Hq * s->N * s->N);
        s->q_fin = fbuf((size_t)NL * BN * qd); s->k_fin = fbuf((size_t)NL * BN * kd); s->v_sav = fbuf((size_t)NL * BN * kd);
    }
    if (!s->use_flash && attn_mfma_supported(s->hd, s->N)) {
        s->kT = fbuf((size_t)NL * s->B * kd * attn_ldt(s->N)); s->vT = fbuf((size_t)NL * s->B * kd * attn_ldt(s->N));
    }
    s->gu_sav = fbuf((size_t)NL * BN * 2 * IS);
    s->tq = fbuf((size_t)NL * BN * (R ? R : 1)); s->tv = fbuf((size_t)NL * BN * (R ? R : 1));
    const bool gemma = s->model_type == MODEL_GEMMA3;
    s->o_raw = gemma ? fbuf((size_t)NL * xsz) : nullptr; s->ff_raw = gemma ? fbuf((size_t)NL * xsz) : nullptr;
    int maxk = D;
    if (qd > maxk) maxk = qd;
    if (2 * IS > maxk) maxk = 2 * IS;
    if (s->nq_ext > maxk) maxk = s->nq_ext;
    s->a16 = hbuf(tiled_elems(BN, maxk)); s->a16_inv = fbuf(BN); s->group_inv = fbuf((size_t)BN * MAX_SCALE_GROUPS);
    s->ones = fbuf(BN);
    launch_fill_f32(at<float>(s->ones), 1.0f, BN);
    s->planes_cap = max_planes_elems(s);
    s->planes = fbuf(s->planes_cap);
    s->logits = fbuf((size_t)BN * V); s->dlogits = nullptr;
    s->dl16 = hbuf(tiled_elems(BN, V)); s->dl_inv = fbuf(BN);
    s->dx[0] = fbuf(xsz); s->dx[1] = fbuf(xsz);
    if (!s->use_flash) { s->dO_red = fbuf((size_t)BN * qd); s->dscore = fbuf((size_t)s->B * s->Hq * s->N * s->N); }
    if (!s->use_flash && attn_mfma_supported(s->hd, s->N) && s->N <= 64) {
        const size_t n = (size_t)((s->N + 31) / 32) * s->Hq * BN * s->hd;
        s->dkp = fbuf(n); s->dvp = fbuf(n);
    }
    const size_t keep = R ? NL : 1;
    s->dq = fbuf((size_t)BN * qd); s->dk = fbuf((size_t)BN * kd); s->dv = fbuf(keep * BN * kd);
    s->dq_f = fbuf(keep * BN * qd); s->dh = fbuf(keep * BN * (R ? 2 * R : 1));
    s->ce_part = metal_buf_create((size_t)BN * CE_CHUNKS * sizeof(float2));

    // ---- full-parameter mode: kept GEMM operands and the transposed pair of one weight gradient ----
    s->st_act = tiled_elems(BN, IS); s->st_attn = tiled_elems(BN, qd);
    if (s->full_param) {
        s->ln2_16 = hbuf((size_t)NL * s->st_ln1); s->ln2_inv = fbuf((size_t)NL * BN);
        s->act16 = hbuf((size_t)NL * s->st_act);  s->act_inv = fbuf((size_t)NL * BN);
        s->attn16 = hbuf((size_t)NL * s->st_attn);
        s->lnf16 = hbuf(s->st_ln1); s->lnf_inv = fbuf(BN);
        int maxy = V > 2 * IS ? V : 2 * IS;
        if (s->nq_ext > maxy) maxy = s->nq_ext;
        if (D > maxy) maxy = D;
        int maxx = IS > qd ? IS : qd;
        if (D > maxx) maxx = D;
        s->yT = hbuf(tiled_elems(maxy, BN)); s->yT_inv = fbuf((size_t)tiled_kb(maxy) * 64);
        s->xT = hbuf(tiled_elems(maxx, BN)); s->xT_inv = fbuf((size_t)tiled_kb(maxx) * 64);
    }

    // the fused QKV weight and its transpose carry fp16 images of A_q, A_v
    refresh_shadow(s);
    metal_flush();
    // products of at most 64 rows on frozen weights (F16 or Q8_0) leave their K-split planes as halves: one factor per matrix
    if (s->R > 0 && BN <= 64) {
        struct Img { int kind; bool T; int N, K; };
        const Img imgs[] = {{W_GU, false, 2 * IS, D}, {W_D, false, D, IS}, {W_D, true, IS, D}, {W_GU, true, D, 2 * IS}, {W_O, true, qd, D}};
        for (const Img &im : imgs) {
            std::vector<float> &v = s->half_scale[im.kind][im.T ? 1 : 0];
            v.resize(s->NL);
            for (int L = 0; L < s->NL; L++) {
                const float l1 = weight_max_row_l1(wop(s, im.kind, L, im.T), im.N, im.K);
                v[L] = l1 > 0.f ? half_plane_scale(l1) : 0.f;          // 0: that product keeps fp32 planes
            }
        }
    }
    return s;
}

void sft_state_free(SFTState *s)
{
    if (!s) return;
    metal_flush();
    for (MetalBuf *b : s->lora_views) metal_buf_free(b);
    for (MetalBuf *b : s->grad_views) metal_buf_free(b);
    MetalBuf *all[] = {s->wqkv, s->wqkvT, s->wo, s->woT, s->wgu, s->wguT, s->wd, s->wdT, s->wlm, s->wlmT, s->zqkv.q, s->zqkv.d, s->zqkv.qT, s->zqkv.dT, s->zo.q, s->zo.d, s->zo.qT, s->zo.dT,
                       s->zgu.q, s->zgu.d, s->zgu.qT, s->zgu.dT, s->zd.q, s->zd.d, s->zd.qT, s->zd.dT, s->zlm.q, s->zlm.d, s->zlm.qT, s->zlm.dT,
                       s->rope_tabs, s->g_in, s->g_post_attn, s->g_pre_ff, s->g_post_ff, s->g_q, s->g_k, s->g_final, s->emb,
                       s->lora, s->lora16, s->lora_grad, s->adam_m, s->adam_v, s->sq_slots, s->grad_norm,
                       s->tokens, s->targets, s->losses, s->hyper, s->x_in_host,
                       s->xs, s->ln1_16, s->ln1_inv, s->q_pre, s->k_pre, s->q_fin, s->k_fin, s->v_sav, s->probs,
                       s->gu_sav, s->tq, s->tv, s->kT, s->vT, s->o_raw, s->ff_raw, s->a16, s->a16_inv, s->group_inv, s->ones, s->planes,
                       s->logits, s->dlogits, s->dl16, s->dl_inv, s->dx[0], s->dx[1], s->dO_red, s->dscore, s->dkp, s->dvp,
                       s->dq, s->dk, s->dv, s->dq_f, s->dh, s->ce_part,
                       s->ln2_16, s->ln2_inv, s->act16, s->act_inv, s->attn16, s->lnf16, s->lnf_inv,
                       s->xT, s->xT_inv, s->yT, s->yT_inv, s->gqkv, s->go, s->ggu, s->gd, s->glm,
                       s->grpo_old_lp, s->grpo_advs, s->grpo_new_lp, s->lora_acc, s->lm_head_out.mbuf,
                       s->fa_q, s->fa_k, s->fa_v, s->fa_O, s->fa_lse, s->fa_do, s->fa_D, s->fa_dkp, s->fa_dvp};
    for (int i = 0; i < 4; i++)
        for (MetalBuf *b : {s->dy16[i], s->dy_inv[i], s->lyT[i], s->lyT_inv[i], s->lxT[i], s->lxT_inv[i]}) metal_buf_free(b);
    for (MetalBuf *b : s->views_out) metal_buf_free(b);
    for (MetalBuf *b : s->gamma_views) metal_buf_free(b);
    for (auto &kv : s->img_slots) metal_buf_free(kv.second);
    for (MetalBuf *b : all) metal_buf_free(b);
    for (WMat &w : s->wmats_out) metal_buf_free(w.mbuf);
    delete s;
    fast_metal_shutdown();
}

static void enqueue_step_kernels(SFTState *s, float lr)
{
    forward_impl(s, true);
    CeArgs ce{};
    ce.logits = at<float>(s->logits); ce.V = s->V; ce.targets = at<uint32_t>(s->targets); ce.losses = at<float>(s->losses);
    ce.dl16 = at<half_t>(s->dl16); ce.inv_scale = at<float>(s->dl_inv); ce.rows_total = s->BN;
    ce.partials = at<float2>(s->ce_part);
    launch_ce_rows(ce, s->BN);
    if (s->full_param) backward_impl(s, s->gqkv ? BWD_ACCUM : BWD_SGD, lr);     // src/nn/fast_sft.c:1136-1140 with :778-786
    else backward_impl(s);
    enqueue_update(s);
}

// The kernels gather embedding rows by token id and read logits[target] without a test of their own, so ids are
// checked here, on the host, before anything is launched (an int32 id < 0 from a token file arrives as a huge uint32).
static bool ids_in_vocab(const SFTState *s, const uint32_t *ids, size_t n, const char *what)
{
    for (size_t i = 0; i < n; i++)
        if (ids[i] >= (uint32_t)s->V) {
            fprintf(stderr, "[FastSFT] %s id %u at position %zu is outside the vocabulary (%d): nothing launched\n", what, ids[i], i, s->V);
            return false;
        }
    return true;
}

void sft_enqueue_train_step(SFTState *s, const uint32_t *input_tokens, const uint32_t *target_tokens, float lr)
{
    // One step in flight: the pinned token / target / optimiser-parameter buffers are read by the kernels of the
    // step that was enqueued last, so a second enqueue first waits for that step.
    if (s->step_in_flight) metal_flush();
    s->step_rejected = !ids_in_vocab(s, input_tokens, (size_t)s->BN, "token") || !ids_in_vocab(s, target_tokens, (size_t)s->BN, "target");
    s->step_in_flight = 1;
    if (s->step_rejected) return;
    memcpy(s->tokens_cpu, input_tokens, (size_t)s->BN * 4);
    memcpy(s->targets_cpu, target_tokens, (size_t)s->BN * 4);
    if (s->R) { s->step_count++; write_hyper(s, lr, s->step_count); }
    enqueue_step_kernels(s, lr);
}

float sft_finish_train_step(SFTState *s)
{
    metal_flush();
    s->step_in_flight = 0;
    if (s->step_rejected) { s->step_rejected = 0; return NAN; }
    float tot = 0.f;
    for (int i = 0; i < s->BN; i++) tot += s->losses_cpu[i];
    return tot / (float)s->BN;
}

float sft_train_step(SFTState *s, const uint32_t *input_tokens, const uint32_t *target_tokens, float lr)
{
    sft_enqueue_train_step(s, input_tokens, target_tokens, lr);
    return sft_finish_train_step(s);
}

void forward_to_logits(SFTState *s)
{
    if (!s->x_in_host) sft_get_x_cpu(s);
    forward_impl(s, false);
}

static void backward_from_dlogits(SFTState *s, int mode, float lr)
{
    MetalBuf *dl = sft_get_dlogits(s);
    launch_rows_to_f16(at<float>(dl), s->V, at<half_t>(s->dl16), at<float>(s->dl_inv), s->BN, s->V);
    backward_impl(s, mode, lr);
}

// sft_backward / sft_backward_sgd / sft_backward_accum, src/nn/fast_sft.c:984-986: all three run
// sft_backward_ex, whose branch depends on the state (LoRA | accumulators allocated | fused SGD).
void sft_backward(SFTState *s) { backward_from_dlogits(s, !s->full_param ? BWD_LORA : (s->gqkv ? BWD_ACCUM : BWD_SGD), 0.f); }
void sft_backward_sgd(SFTState *s, float lr) { backward_from_dlogits(s, !s->full_param ? BWD_LORA : (s->gqkv ? BWD_ACCUM : BWD_SGD), lr); }
void sft_backward_accum(SFTState *s) { sft_backward(s); }

// sft_alloc_grad_accum, src/nn/fast_sft.c:996-1019: zeroed F16 accumulators mirroring every weight.
void sft_alloc_grad_accum(SFTState *s)
{
    if (s->gqkv || !s->full_param) return;
    s->gqkv = hbuf(s->NL * s->st_qkv); s->go = hbuf(s->NL * s->st_o);
    s->ggu = hbuf(s->NL * s->st_gu);   s->gd = hbuf(s->NL * s->st_d);
    s->glm = hbuf(tiled_elems(s->V, s->D));
    for (MetalBuf *b : {s->gqkv, s->go, s->ggu, s->gd, s->glm}) HIP_CHECK(hipMemsetAsync(dptr(b), 0, b->size, stream()));
    const int m_out[4] = {s->D, 2 * s->IS, s->D, s->nq_ext}, n_in[4] = {s->IS, s->D, s->qd, s->D};
    for (int i = 0; i < 4; i++) {
        s->dy16[i] = hbuf(tiled_elems(s->BN, m_out[i])); s->dy_inv[i] = fbuf(s->BN);
        HIP_CHECK(hipMemsetAsync(dptr(s->dy16[i]), 0, s->dy16[i]->size, stream()));      // row and K padding must read as zero
        s->lyT[i] = hbuf(tiled_elems(m_out[i], s->BN)); s->lyT_inv[i] = fbuf((size_t)tiled_kb(m_out[i]) * 64);
        s->lxT[i] = hbuf(tiled_elems(n_in[i], s->BN));  s->lxT_inv[i] = fbuf((size_t)tiled_kb(n_in[i]) * 64);
    }
    const double mb = 2.0 * ((double)s->NL * (s->st_qkv + s->st_o + s->st_gu + s->st_d) + (double)tiled_elems(s->V, s->D)) / (1024.0 * 1024.0);
    printf("[FastSFT] Grad accum buffers allocated: %.2f MB\n", mb);
}

// sft_apply_grad_sgd, src/nn/fast_sft.c:1021-1039: W = half(W - lr G), G = 0, then flush.  Both images
// of every weight (as stored and transposed) are rewritten.
void sft_apply_grad_sgd(SFTState *s, float lr)
{
    if (!s->gqkv) return;
    // one launch per arena: the layers of a kind have one shape and lie at equal distances
    launch_apply_retile(at<half_t>(s->wqkv), at<half_t>(s->gqkv), at<half_t>(s->wqkvT), s->nq_ext, s->D, lr, s->NL, s->st_qkv, s->st_qkvT);
    launch_apply_retile(at<half_t>(s->wo), at<half_t>(s->go), at<half_t>(s->woT), s->D, s->qd, lr, s->NL, s->st_o, s->st_oT);
    launch_apply_retile(at<half_t>(s->wgu), at<half_t>(s->ggu), at<half_t>(s->wguT), 2 * s->IS, s->D, lr, s->NL, s->st_gu, s->st_guT);
    launch_apply_retile(at<half_t>(s->wd), at<half_t>(s->gd), at<half_t>(s->wdT), s->D, s->IS, lr, s->NL, s->st_d, s->st_dT);
    launch_apply_retile(at<half_t>(s->wlm), at<half_t>(s->glm), at<half_t>(s->wlmT), s->V, s->D, lr);
    metal_flush();
}

// Row-major F16 copy of one matrix: which = 0..6 (q, k, v, o, gate, up, down of `layer`) or 7 (lm_head);
// source = 0 the image the forward multiplies with, 1 its transposed twin (must hold the same values),
// 2 the gradient accumulator.
void sft_copy_matrix_f16(SFTState *s, int layer, int which, int source, uint16_t *dst)
{
    const int D = s->D, IS = s->IS, qd = s->qd, kd = s->kd;
    struct Sel { MetalBuf *W, *WT, *G; size_t st, stT; int M, N, row_off, rows; } sel;
    switch (which) {
    case 0: sel = {s->wqkv, s->wqkvT, s->gqkv, s->st_qkv, s->st_qkvT, s->nq_ext, D, 0, qd}; break;
    case 1: sel = {s->wqkv, s->wqkvT, s->gqkv, s->st_qkv, s->st_qkvT, s->nq_ext, D, qd, kd}; break;
    case 2: sel = {s->wqkv, s->wqkvT, s->gqkv, s->st_qkv, s->st_qkvT, s->nq_ext, D, qd + kd, kd}; break;
    case 3: sel = {s->wo, s->woT, s->go, s->st_o, s->st_oT, D, qd, 0, D}; break;
    case 4: sel = {s->wgu, s->wguT, s->ggu, s->st_gu, s->st_guT, 2 * IS, D, 0, IS}; break;
    case 5: sel = {s->wgu, s->wguT, s->ggu, s->st_gu, s->st_guT, 2 * IS, D, IS, IS}; break;
    case 6: sel = {s->wd, s->wdT, s->gd, s->st_d, s->st_dT, D, IS, 0, D}; break;
    case 7: sel = {s->wlm, s->wlmT, s->glm, 0, 0, s->V, D, 0, s->V}; layer = 0; break;
    default: return;
    }
    if (layer < 0 || layer >= s->NL || (source == 2 && !sel.G)) return;
    const size_t n = (size_t)sel.rows * sel.N;
    MetalBuf *tmp = hbuf(n);
    if (s->q8_native) {                                   // dequantised values of the quantised tiles
        const int kind = which <= 2 ? W_QKV : (which == 3 ? W_O : (which <= 5 ? W_GU : (which == 6 ? W_D : W_LM)));
        const WeightOp w = wop(s, kind, layer, source == 1);
        if (source == 1) launch_untile_q8(w.q, w.d, 2, w.kbq, 0, sel.row_off, 1, sel.rows, sel.N, at<half_t>(tmp));
        else launch_untile_q8(w.q, w.d, 1, tiled_kb(sel.N), sel.row_off, 0, 0, sel.rows, sel.N, at<half_t>(tmp));
    } else if (source == 1)
        launch_untile_f16(at<half_t>(sel.WT, layer * sel.stT), tiled_kb(sel.M), 0, sel.row_off, 1, sel.rows, sel.N, at<half_t>(tmp));
    else
        launch_untile_f16(at<half_t>(source == 2 ? sel.G : sel.W, layer * sel.st), tiled_kb(sel.N), sel.row_off, 0, 0, sel.rows, sel.N, at<half_t>(tmp));
    metal_buf_read(tmp, 0, dst, n * 2);
    metal_buf_free(tmp);
}

// "FULL" checkpoint, src/nn/fast_sft.c:1286-1340: nine u32 header words, then per layer
// q, k, v, o, gate, up, down and finally lm_head as row-major F16.
void sft_save_full_checkpoint(SFTState *s, const char *path)
{
    FILE *fp = fopen(path, "wb");
    if (!fp) { fprintf(stderr, "[FastSFT] Failed to open %s for writing\n", path); return; }
    const uint32_t hdr[9] = {0x46554C4Cu, (uint32_t)s->model_type, (uint32_t)s->NL, (uint32_t)s->D, (uint32_t)s->Hq,
                             (uint32_t)s->Hkv, (uint32_t)s->hd, (uint32_t)s->IS, (uint32_t)s->V};
    fwrite(hdr, 4, 9, fp);
    const size_t sizes[8] = {(size_t)s->qd * s->D, (size_t)s->kd * s->D, (size_t)s->kd * s->D, (size_t)s->D * s->qd,
                             (size_t)s->IS * s->D, (size_t)s->IS * s->D, (size_t)s->D * s->IS, (size_t)s->V * s->D};
    std::vector<uint16_t> buf;
    size_t total = 0;
    for (int L = 0; L <= s->NL; L++)
        for (int w = (L < s->NL ? 0 : 7); w < (L < s->NL ? 7 : 8); w++) {
            buf.resize(sizes[w]);
            sft_copy_matrix_f16(s, L < s->NL ? L : 0, w, 0, buf.data());
            fwrite(buf.data(), 2, sizes[w], fp);
            total += sizes[w] * 2;
        }
    fclose(fp);
    printf("[FastSFT] Full checkpoint saved to %s (%.2f MB)\n", path, (float)total / (1024.0f * 1024.0f));
}

void sft_lora_update(SFTState *s, float lr)
{
    // the caller has set the step count (src/nn/fast_grpo.c:488-490); gradients may have been replaced
    // through sft_set_lora_grad, so the sums of squares are recomputed from the gradient arena
    write_hyper(s, lr, s->step_count);
    std::vector<float> g(s->lora_n);
    metal_buf_read(s->lora_grad, 0, g.data(), s->lora_n * 4);
    std::vector<float> slots((size_t)s->slots_per_layer * s->NL, 0.f);
    double sq = 0;
    for (float v : g) sq += (double)v * v;
    slots[0] = (float)sq;
    metal_buf_write(s->sq_slots, 0, slots.data(), slots.size() * 4);
    enqueue_update(s);
    metal_flush();
}

MetalBuf *sft_get_logits(SFTState *s) { return s->logits; }
MetalBuf *sft_get_dlogits(SFTState *s)
{
    if (!s->dlogits) s->dlogits = fbuf((size_t)s->BN * s->V);
    return s->dlogits;
}
float *sft_get_x_cpu(SFTState *s)
{
    if (!s->x_in_host) s->x_in_host = host_buf((size_t)s->BN * s->D * 4, (void **)&s->x_cpu);
    return s->x_cpu;
}
float *sft_get_losses_cpu(SFTState *s) { return s->losses_cpu; }
int sft_get_seq_len(SFTState *s) { return s->BN; }
int sft_get_vocab_size(SFTState *s) { return s->V; }
int sft_get_d_model(SFTState *s) { return s->D; }
int sft_get_lora_rank(SFTState *s) { return s->R; }
int sft_get_n_layers(SFTState *s) { return s->NL; }
float sft_get_emb_scale(SFTState *s) { return s->emb_scale; }
int sft_get_step_count(SFTState *s) { return s->step_count; }
void sft_set_step_count(SFTState *s, int step) { s->step_count = step; }
int sft_get_n_lora_grad_bufs(SFTState *s) { return (int)s->grad_views.size(); }
float *sft_get_lora_grad_ptr(SFTState *s, int idx, int *out_size)
{
    if (idx < 0 || idx >= (int)s->grad_views.size()) return nullptr;
    if (out_size) *out_size = (int)(s->grad_views[idx]->size / 4);
    return (float *)metal_buf_ptr(s->grad_views[idx]);     // migrates the gradient arena to host memory
}
void sft_set_lora_grad(SFTState *s, int idx, const float *data, int size)
{
    if (idx < 0 || idx >= (int)s->grad_views.size()) return;
    metal_buf_write(s->grad_views[idx], 0, data, (size_t)size * 4);
}
MetalBuf *sft_get_lora_weight_buf(SFTState *s, int layer, int sub)
{
    const size_t i = (size_t)layer * 4 + sub;
    return i < s->lora_views.size() ? s->lora_views[i] : nullptr;
}
float sft_get_lora_scaling(SFTState *s) { return s->lora_scaling; }

void hip_gemm_image_budget_mb(int mb) { g_image_budget = mb > 0 ? (size_t)mb << 20 : 0; }

// Sliding-window attention on the local layers.  The reference stores Gemma3's window (src/nn/gemma3.c:20, 99) and
// never applies it: its attention kernels see every earlier key on every layer (shaders/q8_kernels.metal:769-855), which
// is what a state does until this is called.  layer_is_local: [n_layers] flags, or NULL for the pattern the reference
// marks (src/nn/gemma3.c:49-57: every layer but those with L % 6 == 0 on Gemma3; every layer on Qwen3).
void sft_set_sliding_window(SFTState *s, int window, const int *layer_is_local)
{
    s->window = window > 0 ? window : 0;
    for (int L = 0; L < s->NL; L++)
        s->layer_local[L] = layer_is_local ? (layer_is_local[L] != 0) : (s->model_type == MODEL_GEMMA3 ? (L % 6) != 0 : 1);
}
ModelType sft_get_model_type(SFTState *s) { return s->model_type; }
int sft_get_n_q_heads(SFTState *s) { return s->Hq; }
int sft_get_n_kv_heads(SFTState *s) { return s->Hkv; }
int sft_get_head_dim(SFTState *s) { return s->hd; }
int sft_get_intermediate_size(SFTState *s) { return s->IS; }
const float *sft_get_rope_thetas(SFTState *s) { return s->rope_thetas.data(); }
int sft_is_full_param(SFTState *s) { return s->full_param; }
const float *sft_get_token_emb(SFTState *s) { return s->token_emb_host; }
MetalBuf *sft_get_final_norm_g(SFTState *s) { return s->g_final; }
MetalBuf *sft_get_token_emb_buf(SFTState *s) { return s->emb; }

size_t sft_lora_numel(SFTState *s) { return s->lora_n; }
void sft_copy_lora(SFTState *s, float *dst) { if (s->lora_n) metal_buf_read(s->lora, 0, dst, s->lora_n * 4); }
void sft_copy_lora_grads(SFTState *s, float *dst) { if (s->lora_n) metal_buf_read(s->lora_grad, 0, dst, s->lora_n * 4); }
void sft_set_lora(SFTState *s, const float *src)
{
    if (!s->lora_n) return;
    metal_buf_write(s->lora, 0, src, s->lora_n * 4);
    refresh_shadow(s);
    metal_flush();
}
float sft_get_last_grad_norm(SFTState *s)
{
    float v = 0.f;
    metal_buf_read(s->grad_norm, 0, &v, 4);
    return v;
}

// Row-major F16 copies of the seven matrices of every layer (refreshed on every call, since
// full-parameter training changes them) plus windows on the norm gammas: what
// inference_state_create_from_sft borrows (src/nn/fast_inference.c:596-603).  The copies are F16 also
// when the state was built from Q8_0 weights (they hold the dequantised values).
LayerW *sft_get_layers(SFTState *s)
{
    const int NL = s->NL, D = s->D, IS = s->IS, qd = s->qd, kd = s->kd;
    const int rows[7] = {qd, kd, kd, D, IS, IS, D}, cols[7] = {D, D, D, qd, D, D, IS};
    if (s->layers_out.empty()) {
        s->wmats_out.resize((size_t)7 * NL);
        s->layers_out.resize(NL);
        for (int L = 0; L < NL; L++) {
            for (int w = 0; w < 7; w++) {
                WMat &m = s->wmats_out[(size_t)L * 7 + w];
                m.rows = rows[w]; m.cols = cols[w]; m.nb = cols[w] / 32;
                m.mbuf = hbuf((size_t)rows[w] * cols[w]);
            }
            WMat *m = &s->wmats_out[(size_t)L * 7];
            auto view = [&](MetalBuf *arena, int dim) -> MetalBuf * {
                if (!arena) return nullptr;
                MetalBuf *v = metal_buf_view(arena, (size_t)L * dim * 4, (size_t)dim * 4);
                s->views_out.push_back(v);
                return v;
            };
            const bool gemma = s->model_type == MODEL_GEMMA3;
            s->layers_out[L] = LayerW{m, m + 1, m + 2, m + 3, m + 4, m + 5, m + 6,
                                      view(s->g_in, D), view(s->g_post_attn, D),
                                      gemma ? view(s->g_pre_ff, D) : nullptr, gemma ? view(s->g_post_ff, D) : nullptr,
                                      view(s->g_q, s->hd), view(s->g_k, s->hd)};
        }
    }
    for (int L = 0; L < NL; L++) {
        struct Src { MetalBuf *W; size_t st; int N, row_off, kind; };
        const Src src[7] = {{s->wqkv, s->st_qkv, D, 0, W_QKV}, {s->wqkv, s->st_qkv, D, qd, W_QKV}, {s->wqkv, s->st_qkv, D, qd + kd, W_QKV},
                            {s->wo, s->st_o, qd, 0, W_O}, {s->wgu, s->st_gu, D, 0, W_GU}, {s->wgu, s->st_gu, D, IS, W_GU}, {s->wd, s->st_d, IS, 0, W_D}};
        for (int w = 0; w < 7; w++) {
            half_t *out = at<half_t>(s->wmats_out[(size_t)L * 7 + w].mbuf);
            if (s->q8_native) {
                const WeightOp op = wop(s, src[w].kind, L, false);
                launch_untile_q8(op.q, op.d, 1, tiled_kb(src[w].N), src[w].row_off, 0, 0, rows[w], cols[w], out);
            } else {
                launch_untile_f16(at<half_t>(src[w].W, L * src[w].st), tiled_kb(src[w].N), src[w].row_off, 0, 0, rows[w], cols[w], out);
            }
        }
    }
    return s->layers_out.data();
}

WMat *sft_get_lm_head(SFTState *s)
{
    WMat &m = s->lm_head_out;
    if (!m.mbuf) { m.rows = s->V; m.cols = s->D; m.nb = s->D / 32; m.mbuf = hbuf((size_t)s->V * s->D); }
    if (s->q8_native) { const WeightOp op = wop(s, W_LM, 0, false); launch_untile_q8(op.q, op.d, 1, tiled_kb(s->D), 0, 0, 0, s->V, s->D, at<half_t>(m.mbuf)); }
    else launch_untile_f16(at<half_t>(s->wlm), tiled_kb(s->D), 0, 0, 0, s->V, s->D, at<half_t>(m.mbuf));
    return &m;
}

// Phases 3 and 4 of grpo_train_step (src/nn/fast_grpo.c:376-495) for a group of completions that
// has already been sampled and scored: per completion build [prompt tail | completion | zero rows],
// forward, PPO-clip policy gradient scaled by 1/G, backward; then apply.
//   full-parameter + accurate: accumulate F16 gradients, one sft_apply_grad_sgd(lr) at the end;
//   full-parameter otherwise:  fused SGD with lr/G after every completion;
//   LoRA:                      sum the adapter gradients over the group, step_count++, AdamW.
// new_logprobs (optional, [G][rows]) receives the policy's log-probabilities of the actions.
void grpo_apply_completions(SFTState *s, const GRPOCompletions *c, float lr, float *new_logprobs)
{
    const int G = c->group_size, seq_len = s->N, B = s->B;
    if (G <= 0) return;
    const bool accurate = s->full_param && c->accurate;
    if (B > 1 && s->full_param && !accurate) {
        fprintf(stderr, "[FastGRPO] SGD after every completion needs a state built with batch 1 (the weights change between completions)\n");
        return;
    }
    if (s->step_in_flight) { metal_flush(); s->step_in_flight = 0; }
    if (!ids_in_vocab(s, c->prompt, (size_t)(c->prompt_len > 0 ? c->prompt_len : 0), "prompt token")) return;
    for (int i = 0; i < G; i++)
        if (!ids_in_vocab(s, c->gen_tokens[i], (size_t)(c->gen_lengths[i] > 0 ? c->gen_lengths[i] : 0), "completion token")) return;
    if (accurate) sft_alloc_grad_accum(s);
    if (!s->grpo_old_lp) {
        s->grpo_old_lp = host_buf((size_t)s->BN * 4, (void **)&s->grpo_old_lp_cpu);
        s->grpo_advs = host_buf((size_t)s->BN * 4, (void **)&s->grpo_advs_cpu);
        s->grpo_new_lp = host_buf((size_t)s->BN * 4, (void **)&s->grpo_new_lp_cpu);
    }
    if (!s->full_param) {
        if (!s->lora_acc) s->lora_acc = fbuf(s->lora_n);
        HIP_CHECK(hipMemsetAsync(dptr(s->lora_acc), 0, s->lora_n * 4, stream()));
    }
    // A state built with batch B takes B completions per pass (one forward and backward for all of them: every weight
    // is streamed once per pass instead of once per completion); sequence slots beyond the group are all zero rows.
    for (int i0 = 0; i0 < G; i0 += B) {
        int any = 0;
        for (int b = 0; b < B; b++) {
            const int i = i0 + b;
            uint32_t *tok = s->tokens_cpu + (size_t)b * seq_len, *act = s->targets_cpu + (size_t)b * seq_len;
            float *olp = s->grpo_old_lp_cpu + (size_t)b * seq_len, *adv = s->grpo_advs_cpu + (size_t)b * seq_len;
            for (int t = 0; t < seq_len; t++) { tok[t] = ZERO_ROW_TOKEN; act[t] = 0; olp[t] = 0.f; adv[t] = 0.f; }
            if (i >= G) continue;
            int comp_len = c->gen_lengths[i];                  // [:388-400]
            if (comp_len > seq_len) comp_len = seq_len;
            int prompt_use = seq_len - comp_len;
            if (prompt_use > c->prompt_len) prompt_use = c->prompt_len;
            if (prompt_use < 0) prompt_use = 0;
            int total = prompt_use + comp_len;
            if (total > seq_len) { comp_len = seq_len - prompt_use; total = seq_len; }
            if (new_logprobs) memset(new_logprobs + (size_t)i * seq_len, 0, (size_t)seq_len * 4);
            if (total <= 0) continue;                          // nothing but zero rows: no gradient
            any = 1;
            const int prompt_start = c->prompt_len - prompt_use;
            for (int t = 0; t < prompt_use; t++) tok[t] = c->prompt[prompt_start + t];
            for (int t = 0; t < comp_len; t++) {               // actions                      [:430-443]
                const int pos = prompt_use + t;
                tok[pos] = c->gen_tokens[i][t];
                act[pos] = c->gen_tokens[i][t];
                olp[pos] = c->gen_logprobs[i][t];
                adv[pos] = c->advantages[i];
            }
        }
        if (!any) continue;
        forward_impl(s, true, true);
        CeArgs ce{};
        ce.logits = at<float>(s->logits); ce.V = s->V; ce.targets = at<uint32_t>(s->targets); ce.losses = at<float>(s->losses);
        ce.dl16 = at<half_t>(s->dl16); ce.inv_scale = at<float>(s->dl_inv); ce.rows_total = s->BN;
        ce.partials = at<float2>(s->ce_part);
        ce.grpo = 1; ce.old_lp = at<float>(s->grpo_old_lp); ce.advs = at<float>(s->grpo_advs); ce.new_lp = at<float>(s->grpo_new_lp);
        ce.clip_eps = c->clip_eps; ce.dl_scale = 1.0f / (float)G;                 // [:445-452]
        launch_ce_rows(ce, s->BN);
        if (s->full_param) {
            backward_impl(s, s->gqkv ? BWD_ACCUM : BWD_SGD, lr / (float)G);       // [:454-461]
        } else {
            backward_impl(s);                                                     // [:462-473]
            metal_enqueue_add_scaled(s->lora_acc, s->lora_grad, 1.0f, (int)s->lora_n);
        }
        metal_flush();
        if (new_logprobs)
            for (int b = 0; b < B && i0 + b < G; b++)
                memcpy(new_logprobs + (size_t)(i0 + b) * seq_len, s->grpo_new_lp_cpu + (size_t)b * seq_len, (size_t)seq_len * 4);
    }
    if (accurate) {                                                               // [:479-481]
        sft_apply_grad_sgd(s, lr);
    } else if (!s->full_param) {                                                  // [:482-491]
        metal_enqueue_copy(s->lora_acc, s->lora_grad, (int)s->lora_n);
        s->step_count++;
        sft_lora_update(s, lr);
    }
}

// "LORA" adapter file: u32 magic 0x4C4F5241, i32 n_layers, i32 rank, then per layer
// A_q, B_q, A_v, B_v as fp32 (src/nn/fast_sft.c:1255-1285) — exactly the arena order.
void sft_save_lora(SFTState *s, const char *path)
{
    FILE *f = fopen(path, "wb");
    if (!f) { fprintf(stderr, "[FastSFT] Cannot open %s for writing\n", path); return; }
    const uint32_t magic = 0x4C4F5241u;
    const int32_t nl = s->NL, rank = s->R;
    fwrite(&magic, 4, 1, f); fwrite(&nl, 4, 1, f); fwrite(&rank, 4, 1, f);
    std::vector<float> w(s->lora_n);
    sft_copy_lora(s, w.data());
    fwrite(w.data(), 4, w.size(), f);
    fclose(f);
}

// qwen3_load_lora (src/nn/qwen3.c:558-602) for the SFT state: the file sft_save_lora writes (magic "LORA", layers,
// rank, then A_q | B_q | A_v | B_v of every layer, fp32) becomes the state's adapters; optimiser moments are kept.
int sft_load_lora(SFTState *s, const char *path)
{
    FILE *f = fopen(path, "rb");
    if (!f) { fprintf(stderr, "[FastSFT] Cannot open %s for reading\n", path); return -1; }
    uint32_t magic = 0;
    int32_t nl = 0, rank = 0;
    const bool head = fread(&magic, 4, 1, f) == 1 && fread(&nl, 4, 1, f) == 1 && fread(&rank, 4, 1, f) == 1;
    if (!head || magic != 0x4C4F5241u) { fprintf(stderr, "[FastSFT] Invalid LoRA file magic\n"); fclose(f); return -1; }
    if (nl != s->NL || rank != s->R) {
        fprintf(stderr, "[FastSFT] LoRA config mismatch: file(layers=%d,rank=%d) vs state(layers=%d,rank=%d)\n", nl, rank, s->NL, s->R);
        fclose(f);
        return -1;
    }
    std::vector<float> w(s->lora_n);
    const size_t got = fread(w.data(), 4, w.size(), f);
    fclose(f);
    if (got != w.size()) { fprintf(stderr, "[FastSFT] LoRA file %s is truncated\n", path); return -1; }
    sft_set_lora(s, w.data());
    return 0;
}

}  // extern "C"

// internal: see BorrowedLayer
void lmhip::sft_borrow_layer(SFTState *s, int L, BorrowedLayer *out)
{
    if (s->gamma_views.empty()) {
        s->gamma_views.resize((size_t)6 * s->NL, nullptr);
        const bool gemma = s->model_type == MODEL_GEMMA3;
        MetalBuf *arena[6] = {s->g_in, s->g_post_attn, gemma ? s->g_pre_ff : nullptr, gemma ? s->g_post_ff : nullptr, s->g_q, s->g_k};
        const int dim[6] = {s->D, s->D, s->D, s->D, s->hd, s->hd};
        for (int l = 0; l < s->NL; l++)
            for (int g = 0; g < 6; g++)
                if (arena[g]) s->gamma_views[(size_t)l * 6 + g] = metal_buf_view(arena[g], (size_t)l * dim[g] * 4, (size_t)dim[g] * 4);
    }
    MetalBuf **g = &s->gamma_views[(size_t)L * 6];
    *out = BorrowedLayer{wop(s, W_QKV, L, false), wop(s, W_O, L, false), wop(s, W_GU, L, false), wop(s, W_D, L, false),
                         g[0], g[1], g[2], g[3], g[4], g[5]};
}
WeightOp lmhip::sft_borrow_lm_head(SFTState *s) { return wop(s, W_LM, 0, false); }
