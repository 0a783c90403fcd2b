// Launch interface of the fused SFT kernels (fused_kernels.hip).  The host
// pipeline (sft.hip) strings these together with the weight-streaming GEMM:
// activations that feed a GEMM are produced directly as scaled fp16 rows, GEMM
// outputs arrive as K-split partial planes that the consumer sums on load.
#pragma once
#include <cstddef>
#include <stdio.h>
#include <stdlib.h>
#include "backend.h"
#include "devutil.h"
#include "gemm.h"

namespace lmhip {

// K-split partial planes of a GEMM output: value(row, col) = row_scale[row] * sum_s p[s*stride + row*ld + col]
// (40 bytes: with two ints and a pointer in front of it, it fits the arguments that reach a kernel preloaded, kargs.h)
struct Planes {
    const float *p;
    const float *row_scale;   // value(row, col) is multiplied by row_scale[row] when non-null
    uint32_t stride;          // elements between planes
    int S;
    int ld;
    // scale_groups != 0: the operand rows were scaled in that many groups of columns, each the K range of 2^group_shift
    // planes, and plane s is multiplied by row_scale[row * scale_groups + (s >> group_shift)] before it is added
    int16_t group_shift, scale_groups;
    // not 0: the planes hold halves (p points at them, stride and ld count halves), each the chunk's fp32 sum times a
    // power of two that keeps it below the fp16 maximum for any operand row; a value read is multiplied by half_unscale,
    // the inverse of that factor.  Only kernels that read their planes through planes_at4_multi may be given such planes.
    float half_unscale;
};
inline Planes make_planes(const float *p, int S, size_t stride, int ld, const float *row_scale, int group_shift = 0, int scale_groups = 0,
                          float half_unscale = 0.f)
{
    if (stride > 0xffffffffull) { fprintf(stderr, "[fast_hip] planes: more than 2^32 elements per plane\n"); abort(); }
    Planes P;
    P.p = p; P.row_scale = row_scale; P.stride = (uint32_t)stride; P.S = S; P.ld = ld;
    P.group_shift = (int16_t)group_shift; P.scale_groups = (int16_t)scale_groups; P.half_unscale = half_unscale;
    return P;
}
static_assert(sizeof(Planes) == 40, "Planes is part of the kernels' preloaded arguments");

// How a row kernel splits the columns of an fp16 operand row [*, K] among workgroups, each with a power-of-two scale of
// its own: `cols` columns per group (a whole number of K chunks of the GEMM that consumes the operand), `groups` of
// them; cols == 0: one workgroup and one scale per row.
struct ScaleGroups { int cols, groups, shift; };

// Weight tiles of the product that follows a row kernel, for the workgroups the row kernel starts beyond its rows: they
// request, while most CUs have nothing to do, the tiles that the product's workgroups ask for first (its workgroup g
// starts with the K steps rot(g) .. rot(g) + 3 of its chunk).  Hardware counters show that the product fetches them
// again from beyond L2 (no line survives a kernel boundary there), but it then finds them in the memory-side cache, and
// its first K steps stop waiting for HBM.  Which XCD asks makes no difference.  F16 tiles, or the int8 tiles of a Q8_0
// operand (their scales, 6 % of the bytes, are left to the product); base == null: nothing to fetch.
struct WeightPrefetch {
    const char *base;             // tiled F16 weight image, or the int8 tiles of a Q8_0 operand (rotate & 2)
    int Kb, Nb;                   // K steps and 32-row blocks of the image (Q8_0: of its quantised part)
    int nb, steps, S, n_tiles;    // the product's plan: blocks per workgroup, K steps per chunk, chunks, row tiles
    int rotate;                   // bit 0: the product rotates its K steps; bit 1: Q8_0 tiles of 2 KB, `depth` counts pairs of K steps
    int wgs;                      // prefetching workgroups
    int per_wg;                   // product workgroups each of them covers
    int depth;                    // K steps fetched per product workgroup (its waves' first steps)
};

constexpr uint32_t ZERO_ROW_TOKEN = 0xFFFFFFFFu;

struct NormRowsArgs {
    // (the first 56 bytes reach the kernel preloaded: all that the workgroups beyond the rows need, which ask for the next
    // product's weights and are the last to finish; the rows' workgroups read the rest from the argument segment)
    int rows_launched;            // set by the launcher
    int D;
    WeightPrefetch pf;
    const float *x_prev;          // source of the residual stream row, unless it is gathered (emb != null)
    // optional branch added to it: planes, optionally RMS-normalised with g_branch first
    Planes branch;
    const float *emb; const uint32_t *tokens; float emb_scale;      // token gather
    int zero_rows;                // gather only: rows whose token id is ZERO_ROW_TOKEN read as zero (padding of a short sequence)
    const float *g_branch; float *branch_raw_out;
    float *x_out;                 // new residual stream row (may be null when nothing was added)
    const float *g_norm;          // null: no normalised output wanted
    half_t *ln16; float *inv_scale;   // tiled [rows, D]
    float eps;
};
static_assert(offsetof(NormRowsArgs, x_prev) == 56, "NormRowsArgs: preloaded part");
void launch_norm_rows(const NormRowsArgs &a, int rows);

// The matrix-core attention reads K and V once more from copies laid out [batch][Hkv][hd/4][attn_ldt(seq)][4]:
// element (pos, d) of a head at ((d / 4) * ldt + pos) * 4 + d % 4.
__host__ __device__ inline int attn_ldt(int seq) { return seq + 32; }
__host__ __device__ inline size_t attn_t_index(int d, int pos, int ldt) { return ((size_t)(d >> 2) * ldt + pos) * 4 + (d & 3); }

struct QkvPostArgs {
    Planes qkv;                   // [rows][q | k | v | tq(R) | tv(R)]
    const float *Bq, *Bv;         // LoRA B, [Hq*hd][R], [Hkv*hd][R]
    int R; float sc;
    const float *g_q, *g_k; float eps;
    const float2 *rope;           // [seq][hd/2] (cos, sin) of this layer's theta
    int Hq, Hkv, hd, seq;
    float *q_pre, *k_pre, *q_fin, *k_fin, *v_out;   // [rows][H*hd]
    float *tq, *tv;               // [rows][R]
    float *kT, *vT;               // optional: the same k_fin / v_out per head and transposed, [batch][Hkv][hd/4][attn_ldt(seq)][4]
    int rows;
};
void launch_qkv_post(const QkvPostArgs &a, int rows);
// tab[pos][d] = (cos, sin)(pos * theta^(-2d/hd)), pos < seq, d < hd/2
void launch_rope_table(float2 *tab, int seq, int hd, float theta);

// Causal GQA attention over [rows][H*hd] row-major activations, probabilities saved.
struct AttnFwdArgs {
    const float *q, *k, *v; int Hq, Hkv, hd, seq, batch; float scale;
    float *probs;                 // [batch][Hq][seq][seq]
    half_t *out16;                // tiled [rows, Hq*hd], unit scale
    const float *kT;              // k transposed per head [batch][Hkv][hd/4][attn_ldt(seq)][4] (matrix-core path only)
    WeightPrefetch pf;            // matrix-core path: weights of the product that follows
    int window;                   // > 0: query i sees keys i - window + 1 .. i only (sliding window); 0: all keys up to i
};
void launch_attn_fwd(const AttnFwdArgs &a);

struct AttnBwdArgs {
    Planes dO;                    // [rows][Hq*hd]
    const float *probs, *q, *k, *v; int Hq, Hkv, hd, seq, batch; float scale;
    const float *vT;              // v transposed per head [batch][Hkv][hd/4][attn_ldt(seq)][4] (matrix-core path only)
    float *dO_red, *dscore;       // scratch: [rows][Hq*hd], [batch][Hq][seq][seq]
    float *dq, *dk, *dv;          // [rows][Hq*hd], [rows][Hkv*hd] x2 (post-RoPE domain)
    // matrix-core path, at most 64 keys: not null -> one launch that leaves dk / dv as shares per (query block, query
    // head), [ceil(seq/32)][Hq][rows][hd] each, for launch_qkv_bwd to sum (dk, dv, dO_red, dscore are then not written)
    float *dkp, *dvp;
};
void launch_attn_bwd(const AttnBwdArgs &a);
// The same two operations on the fp32 matrix cores (attn_mfma.hip): head_dim a multiple of 32 and a
// 32-row block of scores within the LDS budget; the wave-per-query kernels above remain the general path.
bool attn_mfma_supported(int hd, int seq);
void launch_attn_fwd_mfma(const AttnFwdArgs &a);
void launch_attn_bwd_mfma(const AttnBwdArgs &a);
// dQ and the dK / dV shares in one launch (AttnBwdArgs::dkp): on by default wherever the matrix-core path runs on at
// most 64 keys; the switch is for comparisons with the two-launch path
void set_attn_bwd_one_launch(int on);
bool attn_bwd_one_launch(int hd, int seq);

// The same attention without the [seq, seq] matrices in memory (attn_flash.hip): head_dim 64 or 128, any sequence
// length.  The forward saves the operands of the backward (bf16-pair fragments of q, k, v), the output and one
// number per query row; the backward needs the window again (nothing saved carries it).
struct AttnFlashArgs {
    const float *q, *k, *v;       // forward: [rows][Hq*hd], [rows][Hkv*hd] x2 (post-RoPE)
    Planes dO;                    // backward: [rows][Hq*hd]
    int Hq, Hkv, hd, seq, batch, window; float scale;
    uint4 *q_rt, *q_pt, *k_rt, *k_pt, *v_rt, *v_pt;    // written by the forward, attn_flash_tile_elems() each
    uint4 *do_rt, *do_pt;         // backward scratch, as q_rt
    float *O, *lse;               // written by the forward: [rows][Hq*hd], [batch][Hq][ceil(seq/32)*32]
    float *D;                     // backward scratch, as lse
    half_t *out16;                // forward: tiled [rows, Hq*hd], unit scale
    float *dq, *dk, *dv;          // backward: [rows][Hq*hd], [rows][Hkv*hd] x2
    float *dkp, *dvp;             // backward scratch: [Hq/Hkv][rows][Hkv*hd] each
};
// -1: head_dim 64/128 and enough (128-query block, head, sequence) workgroups for half the CUs, or more than 1024
// positions (default); 0: never; 1: whenever the head size allows
void set_attn_flash_mode(int mode);
bool attn_flash_supported(int hd, int seq, int Hq, int Hkv, int batch);
size_t attn_flash_tile_elems(int hd, int seq, int heads, int batch);     // 16-byte elements of one RT or PT image
// q, k, v null: the fragments are there already (launch_qkv_post_flash)
void launch_attn_fwd_flash(const AttnFlashArgs &a);
// The QKV epilogue (launch_qkv_post) writing this attention's fragments instead of fp32 q_fin / k_fin / v_out: uses
// a.qkv, B, rank, norm weights, rope, q_pre, k_pre, tq, tv of `a` and the fragment pointers of `f`.
void launch_qkv_post_flash(const QkvPostArgs &a, const AttnFlashArgs &f);
void launch_attn_bwd_flash(const AttnFlashArgs &a);

struct QkvBwdArgs {
    const float *dq, *dk, *dv;    // post-RoPE-domain gradients
    // not null: dk and dv come as shares [query block][Hq][rows_total][hd] instead (AttnBwdArgs::dkp): key row j of
    // KV head hk is the sum over the query heads of its group and over the query blocks from j / 32 on; the summed dv
    // is also written to dv_f
    const float *dkp, *dvp; int rows_total;
    const float *q_pre, *k_pre, *g_q, *g_k; float eps;
    const float2 *rope;
    const float *Bq, *Bv; int R; float sc;
    // optional fp16 copies of B_q and B_v (rank 16): every row's workgroup reads all of B for the projection dh, and that
    // read is what a CU's path from L2 spends most of the kernel on; half the bytes.  null: the fp32 matrices are read
    const half_t *Bq16, *Bv16;
    int Hq, Hkv, hd, seq;
    float *dq_f, *dv_f;           // pre-norm-domain dq [rows][Hq*hd], dv copy [rows][Hkv*hd] (for dB)
    float *dh;                    // [rows][2R] = sc * dq B_q | sc * dv B_v
    half_t *out16; float *inv_scale;                // tiled [rows, dq | dk | dv | dh_q | dh_v]
    WeightPrefetch pf; int rows_launched;           // weights of the product that follows; rows_launched: set by the launcher
};
void launch_qkv_bwd(const QkvBwdArgs &a, int rows);

// All pointers address layer 0; layer L of a launch over `layers` layers lies L * (the matching stride) further on.
struct LoraGradArgs {
    const float *dq_f, *dv_f, *tq, *tv, *dh;
    const half_t *ln16; const float *ln_inv_scale;  // tiled [rows, D]
    int rows, D, qd, kd, R; float sc;
    float *grad;                  // arena: dA_q | dB_q | dA_v | dB_v per layer
    float *sq_slots;              // one partial sum of squares per workgroup
    int layers;
    size_t st_dq, st_dv, st_t, st_dh, st_ln16, st_lninv, st_grad, st_slots;   // layer strides in elements
};
int  lora_grad_blocks(int D, int qd, int kd, int R);
void launch_lora_grads(const LoraGradArgs &a);

struct GluArgs {
    // (the first 56 bytes -- the planes, gate_pre, IS and sg.cols -- reach the column-group kernels preloaded, kargs.h)
    Planes in;                    // fwd: [rows][gate | up]; bwd: [rows][d act]
    float *gate_pre;              // fwd: written; bwd: read; rows ld_gu floats apart (gate_pre and up_val are the halves of one [rows][2 IS] array)
    int IS;
    ScaleGroups sg;               // sg.cols != 0: inv_scale is [rows][sg.groups]
    int gelu;
    float *up_val;
    size_t ld_gu;
    int in_place;                 // fwd, one workgroup per row only: `in` is that array (one plane, factors applied): nothing to copy
    half_t *out16; float *inv_scale;                // tiled; fwd: act [rows, IS]; bwd: [rows, dgate | dup]
};
void launch_glu_fwd(const GluArgs &a, int rows);
void launch_glu_bwd(const GluArgs &a, int rows);

struct NormBwdArgs {
    int rows_launched; int D;                           // (first 56 bytes: preloaded, see NormRowsArgs)
    WeightPrefetch pf;
    const float *x_saved;
    Planes dy;
    const float *g; float eps;
    const float *dx_prev; float *dx_out; float clamp;   // clamp <= 0: none
    const float *branch_raw, *g_branch;                 // Gemma3: next GEMM input is RNB(branch_raw, dx_out)
    half_t *d16; float *inv_scale;                      // tiled [rows, D]; may be null on the last kernel of the backward
};
static_assert(offsetof(NormBwdArgs, x_saved) == 56, "NormBwdArgs: preloaded part");
void launch_norm_bwd_rows(const NormBwdArgs &a, int rows);

struct CeArgs {
    const float *logits; int V; const uint32_t *targets; float *losses;
    half_t *dl16; float *inv_scale; int rows_total;     // tiled [rows, V]
    float2 *partials;             // scratch [rows][CE_CHUNKS] (running maximum, sum of exponentials) of the row chunks
    // policy-gradient variant (grpo != 0): targets are the sampled actions; losses is not written
    int grpo; const float *old_lp, *advs; float *new_lp; float clip_eps, dl_scale;
};
constexpr int CE_CHUNKS = 16;
void launch_ce_rows(const CeArgs &a, int rows);

struct AdamArgs {
    float *p, *g, *m, *v; size_t n;
    const float *sq_slots; int n_slots;
    const float *hyper;           // device-visible: [0] lr, [1] 1-b1^t, [2] 1-b2^t, written by the host per step
    float b1, b2, eps, wd, max_norm;
    // fp16 shadows of A_q / A_v: rows a_row0.. of the tiled image wqkv ([*, D]) and columns a_row0.. of the
    // transposed image wqkvT (kbT K blocks per row block)
    half_t *wqkv; size_t wqkv_layer_stride; half_t *wqkvT; size_t wqkvT_layer_stride;
    int a_row0, kbT;
    half_t *p16;                  // optional: fp16 copy of the whole arena, same indexing (k_qkv_bwd_rows reads B_q, B_v there)
    int NL, D, qd, kd, R; size_t layer_size;
    float *grad_norm_out;         // [1]
};
void launch_adamw(const AdamArgs &a);

// fp16 shadow refresh only (after LoRA weights were written from outside)
void launch_lora_shadow(const float *p, size_t n, half_t *wqkv, size_t wqkv_layer_stride, half_t *wqkvT,
                        size_t wqkvT_layer_stride, int D, int qd, int kd, int R, size_t layer_size, int a_row0, int kbT,
                        half_t *p16 = nullptr);

void launch_fill_f32(float *p, float v, size_t n);

// ---- full-parameter mode (fullparam.hip) ----
// out (tiled [F, T]) and out_inv[F] <- transposed in (tiled [T, F]) with in_inv[T]; out_inv needs tiled_kb(F)*64 floats
void launch_transpose_scaled(const half_t *in_tiled, const float *in_inv, int T, int F, half_t *out_tiled, float *out_inv);
// two operands [T, F0] and [T, F1] in one launch
void launch_transpose_scaled_pair(const half_t *in0, const float *in0_inv, int F0, half_t *out0, float *out0_inv,
                                  const half_t *in1, const float *in1_inv, int F1, half_t *out1, float *out1_inv, int T);
// up to eight operands [T, F] in one launch
struct TransposeOperand { const half_t *in; const float *in_inv; int F; half_t *out; float *out_inv; };
void launch_transpose_scaled_jobs(const TransposeOperand *ops, int n, int T);
// target (tiled [M_out, N_in] F16) <- half(target + alpha * Y^T X), XT/YT = transposed operands over T tokens;
// sgd: alpha = -lr (f16_sgd_fused), else alpha = 1 (f16_grad_accum)
void launch_wgrad(const half_t *XT, const float *x_inv, const half_t *YT, const float *y_inv, half_t *target_tiled,
                  int M_out, int N_in, int T, int sgd, float lr);
// the same for up to four matrices in one launch
struct WgradOperands { const half_t *XT; const float *x_inv; const half_t *YT; const float *y_inv; half_t *target_tiled; int M_out, N_in; };
void launch_wgrads(const WgradOperands *w, int n, int T, int sgd, float lr);
// G != null: W = half(W - lr G), G = 0 (f16_sgd_apply); always: WT (tiled [N_in, M_out]) <- W^T.  `matrices` of the same
// shape in one launch, `stride` halves apart in W and G and `strideT` in WT (the layers of an arena).
void launch_apply_retile(half_t *W_tiled, half_t *G_tiled, half_t *WT_tiled, int M_out, int N_in, float lr,
                         int matrices = 1, size_t stride = 0, size_t strideT = 0);
void launch_untile_f16(const half_t *src_tiled, int Kb, int row_off, int k_off, int transpose, int rows, int cols, half_t *dst);

}  // namespace lmhip
