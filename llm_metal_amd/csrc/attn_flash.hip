// Causal GQA attention for long sequences, forward and backward, without the [seq, seq] matrices in memory: the
// forward keeps a running maximum and sum per query row and saves log2(sum) + max, the backward forms the
// probabilities again from the scores and that one number per row.  Same arithmetic as attn_train_fwd /
// attn_bwd_dq / attn_bwd_dkv / repeat_kv_bwd of shaders/q8_kernels.metal:769-992 (saved probabilities there,
// src/nn/fast_sft.c:678-689), on v_mfma_f32_32x32x16_bf16 with every fp32 operand as a bf16 pair (bf16pair.h).
//
// Operands.  Q, K, V and dO of a head are split into bf16 pairs ONCE (k_fa_split) and laid out as the matrix-core
// fragments the kernels need, 1 KB each ([64 lanes][8 bf16]), so that a 32-row block of a head is one contiguous tile
// of HD / 8 fragments that goes from L2 into LDS by global_load_lds (no registers, no conversion in the consumers):
//   RT (rows):        fragment (j, part), j < HD/16: lane (r, hh) holds X[32 blk + r][16 j + 8 hh + 0..7]
//                     -- the operand of a product that reduces over the head's columns
//   PT (transposed):  fragment (db, u, part), db < HD/32, u < 2: lane (c, hh) holds X[32 blk + row(u, hh, e)][32 db + c],
//                     row(u, hh, e) = 16 u + 8 (e / 4) + 4 hh + e % 4 -- the operand of a product that reduces over the
//                     block's 32 rows, in the order in which the accumulator of a 32 x 32 product holds them
//                     (value v of lane half hh is row 8 (v / 4) + 4 hh + v % 4): the accumulator values 8 u .. 8 u + 7
//                     of a lane, split into a bf16 pair, ARE the other operand, without a trip through LDS.
// part 0 holds the upper bf16 values, part 1 the lower ones.
//
// Kernels (a wave owns a 32 x 32 tile position, a workgroup four of them that share the streamed tiles through LDS):
//   k_fa_fwd   wave: 32 queries; streams RT(K), PT(V).      S^T = K Q^T, online softmax, O^T += V^T P^T
//   k_fa_dq    wave: 32 queries; streams RT(K), RT(V), PT(K).  S^T, dP^T = V dO^T, dS^T, dQ^T += K^T dS^T
//   k_fa_dkv   wave: 32 keys of one QUERY head; streams RT(Q), RT(dO), PT(Q), PT(dO).
//              S = Q K^T, dP = dO V^T, dV^T += dO^T P, dK^T += Q^T dS; the query heads of a group leave planes that
//              k_fa_sum_groups adds
// Scores are formed transposed in the first two so that a query is a lane (column of the accumulator): its maximum,
// sum, log-sum and D = rowsum(dO o O) are per-lane scalars, and the row reductions are 16 in-register steps and one
// exchange between the lane halves.
#include "fused.h"
#include "planes.h"
#include "bf16pair.h"

namespace lmhip {
namespace {

#define LAUNCH(kern, grid, block, lds, ...) do { \
    hipLaunchKernelGGL(kern, grid, block, lds, stream(), __VA_ARGS__); HIP_CHECK(hipGetLastError()); } while (0)

typedef __attribute__((address_space(3))) void lds_void;

// "This value is needed here": the compiler places its wait for the load behind x at this point instead of at the
// first real use, which would lie behind requests of later tiles and wait for those as well.
#define FA_TOUCH(x) asm volatile("" :: "v"(x))

__device__ __forceinline__ float16v zero16()
{
    float16v z;
#pragma unroll
    for (int v = 0; v < 16; v++) z[v] = 0.f;
    return z;
}
__device__ __forceinline__ bf16x8 frag(const uint4 *p) { return __builtin_bit_cast(bf16x8, *p); }
__device__ __forceinline__ float16v mfma(bf16x8 a, bf16x8 b, float16v c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }

// row of the 32-row block that element e of step u holds in lane half hh of a PT fragment = row of accumulator value 8 u + e
__device__ __forceinline__ int pt_row(int u, int hh, int e) { return 16 * u + 8 * (e >> 2) + 4 * hh + (e & 3); }

// Workgroup ids go to the eight XCDs in turn (id % 8).
// The kernels' work items are (sequence of tiles to stream) x (position in it), and a position's work grows or
// shrinks with its index (causal mask).  An XCD takes `cnt` consecutive items = cnt / npos whole sequences when that
// divides (else the plain order is kept): it starts the heaviest position of all its sequences first, then the next
// one, ..., so that the workgroups that become free early take the light positions (longest work first), while the
// tiles of its few sequences stay in its L2.  Returns the item as (sequence, rank of the position by weight).
__device__ __forceinline__ void heavy_first_item(int id, int n, int npos, int &seq, int &rank)
{
    const int x = id & 7, per = n >> 3, rem = n & 7;
    const int start = x * per + min(x, rem), cnt = per + (x < rem ? 1 : 0), j = id >> 3;
    if (cnt % npos == 0 && start % npos == 0) {
        const int g = cnt / npos;
        seq = start / npos + j % g; rank = j / g;
    } else { seq = (start + j) / npos; rank = (start + j) % npos; }
}

// query i sees key j
__device__ __forceinline__ bool sees(int i, int j, int window) { return j <= i && (window <= 0 || j > i - window); }

// ---------------------------------------------------------------------------------------------------------------
// Operand split.  grid (blocks of 32 rows, H, batch), block 256.
struct FaSplitArgs {
    const float *X; size_t ldx;          // [rows][ldx], head h at columns h * HD ..; or, when X is null, the planes Xpl
    Planes Xpl;
    int H, seq, batch;
    uint4 *rt, *pt;                      // [batch][H][nblk][HD/8 fragments][64]
    const float *O; float *D;            // optional: D[batch][H][nblk * 32] = rowsum(X o O), O [rows][H * HD]
};

// NBP: planes fetched per batch of loads (1 when the product left a single plane: fewer registers, more workgroups per CU)
template <int HD, int NBP>
__global__ __launch_bounds__(256) void k_fa_split(FaSplitArgs a)
{
    constexpr int LDS_LD = HD + 4, NJ = HD / 16, TILE = HD / 8 * 64, TPR = HD / 4;      // TPR: threads per row
    __shared__ float Xs[32 * LDS_LD];
    const int blk = blockIdx.x, h = blockIdx.y, b = blockIdx.z, nblk = gridDim.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l31 = lane & 31, hh = lane >> 5;
    const size_t r0 = (size_t)b * a.seq;
    const int width = a.H * HD;
    {
        float4 xv[HD / 32];
        size_t rows[HD / 32]; int cols[HD / 32]; bool ok[HD / 32];
#pragma unroll
        for (int u = 0; u < HD / 32; u++) {
            const int idx = tid + 256 * u, rr = idx / TPR, c4 = idx % TPR;
            ok[u] = blk * 32 + rr < a.seq; rows[u] = r0 + (ok[u] ? blk * 32 + rr : 0); cols[u] = h * HD + 4 * c4;
        }
        if (a.X) {
#pragma unroll
            for (int u = 0; u < HD / 32; u++) xv[u] = ok[u] ? ld4(a.X + rows[u] * a.ldx + cols[u]) : make_float4(0.f, 0.f, 0.f, 0.f);
        } else planes_at4_multi<HD / 32, NBP>(a.Xpl, rows, cols, ok, xv);
#pragma unroll
        for (int u = 0; u < HD / 32; u++) {
            const int idx = tid + 256 * u, rr = idx / TPR, c4 = idx % TPR;
            st4(Xs + rr * LDS_LD + 4 * c4, xv[u]);
            if (a.D) {                                      // the TPR threads of a row are neighbours in one wave
                float d = 0.f;
                if (ok[u]) { const float4 o = ld4(a.O + rows[u] * width + cols[u]); d = xv[u].x * o.x + xv[u].y * o.y + xv[u].z * o.z + xv[u].w * o.w; }
#pragma unroll
                for (int s = 1; s < TPR; s <<= 1) d += __shfl_xor(d, s, WAVE);
                if (c4 == 0) a.D[((size_t)b * a.H + h) * nblk * 32 + blk * 32 + rr] = d;
            }
        }
    }
    __syncthreads();
    uint4 *rt = a.rt + (((size_t)b * a.H + h) * nblk + blk) * TILE + lane;
    uint4 *pt = a.pt + (((size_t)b * a.H + h) * nblk + blk) * TILE + lane;
    for (int p = wave; p < HD / 8; p += 4) {
        float x[8];
        if (p < NJ) {                                       // RT pair j = p
            const float *src = Xs + l31 * LDS_LD + 16 * p + 8 * hh;
            const float4 lo4 = ld4(src), hi4 = ld4(src + 4);
            const HL f = split8(lo4, hi4);
            rt[(2 * p) * 64] = __builtin_bit_cast(uint4, f.hi);
            rt[(2 * p + 1) * 64] = __builtin_bit_cast(uint4, f.lo);
        } else {                                            // PT pair (db, u)
            const int q = p - NJ, db = q >> 1, u = q & 1;
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] = Xs[pt_row(u, hh, e) * LDS_LD + 32 * db + l31];
            const HL f = split8(x);
            pt[(2 * q) * 64] = __builtin_bit_cast(uint4, f.hi);
            pt[(2 * q + 1) * 64] = __builtin_bit_cast(uint4, f.lo);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The QKV epilogue for this attention: what k_qkv_post does (plane sums, LoRA term sc * (x A^T) B^T, pre-norm copy,
// per-head RMSNorm, half-split RoPE; src/nn/fast_sft.c:639-669, shaders/q8_kernels.metal:495-538) on a tile of 32
// positions of one head, which then leaves the workgroup as the RT and PT fragments directly: no fp32 copy of the
// final q, k, v is written and read again.  grid (blocks of 32 positions, Hq + 2 Hkv, batch), block 256.
// RK: the LoRA rank compiled in (16), or -1 for any rank up to 64 (0 included).
template <int HD, int RK, int NBP>                           // NBP as in k_fa_split
__global__ __launch_bounds__(256) void k_qkv_post_tile(QkvPostArgs a, uint4 *q_rt, uint4 *q_pt, uint4 *k_rt, uint4 *k_pt, uint4 *v_rt, uint4 *v_pt, int batch)
{
    constexpr int LDS_LD = HD + 4, NJ = HD / 16, TILE = HD / 8 * 64, TPR = HD / 4, HALF = HD / 2;
    __shared__ float Xs[32 * LDS_LD];
    __shared__ float Ts[32 * 64];
    __shared__ float Inv[32];
    const int blk = blockIdx.x, slot = blockIdx.y, b = blockIdx.z, nblk = gridDim.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l31 = lane & 31, hh = lane >> 5;
    const int N = a.seq, qd = a.Hq * HD, kd = a.Hkv * HD, R = RK >= 0 ? RK : a.R;
    const int kind = slot < a.Hq ? 0 : (slot < a.Hq + a.Hkv ? 1 : 2);     // 0 q, 1 k, 2 v
    const int h = kind == 0 ? slot : (kind == 1 ? slot - a.Hq : slot - a.Hq - a.Hkv);
    const int col0 = kind == 0 ? h * HD : (kind == 1 ? qd + h * HD : qd + kd + h * HD);
    const int t0 = qd + 2 * kd + (kind == 2 ? R : 0);
    const bool lora = R > 0 && kind != 1;
    const size_t r0 = (size_t)b * N;
    {   // ---- the tile and its rows of x A^T
        float4 xv[HD / 32];
        size_t rows[HD / 32]; int cols[HD / 32]; bool ok[HD / 32];
#pragma unroll
        for (int u = 0; u < HD / 32; u++) {
            const int idx = tid + 256 * u, rr = idx / TPR, c4 = idx % TPR;
            ok[u] = blk * 32 + rr < N; rows[u] = r0 + (ok[u] ? blk * 32 + rr : 0); cols[u] = col0 + 4 * c4;
        }
        planes_at4_multi<HD / 32, NBP>(a.qkv, rows, cols, ok, xv);
#pragma unroll
        for (int u = 0; u < HD / 32; u++) { const int idx = tid + 256 * u; st4(Xs + (idx / TPR) * LDS_LD + 4 * (idx % TPR), xv[u]); }
        if (lora)
            for (int idx = tid; idx < 32 * R; idx += 256) {
                const int rr = idx / R, k = idx % R;
                const bool okr = blk * 32 + rr < N;
                const float t = okr ? planes_at(a.qkv, r0 + blk * 32 + rr, t0 + k) : 0.f;
                Ts[rr * 64 + k] = t;
                if (okr && h == 0) (kind == 0 ? a.tq : a.tv)[(r0 + blk * 32 + rr) * R + k] = t;
            }
    }
    __syncthreads();
    {   // ---- LoRA term, pre-norm copy: a thread owns one column of HD for 32 * HD / 256 rows
        constexpr int PARTS = 256 / HD, RPP = 32 / PARTS;
        const int d = tid % HD, part = tid / HD;
        float *pre = kind == 0 ? a.q_pre : a.k_pre;
        const int W = kind == 0 ? qd : kd;
        if (lora) {
            const float *B = (kind == 0 ? a.Bq : a.Bv) + (size_t)(h * HD + d) * R;
            if constexpr (RK == 16) {
                float4 w[4];
#pragma unroll
                for (int i = 0; i < 4; i++) w[i] = ld4(B + 4 * i);
#pragma unroll
                for (int q = 0; q < RPP; q++) {
                    const int rr = part * RPP + q;
                    const float *t = Ts + rr * 64;
                    float acc = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; i++) { acc += t[4 * i] * w[i].x; acc += t[4 * i + 1] * w[i].y; acc += t[4 * i + 2] * w[i].z; acc += t[4 * i + 3] * w[i].w; }
                    Xs[rr * LDS_LD + d] += a.sc * acc;
                }
            } else {
                for (int q = 0; q < RPP; q++) {
                    const int rr = part * RPP + q;
                    float acc = 0.f;
                    for (int k = 0; k < R; k++) acc += Ts[rr * 64 + k] * B[k];
                    Xs[rr * LDS_LD + d] += a.sc * acc;
                }
            }
        }
        if (kind != 2)
#pragma unroll
            for (int q = 0; q < RPP; q++) {
                const int rr = part * RPP + q;
                if (blk * 32 + rr < N) pre[(r0 + blk * 32 + rr) * W + h * HD + d] = Xs[rr * LDS_LD + d];
            }
    }
    __syncthreads();
    if (kind != 2) {
        {   // ---- 1 / rms of every row: eight threads per row
            const int rr = tid >> 3, part = tid & 7;
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < HD / 32; c++) { const float4 v = ld4(Xs + rr * LDS_LD + 32 * c + 4 * part); ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w; }
            ss += __shfl_xor(ss, 1, WAVE); ss += __shfl_xor(ss, 2, WAVE); ss += __shfl_xor(ss, 4, WAVE);
            if (part == 0) Inv[rr] = rsqrtf(ss / (float)HD + a.eps);
        }
        __syncthreads();
        {   // ---- weight, RoPE on the pairs (d, d + HD/2): a thread owns one pair for 32 * HALF / 256 rows
            constexpr int PARTS = 256 / HALF, RPP = 32 / PARTS;
            const int d = tid % HALF, part = tid / HALF;
            const float *g = kind == 0 ? a.g_q : a.g_k;
            const float g0 = g[d], g1 = g[d + HALF];
#pragma unroll
            for (int q = 0; q < RPP; q++) {
                const int rr = part * RPP + q, pos = blk * 32 + rr;
                if (pos >= N) continue;
                const float inv = Inv[rr];
                const float n0 = Xs[rr * LDS_LD + d] * inv * g0, n1 = Xs[rr * LDS_LD + d + HALF] * inv * g1;
                const float2 cs = a.rope[(size_t)pos * HALF + d];
                Xs[rr * LDS_LD + d] = n0 * cs.x - n1 * cs.y;
                Xs[rr * LDS_LD + d + HALF] = n0 * cs.y + n1 * cs.x;
            }
        }
        __syncthreads();
    }
    // ---- the tile as fragments
    const int H = kind == 0 ? a.Hq : a.Hkv;
    const size_t tile = (((size_t)b * H + h) * nblk + blk) * TILE + lane;
    uint4 *rt = (kind == 0 ? q_rt : kind == 1 ? k_rt : v_rt) + tile, *pt = (kind == 0 ? q_pt : kind == 1 ? k_pt : v_pt) + tile;
    for (int p = wave; p < HD / 8; p += 4) {
        if (p < NJ) {
            const float *src = Xs + l31 * LDS_LD + 16 * p + 8 * hh;
            const HL f = split8(ld4(src), ld4(src + 4));
            rt[(2 * p) * 64] = __builtin_bit_cast(uint4, f.hi);
            rt[(2 * p + 1) * 64] = __builtin_bit_cast(uint4, f.lo);
        } else {
            const int q = p - NJ, db = q >> 1, u = q & 1;
            float x[8];
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] = Xs[pt_row(u, hh, e) * LDS_LD + 32 * db + l31];
            const HL f = split8(x);
            pt[(2 * q) * 64] = __builtin_bit_cast(uint4, f.hi);
            pt[(2 * q + 1) * 64] = __builtin_bit_cast(uint4, f.lo);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
struct FaArgs {
    const uint4 *q_rt, *q_pt, *k_rt, *k_pt, *v_rt, *v_pt, *do_rt, *do_pt;
    int Hq, Hkv, seq, batch, window;
    float scale, scale_log2;             // 1 / sqrt(hd), and the same times log2(e)
    float *lse;                          // [batch][Hq][nblk * 32]: log2 of the row's sum of 2^(score * scale_log2)
    const float *D;                      // [batch][Hq][nblk * 32]
    float *O;                            // forward: [rows][Hq * HD] fp32
    half_t *out16;                       // forward: tiled [rows, Hq * HD]
    float *dq;                           // [rows][Hq * HD]
    float *dkp, *dvp;                    // [Hq / Hkv][rows][Hkv * HD]: per query head of a group
};

// One wave-wide copy of 1 KB from memory into LDS without passing registers: lane i's 16 bytes land at lds_base + 16 i
// (M0 holds the wave-uniform base).  Written as assembly so that the compiler does not count it among its own loads:
// it cannot tell which LDS bytes a pending copy will write and would wait for ALL copies in flight before every LDS
// read.  The kernels wait for their copies themselves, once per step (FA_WAIT_AND_BARRIER); loads retire in order, so
// a wait that the compiler inserts for a load of its own can only wait longer than it has to, never too short.
__device__ __forceinline__ void copy_to_lds_1k(const uint4 *src_lane, uint4 *lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_void *)lds_base);
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(src_lane), "s"(base) : "memory", "m0");
}

// The tiles of the next step go into the other LDS buffer while the current one is multiplied; every wave requests a
// quarter of the fragments.  NT tiles per step; tile t of block `blk` sits at src[t] + blk * TILE.
template <int HD, int NT>
__device__ __forceinline__ void request_tiles(const uint4 *const (&src)[NT], int blk, uint4 *dst, int wave, int lane)
{
    constexpr int TILE = HD / 8 * 64;
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int f = 0; f < HD / 32; f++)
            copy_to_lds_1k(src[t] + (size_t)blk * TILE + (wave + 4 * f) * 64 + lane, dst + t * TILE + (wave + 4 * f) * 64);
}

// acc (32 x 32) = A-tile rows x B-registers, reduction over the head's columns.  The A fragments come from LDS two
// steps ahead of their use (a ring of three register slots), so that a step's instructions never wait out an LDS
// round trip; two partial sums take the instructions in turn so that none waits for the one before it.
template <int HD>
__device__ __forceinline__ float16v rows_product(const uint4 *a_tile_lane, const bf16x8 (&bh)[HD / 16], const bf16x8 (&bl)[HD / 16])
{
    constexpr int NJ = HD / 16;
    float16v s0 = zero16(), s1 = zero16();
    bf16x8 ah[3], al[3];
#pragma unroll
    for (int j = 0; j < 2; j++) { ah[j] = frag(a_tile_lane + (2 * j) * 64); al[j] = frag(a_tile_lane + (2 * j + 1) * 64); }
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        if (j + 2 < NJ) { ah[(j + 2) % 3] = frag(a_tile_lane + (2 * j + 4) * 64); al[(j + 2) % 3] = frag(a_tile_lane + (2 * j + 5) * 64); }
        s0 = mfma(ah[j % 3], bh[j], s0);
        s1 = mfma(al[j % 3], bh[j], s1);
        if (j & 1) s1 = mfma(ah[j % 3], bl[j], s1); else s0 = mfma(ah[j % 3], bl[j], s0);
    }
    return s0 + s1;
}

// Two such products over the same steps (tiles a0 with b0, a1 with b1), their instructions interleaved: six per LDS
// round trip, fragments one step ahead.
template <int HD>
__device__ __forceinline__ void rows_product2(float16v &r0, float16v &r1, const uint4 *a0_lane, const bf16x8 (&b0h)[HD / 16], const bf16x8 (&b0l)[HD / 16],
                                              const uint4 *a1_lane, const bf16x8 (&b1h)[HD / 16], const bf16x8 (&b1l)[HD / 16])
{
    constexpr int NJ = HD / 16;
    float16v s0 = zero16(), t0 = zero16();                // one sum each: the other product's instructions lie between
    bf16x8 xh[2], xl[2], yh[2], yl[2];
    xh[0] = frag(a0_lane); xl[0] = frag(a0_lane + 64); yh[0] = frag(a1_lane); yl[0] = frag(a1_lane + 64);
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int c = j & 1, n = c ^ 1;
        if (j + 1 < NJ) {
            xh[n] = frag(a0_lane + (2 * j + 2) * 64); xl[n] = frag(a0_lane + (2 * j + 3) * 64);
            yh[n] = frag(a1_lane + (2 * j + 2) * 64); yl[n] = frag(a1_lane + (2 * j + 3) * 64);
        }
        s0 = mfma(xh[c], b0h[j], s0);
        t0 = mfma(yh[c], b1h[j], t0);
        s0 = mfma(xl[c], b0h[j], s0);
        t0 = mfma(yl[c], b1h[j], t0);
        s0 = mfma(xh[c], b0l[j], s0);
        t0 = mfma(yh[c], b1l[j], t0);
    }
    r0 = s0; r1 = t0;
}

// acc[db] (32 head columns x 32) += PT-tile x the 32 x 32 values x (an accumulator's worth, rows = reduction index).
// Steps of two column blocks (four fragments, six instructions on two accumulators in turn), fragments one step ahead.
template <int HD>
__device__ __forceinline__ void cols_product(float16v (&acc)[HD / 32], const uint4 *pt_tile_lane, const float (&x)[16])
{
    constexpr int NDB = HD / 32, NSTEP = NDB;               // steps: (u, pair of column blocks), u-major
    HL b[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const float xe[8] = {x[8 * u], x[8 * u + 1], x[8 * u + 2], x[8 * u + 3], x[8 * u + 4], x[8 * u + 5], x[8 * u + 6], x[8 * u + 7]};
        b[u] = split8(xe);
    }
    bf16x8 ah[2][2], al[2][2];
    auto fetch = [&](int slot, int st) __attribute__((always_inline)) {
        const int u = st / (NDB / 2), d0 = 2 * (st % (NDB / 2));
#pragma unroll
        for (int k = 0; k < 2; k++) {
            ah[slot][k] = frag(pt_tile_lane + (((d0 + k) * 2 + u) * 2) * 64);
            al[slot][k] = frag(pt_tile_lane + (((d0 + k) * 2 + u) * 2 + 1) * 64);
        }
    };
    fetch(0, 0);
#pragma unroll
    for (int st = 0; st < NSTEP; st++) {
        const int c = st & 1, u = st / (NDB / 2), d0 = 2 * (st % (NDB / 2));
        if (st + 1 < NSTEP) fetch(c ^ 1, st + 1);
        acc[d0] = mfma(ah[c][0], b[u].hi, acc[d0]);
        acc[d0 + 1] = mfma(ah[c][1], b[u].hi, acc[d0 + 1]);
        acc[d0] = mfma(al[c][0], b[u].hi, acc[d0]);
        acc[d0 + 1] = mfma(al[c][1], b[u].hi, acc[d0 + 1]);
        acc[d0] = mfma(ah[c][0], b[u].lo, acc[d0]);
        acc[d0 + 1] = mfma(ah[c][1], b[u].lo, acc[d0 + 1]);
    }
}

template <int HD>
__device__ __forceinline__ void load_b_rows(bf16x8 (&bh)[HD / 16], bf16x8 (&bl)[HD / 16], const uint4 *tile_lane)
{
#pragma unroll
    for (int j = 0; j < HD / 16; j++) { bh[j] = frag(tile_lane + (2 * j) * 64); bl[j] = frag(tile_lane + (2 * j + 1) * 64); }
}
template <int HD>
__device__ __forceinline__ void touch_b_rows(const bf16x8 (&bh)[HD / 16], const bf16x8 (&bl)[HD / 16])
{
#pragma unroll
    for (int j = 0; j < HD / 16; j++) { FA_TOUCH(bh[j]); FA_TOUCH(bl[j]); }
}

// Keeps a running accumulator in the accumulation registers across the loop's back edge (without this the compiler
// carries it in ordinary registers and copies all of it in and out around the matrix instructions of every step).
#define FA_PIN_ACC(x) asm volatile("" : "+a"(x))

#define FA_WAIT_AND_BARRIER() asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory")

// grid (blocks of 128 queries * Hq * batch), block 256; LDS: two buffers of [RT(K) | PT(V)]
template <int HD>
__global__ __launch_bounds__(256) void k_fa_fwd(FaArgs a)
{
    constexpr int NDB = HD / 32, TILE = HD / 8 * 64;
    __shared__ uint4 buf0[2 * TILE], buf1[2 * TILE];        // two objects: a read of one does not wait for loads into the other
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l31 = lane & 31, hh = lane >> 5;
    const int N = a.seq, nblk = (N + 31) >> 5;
    // items in the order (batch, KV head, query head of the group, query block from the last one down): the sixteen or
    // so workgroups that stream the tiles of one KV head are neighbours
    const int nq4 = (N + 127) >> 7;
    int bh, rank;
    heavy_first_item(blockIdx.x, gridDim.x, nq4, bh, rank);
    const int qb4 = nq4 - 1 - rank, h = bh % a.Hq, b = bh / a.Hq, hk = h / (a.Hq / a.Hkv);
    const int qb = 4 * qb4 + wave;
    const bool active = qb < nblk;
    const int i = 32 * qb + l31;                            // this lane's query
    bf16x8 qh[HD / 16], ql[HD / 16];
    load_b_rows<HD>(qh, ql, a.q_rt + (((size_t)b * a.Hq + h) * nblk + min(qb, nblk - 1)) * TILE + lane);

    const int kb_hi = min(4 * qb4 + 3, nblk - 1);
    const int kb_lo = a.window > 0 ? max(0, 128 * qb4 - a.window + 1) >> 5 : 0;
    const int my_lo = a.window > 0 ? max(0, 32 * qb - a.window + 1) >> 5 : 0;
    const size_t kv0 = ((size_t)b * a.Hkv + hk) * nblk * TILE;
    const uint4 *const src[2] = {a.k_rt + kv0, a.v_pt + kv0};

    float16v o[NDB];
#pragma unroll
    for (int db = 0; db < NDB; db++) o[db] = zero16();
    float m = -1e30f, l = 0.f;

    request_tiles<HD, 2>(src, kb_lo, buf0, wave, lane);
    touch_b_rows<HD>(qh, ql);
    auto step = [&](int kb, uint4 *cur, uint4 *nxt) __attribute__((always_inline)) {
        FA_WAIT_AND_BARRIER();
#pragma unroll
        for (int db = 0; db < NDB; db++) FA_PIN_ACC(o[db]);
        if (kb < kb_hi) request_tiles<HD, 2>(src, kb + 1, nxt, wave, lane);
        if (!active || kb > qb || kb < my_lo) return;
        float16v s = rows_product<HD>(cur + lane, qh, ql);              // S^T: value v is key 32 kb + pt-row, lane's query
        // Scores stay unscaled; m is in units of the exponent (score * scale_log2).  m follows the row maximum only when
        // that has grown by more than 2^8 since m was set: the terms then stay below 2^8 (no overflow in fp32 for any
        // row length here), the result O / l does not depend on m, and the accumulator is rescaled in few steps only.
        const bool edge = kb == qb || (a.window > 0 && 32 * kb < 32 * qb + 32 - a.window);
        float mx = -1e30f;
        if (edge) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                s[v] = sees(i, 32 * kb + 8 * (v >> 2) + 4 * hh + (v & 3), a.window) ? s[v] : -INFINITY;   // its term is exactly 0
                mx = fmaxf(mx, s[v]);
            }
        } else {
#pragma unroll
            for (int v = 0; v < 16; v++) mx = fmaxf(mx, s[v]);
        }
        mx = fmaxf(mx * a.scale_log2, -1e30f);
        mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
        if (__any(mx > m + 8.0f)) {
            const float m_new = fmaxf(m, mx);
            const float alpha = __builtin_amdgcn_exp2f(m - m_new);
            l *= alpha;
#pragma unroll
            for (int db = 0; db < NDB; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) o[db][v] *= alpha;
            m = m_new;
        }
        float p[16];
#pragma unroll
        for (int v = 0; v < 16; v++) { p[v] = __builtin_amdgcn_exp2f(fmaf(s[v], a.scale_log2, -m)); l += p[v]; }
        cols_product<HD>(o, cur + TILE + lane, p);
    };
    for (int kb = kb_lo; kb <= kb_hi; kb += 2) {
        step(kb, buf0, buf1);
        if (kb + 1 <= kb_hi) step(kb + 1, buf1, buf0);
    }
    if (!active) return;
    l += __shfl_xor(l, 32, WAVE);
    const float inv = 1.0f / l;
    if (hh == 0) a.lse[((size_t)b * a.Hq + h) * nblk * 32 + i] = i < N ? m + log2f(l) : 0.f;
    const int qd = a.Hq * HD, Kb = tiled_kb(qd);
    const size_t row = (size_t)b * N + i;
    if (i < N) {
#pragma unroll
        for (int db = 0; db < NDB; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d = h * HD + 32 * db + 8 * g + 4 * hh;
                const float4 v4 = make_float4(o[db][4 * g] * inv, o[db][4 * g + 1] * inv, o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
                st4(a.O + row * qd + d, v4);
                half4 h4 = {f2h(v4.x), f2h(v4.y), f2h(v4.z), f2h(v4.w)};
                *reinterpret_cast<half4 *>(a.out16 + tiled_a_index((int)row, d, Kb)) = h4;
            }
    }
    if (h == a.Hq - 1 && Kb * 64 > qd)                      // zero the K padding of the operand rows once
        for (int idx = lane; idx < 32 * (Kb * 64 - qd); idx += 64) {
            const int rr = idx / (Kb * 64 - qd), c = qd + idx % (Kb * 64 - qd);
            if (32 * qb + rr < N) a.out16[tiled_a_index((int)((size_t)b * N + 32 * qb + rr), c, Kb)] = (half_t)0;
        }
}

// grid (blocks of 128 queries * Hq * batch), block 256; LDS: two buffers of [RT(K) | RT(V) | PT(K)]
template <int HD>
__global__ __launch_bounds__(256) void k_fa_dq(FaArgs a)
{
    constexpr int NDB = HD / 32, TILE = HD / 8 * 64;
    __shared__ uint4 buf0[3 * TILE], buf1[3 * TILE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l31 = lane & 31, hh = lane >> 5;
    const int N = a.seq, nblk = (N + 31) >> 5;
    // items in the order (batch, KV head, query head of the group, query block from the last one down): the sixteen or
    // so workgroups that stream the tiles of one KV head are neighbours
    const int nq4 = (N + 127) >> 7;
    int bh, rank;
    heavy_first_item(blockIdx.x, gridDim.x, nq4, bh, rank);
    const int qb4 = nq4 - 1 - rank, h = bh % a.Hq, b = bh / a.Hq, hk = h / (a.Hq / a.Hkv);
    const int qb = 4 * qb4 + wave;
    const bool active = qb < nblk;
    const int i = 32 * qb + l31;
    bf16x8 qh[HD / 16], ql[HD / 16], gh[HD / 16], gl[HD / 16];
    const size_t qt = (((size_t)b * a.Hq + h) * nblk + min(qb, nblk - 1)) * TILE + lane;
    load_b_rows<HD>(qh, ql, a.q_rt + qt);
    load_b_rows<HD>(gh, gl, a.do_rt + qt);
    const size_t stat = ((size_t)b * a.Hq + h) * nblk * 32 + min(i, nblk * 32 - 1);
    const float L = a.lse[stat], Dv = a.D[stat];

    const int kb_hi = min(4 * qb4 + 3, nblk - 1);
    const int kb_lo = a.window > 0 ? max(0, 128 * qb4 - a.window + 1) >> 5 : 0;
    const int my_lo = a.window > 0 ? max(0, 32 * qb - a.window + 1) >> 5 : 0;
    const size_t kv0 = ((size_t)b * a.Hkv + hk) * nblk * TILE;
    const uint4 *const src[3] = {a.k_rt + kv0, a.v_rt + kv0, a.k_pt + kv0};

    float16v dqT[NDB];
#pragma unroll
    for (int db = 0; db < NDB; db++) dqT[db] = zero16();

    request_tiles<HD, 3>(src, kb_lo, buf0, wave, lane);
    touch_b_rows<HD>(qh, ql); touch_b_rows<HD>(gh, gl);
    FA_TOUCH(L); FA_TOUCH(Dv);
    auto step = [&](int kb, uint4 *cur, uint4 *nxt) __attribute__((always_inline)) {
        FA_WAIT_AND_BARRIER();
#pragma unroll
        for (int db = 0; db < NDB; db++) FA_PIN_ACC(dqT[db]);
        if (kb < kb_hi) request_tiles<HD, 3>(src, kb + 1, nxt, wave, lane);
        if (!active || kb > qb || kb < my_lo) return;
        float16v s, dp;                                                      // S^T [key, query], dP^T = V dO^T
        rows_product2<HD>(s, dp, cur + lane, qh, ql, cur + TILE + lane, gh, gl);
        const bool edge = kb == qb || (a.window > 0 && 32 * kb < 32 * qb + 32 - a.window);
        float ds[16];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            float p = __builtin_amdgcn_exp2f(fmaf(s[v], a.scale_log2, -L));
            if (edge && !sees(i, 32 * kb + 8 * (v >> 2) + 4 * hh + (v & 3), a.window)) p = 0.f;
            ds[v] = p * (dp[v] - Dv) * a.scale;
        }
        cols_product<HD>(dqT, cur + 2 * TILE + lane, ds);
    };
    for (int kb = kb_lo; kb <= kb_hi; kb += 2) {
        step(kb, buf0, buf1);
        if (kb + 1 <= kb_hi) step(kb + 1, buf1, buf0);
    }
    if (!active || i >= N) return;
    const int qd = a.Hq * HD;
    const size_t row = (size_t)b * N + i;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int g = 0; g < 4; g++)
            st4(a.dq + row * qd + h * HD + 32 * db + 8 * g + 4 * hh, make_float4(dqT[db][4 * g], dqT[db][4 * g + 1], dqT[db][4 * g + 2], dqT[db][4 * g + 3]));
}

// grid (blocks of 128 keys * Hq * batch), block 256; LDS: two buffers of [RT(Q) | RT(dO) | PT(Q) | PT(dO)]
template <int HD>
__global__ __launch_bounds__(256) void k_fa_dkv(FaArgs a)
{
    constexpr int NDB = HD / 32, TILE = HD / 8 * 64;
    __shared__ uint4 buf0[4 * TILE], buf1[4 * TILE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l31 = lane & 31, hh = lane >> 5;
    const int N = a.seq, nblk = (N + 31) >> 5, ratio = a.Hq / a.Hkv;
    // items in the order (batch, query head, key block): the workgroups that stream the tiles of one query head are
    // neighbours, and they walk the query blocks from the last one down, so they start on the same tiles
    const int nk4 = (N + 127) >> 7;
    int bh, kb4;
    heavy_first_item(blockIdx.x, gridDim.x, nk4, bh, kb4);
    const int h = bh % a.Hq, b = bh / a.Hq, hk = h / ratio;
    const int kb = 4 * kb4 + wave;
    const bool active = kb < nblk;
    const int kj = 32 * kb + l31;                           // this lane's key
    bf16x8 kh[HD / 16], kl[HD / 16], vh[HD / 16], vl[HD / 16];
    const size_t kt = (((size_t)b * a.Hkv + hk) * nblk + min(kb, nblk - 1)) * TILE + lane;
    load_b_rows<HD>(kh, kl, a.k_rt + kt);
    load_b_rows<HD>(vh, vl, a.v_rt + kt);

    const int qb_lo = 4 * kb4;
    const int qb_hi = a.window > 0 ? min(nblk - 1, (128 * kb4 + 127 + a.window - 1) >> 5) : nblk - 1;
    const int my_hi = a.window > 0 ? min(nblk - 1, (32 * kb + 31 + a.window - 1) >> 5) : nblk - 1;
    const size_t q0 = ((size_t)b * a.Hq + h) * nblk * TILE;
    const uint4 *const src[4] = {a.q_rt + q0, a.do_rt + q0, a.q_pt + q0, a.do_pt + q0};
    const float *lse = a.lse + ((size_t)b * a.Hq + h) * nblk * 32, *Dp = a.D + ((size_t)b * a.Hq + h) * nblk * 32;

    float16v dkT[NDB], dvT[NDB];
#pragma unroll
    for (int db = 0; db < NDB; db++) { dkT[db] = zero16(); dvT[db] = zero16(); }

    request_tiles<HD, 4>(src, qb_hi, buf0, wave, lane);
    touch_b_rows<HD>(kh, kl); touch_b_rows<HD>(vh, vl);
    auto step = [&](int qb, uint4 *cur, uint4 *nxt) __attribute__((always_inline)) {
        // value v of a lane belongs to query 32 qb + 8 (v / 4) + 4 hh + v % 4.  The row statistics are requested before
        // the next tiles: loads complete in order, so the wait for them leaves the tiles in flight.
        float4 L4[4], D4[4];
#pragma unroll
        for (int g = 0; g < 4; g++) { L4[g] = ld4(lse + 32 * qb + 8 * g + 4 * hh); D4[g] = ld4(Dp + 32 * qb + 8 * g + 4 * hh); }
        FA_WAIT_AND_BARRIER();
#pragma unroll
        for (int g = 0; g < 4; g++) { FA_TOUCH(L4[g].x); FA_TOUCH(L4[g].y); FA_TOUCH(L4[g].z); FA_TOUCH(L4[g].w); FA_TOUCH(D4[g].x); FA_TOUCH(D4[g].y); FA_TOUCH(D4[g].z); FA_TOUCH(D4[g].w); }
#pragma unroll
        for (int db = 0; db < NDB; db++) { FA_PIN_ACC(dkT[db]); FA_PIN_ACC(dvT[db]); }
        if (qb > qb_lo) request_tiles<HD, 4>(src, qb - 1, nxt, wave, lane);
        if (!active || qb < kb || qb > my_hi) return;
        float16v s, dp;                                                          // S [query, key], dP = dO V^T
        rows_product2<HD>(s, dp, cur + lane, kh, kl, cur + TILE + lane, vh, vl);
        const bool edge = qb == kb || (a.window > 0 && 32 * qb + 31 - a.window >= 32 * kb);
        float p[16], ds[16];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float Lq = (&L4[v >> 2].x)[v & 3], Dq = (&D4[v >> 2].x)[v & 3];
            float pv = __builtin_amdgcn_exp2f(fmaf(s[v], a.scale_log2, -Lq));
            if (edge && !sees(32 * qb + 8 * (v >> 2) + 4 * hh + (v & 3), kj, a.window)) pv = 0.f;
            p[v] = pv;
            ds[v] = pv * (dp[v] - Dq) * a.scale;
        }
        cols_product<HD>(dvT, cur + 3 * TILE + lane, p);
        cols_product<HD>(dkT, cur + 2 * TILE + lane, ds);
    };
    for (int qb = qb_hi; qb >= qb_lo; qb -= 2) {
        step(qb, buf0, buf1);
        if (qb - 1 >= qb_lo) step(qb - 1, buf1, buf0);
    }
    if (!active || kj >= N) return;
    const int kd = a.Hkv * HD;
    const size_t off = ((size_t)(h % ratio) * a.batch * N + (size_t)b * N + kj) * kd + hk * HD;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int d = 32 * db + 8 * g + 4 * hh;
            st4(a.dkp + off + d, make_float4(dkT[db][4 * g], dkT[db][4 * g + 1], dkT[db][4 * g + 2], dkT[db][4 * g + 3]));
            st4(a.dvp + off + d, make_float4(dvT[db][4 * g], dvT[db][4 * g + 1], dvT[db][4 * g + 2], dvT[db][4 * g + 3]));
        }
}

// dk, dv = sum over the query heads of a group; n4 = rows * kd / 4 float4 each
__global__ __launch_bounds__(256) void k_fa_sum_groups(const float4 *dkp, const float4 *dvp, float4 *dk, float4 *dv, size_t n4, int ratio)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const float4 *src = blockIdx.y ? dvp : dkp;
    float4 s = src[i];
    for (int g = 1; g < ratio; g++) { const float4 v = src[(size_t)g * n4 + i]; s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w; }
    (blockIdx.y ? dv : dk)[i] = s;
}

template <int HD>
void split_hd(const FaSplitArgs &a)
{
    const dim3 grid((a.seq + 31) / 32, a.H, a.batch);
    if (a.X || a.Xpl.S <= 1) LAUNCH((k_fa_split<HD, 1>), grid, dim3(256), 0, a);
    else LAUNCH((k_fa_split<HD, (HD <= 128 ? 5 : 3)>), grid, dim3(256), 0, a);
}

void split(const FaSplitArgs &a, int hd) { if (hd == 64) split_hd<64>(a); else split_hd<128>(a); }

template <int HD>
void fwd_hd(const FaArgs &a) { LAUNCH(k_fa_fwd<HD>, dim3(((a.seq + 127) / 128) * a.Hq * a.batch), dim3(256), 0, a); }

template <int HD>
void bwd_hd(const FaArgs &a)
{
    LAUNCH(k_fa_dq<HD>, dim3(((a.seq + 127) / 128) * a.Hq * a.batch), dim3(256), 0, a);
    LAUNCH(k_fa_dkv<HD>, dim3(((a.seq + 127) / 128) * a.Hq * a.batch), dim3(256), 0, a);
}

int g_flash_mode = -1;

}  // namespace

void set_attn_flash_mode(int mode) { g_flash_mode = mode < 0 ? -1 : mode > 0 ? 1 : 0; }

// The measured rule (Qwen3-4B widths, MI355X; step time without / with saved probabilities): these kernels run one
// workgroup per 128 queries of a head and want at least half the CUs' worth of them -- 1 x 512 positions x 32 heads = 128
// workgroups 28.6 / 29.0 ms, 2 x 512 44.8 / 49.2, 1 x 1024 48.6 / 56.2, 4 x 256 43.1 / 45.2, 8 x 128 42.2 / 43.7, against
// 1 x 256 (64 workgroups) 18.4 / 17.5 and 1 x 128 12.5 / 11.7 -- and take every sequence beyond the other kernels' 1024 keys.
bool attn_flash_supported(int hd, int seq, int Hq, int Hkv, int batch)
{
    if (g_flash_mode == 0 || !(hd == 64 || hd == 128) || seq < 1 || Hkv < 1 || Hq % Hkv || batch < 1) return false;
    return g_flash_mode == 1 || seq > 1024 || (long)((seq + 127) / 128) * Hq * batch >= 128;
}

size_t attn_flash_tile_elems(int hd, int seq, int heads, int batch)
{
    return (size_t)batch * heads * ((seq + 31) / 32) * (hd / 8) * 64;       // uint4 (16 bytes) each
}

template <int HD>
void qkv_post_hd(const QkvPostArgs &a, const AttnFlashArgs &f)
{
    const dim3 grid((f.seq + 31) / 32, a.Hq + 2 * a.Hkv, f.batch);
    constexpr int NBM = HD <= 128 ? 5 : 3;
    if (a.qkv.S <= 1) {
        if (a.R == 16) LAUNCH((k_qkv_post_tile<HD, 16, 1>), grid, dim3(256), 0, a, f.q_rt, f.q_pt, f.k_rt, f.k_pt, f.v_rt, f.v_pt, f.batch);
        else LAUNCH((k_qkv_post_tile<HD, -1, 1>), grid, dim3(256), 0, a, f.q_rt, f.q_pt, f.k_rt, f.k_pt, f.v_rt, f.v_pt, f.batch);
    } else {
        if (a.R == 16) LAUNCH((k_qkv_post_tile<HD, 16, NBM>), grid, dim3(256), 0, a, f.q_rt, f.q_pt, f.k_rt, f.k_pt, f.v_rt, f.v_pt, f.batch);
        else LAUNCH((k_qkv_post_tile<HD, -1, NBM>), grid, dim3(256), 0, a, f.q_rt, f.q_pt, f.k_rt, f.k_pt, f.v_rt, f.v_pt, f.batch);
    }
}

void launch_qkv_post_flash(const QkvPostArgs &a, const AttnFlashArgs &f)
{
    if (!(f.hd == 64 || f.hd == 128) || a.hd != f.hd || a.R < 0 || a.R > 64 || (a.R & 1) || a.qkv.scale_groups || (a.qkv.ld & 3) || a.seq != f.seq) {
        fprintf(stderr, "[fast_hip] qkv_post_flash: unsupported shape (hd %d, rank %d)\n", a.hd, a.R); abort();
    }
    if (f.hd == 64) qkv_post_hd<64>(a, f); else qkv_post_hd<128>(a, f);
}

void launch_attn_fwd_flash(const AttnFlashArgs &f)
{
    if (!(f.hd == 64 || f.hd == 128)) { fprintf(stderr, "[fast_hip] attn_fwd_flash: unsupported head size %d\n", f.hd); abort(); }
    if (f.q) {                                            // fp32 q, k, v given: split them here (else launch_qkv_post_flash has)
        FaSplitArgs sp{};
        sp.seq = f.seq; sp.batch = f.batch;
        sp.X = f.q; sp.ldx = (size_t)f.Hq * f.hd; sp.H = f.Hq; sp.rt = f.q_rt; sp.pt = f.q_pt; split(sp, f.hd);
        sp.X = f.k; sp.ldx = (size_t)f.Hkv * f.hd; sp.H = f.Hkv; sp.rt = f.k_rt; sp.pt = f.k_pt; split(sp, f.hd);
        sp.X = f.v; sp.rt = f.v_rt; sp.pt = f.v_pt; split(sp, f.hd);
    }
    FaArgs a{};
    a.q_rt = f.q_rt; a.k_rt = f.k_rt; a.v_pt = f.v_pt;
    a.Hq = f.Hq; a.Hkv = f.Hkv; a.seq = f.seq; a.batch = f.batch; a.window = f.window;
    a.scale = f.scale; a.scale_log2 = f.scale * 1.4426950408889634f;
    a.lse = f.lse; a.O = f.O; a.out16 = f.out16;
    if (f.hd == 64) fwd_hd<64>(a); else fwd_hd<128>(a);
}

void launch_attn_bwd_flash(const AttnFlashArgs &f)
{
    if (!(f.hd == 64 || f.hd == 128) || f.dO.scale_groups) { fprintf(stderr, "[fast_hip] attn_bwd_flash: unsupported shape\n"); abort(); }
    FaSplitArgs sp{};
    sp.seq = f.seq; sp.batch = f.batch;
    sp.Xpl = f.dO; sp.H = f.Hq; sp.rt = f.do_rt; sp.pt = f.do_pt; sp.O = f.O; sp.D = f.D; split(sp, f.hd);
    FaArgs a{};
    a.q_rt = f.q_rt; a.q_pt = f.q_pt; a.k_rt = f.k_rt; a.k_pt = f.k_pt; a.v_rt = f.v_rt; a.v_pt = f.v_pt;
    a.do_rt = f.do_rt; a.do_pt = f.do_pt;
    a.Hq = f.Hq; a.Hkv = f.Hkv; a.seq = f.seq; a.batch = f.batch; a.window = f.window;
    a.scale = f.scale; a.scale_log2 = f.scale * 1.4426950408889634f;
    a.lse = f.lse; a.D = f.D; a.dq = f.dq; a.dkp = f.dkp; a.dvp = f.dvp;
    if (f.hd == 64) bwd_hd<64>(a); else bwd_hd<128>(a);
    const size_t n4 = (size_t)f.batch * f.seq * f.Hkv * f.hd / 4;
    LAUNCH(k_fa_sum_groups, dim3((unsigned)((n4 + 255) / 256), 2), dim3(256), 0, reinterpret_cast<const float4 *>(f.dkp),
           reinterpret_cast<const float4 *>(f.dvp), reinterpret_cast<float4 *>(f.dk), reinterpret_cast<float4 *>(f.dv), n4, f.Hq / f.Hkv);
}

}  // namespace lmhip

extern "C" void hip_attention_flash(int mode) { lmhip::set_attn_flash_mode(mode); }
