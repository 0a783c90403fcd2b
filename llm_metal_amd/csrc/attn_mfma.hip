// Causal GQA attention, forward and backward, on the matrix cores.  Every fp32 operand enters as two bf16 values,
// x = hi + lo (hi the upper 16 bits of x, lo those of x - hi), and a product is three v_mfma_f32_32x32x16_bf16:
// hi*hi + lo*hi + hi*lo, accumulated in fp32.  That keeps 16 mantissa bits and the whole fp32 exponent range of
// every operand (gradients of 1e-7 do not underflow as they would in fp16) at a fifth of the matrix-core time of
// the fp32 instruction (v_mfma_f32_32x32x2_f32, 64 cycles for 2 reduction steps).  Same arithmetic as
// attn_train_fwd / attn_bwd_dq / attn_bwd_dkv / repeat_kv_bwd of
// shaders/q8_kernels.metal:769-992, on [rows][H*hd] activations with the KV head
// picked as h / ratio; the probabilities are saved for the backward as the
// reference does (src/nn/fast_sft.c:678-689).
//
// Forward and dQ share one shape: a workgroup owns 32 query rows of one head,
//   phase 1   X[32, keys] = A[32, hd] * B[keys, hd]^T      (Q K^T, or dO V^T)
//   row step  softmax, or dS = P o (dP - rowsum(P o dP)) * scale
//   phase 3   Y[32, hd]   = X[32, keys] * C[keys, hd]       (P V, or dS K)
// with A and X in LDS and B, C read straight from L2 in the order the MFMA
// wants.  dK/dV: a workgroup owns 32 keys x 32 head columns of one KV head, its
// waves split the (query head, query block) pairs and meet in LDS.
#include "fused.h"
#include "planes.h"
#include "bf16pair.h"

namespace lmhip {
namespace {

#define LAUNCH(kern, grid, block, lds, ...) do { \
    hipLaunchKernelGGL(kern, grid, block, lds, stream(), __VA_ARGS__); HIP_CHECK(hipGetLastError()); } while (0)

__device__ __forceinline__ float16v zero16()
{
    float16v z;
#pragma unroll
    for (int v = 0; v < 16; v++) z[v] = 0.f;
    return z;
}

// Two accumulators take the MFMAs in turn, so that no instruction waits for the result of the one before it;
// they are added when the tile is complete.
struct Acc2 { float16v a, b; };

// acc += a b over 16 reduction steps (first operand: rows of the result, second: its columns)
__device__ __forceinline__ void mfma3(float16v &acc, const HL &a, const HL &b)
{
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.hi, b.hi, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.lo, b.hi, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.hi, b.lo, acc, 0, 0, 0);
}

// A 32 x 32 product tile A[32, HD] * Bm[32 rows, HD]^T is formed CB columns of the head at a time (CB = HD up to 128;
// two passes at HD = 256, which keeps the B operands of a pass within 64 registers).  Within a pass the reduction
// index is split between the lane halves (lanes 0-31 take the first CB/2 columns, lanes 32-63 the rest), so a lane
// needs CB/2 floats of its B row: a BTile, read straight from memory a whole pass ahead of its use and split into
// bf16 pairs here.  The A rows sit in LDS already split (Ahi / Alo, bf16, row stride lda halves): 16 bytes of each
// per instruction.
template <int CB> struct BTile { float4 v[CB / 8]; };

// The values come from a copy of the head's matrix laid out as BT[HD/4][ldt][4] (group of four columns, key, column
// in the group; ldt = attn_ldt(seq)): a lane still reads 16 bytes at a time, but the 32 lanes of a half wave read
// 512 contiguous bytes, where the rows themselves (4 KB apart) would cost one cache line per lane and instruction.
template <int CB>
__device__ __forceinline__ void b_tile_load(BTile<CB> &t, const float *bt_lane, int ldt)
{
#pragma unroll
    for (int i = 0; i < CB / 8; i++) t.v[i] = ld4(bt_lane + (size_t)i * ldt * 4);
}

// acc += A[:, col0 .. col0 + CB) * B-pass^T
template <int CB>
__device__ __forceinline__ void tile_abt(Acc2 &acc, const __bf16 *Ahi, const __bf16 *Alo, int lda, int col0, int lane, const BTile<CB> &bt)
{
    constexpr int HALF = CB / 2, NT = HALF / 8;              // instruction triples per pass
    constexpr int CT = NT < 4 ? NT : 4, NC = NT / CT;        // A operands are fetched CT triples at a time, one group ahead
    const size_t off = (size_t)(lane & 31) * lda + col0 + (lane >> 5) * HALF;
    HL a[2][CT];
    auto fetch = [&](int buf, int c) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < CT; t++) {                       // LDS, 16-byte aligned
            a[buf][t].hi = *reinterpret_cast<const bf16x8 *>(Ahi + off + 8 * (c * CT + t));
            a[buf][t].lo = *reinterpret_cast<const bf16x8 *>(Alo + off + 8 * (c * CT + t));
        }
    };
    fetch(0, 0);
#pragma unroll
    for (int c = 0; c < NC; c++) {
        if (c + 1 < NC) fetch((c + 1) & 1, c + 1);
#pragma unroll
        for (int t = 0; t < CT; t++) {
            const int tt = c * CT + t;
            const HL b = split8(bt.v[2 * tt], bt.v[2 * tt + 1]);
            mfma3((t & 1) ? acc.b : acc.a, a[c & 1][t], b);
        }
    }
}

// One 32 x 32 product tile X[32, nk] * C[nk rows, 32 columns], C row-major with row stride ldc; rows beyond n_valid
// are read as row n_valid - 1 (their X column is zero).  X sits in LDS split into bf16 pairs: row r holds the upper
// parts of its nk values at Xh + r * ldxh (halves), the lower parts xlo halves further on.  Inside a chunk of 32 keys
// lanes 0-31 take keys 0-15 and lanes 32-63 keys 16-31 (instruction u of the chunk reduces over keys 16 hh + 8 u +
// 0..7), so a lane reads 16 consecutive X values (two 16-byte LDS reads for each part) and 16 rows of C.  Both are
// requested ahead, unconditionally (past the end the last chunk is read again); `first` holds chunk 0 of C.
struct CChunk { float v[16]; };
struct XChunk { bf16x8 hi[2], lo[2]; };

__device__ __forceinline__ void c_chunk_load(CChunk &c, const float *ccol_lane, size_t ldc, int k0, int hh, int n_valid)
{
#pragma unroll
    for (int t = 0; t < 16; t++) c.v[t] = ccol_lane[(size_t)min(k0 + 16 * hh + t, n_valid - 1) * ldc];
}

__device__ __forceinline__ void x_chunk_load(XChunk &c, const __bf16 *x_row_half, int xlo, int k0)
{
#pragma unroll
    for (int u = 0; u < 2; u++) {
        c.hi[u] = *reinterpret_cast<const bf16x8 *>(x_row_half + k0 + 8 * u);
        c.lo[u] = *reinterpret_cast<const bf16x8 *>(x_row_half + xlo + k0 + 8 * u);
    }
}

__device__ __forceinline__ void c_chunk_mfma(Acc2 &acc, const XChunk &x, const CChunk &c)
{
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const float cv[8] = {c.v[8 * u], c.v[8 * u + 1], c.v[8 * u + 2], c.v[8 * u + 3], c.v[8 * u + 4], c.v[8 * u + 5], c.v[8 * u + 6], c.v[8 * u + 7]};
        mfma3(u ? acc.b : acc.a, HL{x.hi[u], x.lo[u]}, split8(cv));
    }
}

// The C chunks travel in a ring of four (chunk q in slot q % 4), requested three chunks ahead; on entry slots 0-2 hold
// chunks 0-2, which the caller may have requested long before.
struct CRing { CChunk c[4]; };

template <int M32>
__device__ __forceinline__ void c_ring_start(CRing &r, const float *ccol_lane, size_t ldc, int nk, int hh, int n_valid)
{
#pragma unroll
    for (int q = 0; q < (M32 == 2 ? 2 : 3); q++) c_chunk_load(r.c[q], ccol_lane, ldc, min(32 * q, nk - 32), hh, n_valid);
}

// The product for sequences of at most 64 keys: both chunks of C are in the ring already.
__device__ __forceinline__ float16v tile_xc_2(const __bf16 *Xh, int ldxh, int xlo, int nk, int lane, const CRing &ring)
{
    const int hh = lane >> 5;
    const __bf16 *x = Xh + (size_t)(lane & 31) * ldxh + 16 * hh;
    Acc2 acc{zero16(), zero16()};
    XChunk xr[2];
    x_chunk_load(xr[0], x, xlo, 0);
    x_chunk_load(xr[1], x, xlo, nk - 32);
    c_chunk_mfma(acc, xr[0], ring.c[0]);
    if (nk > 32) c_chunk_mfma(acc, xr[1], ring.c[1]);
    return acc.a + acc.b;
}

__device__ __forceinline__ float16v tile_xc(const __bf16 *Xh, int ldxh, int xlo, int nk, const float *ccol_lane, size_t ldc, int n_valid,
                                            int lane, CRing &ring)
{
    const int hh = lane >> 5;
    const __bf16 *x = Xh + (size_t)(lane & 31) * ldxh + 16 * hh;
    Acc2 acc{zero16(), zero16()};
    XChunk xr[2];
    x_chunk_load(xr[0], x, xlo, 0);
    for (int k0 = 0; k0 < nk; k0 += 128) {                // nk is a multiple of 32
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int kc = k0 + 32 * u;
            c_chunk_load(ring.c[(u + 3) & 3], ccol_lane, ldc, min(kc + 96, nk - 32), hh, n_valid);
            x_chunk_load(xr[(u + 1) & 1], x, xlo, min(kc + 32, nk - 32));
            if (kc < nk) c_chunk_mfma(acc, xr[u & 1], ring.c[u]);
        }
    }
    return acc.a + acc.b;
}

struct AttnTileArgs {
    // forward: A = q, B = k, C = v;  dQ: A = dO (planes), B = v, C = k.  B is given transposed per head:
    // BT[batch][Hkv][hd/4][attn_ldt(seq)][4]
    const float *A; Planes Apl;
    const float *BT, *C;
    int Hq, Hkv, hd, seq, batch; float scale;
    float *probs;                 // forward: written; dQ: read          [batch][Hq][seq][seq]
    float *dscore;                // dQ: written
    float *A_out;                 // dQ: plane-summed dO rows [rows][Hq*hd]
    float *out32;                 // dQ: dq [rows][Hq*hd]
    half_t *out16;                // forward: tiled [rows, Hq*hd]
    WeightPrefetch pf;            // weights of the product that follows: fetched by the grid slices z >= batch
    int window;                   // forward: > 0 masks keys older than i - window + 1 (the saved zeros carry it into the backward)
    // dQ with the block's share of dK / dV in the same launch (sequences of at most 64 keys): q [rows][Hq*hd], and the
    // shares [query block][Hq][rows_total][hd] that the consumer of dk / dv sums (attn_dkv_part_index)
    const float *q; float *dkp, *dvp; int rows_total;
};

// Row step: eight threads per row, thread `part` owns the keys 32 m + 4 part + (0..3) for m < M32 and keeps them in
// registers, so every LDS and memory access is a 16-byte one (eight threads cover 128 contiguous bytes) and the
// row reductions need three shuffles.  The finished rows go to memory whole (fp32, zeros right of the diagonal, out to
// column N) and back to LDS for phase 3 as bf16 pairs, in place: the upper parts of keys 0.. at the start of the
// row, the lower parts xlo halves further on.  A row belongs to eight lanes of one wave, which have read all of it
// before they write.
// The saved probabilities this thread needs in the dQ row step (zero right of the diagonal; whole 16-byte groups exist
// when N % 4 == 0, else they go by element).  They depend on nothing computed in the kernel, so short rows (M32 <= 8)
// are requested at the start of the kernel and arrive while the scores are formed.
template <int M32>
__device__ __forceinline__ void load_probs(float4 (&p)[M32], const AttnTileArgs &a, int N, int i0, int b, int h, int tid)
{
    const int rr = tid >> 3, part = tid & 7, i = i0 + rr;
    const size_t goff = (((size_t)b * a.Hq + h) * N + min(i, N - 1)) * N + 4 * part;
#pragma unroll
    for (int m = 0; m < M32; m++) {
        const int j = 32 * m + 4 * part;
        float4 pv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i < N && j <= i) {
            if ((N & 3) == 0) pv = *reinterpret_cast<const float4 *>(a.probs + goff + 32 * m);
            else { float *q = &pv.x; for (int c = 0; c < 4; c++) if (j + c < N) q[c] = a.probs[goff + 32 * m + c]; }
        }
        p[m] = pv;
    }
}

// DKV (dQ only): dS and the probabilities also go to LDS by key (Ts: four images -- upper and lower parts of dS, then of
// P -- of [keys][DKV_TS] halves each, 32 query rows and padding per key), for the shares of dK and dV formed after phase
// 3, whose matrix-core operands are eight consecutive query rows of one key: one 16-byte read each.  dscore stays out of
// memory: nothing reads it.
constexpr int DKV_TS = 40;                                 // halves per key: 80 bytes apart, so that eight lanes' 16-byte reads cover all banks
template <int BWD, int M32, int DKV = 0>
__device__ __forceinline__ void row_step(const AttnTileArgs &a, float *Xs, int ldx, int xlo, int nk, int N, int i0, int b, int h, int tid,
                                         const float4 (&p_early)[BWD ? M32 : 1], uint16_t *Ts = nullptr)
{
    const int rr = tid >> 3, part = tid & 7, i = i0 + rr;
    const bool row_ok = i < N;
    float *xr = Xs + rr * ldx + 4 * part;
    const size_t goff = (((size_t)b * a.Hq + h) * N + min(i, N - 1)) * N + 4 * part;
    float4 v[M32], p[BWD ? M32 : 1];
    if constexpr (BWD) {
        if constexpr (M32 <= 8) {
#pragma unroll
            for (int m = 0; m < M32; m++) p[m] = p_early[m];
        } else load_probs<M32>(p, a, N, i0, b, h, tid);
    }
    float red = BWD ? 0.f : -1e30f;
    const int lo = (!BWD && a.window > 0 && i >= a.window) ? i - a.window + 1 : 0;      // first key row i sees
#pragma unroll
    for (int m = 0; m < M32; m++) {
        const int j = 32 * m + 4 * part;
        v[m] = (j < nk) ? *reinterpret_cast<const float4 *>(xr + 32 * m) : make_float4(0.f, 0.f, 0.f, 0.f);
        float *e = &v[m].x;
        if (BWD) {
            const float4 pv = p[m];
            red += pv.x * e[0] + pv.y * e[1] + pv.z * e[2] + pv.w * e[3];
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++) { e[c] = (j + c <= i && j + c < nk && j + c >= lo) ? e[c] * a.scale : -1e30f; red = fmaxf(red, e[c]); }
        }
    }
    if (BWD) { red += __shfl_xor(red, 1, WAVE); red += __shfl_xor(red, 2, WAVE); red += __shfl_xor(red, 4, WAVE); }
    else { red = fmaxf(red, __shfl_xor(red, 1, WAVE)); red = fmaxf(red, __shfl_xor(red, 2, WAVE)); red = fmaxf(red, __shfl_xor(red, 4, WAVE)); }
    float inv = 1.0f;
    if (!BWD) {
        float sum = 0.f;
#pragma unroll
        for (int m = 0; m < M32; m++) {
            const int j = 32 * m + 4 * part;
            float *e = &v[m].x;
#pragma unroll
            for (int c = 0; c < 4; c++) { e[c] = (j + c <= i && j + c < nk && j + c >= lo) ? expf(e[c] - red) : 0.f; sum += e[c]; }
        }
        sum += __shfl_xor(sum, 1, WAVE); sum += __shfl_xor(sum, 2, WAVE); sum += __shfl_xor(sum, 4, WAVE);
        inv = 1.0f / sum;
    }
    float *gdst = (BWD ? a.dscore : a.probs) + goff;
#pragma unroll
    for (int m = 0; m < M32; m++) {
        const int j = 32 * m + 4 * part;
        float4 o;
        if (BWD) o = make_float4(p[m].x * (v[m].x - red) * a.scale, p[m].y * (v[m].y - red) * a.scale,
                                 p[m].z * (v[m].z - red) * a.scale, p[m].w * (v[m].w - red) * a.scale);
        else o = make_float4(v[m].x * inv, v[m].y * inv, v[m].z * inv, v[m].w * inv);
        if (j < nk) {
            __bf16 *xh = reinterpret_cast<__bf16 *>(Xs + rr * ldx) + j;
            *reinterpret_cast<u32x2 *>(xh) = u32x2{pack_hi(o.x, o.y), pack_hi(o.z, o.w)};
            *reinterpret_cast<u32x2 *>(xh + xlo) = u32x2{pack_hi(rest(o.x), rest(o.y)), pack_hi(rest(o.z), rest(o.w))};
            if constexpr (BWD && DKV) {
                const float ov[4] = {o.x, o.y, o.z, o.w}, pv[4] = {p[m].x, p[m].y, p[m].z, p[m].w};
                const int img = xlo * DKV_TS;                          // xlo: the keys rounded up to 32
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    uint16_t *t = Ts + (j + c) * DKV_TS + rr;
                    t[0] = (uint16_t)(__float_as_uint(ov[c]) >> 16); t[img] = (uint16_t)(__float_as_uint(rest(ov[c])) >> 16);
                    t[2 * img] = (uint16_t)(__float_as_uint(pv[c]) >> 16); t[3 * img] = (uint16_t)(__float_as_uint(rest(pv[c])) >> 16);
                }
            }
        }
        if (!DKV && row_ok && j < N) {
            if ((N & 3) == 0) *reinterpret_cast<float4 *>(gdst + 32 * m) = o;
            else { const float *q = &o.x; for (int c = 0; c < 4; c++) if (j + c < N) gdst[32 * m + c] = q[c]; }
        }
    }
}

// grid (query blocks of 32, Hq, batch), block 256; LDS: Ahi, Alo [32][HD+8] bf16, Xs[32][ldx] fp32 / bf16 pairs
// M32: 32-key blocks a row can hold (2, 8, 16 or 32: sequences up to 64, 256, 512, 1024); a template parameter so
// that the kernel's code is one straight run (the kernel runs once per workgroup, and what it skips it still fetches).
template <int BWD, int HD, int M32, int DKV = 0>
__global__ __launch_bounds__(256) void k_attn_tile(AttnTileArgs a)
{
    extern __shared__ float lds[];
    constexpr int lda = HD + 8;                            // halves; rows 16-byte aligned and 4 banks apart: conflict-free 16-byte reads
    const int N = a.seq;
    if ((int)blockIdx.z >= a.batch) {
        const int per_z = gridDim.x * gridDim.y;
        prefetch_weight_tiles<256>(a.pf, (blockIdx.z - a.batch) * per_z + blockIdx.y * gridDim.x + blockIdx.x);
        return;
    }
    const int qb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l31 = lane & 31, hh = lane >> 5;
    const int qd = a.Hq * HD, kd = a.Hkv * HD, hk = h / (a.Hq / a.Hkv);
    const size_t r0 = (size_t)b * N;
    const int i0 = qb * 32;
    const int nk = min(i0 + 32, (N + 31) & ~31);          // keys this block can see, rounded up to 32
    const int N32 = (N + 31) & ~31, ldx = N32 + 4;
    __bf16 *Ahi = reinterpret_cast<__bf16 *>(lds), *Alo = Ahi + 32 * lda;
    float *Xs = lds + 32 * lda;                           // behind the two bf16 images of A
    uint16_t *Ts = reinterpret_cast<uint16_t *>(Xs + 32 * ldx);      // DKV only: dS and P by key (row_step)

    // ---- the first B pass and the first C chunk of this wave do not depend on anything computed here:
    //      request them before the A rows are staged
    // Work items of a wave in phase 1: (key block jb = wave + 4 (q / NCB), column pass c = q % NCB), q = 0 .. nitems - 1.
    // This lane's part of the transposed B matrix for an item: key jb * 32 + l31, columns c * CB + hh * CB/2 ...
    constexpr int CB = HD > 128 ? 128 : HD, NCB = HD / CB;
    const int ldt = attn_ldt(N);
    const int nkb = nk >> 5;
    const int nitems = wave < nkb ? ((nkb - wave + 3) >> 2) * NCB : 0;
    auto b_item = [&](int q) {
        const int qq = nitems ? min(q, nitems - 1) : 0;
        const int jb = nitems ? wave + 4 * (qq / NCB) : 0, c = qq % NCB;
        return a.BT + ((((size_t)b * a.Hkv + hk) * (HD / 4) + c * (CB / 4) + hh * (CB / 8)) * ldt + min(jb * 32 + l31, N - 1)) * 4;
    };
    BTile<CB> bt0, bt1;
    if (nitems) b_tile_load<CB>(bt0, b_item(0), ldt);     // (uniform per wave; a wave without an item asks for nothing)
    float4 p_early[BWD ? M32 : 1];
    if constexpr (BWD && M32 <= 8) load_probs<M32>(p_early, a, N, i0, b, h, tid);
    // DKV: this lane's q values for the shares formed at the end (query rows 16 u + 8 hh + e of the block, head column
    // dt * 32 + l31 for the wave's blocks dt = wave, wave + 4): requested now, used last
    constexpr int NDT = DKV ? (HD + 127) / 128 : 1;
    float q_early[NDT][2][8];
    if constexpr (BWD && DKV) {
#pragma unroll
        for (int t = 0; t < NDT; t++)
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int i = i0 + 16 * u + 8 * hh + e, d = min((wave + 4 * t) * 32, HD - 32) + l31;
                    q_early[t][u][e] = a.q[(r0 + min(i, N - 1)) * qd + h * HD + d];
                }
    }
    CRing cring;
    const float *c_lane0 = a.C + r0 * kd + hk * HD + l31;
    c_ring_start<M32>(cring, c_lane0 + (wave * 32 < HD ? wave * 32 : 0), (size_t)kd, nk, hh, N);

    // ---- A rows into LDS (rows past the sequence as zeros); the loads of all HD / 32 rounds are issued together
    {
        float4 av[HD / 32];
        if (BWD) {
            size_t rows[HD / 32]; int cols[HD / 32]; bool ok[HD / 32];
#pragma unroll
            for (int u = 0; u < HD / 32; u++) {
                const int idx = tid + 256 * u, rr = idx / (HD >> 2), c4 = idx % (HD >> 2);
                ok[u] = i0 + rr < N; rows[u] = r0 + (ok[u] ? i0 + rr : 0); cols[u] = h * HD + 4 * c4;
            }
            // (a head of 256 columns: eight positions per thread; planes of halves take half the registers, so ten of
            // them -- the chunks of the short products of a model with such heads -- travel in one round trip)
            planes_at4_multi<HD / 32, (HD <= 128 ? 5 : 3), false, (HD <= 128 ? 5 : 5)>(a.Apl, rows, cols, ok, av);
        } else {
#pragma unroll
            for (int u = 0; u < HD / 32; u++) {
                const int idx = tid + 256 * u, rr = idx / (HD >> 2), c4 = idx % (HD >> 2);
                av[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (i0 + rr < N) av[u] = ld4(a.A + (r0 + i0 + rr) * qd + h * HD + 4 * c4);
            }
        }
#pragma unroll
        for (int u = 0; u < HD / 32; u++) {
            const int idx = tid + 256 * u, rr = idx / (HD >> 2), c4 = idx % (HD >> 2);
            if (BWD && !DKV && i0 + rr < N) st4(a.A_out + (r0 + i0 + rr) * qd + h * HD + 4 * c4, av[u]);
            *reinterpret_cast<u32x2 *>(Ahi + rr * lda + 4 * c4) = u32x2{pack_hi(av[u].x, av[u].y), pack_hi(av[u].z, av[u].w)};
            *reinterpret_cast<u32x2 *>(Alo + rr * lda + 4 * c4) = u32x2{pack_hi(rest(av[u].x), rest(av[u].y)), pack_hi(rest(av[u].z), rest(av[u].w))};
        }
    }
    __syncthreads();
    // a head of 256 columns at up to 64 keys: the C values of the wave's second column block are asked for now and
    // arrive during phase 1 and the row step (at the start of the kernel they would not fit among a wave's 63 loads in flight)
    constexpr bool RING2 = HD > 128 && M32 == 2;
    CRing cring2;
    if constexpr (RING2) c_ring_start<M32>(cring2, c_lane0 + (wave + 4) * 32, (size_t)kd, nk, hh, N);

    // ---- phase 1: X = A B^T, one 32-key block per wave and round; the B values of the next item are on their way
    auto put_x = [&](const float16v &acc, int jb) {
#pragma unroll
        for (int v = 0; v < 16; v++) Xs[(8 * (v >> 2) + 4 * hh + (v & 3)) * ldx + jb * 32 + l31] = acc[v];
    };
    {
        Acc2 acc{zero16(), zero16()};
        auto run = [&](int q, const BTile<CB> &bt) __attribute__((always_inline)) {
            const int jb = wave + 4 * (q / NCB), c = q % NCB;
            if (c == 0) { acc.a = zero16(); acc.b = zero16(); }
            tile_abt<CB>(acc, Ahi, Alo, lda, c * CB, lane, bt);
            if (c == NCB - 1) put_x(acc.a + acc.b, jb);
        };
        if constexpr (((M32 + 3) / 4) * NCB == 1) {       // at most one item per wave: no second tile on its way
            if (nitems) run(0, bt0);
        } else if constexpr (((M32 + 3) / 4) * NCB == 2) { // at most two items (two column passes, or two key blocks)
            if (nitems) {
                if (nitems > 1) b_tile_load<CB>(bt1, b_item(1), ldt);
                run(0, bt0);
                if (nitems > 1) run(1, bt1);
            }
        } else {
            for (int q = 0; q < nitems; q += 2) {
                b_tile_load<CB>(bt1, b_item(q + 1), ldt);
                run(q, bt0);
                b_tile_load<CB>(bt0, b_item(q + 2), ldt);
                if (q + 1 < nitems) run(q + 1, bt1);
            }
        }
    }
    __syncthreads();

    // ---- row step
    row_step<BWD, M32, DKV>(a, Xs, ldx, N32, nk, N, i0, b, h, tid, p_early, Ts);    // whole rows of N entries are written
    __syncthreads();

    // ---- phase 3: Y = X C, one 32-column block of the head per wave and round
    const int Kb = tiled_kb(qd);
    auto put_y = [&](const float16v &acc, int dt) __attribute__((always_inline)) {
        const int d = dt * 32 + l31;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int i = i0 + 8 * (v >> 2) + 4 * hh + (v & 3);
            if (i >= N) continue;
            if (BWD) a.out32[(r0 + i) * qd + h * HD + d] = acc[v];
            else a.out16[tiled_a_index((int)(r0 + i), h * HD + d, Kb)] = f2h(acc[v]);
        }
    };
    if constexpr (RING2) {
        put_y(tile_xc_2(reinterpret_cast<const __bf16 *>(Xs), 2 * ldx, N32, nk, lane, cring), wave);
        put_y(tile_xc_2(reinterpret_cast<const __bf16 *>(Xs), 2 * ldx, N32, nk, lane, cring2), wave + 4);
    } else {
        for (int dt = wave; dt * 32 < HD; dt += 4) {
            if (dt != wave) c_ring_start<M32>(cring, c_lane0 + dt * 32, (size_t)kd, nk, hh, N);
            float16v acc;
            if constexpr (M32 == 2) acc = tile_xc_2(reinterpret_cast<const __bf16 *>(Xs), 2 * ldx, N32, nk, lane, cring);
            else acc = tile_xc(reinterpret_cast<const __bf16 *>(Xs), 2 * ldx, N32, nk, c_lane0 + dt * 32, (size_t)kd, N, lane, cring);
            put_y(acc, dt);
        }
    }
    if constexpr (BWD && DKV) {
        // ---- the block's share of dK and dV of its query head, for the keys it sees:
        //      dKp[j, d] = sum_{i in block} dS[i, j] q[i, d],   dVp[j, d] = sum_{i in block} P[i, j] dO[i, d].
        // A wave takes the head columns dt * 32 ..; in an instruction lane (l31, hh) reduces over the query rows
        // 16 u + 8 hh + 0..7 of the block: its key's dS / P values are eight consecutive halves of the images by key,
        // dO comes from the staged A rows a row apart each, q from memory.
        const int img = N32 * DKV_TS;
#pragma unroll
        for (int t = 0; t < NDT; t++) {
            const int dt = wave + 4 * t;
            if (dt * 32 >= HD) break;
            const int d = dt * 32 + l31;
            HL qB[2], oB[2];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                float qv[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int i = i0 + 16 * u + 8 * hh + e;
                    qv[e] = i < N ? q_early[t][u][e] : 0.f;
                    oB[u].hi[e] = Ahi[(16 * u + 8 * hh + e) * lda + d];
                    oB[u].lo[e] = Alo[(16 * u + 8 * hh + e) * lda + d];
                }
                qB[u] = split8(qv);
            }
            for (int jb = 0; jb < nkb; jb++) {
                HL sA[2], pA[2];
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const uint16_t *t = Ts + (jb * 32 + l31) * DKV_TS + 16 * u + 8 * hh;
                    sA[u].hi = *reinterpret_cast<const bf16x8 *>(t); sA[u].lo = *reinterpret_cast<const bf16x8 *>(t + img);
                    pA[u].hi = *reinterpret_cast<const bf16x8 *>(t + 2 * img); pA[u].lo = *reinterpret_cast<const bf16x8 *>(t + 3 * img);
                }
                float16v aK = zero16(), aV = zero16();
#pragma unroll
                for (int u = 0; u < 2; u++) { mfma3(aK, sA[u], qB[u]); mfma3(aV, pA[u], oB[u]); }
                const size_t base = (((size_t)qb * a.Hq + h) * a.rows_total + r0) * HD + d;
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int jj = jb * 32 + 8 * (v >> 2) + 4 * hh + (v & 3);
                    if (jj >= N) continue;
                    a.dkp[base + (size_t)jj * HD] = aK[v];
                    a.dvp[base + (size_t)jj * HD] = aV[v];
                }
            }
        }
    }
    if (!BWD && h == a.Hq - 1)                             // zero the K padding of the operand rows once
        for (int idx = tid; idx < 32 * (Kb * 64 - qd); idx += 256) {
            const int rr = idx / (Kb * 64 - qd), c = qd + idx % (Kb * 64 - qd);
            if (i0 + rr < N) a.out16[tiled_a_index((int)(r0 + i0 + rr), c, Kb)] = (half_t)0;
        }
}

struct AttnDkvArgs {
    const float *probs, *dscore, *q, *dO;   // [batch][Hq][seq][seq] x2, [rows][Hq*hd] x2
    int Hq, Hkv, hd, seq, batch;
    float *dk, *dv;                          // [rows][Hkv*hd]
};

// grid (key blocks of 32 * head-column blocks of 32, Hkv, batch), block 256.
// dV[j, d] = sum_{g, i >= j} P[g, i, j] dO[g, i, d];  dK[j, d] = sum dS[g, i, j] q[g, i, d]  (g: query heads of the group)
__global__ __launch_bounds__(256) void k_attn_dkv_tile(AttnDkvArgs a)
{
    __shared__ float red[3][2][16][64];
    const int N = a.seq, hd = a.hd, ratio = a.Hq / a.Hkv;
    const int ndt = hd >> 5;
    const int jb = blockIdx.x / ndt, dt = blockIdx.x % ndt, hk = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l31 = lane & 31, hh = lane >> 5;
    const int qd = a.Hq * hd, kd = a.Hkv * hd;
    const size_t r0 = (size_t)b * N;
    const int nqb = (N + 31) >> 5;
    const int j = min(jb * 32 + l31, N - 1);
    float16v accK = zero16(), accV = zero16();
    const int npairs = ratio * (nqb - jb);
    for (int p = wave; p < npairs; p += 4) {
        const int g = p / (nqb - jb), ib = jb + p % (nqb - jb);
        const int hq = hk * ratio + g;
        const float *P = a.probs + ((size_t)b * a.Hq + hq) * N * N + j;
        const float *S = a.dscore + ((size_t)b * a.Hq + hq) * N * N + j;
        const float *Q = a.q + r0 * qd + hq * hd + dt * 32 + l31;
        const float *O = a.dO + r0 * qd + hq * hd + dt * 32 + l31;
        // lane half hh takes the query rows ib * 32 + 2 s + hh, s = 0..15; instruction u reduces over s = 8 u + 0..7
        float pv[16], sv[16], qv[16], ov[16];
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int i = ib * 32 + 2 * t + hh;
            const int ic = min(i, N - 1);
            const bool ok = i < N;
            pv[t] = ok ? P[(size_t)ic * N] : 0.f;
            sv[t] = ok ? S[(size_t)ic * N] : 0.f;
            qv[t] = Q[(size_t)ic * qd];
            ov[t] = O[(size_t)ic * qd];
        }
#pragma unroll
        for (int u = 0; u < 2; u++) {
            float x[4][8];
#pragma unroll
            for (int e = 0; e < 8; e++) { x[0][e] = pv[8 * u + e]; x[1][e] = ov[8 * u + e]; x[2][e] = sv[8 * u + e]; x[3][e] = qv[8 * u + e]; }
            mfma3(accV, split8(x[0]), split8(x[1]));
            mfma3(accK, split8(x[2]), split8(x[3]));
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int v = 0; v < 16; v++) { red[wave - 1][0][v][lane] = accK[v]; red[wave - 1][1][v][lane] = accV[v]; }
    }
    __syncthreads();
    if (wave != 0) return;
    const int d = dt * 32 + l31;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int jj = jb * 32 + 8 * (v >> 2) + 4 * hh + (v & 3);
        if (jj >= N) continue;
        a.dk[(r0 + jj) * kd + hk * hd + d] = accK[v] + red[0][0][v][lane] + red[1][0][v][lane] + red[2][0][v][lane];
        a.dv[(r0 + jj) * kd + hk * hd + d] = accV[v] + red[0][1][v][lane] + red[1][1][v][lane] + red[2][1][v][lane];
    }
}

size_t tile_lds_bytes(int hd, int seq, int dkv = 0)
{
    const size_t n32 = (seq + 31) & ~31;
    return (size_t)32 * (hd + 8 + n32 + 4) * sizeof(float) + (dkv ? 4 * n32 * DKV_TS * sizeof(uint16_t) : 0);
}

template <int BWD, int HD, int M32, int DKV = 0>
void launch_tile_m(const AttnTileArgs &a)
{
    static bool attr_set = false;
    if (!attr_set) { HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_attn_tile<BWD, HD, M32, DKV>), hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024)); attr_set = true; }
    const size_t lds = tile_lds_bytes(HD, a.seq, DKV);
    const int per_z = ((a.seq + 31) / 32) * a.Hq;
    const int extra = a.pf.base ? a.pf.wgs / per_z : 0;   // the planner made pf.wgs a multiple of per_z
    LAUNCH((k_attn_tile<BWD, HD, M32, DKV>), dim3((a.seq + 31) / 32, a.Hq, a.batch + extra), dim3(256), lds, a);
}

template <int BWD, int HD>
void launch_tile_hd(const AttnTileArgs &a)
{
    if (BWD && a.dkp) { launch_tile_m<BWD, HD, 2, BWD>(a); return; }     // at most 64 keys (the caller checked)
    if (a.seq <= 64) launch_tile_m<BWD, HD, 2>(a);
    else if (a.seq <= 256) launch_tile_m<BWD, HD, 8>(a);
    else if (a.seq <= 512) launch_tile_m<BWD, HD, 16>(a);
    else launch_tile_m<BWD, HD, 32>(a);
}

template <int BWD>
void launch_tile(const AttnTileArgs &a)
{
    switch (a.hd) {
    case 32: launch_tile_hd<BWD, 32>(a); break;
    case 64: launch_tile_hd<BWD, 64>(a); break;
    case 128: launch_tile_hd<BWD, 128>(a); break;
    default: launch_tile_hd<BWD, 256>(a); break;
    }
}



}  // namespace

namespace { int g_bwd_one_launch = 1; }
void set_attn_bwd_one_launch(int on) { g_bwd_one_launch = on ? 1 : 0; }
bool attn_bwd_one_launch(int hd, int seq)
{
    return g_bwd_one_launch && attn_mfma_supported(hd, seq) && seq <= 64 && tile_lds_bytes(hd, seq, 1) <= 150 * 1024;
}

bool attn_mfma_supported(int hd, int seq)
{
    return (hd == 32 || hd == 64 || hd == 128 || hd == 256) && seq >= 1 && seq <= 1024 && tile_lds_bytes(hd, seq) <= 150 * 1024;
}

void launch_attn_fwd_mfma(const AttnFwdArgs &f)
{
    if (!attn_mfma_supported(f.hd, f.seq) || !f.kT) { fprintf(stderr, "[fast_hip] attn_fwd_mfma: unsupported shape\n"); abort(); }
    AttnTileArgs a{};
    a.A = f.q; a.BT = f.kT; a.C = f.v;
    a.Hq = f.Hq; a.Hkv = f.Hkv; a.hd = f.hd; a.seq = f.seq; a.batch = f.batch; a.scale = f.scale;
    a.probs = f.probs; a.out16 = f.out16;
    a.pf = f.pf; a.window = f.window;
    launch_tile<0>(a);
}

void launch_attn_bwd_mfma(const AttnBwdArgs &g)
{
    if (!attn_mfma_supported(g.hd, g.seq) || !g.vT || g.dO.scale_groups) { fprintf(stderr, "[fast_hip] attn_bwd_mfma: unsupported shape\n"); abort(); }
    AttnTileArgs a{};
    a.Apl = g.dO; a.BT = g.vT; a.C = g.k;
    a.Hq = g.Hq; a.Hkv = g.Hkv; a.hd = g.hd; a.seq = g.seq; a.batch = g.batch; a.scale = g.scale;
    a.probs = const_cast<float *>(g.probs); a.dscore = g.dscore; a.A_out = g.dO_red; a.out32 = g.dq;
    if (g.dkp) {                                          // one launch: the consumer of dk / dv sums the shares
        if (g.seq > 64) { fprintf(stderr, "[fast_hip] attn_bwd_mfma: dK / dV shares need a sequence of at most 64\n"); abort(); }
        a.q = g.q; a.dkp = g.dkp; a.dvp = g.dvp; a.rows_total = g.batch * g.seq;
        launch_tile<1>(a);
        return;
    }
    launch_tile<1>(a);
    AttnDkvArgs d{};
    d.probs = g.probs; d.dscore = g.dscore; d.q = g.q; d.dO = g.dO_red;
    d.Hq = g.Hq; d.Hkv = g.Hkv; d.hd = g.hd; d.seq = g.seq; d.batch = g.batch;
    d.dk = g.dk; d.dv = g.dv;
    LAUNCH(k_attn_dkv_tile, dim3(((g.seq + 31) / 32) * (g.hd / 32), g.Hkv, g.batch), dim3(256), 0, d);
}

}  // namespace lmhip

extern "C" void hip_attention_backward_one_launch(int on) { lmhip::set_attn_bwd_one_launch(on); }
