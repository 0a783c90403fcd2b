// Causal GQA attention, forward and backward, on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32: operands are not rounded).  Same arithmetic as
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

// One 32 x 32 product tile A[32, HD] (LDS, row stride lda) * Bm[32 rows, HD]^T, with the 32 B rows read straight from
// memory.  The reduction index is split between the lane halves (lanes 0-31 take columns [0, HD/2), lanes 32-63
// the rest), so a lane reads one contiguous half row of its B row in chunks of CH floats.  Every load is
// unconditional and issued one chunk ahead of its MFMAs: `first` arrives holding chunk 0 and leaves holding chunk 0
// of `next_half_row` (the tile this wave multiplies next; any valid row when there is none).
template <int HD> struct BCfg { static constexpr int HALF = HD / 2, CH = HALF < 32 ? HALF : 32, NCH = HALF / CH; };
template <int HD> struct BChunk { float4 v[BCfg<HD>::CH / 4]; };

template <int HD>
__device__ __forceinline__ void b_chunk_load(BChunk<HD> &c, const float *b_half_row, int c0)
{
#pragma unroll
    for (int t = 0; t < BCfg<HD>::CH / 4; t++) c.v[t] = ld4(b_half_row + c0 + 4 * t);
}

template <int HD>
__device__ __forceinline__ float16v tile_abt(const float *As, int lda, const float *b_half_row, int lane,
                                             BChunk<HD> &first, const float *next_half_row)
{
    constexpr int CH = BCfg<HD>::CH, NCH = BCfg<HD>::NCH;
    const float *a = As + (lane & 31) * lda + (lane >> 5) * BCfg<HD>::HALF;
    Acc2 acc{zero16(), zero16()};
    BChunk<HD> buf[2];
    buf[0] = first;
#pragma unroll
    for (int ci = 0; ci < NCH; ci++) {
        if (ci + 1 < NCH) b_chunk_load<HD>(buf[(ci + 1) & 1], b_half_row, (ci + 1) * CH);
        else b_chunk_load<HD>(buf[(ci + 1) & 1], next_half_row, 0);
        const BChunk<HD> &c = buf[ci & 1];
#pragma unroll
        for (int t = 0; t < CH / 4; t++) {
            acc.a = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ci * CH + 4 * t + 0], c.v[t].x, acc.a, 0, 0, 0);
            acc.b = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ci * CH + 4 * t + 1], c.v[t].y, acc.b, 0, 0, 0);
            acc.a = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ci * CH + 4 * t + 2], c.v[t].z, acc.a, 0, 0, 0);
            acc.b = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ci * CH + 4 * t + 3], c.v[t].w, acc.b, 0, 0, 0);
        }
    }
    first = buf[NCH & 1];
    return acc.a + acc.b;
}

// One 32 x 32 product tile X[32, nk] (LDS, row stride ldx) * C[nk rows, 32 columns], C row-major with row stride ldc;
// rows beyond n_valid are read as row n_valid - 1 (their X column is zero).  Chunks of 32 rows of C (16 loads) are
// requested one chunk ahead, unconditionally (past the end the last chunk is read again); `first` holds chunk 0.
struct CChunk { float v[16]; };

__device__ __forceinline__ void c_chunk_load(CChunk &c, const float *ccol_lane, size_t ldc, int k0, int hh, int n_valid)
{
#pragma unroll
    for (int t = 0; t < 16; t++) c.v[t] = ccol_lane[(size_t)min(k0 + 2 * t + hh, n_valid - 1) * ldc];
}

__device__ __forceinline__ void c_chunk_mfma(Acc2 &acc, const float *x, const CChunk &c)
{
#pragma unroll
    for (int t = 0; t < 16; t += 2) {
        acc.a = __builtin_amdgcn_mfma_f32_32x32x2f32(x[2 * t], c.v[t], acc.a, 0, 0, 0);
        acc.b = __builtin_amdgcn_mfma_f32_32x32x2f32(x[2 * t + 2], c.v[t + 1], acc.b, 0, 0, 0);
    }
}

__device__ __forceinline__ float16v tile_xc(const float *Xs, int ldx, int nk, const float *ccol_lane, size_t ldc, int n_valid, int lane,
                                            CChunk &first)
{
    const int hh = lane >> 5;
    const float *x = Xs + (lane & 31) * ldx + hh;
    Acc2 acc{zero16(), zero16()};
    CChunk other;
    for (int k0 = 0; k0 < nk; k0 += 64) {                 // nk is a multiple of 32
        c_chunk_load(other, ccol_lane, ldc, min(k0 + 32, nk - 32), hh, n_valid);
        c_chunk_mfma(acc, x + k0, first);
        c_chunk_load(first, ccol_lane, ldc, min(k0 + 64, nk - 32), hh, n_valid);
        if (k0 + 32 < nk) c_chunk_mfma(acc, x + k0 + 32, other);
    }
    return acc.a + acc.b;
}

struct AttnTileArgs {
    // forward: A = q, B = k, C = v;  dQ: A = dO (planes), B = v, C = k
    const float *A; Planes Apl;
    const float *B, *C;
    int Hq, Hkv, hd, seq, batch; float scale;
    float *probs;                 // forward: written; dQ: read          [batch][Hq][seq][seq]
    float *dscore;                // dQ: written
    float *A_out;                 // dQ: plane-summed dO rows [rows][Hq*hd]
    float *out32;                 // dQ: dq [rows][Hq*hd]
    half_t *out16;                // forward: tiled [rows, Hq*hd]
};

// Row step for four rows at a time: a wave holds NE elements per lane of each row (keys lane, lane + 64, ...), so
// the LDS reads of a row are in flight together and the four rows' wave reductions interleave.  The finished rows
// go back to LDS for phase 3 and, whole (zeros right of the diagonal), to memory.
template <int BWD, int NE>
__device__ __forceinline__ void row_step(const AttnTileArgs &a, float *Xs, int ldx, int nk, int N, int i0, int b, int h, int wave, int lane)
{
    for (int r4 = 0; r4 < 8; r4 += 4) {
        float v[4][NE], p[4][NE];
        float red[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int rr = wave * 8 + r4 + q, i = i0 + rr;
            const float *prow = a.probs + (((size_t)b * a.Hq + h) * N + min(i, N - 1)) * N;
            red[q] = BWD ? 0.f : -1e30f;
#pragma unroll
            for (int e = 0; e < NE; e++) {
                const int j = lane + 64 * e;
                const bool ok = j <= i && j < nk && i < N;
                v[q][e] = Xs[rr * ldx + min(j, nk - 1)];
                if (BWD) { p[q][e] = ok ? prow[j] : 0.f; red[q] += p[q][e] * v[q][e]; }
                else { v[q][e] = ok ? v[q][e] * a.scale : -1e30f; red[q] = fmaxf(red[q], v[q][e]); }
            }
        }
#pragma unroll
        for (int q = 0; q < 4; q++) red[q] = BWD ? wave_sum(red[q]) : wave_max(red[q]);
        if (!BWD) {
            float sum[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                sum[q] = 0.f;
#pragma unroll
                for (int e = 0; e < NE; e++) {
                    const int j = lane + 64 * e;
                    v[q][e] = (j <= i0 + wave * 8 + r4 + q && j < nk) ? expf(v[q][e] - red[q]) : 0.f;
                    sum[q] += v[q][e];
                }
            }
#pragma unroll
            for (int q = 0; q < 4; q++) red[q] = 1.0f / wave_sum(sum[q]);
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int rr = wave * 8 + r4 + q, i = i0 + rr;
            float *grow = (BWD ? a.dscore : a.probs) + (((size_t)b * a.Hq + h) * N + min(i, N - 1)) * N;
#pragma unroll
            for (int e = 0; e < NE; e++) {
                const int j = lane + 64 * e;
                const float o = BWD ? p[q][e] * (v[q][e] - red[q]) * a.scale : v[q][e] * red[q];
                if (j < nk) Xs[rr * ldx + j] = o;
                if (j < N && i < N) grow[j] = (j < nk) ? o : 0.f;
            }
        }
    }
}

// grid (query blocks of 32, Hq, batch), block 256; LDS: As[32][HD+1], Xs[32][ldx]
template <int BWD, int HD>
__global__ __launch_bounds__(256) void k_attn_tile(AttnTileArgs a)
{
    extern __shared__ float lds[];
    constexpr int lda = HD + 1, half = HD / 2;
    const int N = a.seq;
    const int qb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l31 = lane & 31, hh = lane >> 5;
    const int qd = a.Hq * HD, kd = a.Hkv * HD, hk = h / (a.Hq / a.Hkv);
    const size_t r0 = (size_t)b * N;
    const int i0 = qb * 32;
    const int nk = min(i0 + 32, (N + 31) & ~31);          // keys this block can see, rounded up to 32
    const int ldx = ((N + 63) & ~63) + 1;
    float *As = lds, *Xs = As + 32 * lda;

    // ---- the first B tile and the first C chunk of this wave do not depend on anything computed here:
    //      request them before the A rows are staged (waves without a tile of their own read tile 0)
    auto b_row = [&](int jb) { return a.B + (r0 + min(jb * 32 + l31, N - 1)) * kd + hk * HD + hh * half; };
    const int nkb = nk >> 5;
    BChunk<HD> bfirst;
    b_chunk_load<HD>(bfirst, b_row(wave < nkb ? wave : 0), 0);
    CChunk cfirst;
    const float *c_lane0 = a.C + r0 * kd + hk * HD + l31;
    c_chunk_load(cfirst, c_lane0 + (wave * 32 < HD ? wave * 32 : 0), (size_t)kd, 0, hh, N);

    // ---- A rows into LDS (rows past the sequence as zeros)
    for (int idx = tid; idx < 32 * (HD >> 2); idx += 256) {
        const int rr = idx / (HD >> 2), c4 = idx % (HD >> 2);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i0 + rr < N) {
            if (BWD) {
                v = planes_at4(a.Apl, r0 + i0 + rr, h * HD + 4 * c4);
                st4(a.A_out + (r0 + i0 + rr) * qd + h * HD + 4 * c4, v);
            } else {
                v = ld4(a.A + (r0 + i0 + rr) * qd + h * HD + 4 * c4);
            }
        }
        float *d = As + rr * lda + 4 * c4;
        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
    }
    __syncthreads();

    // ---- phase 1: X = A B^T, one 32-key block per wave and round
    for (int jb = wave; jb < nkb; jb += 4) {
        const float16v acc = tile_abt<HD>(As, lda, b_row(jb), lane, bfirst, b_row(jb + 4 < nkb ? jb + 4 : jb));
#pragma unroll
        for (int v = 0; v < 16; v++) Xs[(8 * (v >> 2) + 4 * hh + (v & 3)) * ldx + jb * 32 + l31] = acc[v];
    }
    __syncthreads();

    // ---- row step
    if (N <= 64) row_step<BWD, 1>(a, Xs, ldx, nk, N, i0, b, h, wave, lane);          // whole rows of N entries are written
    else if (N <= 256) row_step<BWD, 4>(a, Xs, ldx, nk, N, i0, b, h, wave, lane);
    else if (N <= 512) row_step<BWD, 8>(a, Xs, ldx, nk, N, i0, b, h, wave, lane);
    else row_step<BWD, 16>(a, Xs, ldx, nk, N, i0, b, h, wave, lane);
    __syncthreads();

    // ---- phase 3: Y = X C, one 32-column block of the head per wave and round
    const int Kb = tiled_kb(qd);
    for (int dt = wave; dt * 32 < HD; dt += 4) {
        if (dt != wave) c_chunk_load(cfirst, c_lane0 + dt * 32, (size_t)kd, 0, hh, N);
        const float16v acc = tile_xc(Xs, ldx, nk, c_lane0 + dt * 32, (size_t)kd, N, lane, cfirst);
        const int d = dt * 32 + l31;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int i = i0 + 8 * (v >> 2) + 4 * hh + (v & 3);
            if (i >= N) continue;
            if (BWD) a.out32[(r0 + i) * qd + h * HD + d] = acc[v];
            else a.out16[tiled_index((int)(r0 + i), h * HD + d, Kb)] = f2h(acc[v]);
        }
    }
    if (!BWD && h == a.Hq - 1)                             // zero the K padding of the operand rows once
        for (int idx = tid; idx < 32 * (Kb * 64 - qd); idx += 256) {
            const int rr = idx / (Kb * 64 - qd), c = qd + idx % (Kb * 64 - qd);
            if (i0 + rr < N) a.out16[tiled_index((int)(r0 + i0 + rr), c, Kb)] = (half_t)0;
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
#pragma unroll
        for (int k0 = 0; k0 < 32; k0 += 8) {
            float pv[4], sv[4], qv[4], ov[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int i = ib * 32 + k0 + 2 * t + hh;
                const int ic = min(i, N - 1);
                const bool ok = i < N;
                pv[t] = ok ? P[(size_t)ic * N] : 0.f;
                sv[t] = ok ? S[(size_t)ic * N] : 0.f;
                qv[t] = Q[(size_t)ic * qd];
                ov[t] = O[(size_t)ic * qd];
            }
#pragma unroll
            for (int t = 0; t < 4; t++) {
                accV = __builtin_amdgcn_mfma_f32_32x32x2f32(pv[t], ov[t], accV, 0, 0, 0);
                accK = __builtin_amdgcn_mfma_f32_32x32x2f32(sv[t], qv[t], accK, 0, 0, 0);
            }
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

template <int BWD, int HD>
void launch_tile_hd(const AttnTileArgs &a)
{
    static bool attr_set = false;
    if (!attr_set) { HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_attn_tile<BWD, HD>), hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024)); attr_set = true; }
    const size_t lds = (size_t)32 * (HD + 1 + ((a.seq + 63) & ~63) + 1) * sizeof(float);
    LAUNCH((k_attn_tile<BWD, HD>), dim3((a.seq + 31) / 32, a.Hq, a.batch), dim3(256), lds, a);
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

size_t tile_lds_bytes(int hd, int seq) { return (size_t)32 * (hd + 1 + ((seq + 63) & ~63) + 1) * sizeof(float); }

}  // namespace

bool attn_mfma_supported(int hd, int seq)
{
    return (hd == 32 || hd == 64 || hd == 128 || hd == 256) && seq >= 1 && seq <= 1024 && tile_lds_bytes(hd, seq) <= 150 * 1024;
}

void launch_attn_fwd_mfma(const AttnFwdArgs &f)
{
    if (!attn_mfma_supported(f.hd, f.seq)) { fprintf(stderr, "[fast_hip] attn_fwd_mfma: unsupported shape\n"); abort(); }
    AttnTileArgs a{};
    a.A = f.q; a.B = f.k; a.C = f.v;
    a.Hq = f.Hq; a.Hkv = f.Hkv; a.hd = f.hd; a.seq = f.seq; a.batch = f.batch; a.scale = f.scale;
    a.probs = f.probs; a.out16 = f.out16;
    launch_tile<0>(a);
}

void launch_attn_bwd_mfma(const AttnBwdArgs &g)
{
    if (!attn_mfma_supported(g.hd, g.seq)) { fprintf(stderr, "[fast_hip] attn_bwd_mfma: unsupported shape\n"); abort(); }
    AttnTileArgs a{};
    a.Apl = g.dO; a.B = g.v; a.C = g.k;
    a.Hq = g.Hq; a.Hkv = g.Hkv; a.hd = g.hd; a.seq = g.seq; a.batch = g.batch; a.scale = g.scale;
    a.probs = const_cast<float *>(g.probs); a.dscore = g.dscore; a.A_out = g.dO_red; a.out32 = g.dq;
    launch_tile<1>(a);
    AttnDkvArgs d{};
    d.probs = g.probs; d.dscore = g.dscore; d.q = g.q; d.dO = g.dO_red;
    d.Hq = g.Hq; d.Hkv = g.Hkv; d.hd = g.hd; d.seq = g.seq; d.batch = g.batch;
    d.dk = g.dk; d.dv = g.dv;
    LAUNCH(k_attn_dkv_tile, dim3(((g.seq + 31) / 32) * (g.hd / 32), g.Hkv, g.batch), dim3(256), 0, d);
}

}  // namespace lmhip
