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

// acc[32 x 32] += A[32, hd] (LDS, row stride lda) * Bm[32 rows of a row-major matrix with row stride ldb]^T.
// The reduction index is split between the lane halves (lanes 0-31 take columns [0, hd/2), lanes 32-63 the
// rest), so a lane reads one contiguous half row of its B row as 16-byte loads.
__device__ __forceinline__ float16v tile_abt(const float *As, int lda, const float *Brow, int hd, int lane)
{
    const int half = hd >> 1, hh = lane >> 5;
    const float *a = As + (lane & 31) * lda + hh * half;
    const float *b = Brow + hh * half;
    float16v acc = zero16();
    for (int c0 = 0; c0 < half; c0 += 16) {
        float4 bv[4];
#pragma unroll
        for (int t = 0; t < 4; t++) bv[t] = ld4(b + c0 + 4 * t);
#pragma unroll
        for (int t = 0; t < 4; t++) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c0 + 4 * t + 0], bv[t].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c0 + 4 * t + 1], bv[t].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c0 + 4 * t + 2], bv[t].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c0 + 4 * t + 3], bv[t].w, acc, 0, 0, 0);
        }
    }
    return acc;
}

// acc[32 x 32] = X[32, nk] (LDS, row stride ldx) * C[nk rows, 32 columns starting at Ccol], C row-major with
// row stride ldc; rows beyond n_valid are read as row n_valid - 1 (their X column is zero).
__device__ __forceinline__ float16v tile_xc(const float *Xs, int ldx, int nk, const float *Ccol, size_t ldc, int n_valid, int lane)
{
    const int hh = lane >> 5;
    const float *x = Xs + (lane & 31) * ldx + hh;
    const float *c = Ccol + (lane & 31);
    float16v acc = zero16();
    for (int k0 = 0; k0 < nk; k0 += 16) {                 // nk is a multiple of 32
        float cv[8];
#pragma unroll
        for (int t = 0; t < 8; t++) cv[t] = c[(size_t)min(k0 + 2 * t + hh, n_valid - 1) * ldc];
#pragma unroll
        for (int t = 0; t < 8; t++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[k0 + 2 * t], cv[t], acc, 0, 0, 0);
    }
    return acc;
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

// grid (query blocks of 32, Hq, batch), block 256; LDS: As[32][hd+1], Xs[32][nk_max+1], red[64]
template <int BWD>
__global__ __launch_bounds__(256) void k_attn_tile(AttnTileArgs a)
{
    extern __shared__ float lds[];
    const int N = a.seq, hd = a.hd, lda = hd + 1;
    const int qb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l31 = lane & 31, hh = lane >> 5;
    const int qd = a.Hq * hd, kd = a.Hkv * hd, hk = h / (a.Hq / a.Hkv);
    const size_t r0 = (size_t)b * N;
    const int i0 = qb * 32;
    const int nk = min(i0 + 32, (N + 31) & ~31);          // keys this block can see, rounded up to 32
    const int ldx = ((N + 31) & ~31) + 1;
    float *As = lds, *Xs = As + 32 * lda;

    // ---- A rows into LDS (rows past the sequence as zeros)
    for (int idx = tid; idx < 32 * (hd >> 2); idx += 256) {
        const int rr = idx / (hd >> 2), c4 = idx % (hd >> 2);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i0 + rr < N) {
            if (BWD) {
                v = planes_at4(a.Apl, r0 + i0 + rr, h * hd + 4 * c4);
                st4(a.A_out + (r0 + i0 + rr) * qd + h * hd + 4 * c4, v);
            } else {
                v = ld4(a.A + (r0 + i0 + rr) * qd + h * hd + 4 * c4);
            }
        }
        float *d = As + rr * lda + 4 * c4;
        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
    }
    __syncthreads();

    // ---- phase 1: X = A B^T, one 32-key block per wave and round
    for (int jb = wave; jb * 32 < nk; jb += 4) {
        const int key = min(jb * 32 + l31, N - 1);
        const float16v acc = tile_abt(As, lda, a.B + (r0 + key) * kd + hk * hd, hd, lane);
#pragma unroll
        for (int v = 0; v < 16; v++) Xs[(8 * (v >> 2) + 4 * hh + (v & 3)) * ldx + jb * 32 + l31] = acc[v];
    }
    __syncthreads();

    // ---- row step: eight threads per row
    {
        const int rr = tid >> 3, part = tid & 7, i = i0 + rr;
        float *xr = Xs + rr * ldx;
        const size_t prow = (((size_t)b * a.Hq + h) * N + min(i, N - 1)) * N;
        if (!BWD) {
            float mx = -1e30f;
            for (int j = part; j < nk; j += 8) { const float s = (j <= i) ? xr[j] * a.scale : -1e30f; xr[j] = s; mx = fmaxf(mx, s); }
            mx = fmaxf(mx, __shfl_xor(mx, 1, WAVE)); mx = fmaxf(mx, __shfl_xor(mx, 2, WAVE)); mx = fmaxf(mx, __shfl_xor(mx, 4, WAVE));
            float sum = 0.f;
            for (int j = part; j < nk; j += 8) { const float e = (j <= i) ? expf(xr[j] - mx) : 0.f; xr[j] = e; sum += e; }
            sum += __shfl_xor(sum, 1, WAVE); sum += __shfl_xor(sum, 2, WAVE); sum += __shfl_xor(sum, 4, WAVE);
            const float inv = 1.0f / sum;
            for (int j = part; j < nk; j += 8) xr[j] *= inv;
        } else {
            float dp = 0.f;
            for (int j = part; j < nk; j += 8) if (j <= i && i < N) dp += a.probs[prow + j] * xr[j];
            dp += __shfl_xor(dp, 1, WAVE); dp += __shfl_xor(dp, 2, WAVE); dp += __shfl_xor(dp, 4, WAVE);
            for (int j = part; j < nk; j += 8) xr[j] = (j <= i && i < N) ? a.probs[prow + j] * (xr[j] - dp) * a.scale : 0.f;
        }
    }
    __syncthreads();
    // the whole rows (zeros right of the diagonal) go to memory, coalesced along the keys
    {
        float *dst = BWD ? a.dscore : a.probs;
        for (int idx = tid; idx < 32 * N; idx += 256) {
            const int rr = idx / N, j = idx % N, i = i0 + rr;
            if (i < N) dst[(((size_t)b * a.Hq + h) * N + i) * N + j] = (j < nk) ? Xs[rr * ldx + j] : 0.f;
        }
    }

    // ---- phase 3: Y = X C, one 32-column block of the head per wave and round
    const int Kb = tiled_kb(qd);
    for (int dt = wave; dt * 32 < hd; dt += 4) {
        const float16v acc = tile_xc(Xs, ldx, nk, a.C + r0 * kd + hk * hd + dt * 32, (size_t)kd, N, lane);
        const int d = dt * 32 + l31;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int i = i0 + 8 * (v >> 2) + 4 * hh + (v & 3);
            if (i >= N) continue;
            if (BWD) a.out32[(r0 + i) * qd + h * hd + d] = acc[v];
            else a.out16[tiled_index((int)(r0 + i), h * hd + d, Kb)] = f2h(acc[v]);
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

size_t tile_lds_bytes(int hd, int seq) { return (size_t)32 * (hd + 1 + ((seq + 31) & ~31) + 1) * sizeof(float); }

}  // namespace

bool attn_mfma_supported(int hd, int seq)
{
    return hd >= 32 && (hd % 32) == 0 && seq >= 1 && tile_lds_bytes(hd, seq) <= 150 * 1024;
}

void launch_attn_fwd_mfma(const AttnFwdArgs &f)
{
    if (!attn_mfma_supported(f.hd, f.seq)) { fprintf(stderr, "[fast_hip] attn_fwd_mfma: unsupported shape\n"); abort(); }
    AttnTileArgs a{};
    a.A = f.q; a.B = f.k; a.C = f.v;
    a.Hq = f.Hq; a.Hkv = f.Hkv; a.hd = f.hd; a.seq = f.seq; a.batch = f.batch; a.scale = f.scale;
    a.probs = f.probs; a.out16 = f.out16;
    static bool attr_set = false;
    if (!attr_set) { HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_attn_tile<0>), hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024)); attr_set = true; }
    LAUNCH(k_attn_tile<0>, dim3((f.seq + 31) / 32, f.Hq, f.batch), dim3(256), tile_lds_bytes(f.hd, f.seq), a);
}

void launch_attn_bwd_mfma(const AttnBwdArgs &g)
{
    if (!attn_mfma_supported(g.hd, g.seq)) { fprintf(stderr, "[fast_hip] attn_bwd_mfma: unsupported shape\n"); abort(); }
    AttnTileArgs a{};
    a.Apl = g.dO; a.B = g.v; a.C = g.k;
    a.Hq = g.Hq; a.Hkv = g.Hkv; a.hd = g.hd; a.seq = g.seq; a.batch = g.batch; a.scale = g.scale;
    a.probs = const_cast<float *>(g.probs); a.dscore = g.dscore; a.A_out = g.dO_red; a.out32 = g.dq;
    static bool attr_set = false;
    if (!attr_set) { HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_attn_tile<1>), hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024)); attr_set = true; }
    LAUNCH(k_attn_tile<1>, dim3((g.seq + 31) / 32, g.Hq, g.batch), dim3(256), tile_lds_bytes(g.hd, g.seq), a);
    AttnDkvArgs d{};
    d.probs = g.probs; d.dscore = g.dscore; d.q = g.q; d.dO = g.dO_red;
    d.Hq = g.Hq; d.Hkv = g.Hkv; d.hd = g.hd; d.seq = g.seq; d.batch = g.batch;
    d.dk = g.dk; d.dv = g.dv;
    LAUNCH(k_attn_dkv_tile, dim3(((g.seq + 31) / 32) * (g.hd / 32), g.Hkv, g.batch), dim3(256), 0, d);
}

}  // namespace lmhip
