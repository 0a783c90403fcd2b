// Large-M GEMM: C[M, N] = inv_scale[m] * A16[M, K] * W[N, K]^T for M of several hundred rows and more
// (batch * seq = 2048 in the Q8_0 configuration), where a weight tile is reused by enough activation rows
// that the matrix cores, not HBM, bound the product.  Same operands as the weight-streaming kernel
// (gemm.h: tiled fp16 activations with per-row power-of-two factors; F16 or Q8_0 weight tiles), same
// arithmetic (v_mfma_f32_32x32x16_f16, fp32 accumulation), one launch, no K split.
//
// A workgroup of four waves owns a 128 x 128 block of C and walks K in steps of 64.  Per step every wave
// fetches one 32-row block of the activation tile and one of the weight tile from L2/HBM in the MFMA
// register layout, Q8_0 blocks are unpacked to fp16 there (int8 * fp16 scale, once per tile instead of once
// per consumer), and both go to LDS in the same [j][lane][8 halves] order, so a wave reads any row block back
// with conflict-free 16-byte loads.  LDS is double buffered: the global loads of step k+1 are issued before the
// MFMAs of step k and written to the other buffer after them; one barrier per step.
#include "backend.h"
#include "devutil.h"
#include "gemm.h"
#include "gemm_kernel.h"
#include <hip/hip_ext.h>

namespace lmhip {
namespace {

struct Stage {                       // what one thread holds of the next K step: one row block of A, one of W
    half8 a[4];
    half8 w[4];
};

template <int WF>
__device__ __forceinline__ void fetch(Stage &s, const GemmKArgs &g, int mb, int nb, bool w_q8_rows, int kt, int lane)
{
    const half8 *ap = g.A + ((size_t)mb * g.Kb + kt) * 256 + lane;
#pragma unroll
    for (int j = 0; j < 4; j++) s.a[j] = ap[j * 64];
    if (WF == 0) load_w_f16(s.w, g.W.w16, nb, g.Kb, kt, lane);
    else if (WF == 1) {
        if (w_q8_rows) load_w_q8_rows(s.w, g.W, nb, g.Kb, kt, lane);
        else load_w_f16(s.w, g.W.w16, nb - g.W.nbq, g.Kb, kt, lane);
    } else {
        if (kt < g.W.kbq) load_w_q8_cols(s.w, g.W, nb, g.W.kbq, kt, lane);
        else load_w_f16(s.w, g.W.w16, nb, g.Kb - g.W.kbq, kt - g.W.kbq, lane);
    }
}

// grid: x = ceil(N / 128), y = ceil(M / 128); block 256; LDS 2 x (4 + 4) row blocks x 4 KB = 64 KB
template <int WF>
__global__ __launch_bounds__(256, 2) void gemm_big(GemmKArgs g)
{
    extern __shared__ half8 tiles[];                      // [buf][A blocks 0-3 | W blocks 0-3][j][lane]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int nb0 = blockIdx.x * 4, mb0 = blockIdx.y * 4;
    const int wm = wave >> 1, wn = wave & 1;              // this wave's 64 x 64 quadrant of the block
    // the row blocks this wave fetches (clamped: rows past the end are computed and never stored)
    const int mb_ld = min(mb0 + wave, g.Mb - 1), nb_ld = min(nb0 + wave, g.Nb - 1);
    const bool q8r = WF == 1 && nb_ld < g.W.nbq;

    float16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    Stage st;
    fetch<WF>(st, g, mb_ld, nb_ld, q8r, 0, lane);
    {
        half8 *buf = tiles;
#pragma unroll
        for (int j = 0; j < 4; j++) { buf[(wave * 4 + j) * 64 + lane] = st.a[j]; buf[((4 + wave) * 4 + j) * 64 + lane] = st.w[j]; }
    }
    __syncthreads();
    for (int kt = 0; kt < g.Kb; kt++) {
        const half8 *cur = tiles + (size_t)(kt & 1) * 2048;
        half8 *nxt = tiles + (size_t)((kt + 1) & 1) * 2048;
        const bool more = kt + 1 < g.Kb;
        if (more) fetch<WF>(st, g, mb_ld, nb_ld, q8r, kt + 1, lane);
        half8 a[2][4], w[2][4];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                a[i][j] = cur[((2 * wm + i) * 4 + j) * 64 + lane];
                w[i][j] = cur[((4 + 2 * wn + i) * 4 + j) * 64 + lane];
            }
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int k = 0; k < 2; k++)
                    acc[i][k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i][j], w[k][j], acc[i][k], 0, 0, 0);
        if (more) {
#pragma unroll
            for (int j = 0; j < 4; j++) { nxt[(wave * 4 + j) * 64 + lane] = st.a[j]; nxt[((4 + wave) * 4 + j) * 64 + lane] = st.w[j]; }
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            // D layout of v_mfma_f32_32x32x16: column = lane & 31, row = 8*(v/4) + 4*(lane/32) + v%4
            const int m = (mb0 + 2 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
            if (m >= g.M) continue;
            const float sc = g.a_inv_scale ? g.a_inv_scale[m] : 1.0f;
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const int n = (nb0 + 2 * wn + k) * 32 + r;
                if (n < g.N) g.P[(size_t)m * g.ldp + n] = acc[i][k][v] * sc;
            }
        }
}

}  // namespace

void launch_gemm_big(const half_t *A, const float *a_inv_scale, const WeightOp &W, float *C, int ldc, int M, int N, int K)
{
    if (M <= 0 || N <= 0 || K <= 0) return;
    const int Kb = tiled_kb(K), Nb = tiled_rb(N), Mb = tiled_rb(M);
    bool ok = ldc >= N && W.fmt >= 0 && W.fmt <= 2;
    if (W.fmt == 0) ok = ok && W.w16;
    if (W.fmt == 1) ok = ok && W.q && W.d && W.nbq >= 0 && W.nbq <= Nb && (W.nbq == Nb || W.w16);
    if (W.fmt == 2) ok = ok && W.q && W.d && W.kbq >= 0 && W.kbq <= Kb && (W.kbq == Kb || W.w16);
    if (!ok) { fprintf(stderr, "[fast_hip] gemm_big: bad launch M=%d N=%d K=%d ldc=%d fmt=%d\n", M, N, K, ldc, W.fmt); abort(); }
    GemmKArgs g{};
    g.A = reinterpret_cast<const half8 *>(A); g.a_inv_scale = a_inv_scale; g.W = W;
    g.P = C; g.ldp = ldc; g.plane_stride = 0;
    g.M = M; g.N = N; g.Mb = Mb; g.Nb = Nb; g.Kb = Kb; g.steps_per_chunk = Kb;
    const dim3 grid((N + 127) / 128, (M + 127) / 128), block(256);
    const size_t lds = 2 * 2048 * sizeof(half8);
    static bool attr_set = false;
    if (!attr_set) {
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_big<0>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_big<1>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_big<2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    hipEvent_t ev_a = nullptr, ev_b = nullptr;
    if (gemm_prof_begin(weight_stream_bytes(W, N, K), 2.0 * M * N * K, &ev_a, &ev_b)) {
        if (W.fmt == 0) hipExtLaunchKernelGGL(gemm_big<0>, grid, block, lds, stream(), ev_a, ev_b, 0, g);
        else if (W.fmt == 1) hipExtLaunchKernelGGL(gemm_big<1>, grid, block, lds, stream(), ev_a, ev_b, 0, g);
        else hipExtLaunchKernelGGL(gemm_big<2>, grid, block, lds, stream(), ev_a, ev_b, 0, g);
    } else {
        if (W.fmt == 0) hipLaunchKernelGGL(gemm_big<0>, grid, block, lds, stream(), g);
        else if (W.fmt == 1) hipLaunchKernelGGL(gemm_big<1>, grid, block, lds, stream(), g);
        else hipLaunchKernelGGL(gemm_big<2>, grid, block, lds, stream(), g);
    }
    HIP_CHECK(hipGetLastError());
}

}  // namespace lmhip
