// The weight-streaming GEMM kernel (device code only; included by gemm.hip).
#pragma once
#include "devutil.h"

namespace lmhip {

// grid: x = ceil(Nb / NB) weight-row tiles, y = S (K chunks), z = ceil(M / 64); block = NW waves of 64.
// Kb = number of 64-wide K steps of the (padded) reduction; Nb, Mb = 32-row blocks of W and A.
//
// Each wave loads one K step (NB weight tiles + 2 activation tiles), waits, issues its MFMAs and
// moves on; there is no register double buffering.  Measured on MI355X, the lower register count
// (four resident workgroups per CU instead of two) hides the load latency better than a second
// register stage does.  ROTATE starts every workgroup at a different step of its chunk: without
// it all workgroups of a chunk ask L2 for the same activation lines at the same moment.
// SCALE: multiply row m of the result by a_inv_scale[m] here (used when the output is final, S == 1);
// otherwise the consumer of the partial planes applies the row factors.
// NW (4, 8 or 16 waves) trades partial planes for workgroup size: the waves of a workgroup split its K chunk
// and add their accumulators through LDS, so a larger workgroup covers a longer chunk and the launch writes
// fewer planes for the same number of waves in flight.
template <int NB, int NW, int ROTATE, int SCALE>
__global__ __launch_bounds__(NW * 64, 2) void gemm_tiled_f16(
    const half8 *__restrict__ A, const float *__restrict__ a_inv_scale, const half8 *__restrict__ W,
    float *__restrict__ P, int ldp, size_t plane_stride,
    int M, int N, int Mb, int Nb, int Kb, int steps_per_chunk)
{
    extern __shared__ float red[];                       // [NW/2][2*NB*16 regs][64 lanes]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int nb0 = blockIdx.x * NB, mb0 = blockIdx.z * 2;
    const int kb_beg = blockIdx.y * steps_per_chunk;
    const int nsteps = min(Kb, kb_beg + steps_per_chunk) - kb_beg;

    const half8 *wp[NB];
    const half8 *ap[2];
#pragma unroll
    for (int b = 0; b < NB; b++) wp[b] = W + (size_t)min(nb0 + b, Nb - 1) * Kb * 256 + lane;
#pragma unroll
    for (int mb = 0; mb < 2; mb++) ap[mb] = A + (size_t)min(mb0 + mb, Mb - 1) * Kb * 256 + lane;

    // row factors of the 2 x 16 rows this lane stores, fetched before the K loop so that the
    // epilogue of the last wave does not wait for them
    float rsc[2][16];
    if (SCALE) {
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = (mb0 + mb) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                rsc[mb][v] = a_inv_scale[min(m, M - 1)];
            }
    }

    float16v acc[2][NB];
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[mb][b][v] = 0.f;

    // wave w takes the K steps w, w+NW, w+2NW, ... of this workgroup's chunk (rotated)
    const int rot = ROTATE ? (int)((blockIdx.x * 7u + blockIdx.y * 3u) % (unsigned)nsteps) : 0;
    for (int i = wave; i < nsteps; i += NW) {
        int kk = i + rot;
        if (kk >= nsteps) kk -= nsteps;
        const size_t o = (size_t)(kb_beg + kk) * 256;    // 4 x 64 half8 per K step
        half8 a[2][4], w[NB][4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
#pragma unroll
            for (int b = 0; b < NB; b++) w[b][j] = __builtin_nontemporal_load(&wp[b][o + j * 64]);   // streamed once
#pragma unroll
            for (int mb = 0; mb < 2; mb++) a[mb][j] = ap[mb][o + j * 64];
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int b = 0; b < NB; b++)
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
                    acc[mb][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mb][j], w[b][j], acc[mb][b], 0, 0, 0);
    }

    // add the waves' accumulators in log2(NW) rounds through LDS (lane fastest => conflict-free):
    // in every round the upper half of the remaining waves parks its registers and the lower half adds them
    constexpr int REGS = 2 * NB * 16;
#pragma unroll
    for (int half = NW / 2; half >= 1; half >>= 1) {
        if (wave >= half && wave < 2 * half) {
            float *slot = red + (size_t)(wave - half) * REGS * 64;
#pragma unroll
            for (int mb = 0; mb < 2; mb++)
#pragma unroll
                for (int b = 0; b < NB; b++)
#pragma unroll
                    for (int v = 0; v < 16; v++) slot[((mb * NB + b) * 16 + v) * 64 + lane] = acc[mb][b][v];
        }
        __syncthreads();
        if (wave < half) {
            const float *slot = red + (size_t)wave * REGS * 64;
#pragma unroll
            for (int mb = 0; mb < 2; mb++)
#pragma unroll
                for (int b = 0; b < NB; b++)
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[mb][b][v] += slot[((mb * NB + b) * 16 + v) * 64 + lane];
        }
        if (half > 1) __syncthreads();
    }
    if (wave != 0) return;
    float *Pp = P + (size_t)blockIdx.y * plane_stride;
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float sres = acc[mb][b][v];
                // D layout of v_mfma_f32_32x32x16: column = lane & 31, row = 8*(v/4) + 4*(lane/32) + v%4
                const int m = (mb0 + mb) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                const int n = (nb0 + b) * 32 + r;
                if (m < M && n < N) {
                    if (SCALE) sres *= rsc[mb][v];
                    Pp[(size_t)m * ldp + n] = sres;
                }
            }
}

}  // namespace lmhip
