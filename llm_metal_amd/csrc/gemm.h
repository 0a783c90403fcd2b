// Internal interface of the weight-streaming GEMM (gemm.hip).
#pragma once
#include "backend.h"
#include "devutil.h"

namespace lmhip {

struct GemmPlan {
    int nb;        // 32-row weight blocks per wave (1 or 2)
    int S;         // K chunks = partial planes written
    int k_chunk;   // elements of K per chunk (multiple of 256)
    int n_tiles, m_tiles;
};

GemmPlan plan_gemm(int M, int N, int K);

// P[s][m][n] (s < plan.S, plane s at P + s*plane_stride, row stride ldp) =
//   inv_scale[m] * sum_{k in chunk s} A[m][k] * W[n][k]
void launch_gemm(const half_t *A, int lda, const float *a_inv_scale, const half_t *W, int ldw,
                 float *P, int ldp, size_t plane_stride, int M, int N, int K, const GemmPlan &p);

// out[m][0..ldo) = fp16(X[m][k] * s_m) (zero beyond K), inv_scale[m] = 1/s_m
void launch_rows_to_f16(const float *X, int ldx, half_t *out, int ldo, float *inv_scale, int M, int K);
void launch_reduce_planes(const float *P, int S, size_t plane_stride, int ldp, float *C, int M, int N);
void launch_transpose_f16(const half_t *src, half_t *dst, int rows, int cols, int ld_dst);
void gemm_f32a(const float *A, const half_t *W, int ldw, float *C, int M, int N, int K);

}  // namespace lmhip
