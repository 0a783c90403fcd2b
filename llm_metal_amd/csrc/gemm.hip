// Weight-streaming skinny GEMM for gfx950 and its entry points.
//
//   P[s][m][n] = inv_scale[m] * sum_{k in chunk s} A16[m][k] * W16[n][k]
//
// A16 is the fp16 image of an fp32 activation matrix whose rows were multiplied
// by a per-row power of two (inv_scale undoes it), W16 the frozen F16 weight,
// row-major [N, K] exactly as wmat_create_f16 lays it out (src/nn/wmat.c:63-75).
// Replaces f16_matmul / f16_matmul_nt of shaders/q8_kernels.metal:383-435.
//
// Shape of the problem: M = batch*seq is 64..160 while N*K is up to 389 M, so
// every weight byte is used 2*M times and the kernel is bound by streaming W
// from HBM once.  Design:
//   * one wave owns NB*32 weight rows and walks K in steps of 64; each lane
//     pulls 64 contiguous bytes of "its" row per step (two lanes cover a 128 B
//     line) straight into the B operand registers of v_mfma_f32_32x32x16_f16 —
//     no LDS round trip for data that is used by exactly one wave.  The K order
//     inside a step is permuted identically for A and W, which a dot product
//     does not see.
//   * the 64 activation rows of the tile come through L2 in the same per-lane
//     layout (the activation matrix is at most a few MB and shared by all
//     workgroups), so one W fragment feeds two MFMAs (rows 0-31 and 32-63).
//   * the four waves of a workgroup split the K chunk between them and add
//     their accumulators through LDS; chunks of different workgroups land in
//     separate partial planes P[s] that the consumer kernel sums on load
//     (deterministic, no atomics, no zero-fill).
#include "backend.h"
#include "devutil.h"
#include "gemm.h"
#include <vector>

namespace {

__device__ __forceinline__ half8 ld8(const half_t *p, bool ok)
{
    half8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    return ok ? *reinterpret_cast<const half8 *>(p) : z;
}

template <int NB>
struct Stage {
    half8 a[2][4];
    half8 w[NB][4];
};

template <int NB>
__device__ __forceinline__ void load_stage(Stage<NB> &st, const half_t *const (&arow)[2],
                                           const half_t *const (&wrow)[NB], int k, int kend)
{
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const bool ok = (k + 8 * j + 8) <= kend;
#pragma unroll
        for (int b = 0; b < NB; b++) st.w[b][j] = ld8(wrow[b] + k + 8 * j, ok);
#pragma unroll
        for (int mb = 0; mb < 2; mb++) st.a[mb][j] = ld8(arow[mb] + k + 8 * j, ok);
    }
}

template <int NB>
__device__ __forceinline__ void mma_stage(const Stage<NB> &st, float16v (&acc)[2][NB])
{
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
            for (int b = 0; b < NB; b++)
                acc[mb][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(st.a[mb][j], st.w[b][j], acc[mb][b], 0, 0, 0);
}

// grid: x = ceil(N / (32*NB)), y = S (K chunks), z = ceil(M / 64); block = 256.
// K must be a multiple of 8 and lda, ldw multiples of 8 (16-byte row alignment).
template <int NB>
__global__ __launch_bounds__(256, 2) void gemm_skinny_f16(
    const half_t *__restrict__ A, int lda, const float *__restrict__ a_inv_scale,
    const half_t *__restrict__ W, int ldw,
    float *__restrict__ P, int ldp, size_t plane_stride,
    int M, int N, int K, int k_chunk)
{
    extern __shared__ float red[];                       // [4 waves][2*NB*16 regs][64 lanes]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int n0 = blockIdx.x * (32 * NB), m0 = blockIdx.z * 64;
    const int kbeg = blockIdx.y * k_chunk;
    const int kend = min(K, kbeg + k_chunk);

    const half_t *wrow[NB];
    const half_t *arow[2];
#pragma unroll
    for (int b = 0; b < NB; b++) wrow[b] = W + (size_t)min(n0 + b * 32 + r, N - 1) * ldw + h * 32;
#pragma unroll
    for (int mb = 0; mb < 2; mb++) arow[mb] = A + (size_t)min(m0 + mb * 32 + r, M - 1) * lda + h * 32;

    float16v acc[2][NB];
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[mb][b][v] = 0.f;

    // wave w takes the 64-wide K steps w, w+4, w+8, ... of this workgroup's chunk
    const int kstep = 4 * 64;
    int k = kbeg + wave * 64;
    // a lane's 32 elements of a step start at k + h*32 (folded into the row pointers);
    // validity is judged on the un-offset position plus the lane's half
    const int kend_l = kend - h * 32;
    Stage<NB> s0, s1;
    if (k < kend) load_stage<NB>(s0, arow, wrow, k, kend_l);
    while (k < kend) {
        const int k1 = k + kstep;
        if (k1 < kend) load_stage<NB>(s1, arow, wrow, k1, kend_l);
        mma_stage<NB>(s0, acc);
        k = k1;
        if (k >= kend) break;
        const int k2 = k + kstep;
        if (k2 < kend) load_stage<NB>(s0, arow, wrow, k2, kend_l);
        mma_stage<NB>(s1, acc);
        k = k2;
    }

    // add the four waves' accumulators: red[wave][reg][lane], lane fastest => conflict-free
    constexpr int REGS = 2 * NB * 16;
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                red[(wave * REGS + (mb * NB + b) * 16 + v) * 64 + lane] = acc[mb][b][v];
    __syncthreads();

    float *Pp = P + (size_t)blockIdx.y * plane_stride;
#pragma unroll
    for (int i = 0; i < REGS / 4; i++) {
        const int reg = wave + 4 * i;                      // this thread finishes (reg, lane)
        float s = red[(0 * REGS + reg) * 64 + lane] + red[(1 * REGS + reg) * 64 + lane]
                + red[(2 * REGS + reg) * 64 + lane] + red[(3 * REGS + reg) * 64 + lane];
        const int v = reg & 15, blk = reg >> 4;
        const int b = blk % NB, mb = blk / NB;
        // D layout of v_mfma_f32_32x32x16: column = lane & 31, row = 8*(v/4) + 4*(lane/32) + v%4
        const int m = m0 + mb * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        const int n = n0 + b * 32 + r;
        if (m < M && n < N) {
            if (a_inv_scale) s *= a_inv_scale[m];
            Pp[(size_t)m * ldp + n] = s;
        }
    }
}

// One workgroup per row: fp32 row -> fp16 row scaled by a power of two, plus 1/scale.
__global__ __launch_bounds__(256) void rows_to_f16_scaled(
    const float *__restrict__ X, int ldx, half_t *__restrict__ out, int ldo,
    float *__restrict__ inv_scale, int K)
{
    __shared__ float sm[16];
    const int row = blockIdx.x;
    const float *x = X + (size_t)row * ldx;
    float amax = 0.f;
    for (int i = threadIdx.x; i < K; i += blockDim.x) amax = fmaxf(amax, fabsf(x[i]));
    amax = block_max(amax, sm);
    const float s = row_scale_for(amax);
    half_t *o = out + (size_t)row * ldo;
    for (int i = threadIdx.x; i < ldo; i += blockDim.x) o[i] = (i < K) ? f2h(x[i] * s) : (half_t)0;
    if (threadIdx.x == 0) inv_scale[row] = 1.0f / s;
}

__global__ void reduce_planes(const float *__restrict__ P, int S, size_t plane_stride, int ldp,
                              float *__restrict__ C, int M, int N)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)M * N) return;
    const int m = (int)(idx / N), n = (int)(idx % N);
    float s = 0.f;
    for (int p = 0; p < S; p++) s += P[p * plane_stride + (size_t)m * ldp + n];
    C[idx] = s;
}

// dst[c][r] = src[r][c] for an F16 matrix [rows, cols]; 64x64 tiles through LDS.
__global__ __launch_bounds__(256) void transpose_f16(const half_t *__restrict__ src, half_t *__restrict__ dst,
                                                      int rows, int cols, int ld_dst)
{
    __shared__ half_t tile[64][66];
    const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        const int rr = r0 + i, cc = c0 + tx;
        tile[i][tx] = (rr < rows && cc < cols) ? src[(size_t)rr * cols + cc] : (half_t)0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int cc = c0 + i, rr = r0 + tx;
        if (cc < cols && rr < rows) dst[(size_t)cc * ld_dst + rr] = tile[tx][i];
    }
}

struct ProfRec { hipEvent_t a, b; double wbytes; };
int g_prof_on = 0;
std::vector<ProfRec> g_prof;

}  // namespace

namespace lmhip {

GemmPlan plan_gemm(int M, int N, int K)
{
    GemmPlan p;
    const int m_tiles = (M + 63) / 64;
    p.nb = (N >= 2048 || N % 64 == 0) ? 2 : 1;
    int n_tiles = (N + 32 * p.nb - 1) / (32 * p.nb);
    const int target = 2 * (num_cus() > 0 ? num_cus() : 256);       // two resident workgroups per CU
    if (n_tiles * m_tiles * 2 <= target && p.nb == 2) {                // too few tiles: halve the tile
        p.nb = 1;
        n_tiles = (N + 31) / 32;
    }
    int S = 1;
    if (n_tiles * m_tiles < target) {
        S = (target + n_tiles * m_tiles - 1) / (n_tiles * m_tiles);
        const int max_s = (K + 255) / 256;                              // each chunk gives every wave >= 1 step
        if (S > max_s) S = max_s;
        if (S < 1) S = 1;
    }
    int kc = (K + S - 1) / S;
    kc = ((kc + 255) / 256) * 256;
    p.k_chunk = kc;
    p.S = (K + kc - 1) / kc;
    p.n_tiles = n_tiles;
    p.m_tiles = m_tiles;
    return p;
}

void launch_gemm(const half_t *A, int lda, const float *a_inv_scale, const half_t *W, int ldw,
                 float *P, int ldp, size_t plane_stride, int M, int N, int K, const GemmPlan &p)
{
    if (M <= 0 || N <= 0 || K <= 0) return;
    if ((K & 7) || (lda & 7) || (ldw & 7) || lda < K || ldw < K || ldp < N) {
        fprintf(stderr, "[fast_hip] gemm: unsupported shape M=%d N=%d K=%d lda=%d ldw=%d ldp=%d "
                        "(K and the leading dimensions must be multiples of 8)\n", M, N, K, lda, ldw, ldp);
        abort();
    }
    dim3 grid(p.n_tiles, p.S, p.m_tiles), block(256);
    const size_t lds = (size_t)4 * (2 * p.nb * 16) * 64 * sizeof(float);
    ProfRec rec{};
    if (g_prof_on) {
        HIP_CHECK(hipEventCreate(&rec.a));
        HIP_CHECK(hipEventCreate(&rec.b));
        rec.wbytes = 2.0 * (double)N * (double)K * p.m_tiles;
        HIP_CHECK(hipEventRecord(rec.a, stream()));
    }
    if (p.nb == 2)
        hipLaunchKernelGGL(gemm_skinny_f16<2>, grid, block, lds, stream(), A, lda, a_inv_scale, W, ldw,
                           P, ldp, plane_stride, M, N, K, p.k_chunk);
    else
        hipLaunchKernelGGL(gemm_skinny_f16<1>, grid, block, lds, stream(), A, lda, a_inv_scale, W, ldw,
                           P, ldp, plane_stride, M, N, K, p.k_chunk);
    HIP_CHECK(hipGetLastError());
    if (g_prof_on) {
        HIP_CHECK(hipEventRecord(rec.b, stream()));
        g_prof.push_back(rec);
    }
}

void launch_rows_to_f16(const float *X, int ldx, half_t *out, int ldo, float *inv_scale, int M, int K)
{
    hipLaunchKernelGGL(rows_to_f16_scaled, dim3(M), dim3(256), 0, stream(), X, ldx, out, ldo, inv_scale, K);
    HIP_CHECK(hipGetLastError());
}

void launch_reduce_planes(const float *P, int S, size_t plane_stride, int ldp, float *C, int M, int N)
{
    const size_t n = (size_t)M * N;
    hipLaunchKernelGGL(reduce_planes, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream(),
                       P, S, plane_stride, ldp, C, M, N);
    HIP_CHECK(hipGetLastError());
}

void launch_transpose_f16(const half_t *src, half_t *dst, int rows, int cols, int ld_dst)
{
    hipLaunchKernelGGL(transpose_f16, dim3((cols + 63) / 64, (rows + 63) / 64), dim3(256), 0, stream(),
                       src, dst, rows, cols, ld_dst);
    HIP_CHECK(hipGetLastError());
}

// C[M,N] fp32 = A[M,K] fp32 * W16[N,K]^T through the skinny kernel (convert, multiply, sum planes).
void gemm_f32a(const float *A, const half_t *W, int ldw, float *C, int M, int N, int K)
{
    const int Kp = (K + 7) & ~7;
    half_t *a16 = (half_t *)scratch(SCR_A16, (size_t)M * Kp * sizeof(half_t));
    float *inv = (float *)scratch(SCR_SCALE, (size_t)M * sizeof(float));
    launch_rows_to_f16(A, K, a16, Kp, inv, M, K);
    GemmPlan p = plan_gemm(M, N, Kp);
    if (p.S == 1) {
        launch_gemm(a16, Kp, inv, W, ldw, C, N, 0, M, N, Kp, p);
    } else {
        const size_t plane = (size_t)M * N;
        float *P = (float *)scratch(SCR_PARTIAL, plane * p.S * sizeof(float));
        launch_gemm(a16, Kp, inv, W, ldw, P, N, plane, M, N, Kp, p);
        launch_reduce_planes(P, p.S, plane, N, C, M, N);
    }
}

}  // namespace lmhip

using namespace lmhip;

extern "C" {

// f16_matmul, shaders/q8_kernels.metal:383-407; dispatch src/nn/fast_metal.m:562-577.
void metal_enqueue_f16_matmul(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K)
{
    REQUIRE_BYTES(A, (size_t)M * K * 4, "f16_matmul");
    REQUIRE_BYTES(W, (size_t)N * K * 2, "f16_matmul");
    REQUIRE_BYTES(C, (size_t)M * N * 4, "f16_matmul");
    if (K & 7) { fprintf(stderr, "[fast_hip] f16_matmul: K=%d must be a multiple of 8\n", K); return; }
    gemm_f32a(dptr_as<float>(A), dptr_as<half_t>(W), K, dptr_as<float>(C), M, N, K);
    mark_written(C);
}

// f16_matmul_nt, shaders/q8_kernels.metal:411-435; dispatch src/nn/fast_metal.m:579-594.
// C[M,K] = A[M,N] W[N,K]: the reduction runs over W's rows, so the multiply uses a
// transposed copy of W ([K, N], row stride N padded to 8) that is built on first use
// and kept with the buffer until something writes the buffer.
void metal_enqueue_f16_matmul_nt(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K)
{
    REQUIRE_BYTES(A, (size_t)M * N * 4, "f16_matmul_nt");
    REQUIRE_BYTES(W, (size_t)N * K * 2, "f16_matmul_nt");
    REQUIRE_BYTES(C, (size_t)M * K * 4, "f16_matmul_nt");
    const int ldt = (N + 7) & ~7;
    const bool cacheable = W->owns && !W->host && !W->parent;
    half_t *wt;
    if (cacheable) {
        if (!W->t_dev || W->t_rows != K || W->t_cols != N || W->t_version != W->version) {
            if (W->t_dev && (W->t_rows != K || W->t_cols != N)) {
                HIP_CHECK(hipStreamSynchronize(stream()));
                HIP_CHECK(hipFree(W->t_dev));
                W->t_dev = nullptr;
            }
            if (!W->t_dev) {
                HIP_CHECK(hipMalloc(&W->t_dev, (size_t)K * ldt * sizeof(half_t)));
                HIP_CHECK(hipMemsetAsync(W->t_dev, 0, (size_t)K * ldt * sizeof(half_t), stream()));
            }
            launch_transpose_f16(dptr_as<half_t>(W), (half_t *)W->t_dev, N, K, ldt);
            W->t_rows = K; W->t_cols = N; W->t_version = W->version;
        }
        wt = (half_t *)W->t_dev;
    } else {
        wt = (half_t *)scratch(SCR_MISC, (size_t)K * ldt * sizeof(half_t));
        if (ldt != N) HIP_CHECK(hipMemsetAsync(wt, 0, (size_t)K * ldt * sizeof(half_t), stream()));
        launch_transpose_f16(dptr_as<half_t>(W), wt, N, K, ldt);
    }
    // C[M,K] = A[M,N] * Wt[K,N]^T; A's reduction length N is padded to 8 inside gemm_f32a
    const int Np = ldt;
    half_t *a16 = (half_t *)scratch(SCR_A16, (size_t)M * Np * sizeof(half_t));
    float *inv = (float *)scratch(SCR_SCALE, (size_t)M * sizeof(float));
    launch_rows_to_f16(dptr_as<float>(A), N, a16, Np, inv, M, N);
    GemmPlan p = plan_gemm(M, K, Np);
    if (p.S == 1) {
        launch_gemm(a16, Np, inv, wt, ldt, dptr_as<float>(C), K, 0, M, K, Np, p);
    } else {
        const size_t plane = (size_t)M * K;
        float *P = (float *)scratch(SCR_PARTIAL, plane * p.S * sizeof(float));
        launch_gemm(a16, Np, inv, wt, ldt, P, K, plane, M, K, Np, p);
        launch_reduce_planes(P, p.S, plane, K, dptr_as<float>(C), M, K);
    }
    mark_written(C);
}

void hip_gemm_profile_enable(int on)
{
    HIP_CHECK(hipStreamSynchronize(stream()));
    for (auto &r : g_prof) { hipEventDestroy(r.a); hipEventDestroy(r.b); }
    g_prof.clear();
    g_prof_on = on;
}

int hip_gemm_profile_read(double *total_ms, double *total_weight_bytes)
{
    HIP_CHECK(hipStreamSynchronize(stream()));
    double ms = 0, wb = 0;
    for (auto &r : g_prof) {
        float t = 0;
        HIP_CHECK(hipEventElapsedTime(&t, r.a, r.b));
        ms += t;
        wb += r.wbytes;
    }
    if (total_ms) *total_ms = ms;
    if (total_weight_bytes) *total_weight_bytes = wb;
    return (int)g_prof.size();
}

}  // extern "C"
