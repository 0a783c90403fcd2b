// Weight-streaming skinny GEMM for gfx950 and its entry points.
//
//   P[s][m][n] = inv_scale[m] * sum_{k in chunk s} A16[m][k] * W16[n][k]
//
// A16 is the fp16 image of an fp32 activation matrix whose rows were multiplied
// by a per-row power of two (inv_scale undoes it), W16 the frozen F16 weight.
// Replaces f16_matmul / f16_matmul_nt of shaders/q8_kernels.metal:383-435.
//
// Shape of the problem: M = batch*seq is 64..160 while N*K is up to 389 M, so
// every weight byte is used 2*M times and the kernel is bound by streaming W
// from HBM once.  Design:
//   * both operands live in the tiled layout of gemm.h: a wave-wide 16-byte load
//     is 1 KB of contiguous memory and lands directly in the operand registers
//     of v_mfma_f32_32x32x16_f16 — no LDS round trip for weight data that
//     exactly one wave uses, no shuffles;
//   * one wave owns NB*32 weight rows and walks K in steps of 64; the 64
//     activation rows of the tile come through L2 in the same layout (the
//     activation matrix is at most a few MB and shared by all workgroups), so
//     one W fragment feeds two MFMAs (rows 0-31 and 32-63);
//   * the four waves of a workgroup split the K chunk between them and add
//     their accumulators through LDS; chunks of different workgroups land in
//     separate partial planes P[s] that the consumer kernel sums on load
//     (deterministic, no atomics, no zero-fill).
#include "backend.h"
#include "devutil.h"
#include "gemm.h"
#include <vector>

namespace {

template <int NB>
struct Stage {
    half8 a[2][4];
    half8 w[NB][4];
};

template <int NB>
__device__ __forceinline__ void load_stage(Stage<NB> &st, const half8 *const (&ap)[2],
                                           const half8 *const (&wp)[NB], int kb)
{
    const size_t o = (size_t)kb * 256;                   // 4 x 64 half8 per K step
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int b = 0; b < NB; b++) st.w[b][j] = __builtin_nontemporal_load(&wp[b][o + j * 64]);   // streamed once: keep L2 for A
#pragma unroll
        for (int mb = 0; mb < 2; mb++) st.a[mb][j] = ap[mb][o + j * 64];
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

// grid: x = ceil(Nb / NB) weight-row tiles, y = S (K chunks), z = ceil(M / 64); block = 256.
// Kb = number of 64-wide K steps of the (padded) reduction; Nb, Mb = 32-row blocks of W and A.
template <int NB>
__global__ __launch_bounds__(256, 2) void gemm_tiled_f16(
    const half8 *__restrict__ A, const float *__restrict__ a_inv_scale, const half8 *__restrict__ W,
    float *__restrict__ P, int ldp, size_t plane_stride,
    int M, int N, int Mb, int Nb, int Kb, int steps_per_chunk)
{
    extern __shared__ float red[];                       // [4 waves][2*NB*16 regs][64 lanes]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int nb0 = blockIdx.x * NB, mb0 = blockIdx.z * 2;
    const int kb_beg = blockIdx.y * steps_per_chunk;
    const int kb_end = min(Kb, kb_beg + steps_per_chunk);

    const half8 *wp[NB];
    const half8 *ap[2];
#pragma unroll
    for (int b = 0; b < NB; b++) wp[b] = W + (size_t)min(nb0 + b, Nb - 1) * Kb * 256 + lane;
#pragma unroll
    for (int mb = 0; mb < 2; mb++) ap[mb] = A + (size_t)min(mb0 + mb, Mb - 1) * Kb * 256 + lane;

    float16v acc[2][NB];
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[mb][b][v] = 0.f;

    // wave w takes the K steps w, w+4, w+8, ... of this workgroup's chunk
    int kb = kb_beg + wave;
    Stage<NB> s0, s1;
    if (kb < kb_end) load_stage<NB>(s0, ap, wp, kb);
    while (kb < kb_end) {
        if (kb + 4 < kb_end) load_stage<NB>(s1, ap, wp, kb + 4);
        mma_stage<NB>(s0, acc);
        kb += 4;
        if (kb >= kb_end) break;
        if (kb + 4 < kb_end) load_stage<NB>(s0, ap, wp, kb + 4);
        mma_stage<NB>(s1, acc);
        kb += 4;
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
        const int m = (mb0 + mb) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        const int n = (nb0 + b) * 32 + r;
        if (m < M && n < N) {
            if (a_inv_scale) s *= a_inv_scale[m];
            Pp[(size_t)m * ldp + n] = s;
        }
    }
}

// One workgroup per row: fp32 row -> tiled fp16 row scaled by a power of two, plus 1/scale.
__global__ __launch_bounds__(256) void rows_to_f16_scaled(
    const float *__restrict__ X, int ldx, half_t *__restrict__ out, float *__restrict__ inv_scale, int K, int Kb)
{
    __shared__ float sm[16];
    const int row = blockIdx.x;
    const float *x = X + (size_t)row * ldx;
    float amax = 0.f;
    for (int i = threadIdx.x; i < K; i += blockDim.x) amax = fmaxf(amax, fabsf(x[i]));
    amax = block_max(amax, sm);
    const float s = row_scale_for(amax);
    for (int i = threadIdx.x; i < Kb * 64; i += blockDim.x)
        out[lmhip::tiled_index(row, i, Kb)] = (i < K) ? f2h(x[i] * s) : (half_t)0;
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

// Row-major F16 [rows, cols] -> tiled layout, optionally transposed; 64x64 element tiles via LDS
// so that both the reads (along cols) and the writes (16-byte groups along the destination K) coalesce.
__global__ __launch_bounds__(256) void tile_f16(const half_t *__restrict__ src, int rows, int cols,
                                                 half_t *__restrict__ dst, int Kb_dst, int row_off, int k_off,
                                                 int transpose)
{
    __shared__ half_t t[64][66];
    const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        const int rr = r0 + i, cc = c0 + tx;
        t[i][tx] = (rr < rows && cc < cols) ? src[(size_t)rr * cols + cc] : (half_t)0;
    }
    __syncthreads();
    // destination element (dr, dk): dr indexes tiled rows, dk the tiled K
    for (int i = ty; i < 64; i += 4) {
        int dr, dk;
        half_t v;
        if (!transpose) { dr = r0 + i; dk = c0 + tx; v = t[i][tx]; if (dr >= rows || dk >= cols) continue; }
        else            { dr = c0 + i; dk = r0 + tx; v = t[tx][i]; if (dr >= cols || dk >= rows) continue; }
        dst[lmhip::tiled_index(row_off + dr, k_off + dk, Kb_dst)] = v;
    }
}

struct ProfRec { hipEvent_t a, b; double wbytes; };
int g_prof_on = 0;
std::vector<ProfRec> g_prof;
int g_force_nb = 0, g_force_S = 0;

}  // namespace

namespace lmhip {

// Tile height and K split.  Measured on MI355X at M = 64: one 32-row block per wave (lower
// register use, three resident workgroups per CU) beats two at every shape of the step, and
// the kernel wants at least ~2.5 workgroups per CU even when that leaves each with only a
// couple of K steps per wave; beyond that, splitting K only adds partial-plane traffic.
GemmPlan plan_gemm(int M, int N, int K)
{
    const int Kb = tiled_kb(K), Nb = tiled_rb(N), m_tiles = (M + 63) / 64;
    const int cus = num_cus() > 0 ? num_cus() : 256;
    GemmPlan p{};
    p.nb = g_force_nb ? g_force_nb : 1;
    p.n_tiles = (Nb + p.nb - 1) / p.nb;
    p.m_tiles = m_tiles;
    const int base = p.n_tiles * m_tiles;
    int S = g_force_S ? g_force_S : (5 * cus / 2 + base - 1) / base;
    const int max_s = Kb >= 8 ? Kb / 8 : 1;                // at least two K steps per wave
    if (!g_force_S && S > max_s) S = max_s;
    if (S < 1) S = 1;
    int steps = (Kb + S - 1) / S;
    steps = (steps + 3) & ~3;                              // whole steps for each of the four waves
    p.steps = steps;
    p.S = (Kb + steps - 1) / steps;
    return p;
}

void launch_gemm(const half_t *A, const float *a_inv_scale, const half_t *W,
                 float *P, int ldp, size_t plane_stride, int M, int N, int K, const GemmPlan &p)
{
    if (M <= 0 || N <= 0 || K <= 0) return;
    if (ldp < N || p.S < 1 || p.steps < 1 || (p.nb != 1 && p.nb != 2)) {
        fprintf(stderr, "[fast_hip] gemm: bad launch M=%d N=%d K=%d ldp=%d plan(nb=%d S=%d steps=%d)\n",
                M, N, K, ldp, p.nb, p.S, p.steps);
        abort();
    }
    const int Kb = tiled_kb(K), Nb = tiled_rb(N), Mb = tiled_rb(M);
    dim3 grid(p.n_tiles, p.S, p.m_tiles), block(256);
    const size_t lds = (size_t)4 * (2 * p.nb * 16) * 64 * sizeof(float);
    ProfRec rec{};
    if (g_prof_on) {
        HIP_CHECK(hipEventCreate(&rec.a));
        HIP_CHECK(hipEventCreate(&rec.b));
        rec.wbytes = 2.0 * (double)N * (double)K * p.m_tiles;
        HIP_CHECK(hipEventRecord(rec.a, stream()));
    }
    const half8 *A8 = reinterpret_cast<const half8 *>(A), *W8 = reinterpret_cast<const half8 *>(W);
    if (p.nb == 2)
        hipLaunchKernelGGL(gemm_tiled_f16<2>, grid, block, lds, stream(), A8, a_inv_scale, W8,
                           P, ldp, plane_stride, M, N, Mb, Nb, Kb, p.steps);
    else
        hipLaunchKernelGGL(gemm_tiled_f16<1>, grid, block, lds, stream(), A8, a_inv_scale, W8,
                           P, ldp, plane_stride, M, N, Mb, Nb, Kb, p.steps);
    HIP_CHECK(hipGetLastError());
    if (g_prof_on) {
        HIP_CHECK(hipEventRecord(rec.b, stream()));
        g_prof.push_back(rec);
    }
}

void launch_rows_to_f16(const float *X, int ldx, half_t *out_tiled, float *inv_scale, int M, int K)
{
    hipLaunchKernelGGL(rows_to_f16_scaled, dim3(M), dim3(256), 0, stream(), X, ldx, out_tiled, inv_scale, K, tiled_kb(K));
    HIP_CHECK(hipGetLastError());
}

void launch_reduce_planes(const float *P, int S, size_t plane_stride, int ldp, float *C, int M, int N)
{
    const size_t n = (size_t)M * N;
    hipLaunchKernelGGL(reduce_planes, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream(),
                       P, S, plane_stride, ldp, C, M, N);
    HIP_CHECK(hipGetLastError());
}

void launch_tile_f16(const half_t *src, int rows, int cols, half_t *dst_tiled, int Kb_dst,
                     int row_off, int k_off, int transpose)
{
    if (rows <= 0 || cols <= 0) return;
    hipLaunchKernelGGL(tile_f16, dim3((cols + 63) / 64, (rows + 63) / 64), dim3(256), 0, stream(),
                       src, rows, cols, dst_tiled, Kb_dst, row_off, k_off, transpose);
    HIP_CHECK(hipGetLastError());
}

}  // namespace lmhip

using namespace lmhip;

namespace {

// Tiled image of a row-major F16 weight buffer W[rows, cols] (transposed: of W^T), kept with the
// buffer until something writes it.  Host-visible buffers and views are re-tiled on every call.
const half_t *tiled_copy_of(MetalBuf *W, int rows, int cols, int transposed)
{
    const int R = transposed ? cols : rows, K = transposed ? rows : cols;
    const size_t bytes = tiled_elems(R, K) * sizeof(half_t);
    const bool cacheable = W->owns && !W->host && !W->parent;
    if (!cacheable) {
        half_t *t = (half_t *)scratch(SCR_MISC, bytes);
        HIP_CHECK(hipMemsetAsync(t, 0, bytes, stream()));
        launch_tile_f16(dptr_as<half_t>(W), rows, cols, t, tiled_kb(K), 0, 0, transposed);
        return t;
    }
    MetalBuf::Tiled &c = W->tiled[transposed ? 1 : 0];
    if (!c.dev || c.rows != rows || c.cols != cols || c.version != W->version) {
        if (c.dev && (c.rows != rows || c.cols != cols)) {
            HIP_CHECK(hipStreamSynchronize(stream()));
            HIP_CHECK(hipFree(c.dev));
            c.dev = nullptr;
        }
        if (!c.dev) {
            HIP_CHECK(hipMalloc(&c.dev, bytes));
            HIP_CHECK(hipMemsetAsync(c.dev, 0, bytes, stream()));
        }
        launch_tile_f16(dptr_as<half_t>(W), rows, cols, (half_t *)c.dev, tiled_kb(K), 0, 0, transposed);
        c.rows = rows; c.cols = cols; c.version = W->version;
    }
    return (const half_t *)c.dev;
}

// C[M, Nout] fp32 = A[M, Kred] fp32 * Wt^T with Wt the tiled [Nout, Kred] operand
void gemm_f32a(const float *A, const half_t *Wt, float *C, int M, int Nout, int Kred)
{
    half_t *a16 = (half_t *)scratch(SCR_A16, tiled_elems(M, Kred) * sizeof(half_t));
    float *inv = (float *)scratch(SCR_SCALE, (size_t)M * sizeof(float));
    launch_rows_to_f16(A, Kred, a16, inv, M, Kred);
    GemmPlan p = plan_gemm(M, Nout, Kred);
    if (p.S == 1) {
        launch_gemm(a16, inv, Wt, C, Nout, 0, M, Nout, Kred, p);
    } else {
        const size_t plane = (size_t)M * Nout;
        float *P = (float *)scratch(SCR_PARTIAL, plane * p.S * sizeof(float));
        launch_gemm(a16, inv, Wt, P, Nout, plane, M, Nout, Kred, p);
        launch_reduce_planes(P, p.S, plane, Nout, C, M, Nout);
    }
}

}  // namespace

extern "C" {

// f16_matmul, shaders/q8_kernels.metal:383-407; dispatch src/nn/fast_metal.m:562-577.
void metal_enqueue_f16_matmul(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K)
{
    REQUIRE_BYTES(A, (size_t)M * K * 4, "f16_matmul");
    REQUIRE_BYTES(W, (size_t)N * K * 2, "f16_matmul");
    REQUIRE_BYTES(C, (size_t)M * N * 4, "f16_matmul");
    if (M <= 0 || N <= 0 || K <= 0) return;
    gemm_f32a(dptr_as<float>(A), tiled_copy_of(W, N, K, 0), dptr_as<float>(C), M, N, K);
    mark_written(C);
}

// f16_matmul_nt, shaders/q8_kernels.metal:411-435; dispatch src/nn/fast_metal.m:579-594.
// C[M,K] = A[M,N] W[N,K]: the reduction runs over W's rows, so the multiply uses the tiled
// image of W^T.
void metal_enqueue_f16_matmul_nt(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K)
{
    REQUIRE_BYTES(A, (size_t)M * N * 4, "f16_matmul_nt");
    REQUIRE_BYTES(W, (size_t)N * K * 2, "f16_matmul_nt");
    REQUIRE_BYTES(C, (size_t)M * K * 4, "f16_matmul_nt");
    if (M <= 0 || N <= 0 || K <= 0) return;
    gemm_f32a(dptr_as<float>(A), tiled_copy_of(W, N, K, 1), dptr_as<float>(C), M, K, N);
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

// Times `iters` launches of the GEMM alone on synthetic tiled operands of the given shape
// (HIP events on the library's stream).  nb / S = 0 let the planner choose; otherwise they
// force the tile height and K split.  Returns the average milliseconds per launch.
double hip_gemm_time_shape(int M, int N, int K, int nb, int S, int iters, int *used_nb, int *used_S)
{
    g_force_nb = nb; g_force_S = S;
    GemmPlan p = plan_gemm(M, N, K);
    g_force_nb = 0; g_force_S = 0;
    if (used_nb) *used_nb = p.nb;
    if (used_S) *used_S = p.S;
    void *A = nullptr, *W = nullptr, *P = nullptr, *inv = nullptr;
    const size_t ab = tiled_elems(M, K) * 2, wb = tiled_elems(N, K) * 2, pb = (size_t)p.S * M * N * 4;
    // rotate through enough distinct weight images that no launch finds its weights in a cache
    const int nbuf = (int)((size_t)1200 * 1024 * 1024 / wb) + 1;
    HIP_CHECK(hipMalloc(&A, ab)); HIP_CHECK(hipMalloc(&W, wb * nbuf)); HIP_CHECK(hipMalloc(&P, pb)); HIP_CHECK(hipMalloc(&inv, (size_t)M * 4));
    HIP_CHECK(hipMemsetAsync(A, 0x11, ab, stream())); HIP_CHECK(hipMemsetAsync(W, 0x11, wb * nbuf, stream()));
    HIP_CHECK(hipMemsetAsync(inv, 0, (size_t)M * 4, stream()));
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0)); HIP_CHECK(hipEventCreate(&e1));
    const int saved = g_prof_on;
    g_prof_on = 0;
    for (int i = 0; i < 3; i++) launch_gemm((half_t *)A, (float *)inv, (half_t *)W, (float *)P, N, (size_t)M * N, M, N, K, p);
    HIP_CHECK(hipEventRecord(e0, stream()));
    for (int i = 0; i < iters; i++)
        launch_gemm((half_t *)A, (float *)inv, (half_t *)((char *)W + (size_t)(i % nbuf) * wb), (float *)P, N, (size_t)M * N, M, N, K, p);
    HIP_CHECK(hipEventRecord(e1, stream()));
    HIP_CHECK(hipStreamSynchronize(stream()));
    g_prof_on = saved;
    float ms = 0;
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    hipEventDestroy(e0); hipEventDestroy(e1);
    hipFree(A); hipFree(W); hipFree(P); hipFree(inv);
    return (double)ms / iters;
}

}  // extern "C"
