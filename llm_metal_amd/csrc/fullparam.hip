// Full-parameter mode: weight gradients dW = dY^T X on the matrix cores, straight
// into the tiled F16 images the GEMMs read.
//
// Replaces f16_grad_accum / f16_sgd_fused / f16_sgd_apply of
// shaders/q8_kernels.metal:1097-1125, 1164-1206 as the fused pipeline uses them
// (src/nn/fast_sft.c:778-946, 1021-1039).
//
// The contraction of a weight gradient runs over the tokens, so both operands are
// first transposed: the token-major fp16 operand rows that the backward already
// holds (each with its own row factor) become feature-major rows with one
// power-of-two factor per FEATURE — factors of the output's row and column, which
// can be taken out of the sum.  k_wgrad then forms 64 x 64 blocks of dW per wave
// with v_mfma_f32_32x32x16_f16 and does the read-modify-write of the F16 target
// (accumulator G or weight W) in the operand layout of gemm.h, 8 bytes per lane,
// 512 contiguous bytes per wave instruction.  The kernel is bound by that
// read-modify-write: 4 bytes of HBM traffic per weight and call.
#include "backend.h"
#include "devutil.h"
#include "gemm.h"
#include "fused.h"
#include <hip/hip_ext.h>

using namespace lmhip;

// The F16 update rules are specified as separate fp32 operations (multiply, then add, then one
// rounding to F16); a fused multiply-add would change results at rounding ties.
#pragma clang fp contract(off)

namespace {

#define LAUNCH(kern, grid, block, lds, ...) do { \
    hipLaunchKernelGGL(kern, grid, block, lds, stream(), __VA_ARGS__); HIP_CHECK(hipGetLastError()); } while (0)
// The same, timed with the products when per-launch events are being recorded (hip_gemm_profile_enable): `bytes` are the
// HBM bytes the launch has to move at least (the F16 targets it reads and writes; operand transposes move none that the
// step's arithmetic asks for, so their time counts and their bytes do not), `flops` its multiply-adds times two.
#define LAUNCH_TIMED(bytes, flops, kern, grid, block, lds, ...) do { \
    hipEvent_t ev_a_ = nullptr, ev_b_ = nullptr; \
    if (gemm_prof_begin((bytes), (flops), &ev_a_, &ev_b_)) hipExtLaunchKernelGGL(kern, grid, block, lds, stream(), ev_a_, ev_b_, 0, __VA_ARGS__); \
    else hipLaunchKernelGGL(kern, grid, block, lds, stream(), __VA_ARGS__); \
    HIP_CHECK(hipGetLastError()); } while (0)

// in:  tiled [T tokens, F features] fp16, value(t, f) = in[t][f] * in_inv[t]
// out: tiled [F, T] fp16, value(f, t) = out[f][t] * out_inv[f]; zero in the K (token) padding and in
//      rows >= F; out_inv has room for a multiple of 64 entries and gets 0 beyond F.
// One workgroup per block of 64 features; two sweeps over the tokens (row maxima, then the data).
__device__ __forceinline__ void transpose_scaled_block(const half8 *__restrict__ in, const float *__restrict__ in_inv,
                                                       int T, int F, half8 *__restrict__ out, float *__restrict__ out_inv, int fb)
{
    __shared__ float amax[64], scl[64];
    __shared__ half_t t[64][72];
    const int tid = threadIdx.x;
    const int KbIn = tiled_kb(F), TbIn = tiled_rb(T), KbOut = tiled_kb(T), FbOut = tiled_rb(F);
    if (tid < 64) amax[tid] = 0.f;
    __syncthreads();
    {
        // Requests in batches of four token blocks, none under a condition (indices clamped, the factor of a token that
        // does not exist is 0): loads under a bounds test are waited for one at a time.  Per-thread maxima first, then
        // one LDS atomic per feature.
        const int j = tid >> 6, lp = tid & 63, f0 = (lp >> 5) * 32 + 8 * j;
        float lm[8];
#pragma unroll
        for (int e = 0; e < 8; e++) lm[e] = 0.f;
        for (int tb0 = 0; tb0 < TbIn; tb0 += 4) {
            half8 hb[4]; float sb[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int tb = tb0 + u, token = tb * 32 + (lp & 31);
                hb[u] = in[((size_t)min(tb, TbIn - 1) * KbIn + fb) * 256 + (tid & ~63) + a_lane(tid & 63)];
                sb[u] = in_inv[min(token, T - 1)];
                if (token >= T) sb[u] = 0.f;
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int e = 0; e < 8; e++) lm[e] = fmaxf(lm[e], fabsf(h2f(hb[u][e]) * sb[u]));
        }
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (lm[e] > 0.f) atomicMax(reinterpret_cast<unsigned *>(&amax[f0 + e]), __float_as_uint(lm[e]));
    }
    __syncthreads();
    if (tid < 64) {
        const int f = fb * 64 + tid;
        const float s = f < F ? row_scale_for(amax[tid]) : 0.f;
        scl[tid] = s;
        out_inv[f] = f < F ? 1.0f / s : 0.f;
    }
    __syncthreads();
    // thread tid handles the quarter-tile slots q = tid (token half 0) and q = tid + 256 (token half 1) of every K step
    const int j = tid >> 6, lp = tid & 63, f0 = (lp >> 5) * 32 + 8 * j;
    auto request = [&](int tb2, half8 (&h)[2], float (&sc)[2]) {
#pragma unroll
        for (int th = 0; th < 2; th++) {
            const int tile = tb2 * 2 + th, token = tb2 * 64 + th * 32 + (lp & 31);
            h[th] = in[((size_t)min(tile, TbIn - 1) * KbIn + fb) * 256 + (tid & ~63) + a_lane(tid & 63)];
            sc[th] = in_inv[min(token, T - 1)];
            if (tile >= TbIn || token >= T) { sc[th] = 0.f; h[th] = half8{0, 0, 0, 0, 0, 0, 0, 0}; }
        }
    };
    half8 h[2], hn[2];
    float sc[2], scn[2];
    request(0, h, sc);
    for (int tb2 = 0; tb2 < KbOut; tb2++) {
#pragma unroll
        for (int th = 0; th < 2; th++) {
            const int tl = th * 32 + (lp & 31);
#pragma unroll
            for (int e = 0; e < 8; e++) t[tl][f0 + e] = f2h(h2f(h[th][e]) * sc[th] * scl[f0 + e]);
        }
        __syncthreads();
        request(min(tb2 + 1, KbOut - 1), hn, scn);            // the next step's tiles travel while this one is written out
#pragma unroll
        for (int th = 0; th < 2; th++) {
            const int rowtile = fb * 2 + th;
            if (rowtile >= FbOut) continue;
            const int fl = th * 32 + (lp & 31), k0 = (lp >> 5) * 32 + 8 * j;
            half8 o;
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] = t[k0 + e][fl];
            out[((size_t)rowtile * KbOut + tb2) * 256 + tid] = o;
        }
        __syncthreads();
#pragma unroll
        for (int th = 0; th < 2; th++) { h[th] = hn[th]; sc[th] = scn[th]; }
    }
}

__global__ __launch_bounds__(256) void k_transpose_scaled(const half8 *__restrict__ in, const float *__restrict__ in_inv,
                                                           int T, int F, half8 *__restrict__ out, float *__restrict__ out_inv)
{
    transpose_scaled_block(in, in_inv, T, F, out, out_inv, blockIdx.x);
}

// Both operands of one weight gradient in one launch: the first nb0 workgroups transpose job 0, the rest job 1.
struct TransposeJob { const half8 *in; const float *in_inv; int F; half8 *out; float *out_inv; };
__global__ __launch_bounds__(256) void k_transpose_scaled_pair(TransposeJob j0, TransposeJob j1, int T, int nb0)
{
    const bool first = (int)blockIdx.x < nb0;             // uniform per workgroup
    const TransposeJob &j = first ? j0 : j1;
    transpose_scaled_block(j.in, j.in_inv, T, j.F, j.out, j.out_inv, first ? blockIdx.x : blockIdx.x - nb0);
}

// Up to eight operands in one launch (both operands of the four weight gradients of a layer): workgroup id -> job by the
// jobs' first ids.
struct TransposeJobs { TransposeJob j[8]; int first[9]; int n; };
__global__ __launch_bounds__(256) void k_transpose_scaled_jobs(TransposeJobs js, int T)
{
    int k = 0;
#pragma unroll
    for (int i = 1; i < 8; i++) if (i < js.n && (int)blockIdx.x >= js.first[i]) k = i;      // uniform per workgroup
    const TransposeJob &j = js.j[k];
    transpose_scaled_block(j.in, j.in_inv, T, j.F, j.out, j.out_inv, blockIdx.x - js.first[k]);
}

// Target[m][n] (tiled [M_out, N_in] F16) <- half(float(Target) + alpha * sum_t Y[t][m] X[t][n])
// with XT = tiled [N_in, T], YT = tiled [M_out, T] and their row factors.  SGD: alpha = -lr, else 1.
// grid: x = ceil(Kb / 4) (each wave one 64-wide column block), y = ceil(Mb / 2); block 256.
// The MFMA's first operand supplies the rows of its result, so feeding X there puts four
// consecutive n into each lane's registers: exactly the 8-byte groups of the tiled target.
// One to four weight gradients per launch (the four matrices of a layer in accumulate mode).  Workgroup ids go to the
// eight XCDs in turn; an XCD takes a contiguous share of the list of (matrix, row pair, column group) items, so the
// workgroups that read the same two row blocks of Y^T run on one XCD, one after the other, and fetch them into one L2
// instead of one each.
struct WgradJob { const half8 *XT; const float *x_inv; const half8 *YT; const float *y_inv; half_t *target; int M_out, N_in; };
struct WgradJobs { WgradJob j[4]; int first[5]; int n; };

template <int SGD>
__global__ __launch_bounds__(256) void k_wgrad(WgradJobs js, int Kt, float lr)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l31 = lane & 31, h = lane >> 5;
    const int total = js.first[js.n], per_xcd = (total + 7) >> 3;
    int item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (item >= total || (int)(blockIdx.x >> 3) >= per_xcd) return;
    int k = 0;
#pragma unroll
    for (int i = 1; i < 4; i++) if (i < js.n && item >= js.first[i]) k = i;                  // uniform per workgroup
    item -= js.first[k];
    const half8 *__restrict__ XT = js.j[k].XT, *__restrict__ YT = js.j[k].YT;
    const float *__restrict__ x_inv = js.j[k].x_inv, *__restrict__ y_inv = js.j[k].y_inv;
    half_t *__restrict__ target = js.j[k].target;
    const int M_out = js.j[k].M_out, N_in = js.j[k].N_in;
    const int KbG = tiled_kb(N_in), MbG = tiled_rb(M_out), NbX = tiled_rb(N_in);
    const int gx = (KbG + 3) >> 2;
    const int nk = (item % gx) * 4 + wave, mb0 = (item / gx) * 2;
    const bool active = nk < KbG;                         // a wave past the last column block still fetches its share of Y
    const half8 *xp[2], *yp[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        xp[i] = XT + (size_t)min(nk * 2 + i, NbX - 1) * Kt * 256 + lane;
        yp[i] = YT + (size_t)min(mb0 + i, MbG - 1) * Kt * 256 + lane;
    }
    float16v acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;
    // The four waves of a workgroup multiply the same two row blocks of Y^T: each fetches a quarter of them (block
    // wave & 1, MFMA slices 2 (wave >> 1) and + 1) and they exchange through LDS, double buffered, one barrier per step.
    __shared__ half8 ysh[2][2][4][64];
    auto contract_tokens = [&]() {
        const int yi = wave & 1, yj = (wave >> 1) * 2;
        for (int kt = 0; kt < Kt; kt++) {
            const size_t o = (size_t)kt * 256;
            half8 x[2][4], y[2][4];
            const half8 ya = yp[yi][o + yj * 64], yb = yp[yi][o + (yj + 1) * 64];
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 2; i++) x[i][j] = xp[i][o + j * 64];
            ysh[kt & 1][yi][yj][lane] = ya;
            ysh[kt & 1][yi][yj + 1][lane] = yb;
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 2; i++) y[i][j] = ysh[kt & 1][i][j][lane];
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int mt = 0; mt < 2; mt++)
#pragma unroll
                    for (int nh = 0; nh < 2; nh++)
                        acc[mt][nh] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[nh][j], y[mt][j], acc[mt][nh], 0, 0, 0);
        }
    };
    if (active && (mb0 + 2) * 32 <= M_out && nk * 64 + 64 <= N_in) {
        // Block inside the matrix: everything the read-modify-write needs is requested at once, before the contraction
        // (whose loads it then travels with), then computed, then stored.  With the bounds tests of the general path
        // below between them, each of the wave's sixteen load-update-store groups waits for the one before it.
        float sy[2];
        float4 xi[2][4];
        half4 g[2][2][4];
        half4 *gp[2][2][4];
#pragma unroll
        for (int mt = 0; mt < 2; mt++) sy[mt] = y_inv[(mb0 + mt) * 32 + l31];
#pragma unroll
        for (int nh = 0; nh < 2; nh++)
#pragma unroll
            for (int j4 = 0; j4 < 4; j4++) xi[nh][j4] = *reinterpret_cast<const float4 *>(x_inv + nk * 64 + nh * 32 + 8 * j4 + 4 * h);
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
            for (int nh = 0; nh < 2; nh++)
#pragma unroll
                for (int j4 = 0; j4 < 4; j4++) {
                    gp[mt][nh][j4] = reinterpret_cast<half4 *>(
                        target + ((((size_t)(mb0 + mt) * KbG + nk) * 4 + j4) * 64 + nh * 32 + l31) * 8 + 4 * h);
                    g[mt][nh][j4] = __builtin_nontemporal_load(gp[mt][nh][j4]);     // touched once per launch: past the caches, which hold the operands
                }
        contract_tokens();
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
            for (int nh = 0; nh < 2; nh++)
#pragma unroll
                for (int j4 = 0; j4 < 4; j4++) {
                    const float xs[4] = {xi[nh][j4].x, xi[nh][j4].y, xi[nh][j4].z, xi[nh][j4].w};
                    half4 o = g[mt][nh][j4];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float a = acc[mt][nh][4 * j4 + i] * sy[mt] * xs[i];
                        o[i] = SGD ? f2h(h2f(o[i]) - lr * a) : f2h(h2f(o[i]) + a);
                    }
                    __builtin_nontemporal_store(o, gp[mt][nh][j4]);
                }
        return;
    }
    contract_tokens();
    if (!active) return;
#pragma unroll
    for (int mt = 0; mt < 2; mt++) {
        const int m = (mb0 + mt) * 32 + l31;
        if (mb0 + mt >= MbG || m >= M_out) continue;
        const float sy = y_inv[m];
#pragma unroll
        for (int nh = 0; nh < 2; nh++)
#pragma unroll
            for (int j4 = 0; j4 < 4; j4++) {
                const int n0 = nk * 64 + nh * 32 + 8 * j4 + 4 * h;
                if (n0 >= N_in) continue;
                const size_t addr = ((((size_t)(mb0 + mt) * KbG + nk) * 4 + j4) * 64 + nh * 32 + l31) * 8 + 4 * h;
                half4 g = *reinterpret_cast<half4 *>(target + addr);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    if (n0 + i >= N_in) continue;
                    const float a = acc[mt][nh][4 * j4 + i] * sy * x_inv[n0 + i];
                    g[i] = SGD ? f2h(h2f(g[i]) - lr * a) : f2h(h2f(g[i]) + a);        // contraction is off in this file
                }
                *reinterpret_cast<half4 *>(target + addr) = g;
            }
    }
}

// 64 x 64 blocks of W (tiled [Mo, Ni]):  if G: W = half(W - lr * G), G = 0 (f16_sgd_apply);
// then the block is written, transposed, into WT (tiled [Ni, Mo]).
// grid: x = K blocks of W, y = ceil(row tiles / 2), z = matrices of this shape (the layers of an arena, st / stT half8
// apart in W and G / in WT); block 256.
__global__ __launch_bounds__(256) void k_apply_retile(half8 *__restrict__ W, half8 *__restrict__ G, half8 *__restrict__ WT,
                                                       int Mo, int Ni, float lr, size_t st, size_t stT)
{
    __shared__ half_t t[64][72];
    const int tid = threadIdx.x, bx = blockIdx.x, by = blockIdx.y;
    W += blockIdx.z * st; WT += blockIdx.z * stT;
    if (G) G += blockIdx.z * st;
    const int KbW = tiled_kb(Ni), MbW = tiled_rb(Mo), KbT = tiled_kb(Mo), NbT = tiled_rb(Ni);
    // both 32-row tiles of the block: their loads are issued together (one memory round trip for the thread's two pieces)
    half8 w[2], g[2];
    size_t at[2];
#pragma unroll
    for (int th = 0; th < 2; th++) {
        const int mbt = by * 2 + th;
        at[th] = ((size_t)min(mbt, MbW - 1) * KbW + bx) * 256 + tid;
        w[th] = half8{0, 0, 0, 0, 0, 0, 0, 0}; g[th] = w[th];
        if (mbt < MbW) {
            w[th] = __builtin_nontemporal_load(&W[at[th]]);
            if (G) g[th] = __builtin_nontemporal_load(&G[at[th]]);
        }
    }
#pragma unroll
    for (int th = 0; th < 2; th++) {
        const int mbt = by * 2 + th;
        const int j = tid >> 6, lp = tid & 63, ml = th * 32 + (lp & 31), n0 = (lp >> 5) * 32 + 8 * j;
        if (mbt < MbW && G) {
#pragma unroll
            for (int e = 0; e < 8; e++) w[th][e] = f2h(h2f(w[th][e]) - lr * h2f(g[th][e]));   // two roundings: contraction is off
            __builtin_nontemporal_store(w[th], &W[at[th]]);
            const half8 z = {0, 0, 0, 0, 0, 0, 0, 0};
            __builtin_nontemporal_store(z, &G[at[th]]);
        }
#pragma unroll
        for (int e = 0; e < 8; e++) t[ml][n0 + e] = w[th][e];
    }
    __syncthreads();
    for (int q = tid; q < 512; q += 256) {
        const int th = q >> 8, qq = q & 255, nbt = bx * 2 + th;
        if (nbt >= NbT) continue;
        const int j = qq >> 6, lp = qq & 63, nl = th * 32 + (lp & 31), m0 = (lp >> 5) * 32 + 8 * j;
        half8 o;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = t[m0 + e][nl];
        __builtin_nontemporal_store(o, &WT[((size_t)nbt * KbT + by) * 256 + qq]);
    }
}

// dst row-major F16 [rows, cols] <- tiled image: element (r, c) from tiled(row_off + r, k_off + c),
// or from tiled(row_off + c, k_off + r) when the image holds the transposed matrix.
__global__ void k_untile_f16(const half_t *__restrict__ src, int Kb, int row_off, int k_off, int transpose,
                             int rows, int cols, half_t *__restrict__ dst)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)rows * cols) return;
    const int r = (int)(idx / cols), c = (int)(idx % cols);
    dst[idx] = transpose ? src[tiled_index(row_off + c, k_off + r, Kb)] : src[tiled_index(row_off + r, k_off + c, Kb)];
}

}  // namespace

namespace lmhip {

void launch_transpose_scaled(const half_t *in_tiled, const float *in_inv, int T, int F, half_t *out_tiled, float *out_inv)
{
    if (T <= 0 || F <= 0) return;
    LAUNCH_TIMED(0.0, 0.0, k_transpose_scaled, dim3(tiled_kb(F)), dim3(256), 0, reinterpret_cast<const half8 *>(in_tiled), in_inv, T, F,
           reinterpret_cast<half8 *>(out_tiled), out_inv);
}

void launch_transpose_scaled_pair(const half_t *in0, const float *in0_inv, int F0, half_t *out0, float *out0_inv,
                                  const half_t *in1, const float *in1_inv, int F1, half_t *out1, float *out1_inv, int T)
{
    if (T <= 0 || F0 <= 0 || F1 <= 0) { fprintf(stderr, "[fast_hip] transpose_scaled_pair: empty operand\n"); abort(); }
    const TransposeJob j0{reinterpret_cast<const half8 *>(in0), in0_inv, F0, reinterpret_cast<half8 *>(out0), out0_inv};
    const TransposeJob j1{reinterpret_cast<const half8 *>(in1), in1_inv, F1, reinterpret_cast<half8 *>(out1), out1_inv};
    const int nb0 = tiled_kb(F0);
    LAUNCH_TIMED(0.0, 0.0, k_transpose_scaled_pair, dim3(nb0 + tiled_kb(F1)), dim3(256), 0, j0, j1, T, nb0);
}

void launch_transpose_scaled_jobs(const TransposeOperand *ops, int n, int T)
{
    if (n <= 0 || n > 8 || T <= 0) { fprintf(stderr, "[fast_hip] transpose_scaled_jobs: %d operands\n", n); abort(); }
    TransposeJobs js{};
    js.n = n;
    int total = 0;
    for (int i = 0; i < n; i++) {
        if (ops[i].F <= 0) { fprintf(stderr, "[fast_hip] transpose_scaled_jobs: empty operand\n"); abort(); }
        js.j[i] = TransposeJob{reinterpret_cast<const half8 *>(ops[i].in), ops[i].in_inv, ops[i].F, reinterpret_cast<half8 *>(ops[i].out), ops[i].out_inv};
        js.first[i] = total;
        total += tiled_kb(ops[i].F);
    }
    js.first[n] = total;
    LAUNCH_TIMED(0.0, 0.0, k_transpose_scaled_jobs, dim3(total), dim3(256), 0, js, T);
}

void launch_wgrads(const WgradOperands *w, int n, int T, int sgd, float lr)
{
    if (n <= 0 || n > 4 || T <= 0) { fprintf(stderr, "[fast_hip] wgrads: %d matrices\n", n); abort(); }
    WgradJobs js{};
    js.n = n;
    int total = 0;
    for (int i = 0; i < n; i++) {
        if (w[i].M_out <= 0 || w[i].N_in <= 0) { fprintf(stderr, "[fast_hip] wgrads: empty matrix\n"); abort(); }
        js.j[i] = WgradJob{reinterpret_cast<const half8 *>(w[i].XT), w[i].x_inv, reinterpret_cast<const half8 *>(w[i].YT), w[i].y_inv,
                           w[i].target_tiled, w[i].M_out, w[i].N_in};
        js.first[i] = total;
        total += ((tiled_kb(w[i].N_in) + 3) / 4) * ((tiled_rb(w[i].M_out) + 1) / 2);
    }
    for (int i = n; i <= 4; i++) js.first[i] = total;
    const dim3 grid((total + 7) / 8 * 8);                 // whole rounds of the eight XCDs; k_wgrad maps ids to tiles
    double weights = 0.0;
    for (int i = 0; i < n; i++) weights += (double)w[i].M_out * w[i].N_in;
    // the F16 target is read and written once: 4 bytes per weight
    if (sgd) LAUNCH_TIMED(4.0 * weights, 2.0 * T * weights, k_wgrad<1>, grid, dim3(256), 0, js, tiled_kb(T), lr);
    else     LAUNCH_TIMED(4.0 * weights, 2.0 * T * weights, k_wgrad<0>, grid, dim3(256), 0, js, tiled_kb(T), lr);
}

void launch_wgrad(const half_t *XT, const float *x_inv, const half_t *YT, const float *y_inv, half_t *target_tiled,
                  int M_out, int N_in, int T, int sgd, float lr)
{
    if (M_out <= 0 || N_in <= 0 || T <= 0) return;
    const WgradOperands w{XT, x_inv, YT, y_inv, target_tiled, M_out, N_in};
    launch_wgrads(&w, 1, T, sgd, lr);
}

void launch_apply_retile(half_t *W_tiled, half_t *G_tiled, half_t *WT_tiled, int M_out, int N_in, float lr,
                         int matrices, size_t stride, size_t strideT)
{
    if (M_out <= 0 || N_in <= 0 || matrices <= 0) return;
    if (matrices > 65535 || (stride & 7) || (strideT & 7)) { fprintf(stderr, "[fast_hip] apply_retile: bad strides\n"); abort(); }
    // W read and written, the transposed image written, and with an accumulator G read and cleared: 10 (6) bytes per weight
    const double weights = (double)M_out * N_in * matrices;
    LAUNCH_TIMED((G_tiled ? 10.0 : 6.0) * weights, 0.0, k_apply_retile, dim3(tiled_kb(N_in), (tiled_rb(M_out) + 1) / 2, matrices), dim3(256), 0, reinterpret_cast<half8 *>(W_tiled),
           reinterpret_cast<half8 *>(G_tiled), reinterpret_cast<half8 *>(WT_tiled), M_out, N_in, lr, stride / 8, strideT / 8);
}

void launch_untile_f16(const half_t *src_tiled, int Kb, int row_off, int k_off, int transpose, int rows, int cols, half_t *dst)
{
    const size_t n = (size_t)rows * cols;
    if (!n) return;
    LAUNCH(k_untile_f16, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, src_tiled, Kb, row_off, k_off, transpose, rows, cols, dst);
}

}  // namespace lmhip
