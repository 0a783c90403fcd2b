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
#include "gemm_kernel.h"
#include <hip/hip_ext.h>
#include <vector>
#include <algorithm>

namespace {

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
        out[lmhip::tiled_a_index(row, i, Kb)] = (i < K) ? f2h(x[i] * s) : (half_t)0;
    if (threadIdx.x == 0) inv_scale[row] = 1.0f / s;
}

// The same, keeping 22 bits of every element: row m of the tiled operand holds the fp16 image of x, row M + m the
// fp16 image of what that rounding lost (x - fp16(x s) / s is exact in fp32), each with its own power-of-two scale.
__global__ __launch_bounds__(256) void rows_to_f16_split(
    const float *__restrict__ X, int ldx, half_t *__restrict__ out, float *__restrict__ inv_scale, int M, int K, int Kb)
{
    __shared__ float sm[16];
    const int row = blockIdx.x;
    const float *x = X + (size_t)row * ldx;
    float amax = 0.f;
    for (int i = threadIdx.x; i < K; i += blockDim.x) amax = fmaxf(amax, fabsf(x[i]));
    amax = block_max(amax, sm);
    const float s = row_scale_for(amax), inv = 1.0f / s;
    float lmax = 0.f;
    for (int i = threadIdx.x; i < Kb * 64; i += blockDim.x) {
        const half_t h = (i < K) ? f2h(x[i] * s) : (half_t)0;
        out[lmhip::tiled_a_index(row, i, Kb)] = h;
        if (i < K) lmax = fmaxf(lmax, fabsf(x[i] - h2f(h) * inv));
    }
    lmax = block_max(lmax, sm);
    const float s2 = row_scale_for(lmax);
    for (int i = threadIdx.x; i < Kb * 64; i += blockDim.x) {
        half_t l = (half_t)0;
        if (i < K) { const half_t h = f2h(x[i] * s); l = f2h((x[i] - h2f(h) * inv) * s2); }
        out[lmhip::tiled_a_index(M + row, i, Kb)] = l;
    }
    if (threadIdx.x == 0) { inv_scale[row] = inv; inv_scale[M + row] = 1.0f / s2; }
}

// The same for rows a workgroup of 1024 threads can hold in registers (K <= 8192 * CPT, K % 4 == 0, X 16-byte aligned):
// a thread owns CPT chunks of 8 consecutive elements, each one 16-byte store into the tiled image, and the row is read
// once.  Same values as rows_to_f16_split.
template <int CPT>
__global__ __launch_bounds__(1024) void rows_to_f16_split_vec(
    const float *__restrict__ X, int ldx, half_t *__restrict__ out, float *__restrict__ inv_scale, int M, int K, int Kb)
{
    __shared__ float sm[16];
    typedef _Float16 half8 __attribute__((ext_vector_type(8)));
    const int row = blockIdx.x;
    const float *x = X + (size_t)row * ldx;
    float v[CPT][8];
    float amax = 0.f;
#pragma unroll
    for (int u = 0; u < CPT; u++) {
        const int k0 = (threadIdx.x + 1024 * u) * 8;
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
        if (k0 < K) a = *reinterpret_cast<const float4 *>(x + k0);
        if (k0 + 4 < K) b = *reinterpret_cast<const float4 *>(x + k0 + 4);
        v[u][0] = a.x; v[u][1] = a.y; v[u][2] = a.z; v[u][3] = a.w; v[u][4] = b.x; v[u][5] = b.y; v[u][6] = b.z; v[u][7] = b.w;
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[u][e]));
    }
    amax = block_max(amax, sm);
    const float s = row_scale_for(amax), inv = 1.0f / s;
    float lmax = 0.f;
#pragma unroll
    for (int u = 0; u < CPT; u++) {
        const int k0 = (threadIdx.x + 1024 * u) * 8;
        half8 h;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            h[e] = f2h(v[u][e] * s);
            v[u][e] = v[u][e] - h2f(h[e]) * inv;                            // what the rounding lost, exact in fp32
            lmax = fmaxf(lmax, fabsf(v[u][e]));
        }
        if (k0 < Kb * 64) *reinterpret_cast<half8 *>(out + lmhip::tiled_a_index(row, k0, Kb)) = h;
    }
    lmax = block_max(lmax, sm);
    const float s2 = row_scale_for(lmax);
#pragma unroll
    for (int u = 0; u < CPT; u++) {
        const int k0 = (threadIdx.x + 1024 * u) * 8;
        half8 l;
#pragma unroll
        for (int e = 0; e < 8; e++) l[e] = f2h(v[u][e] * s2);
        if (k0 < Kb * 64) *reinterpret_cast<half8 *>(out + lmhip::tiled_a_index(M + row, k0, Kb)) = l;
    }
    if (threadIdx.x == 0) { inv_scale[row] = inv; inv_scale[M + row] = 1.0f / s2; }
}

// pseudo-random fp16 values in (-1, 1) for the timing entry points: constant operands would flatter the matrix cores,
// whose power (and with it the clock the GPU holds) depends on how many operand bits toggle
__global__ void fill_random_f16(half_t *p, size_t n, uint32_t seed)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint32_t x = (uint32_t)i * 2654435761u ^ seed;
    x ^= x >> 15; x *= 2246822519u; x ^= x >> 13; x *= 3266489917u; x ^= x >> 16;
    p[i] = (half_t)(((int)(x & 0xffff) - 32768) * (1.0f / 32768.0f));
}

// C[m, n] = sum over planes of row m and of row M + m, each times its row factor
__global__ void reduce_planes_split(const float *__restrict__ P, int S, size_t plane_stride, int ldp,
                                    const float *__restrict__ row_scale, float *__restrict__ C, int M, int N)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)M * N) return;
    const int m = (int)(idx / N), n = (int)(idx % N);
    C[idx] = lmhip::split_planes_value(P, S, plane_stride, ldp, row_scale, M, m, n);
}

__global__ void reduce_planes(const float *__restrict__ P, int S, size_t plane_stride, int ldp,
                              const float *__restrict__ row_scale, float *__restrict__ C, int M, int N)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)M * N) return;
    const int m = (int)(idx / N), n = (int)(idx % N);
    float s = 0.f;
    for (int p = 0; p < S; p++) s += P[p * plane_stride + (size_t)m * ldp + n];
    C[idx] = row_scale ? s * row_scale[m] : s;
}

// F16 tile image of a Q8_0 (or mixed Q8_0 / F16) weight operand: one wave per 32 x 64 tile loads the tile the way
// the streaming GEMM does (codes unpacked and scaled in registers, F16 tiles as they are) and stores the four operand
// vectors of every lane at the tile's place in a plain F16 operand, out[(nb * Kb + kt) * 256 + j * 64 + lane].
// f16_only: only the tiles that are F16 in W (adapter rows of a fused matrix) are copied; the rest of `out` is kept.
__global__ __launch_bounds__(256) void q8_operand_to_f16(lmhip::WeightOp W, int Nb, int Kb, half8 *__restrict__ out, int f16_only)
{
    const int lane = threadIdx.x & 63;
    const size_t t = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    int nb, kt;
    if (!f16_only) {
        if (t >= (size_t)Nb * Kb) return;
        nb = (int)(t / Kb); kt = (int)(t % Kb);
    } else if (W.fmt == 1) {                               // the row blocks from nbq on
        if (t >= (size_t)(Nb - W.nbq) * Kb) return;
        nb = W.nbq + (int)(t / Kb); kt = (int)(t % Kb);
    } else {                                              // the K steps from kbq on, of every row block
        const int kf = Kb - W.kbq;
        if (kf <= 0 || t >= (size_t)Nb * kf) return;
        nb = (int)(t / kf); kt = W.kbq + (int)(t % kf);
    }
    const size_t tile = (size_t)nb * Kb + kt;
    half8 w[4];
    if (W.fmt == 1) {
        if (nb < W.nbq) lmhip::load_w_q8_rows(w, W, nb, Kb, kt, lane);
        else lmhip::load_w_f16(w, W.w16, nb - W.nbq, Kb, kt, lane);
    } else {
        if (kt < W.kbq) lmhip::load_w_q8_cols(w, W, nb, W.kbq, kt, lane);
        else lmhip::load_w_f16(w, W.w16, nb, Kb - W.kbq, kt - W.kbq, lane);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) out[tile * 256 + j * 64 + lane] = w[j];
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

// Q8_0 blocks (34 bytes: fp16 scale, 32 int8; row-major [rows][cols/32]) -> GEMM tiles, see WeightOp in gemm.h.
// One thread per source block.
__global__ __launch_bounds__(256) void tile_q8(const uint8_t *__restrict__ blocks, int rows, int nbk,
                                                uint8_t *__restrict__ qt, half_t *__restrict__ dt, int Kb_dst,
                                                int row_off, int k_off, int transpose)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)rows * nbk) return;
    const int r = (int)(idx / nbk), b = (int)(idx % nbk);
    const uint8_t *p = blocks + idx * 34;
    const half_t d = __builtin_bit_cast(half_t, (uint16_t)(p[0] | (p[1] << 8)));
    for (int i = 0; i < 32; i++) {
        const int c = b * 32 + i;
        const int R = transpose ? row_off + c : row_off + r, Kc = transpose ? k_off + r : k_off + c;
        const size_t tile = (size_t)(R >> 5) * Kb_dst + (Kc >> 6);
        const int cc = Kc & 63, j = (cc & 31) >> 3, lane = (cc >> 5) * 32 + (R & 31);
        qt[((tile * 2 + (j >> 1)) * 64 + lane) * 16 + (j & 1) * 8 + (cc & 7)] = p[2 + i];
        if (transpose && i == 0) dt[tile * 64 + cc] = d;            // one scale per (column Kc, 32-row block)
    }
    if (!transpose) {
        const int R = row_off + r, Kc = k_off + b * 32;
        const size_t tile = (size_t)(R >> 5) * Kb_dst + (Kc >> 6);
        dt[tile * 64 + ((Kc >> 5) & 1) * 32 + (R & 31)] = d;
    }
}

// Row-major F16 copy of a window of a Q8_0 tiled operand: dst[r][c] = half(d * q) of tiled element
// (row_off + r, k_off + c), or (row_off + c, k_off + r) when transposed.  fmt as in WeightOp.
__global__ void untile_q8(const uint8_t *__restrict__ qt, const half_t *__restrict__ dt, int fmt, int Kb,
                          int row_off, int k_off, int transpose, int rows, int cols, half_t *__restrict__ dst)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)rows * cols) return;
    const int r = (int)(idx / cols), c = (int)(idx % cols);
    const int R = transpose ? row_off + c : row_off + r, Kc = transpose ? k_off + r : k_off + c;
    const size_t tile = (size_t)(R >> 5) * Kb + (Kc >> 6);
    const int cc = Kc & 63, j = (cc & 31) >> 3, lane = (cc >> 5) * 32 + (R & 31);
    const int8_t q = (int8_t)qt[((tile * 2 + (j >> 1)) * 64 + lane) * 16 + (j & 1) * 8 + (cc & 7)];
    const half_t d = fmt == 1 ? dt[tile * 64 + lane] : dt[tile * 64 + cc];
    dst[idx] = (half_t)__fmul_rn(h2f(d), (float)q);
}

struct ProfRec { hipEvent_t a, b; double wbytes, flops; };
// Events that ride on a dispatch to time it release to the device only: the default (a release to the system, for a host
// that reads results after the event) makes every timed kernel end with a write-back of all of L2 to system scope, which
// the untimed step does not do -- the timed products ran 1.4 us longer each than the same products in a kernel trace.
constexpr unsigned PROF_EVENT_FLAGS = hipEventReleaseToDevice;
int g_prof_on = 0;
std::vector<ProfRec> g_prof;
int g_force_nb = 0, g_force_S = 0;
int g_wide_wg = 1;                     // eight-wave workgroups where K would be cut into ten or more chunks
int g_ring = 1;                        // gemm_ring for one-tile products (F16 or Q8_0 weights)
int g_ring_wide = 1;                   // gemm_ring_wide where the product has enough row tiles for it

}  // namespace

namespace lmhip {

// Tile height and K split, from measurements on MI355X at M = 64: two 32-row blocks per wave
// (activation bytes through L1/L2 = weight bytes), about three workgroups per CU, chunks of at
// least 4 and at most 40 K steps (long chunks gain nothing and short ones spread the
// activation reads over more L2 lines); beyond that, splitting K only adds plane traffic.
// K chunks for gemm_ring.  Measured on MI355X (256 CUs; Qwen3-4B and Gemma3-1B layer shapes at 64 rows, cold weights):
// the launch is fastest when every CU has the same number of workgroups — one for up to 256 of them, two for up to 512
// (64 KB of LDS each) — and loses when some CUs have one more than others (320 workgroups: 9.2 us against 8.1 for 240
// on 2560 x 4096) or when not all are resident at once (beyond 512).  Among equally balanced splits the one with fewer
// planes wins: a plane costs the product its stores and the consumer its loads (the more the shorter K is).
static int ring_chunks(int n_tiles, int Kb, int K, int cus)
{
    int best = 1;
    double best_score = -1e9;
    for (int S = 1; S <= 32 && S <= Kb; S++) {
        const int steps = (Kb + S - 1) / S;
        if ((Kb + steps - 1) / steps != S) continue;       // this S does not exist (the last chunk would be empty)
        const long wgs = (long)n_tiles * S;
        const long slots = wgs <= 2L * cus ? cus : 2L * cus;
        double eff = (double)wgs / (double)(slots * ((wgs + slots - 1) / slots));
        if (wgs > 2L * cus) eff *= 0.85;
        const double score = eff - 0.05 * S * (K > 2560 ? 2560.0 / K : 1.0);
        if (score > best_score + 1e-9) { best_score = score; best = S; }
    }
    return best;
}

GemmPlan plan_gemm(int M, int N, int K, int nbq, int fmt)
{
    const int Kb = tiled_kb(K), Nb = tiled_rb(N), m_tiles = (M + 63) / 64;
    const int cus = num_cus() > 0 ? num_cus() : 256;
    GemmPlan p{};
    p.nw = 4;
    p.m_tiles = m_tiles;
    if (g_ring && m_tiles == 1 && !g_force_nb) {            // any weight format: Q8_0 tiles travel through the ring quantised
        p.ring = 1; p.kg = 2; p.nw = 8; p.nb = 2;
        p.n_tiles = (Nb + 1) / 2;
        const int S = g_force_S ? std::min(g_force_S, Kb) : ring_chunks(p.n_tiles, Kb, K, cus);
        p.steps = (Kb + S - 1) / S;
        p.S = (Kb + p.steps - 1) / p.steps;
        p.rotate = 0;
        // four weight row blocks per workgroup (up to three workgroups per CU) with the same K chunks, when every CU
        // still gets such a workgroup (with 0.9 of them -- 9728 x 2560 and 6176 x 2560 in three and five chunks -- the
        // products alone gain 2-7 %, the step nothing with F16 weights and it loses 1 % with Q8_0); more than 32 rows: with one
        // activation block (20 KB stages, two waves requesting nothing) batched generation on a training state's tiles
        // took 3.66 instead of 3.63 ms per step of eight tokens
        if (g_ring_wide && M > 32 && (!g_force_S || g_ring_wide == 2)) {
            const int nt4 = (Nb + 3) / 4;
            bool wide = g_ring_wide == 2 || (long)nt4 * p.S >= (long)cus;
            // under a long K twice the chunks, up to 16, cost little: the planes stay a few percent of the weights.  The
            // lm_head backward (2560 x 151936: 157 -> 139 us alone; with 28 chunks on 1152 x 262144 it loses, 122 -> 126 us),
            // and with F16 weights the down forward and the gate|up backward (K = 9728, 19456; six -> twelve chunks: the
            // step 7.17 -> 7.09 ms; from K = 4096 on the same; with Q8_0 weights the step loses 0.4 %)
            if (!wide && !g_force_S && K >= (fmt == 0 ? 8192 : 32768) && 2 * p.S <= 16) {
                const int steps2 = (Kb + 2 * p.S - 1) / (2 * p.S), S2 = (Kb + steps2 - 1) / steps2;
                if ((long)nt4 * S2 >= (long)cus * 7 / 8) { wide = true; p.steps = steps2; p.S = S2; }
            }
            if (wide) { p.wide = 1; p.nb = 4; p.kg = 1; p.nw = 8; p.n_tiles = nt4; }
        }
        return p;
    }
    auto split = [&](int nb) {
        p.nb = nb;
        p.n_tiles = (Nb + nb - 1) / nb;
        const int base = p.n_tiles * m_tiles;
        // about twelve waves per CU in flight, whatever the workgroup size
        int S = g_force_S ? g_force_S : (12 * cus / p.nw + base - 1) / base;
        if (S < 1) S = 1;
        int steps = (Kb + S - 1) / S;
        if (!g_force_S) {
            if (steps < p.nw) steps = p.nw;
            if (steps > 10 * p.nw) steps = 10 * p.nw;
        }
        steps = (steps + p.nw - 1) / p.nw * p.nw;          // whole steps for each wave
        if (steps > Kb) steps = Kb;
        p.steps = steps;
        p.S = (Kb + steps - 1) / steps;
    };
    int nb = g_force_nb ? g_force_nb : (Nb >= 2 ? 2 : 1);
    if (nbq & 1) nb = 1;                                   // a workgroup must not straddle the Q8_0 / F16 boundary
    split(nb);
    // a product too small to give every CU a workgroup of 64 weight rows (K is short as well) takes 32-row workgroups:
    // measured on 1152 x 1024 .. 1568 x 1152 at 64 rows, 4.3-4.6 us against 5.2-5.5
    if (!g_force_nb && p.nb == 2 && m_tiles == 1 && p.n_tiles * p.S < cus) split(1);
    // few weight rows under a long K would be cut into ten or more chunks: eight waves per workgroup split K among
    // themselves instead and leave half as many planes to write and to add
    if (g_wide_wg && !g_force_S && m_tiles == 1 && p.S >= 20) { p.nw = 8; split(p.nb); }
    // rotate the K order unless the activation matrix is too big to stay in an XCD's L2
    p.rotate = (size_t)tiled_rb(M) * 32 * Kb * 64 * 2 <= (size_t)4 << 20;
    return p;
}

void launch_gemm(const half_t *A, const float *a_inv_scale, const WeightOp &W,
                 float *P, int ldp, size_t plane_stride, int M, int N, int K, const GemmPlan &p, float half_scale)
{
    if (half_scale != 0.f && (!p.ring || a_inv_scale)) { fprintf(stderr, "[fast_hip] gemm: half planes need a ring plan without row factors\n"); abort(); }
    if (M <= 0 || N <= 0 || K <= 0) return;
    const int Kb = tiled_kb(K), Nb = tiled_rb(N), Mb = tiled_rb(M);
    bool ok = ldp >= N && p.S >= 1 && p.steps >= 1 && (p.nb == 1 || p.nb == 2 || (p.ring && p.wide && p.nb == 4)) &&
              (p.nw == 4 || (p.nw == 8 && p.m_tiles == 1)) && W.fmt >= 0 && W.fmt <= 2;
    if (W.fmt == 0) ok = ok && W.w16;
    if (W.fmt == 1) ok = ok && W.q && W.d && W.nbq >= 0 && W.nbq <= Nb && (W.nbq == Nb || (W.w16 && (p.ring || (W.nbq % p.nb) == 0)));
    if (W.fmt == 2) ok = ok && W.q && W.d && W.kbq >= 0 && W.kbq <= Kb && (W.kbq == Kb || W.w16);
    if (!ok) {
        fprintf(stderr, "[fast_hip] gemm: bad launch M=%d N=%d K=%d ldp=%d fmt=%d nbq=%d kbq=%d plan(nb=%d S=%d steps=%d)\n",
                M, N, K, ldp, W.fmt, W.nbq, W.kbq, p.nb, p.S, p.steps);
        abort();
    }
    if (p.ring) {
        if (p.m_tiles != 1 || M > 64 || (p.kg != 1 && p.kg != 2 && p.kg != 4) || p.n_tiles != (p.wide ? (Nb + 3) / 4 : (Nb + 1) / 2) ||
            (p.wide && (p.kg != 1 || M <= 32)) ||
            (long)p.S * p.steps < Kb || (long)(p.S - 1) * p.steps >= Kb || (W.fmt != 0 && ((!p.wide && p.kg != 2) || (half_scale != 0.f && a_inv_scale)))) {
            fprintf(stderr, "[fast_hip] gemm_ring: bad launch M=%d N=%d K=%d fmt=%d plan(kg=%d S=%d steps=%d tiles=%d)\n", M, N, K, W.fmt, p.kg, p.S, p.steps, p.n_tiles);
            abort();
        }
        ProfRec rrec{};
        hipEvent_t ra = nullptr, rb = nullptr;
        if (g_prof_on) {
            HIP_CHECK(hipEventCreateWithFlags(&rrec.a, PROF_EVENT_FLAGS)); HIP_CHECK(hipEventCreateWithFlags(&rrec.b, PROF_EVENT_FLAGS));
            rrec.wbytes = weight_stream_bytes(W, N, K); rrec.flops = 2.0 * M * N * K;
            ra = rrec.a; rb = rrec.b;
        }
        GemmKArgs g{};
        g.A = reinterpret_cast<const half8 *>(A); g.a_inv_scale = a_inv_scale; g.W = W;
        g.P = P; g.ldp = ldp; g.plane_stride = plane_stride;
        g.M = M; g.N = N; g.Mb = Mb; g.Nb = Nb; g.Kb = Kb; g.steps_per_chunk = p.steps;
        g.n_tiles = p.n_tiles; g.S = p.S; g.m_tiles = 1; g.half_scale = half_scale; g.w16_ring = W.w16;
        const dim3 rgrid((unsigned)(p.n_tiles * p.S)), rblock(p.wide ? 512 : 256 * p.kg);
        if (p.wide) {
#define WIDE_LAUNCH(SC, HP, WFV) launch_kargs<24>(gemm_ring_wide<SC, HP, WFV>, rgrid, rblock, 0, stream(), g, g_prof_on ? ra : nullptr, g_prof_on ? rb : nullptr)
#define WIDE_PICK(WFV) do { if (a_inv_scale) WIDE_LAUNCH(1, 0, WFV); else if (half_scale != 0.f) WIDE_LAUNCH(0, 1, WFV); else WIDE_LAUNCH(0, 0, WFV); } while (0)
            if (W.fmt == 1) WIDE_PICK(1); else if (W.fmt == 2) WIDE_PICK(2); else WIDE_PICK(0);
#undef WIDE_PICK
#undef WIDE_LAUNCH
            HIP_CHECK(hipGetLastError());
            if (g_prof_on) g_prof.push_back(rrec);
            return;
        }
#define RING_LAUNCH(KGV, SC, HP) launch_kargs<24>(gemm_ring<KGV, SC, HP>, rgrid, rblock, 0, stream(), g, g_prof_on ? ra : nullptr, g_prof_on ? rb : nullptr)
#define RING_PICK(KGV) do { if (a_inv_scale) RING_LAUNCH(KGV, 1, 0); else if (half_scale != 0.f) RING_LAUNCH(KGV, 0, 1); else RING_LAUNCH(KGV, 0, 0); } while (0)
#define RING_LAUNCH_Q8(SC, HP, WFV) launch_kargs<24>(gemm_ring<2, SC, HP, WFV>, rgrid, rblock, 0, stream(), g, g_prof_on ? ra : nullptr, g_prof_on ? rb : nullptr)
        if (W.fmt == 1) { if (a_inv_scale) RING_LAUNCH_Q8(1, 0, 1); else if (half_scale != 0.f) RING_LAUNCH_Q8(0, 1, 1); else RING_LAUNCH_Q8(0, 0, 1); }
        else if (W.fmt == 2) { if (a_inv_scale) RING_LAUNCH_Q8(1, 0, 2); else if (half_scale != 0.f) RING_LAUNCH_Q8(0, 1, 2); else RING_LAUNCH_Q8(0, 0, 2); }
        else if (p.kg == 1) RING_PICK(1); else if (p.kg == 2) RING_PICK(2); else RING_PICK(4);
#undef RING_LAUNCH_Q8
#undef RING_PICK
#undef RING_LAUNCH
        HIP_CHECK(hipGetLastError());
        if (g_prof_on) g_prof.push_back(rrec);
        return;
    }
    dim3 grid(p.n_tiles, p.S, p.m_tiles), block(p.nw * 64);
    if (p.m_tiles > 1) grid = dim3((unsigned)(((size_t)p.n_tiles * p.S + 7) / 8 * 8 * p.m_tiles), 1, 1);   // see gemm_tiled
    const size_t lds = (size_t)(p.nw / 2) * (2 * p.nb * 16) * 64 * sizeof(float);
    // When profiling, the events ride on the dispatch itself (hipExtLaunchKernelGGL), so their
    // difference is the kernel's own execution time without the gaps a separate record adds.
    ProfRec rec{};
    hipEvent_t ev_a = nullptr, ev_b = nullptr;
    if (g_prof_on) {
        HIP_CHECK(hipEventCreateWithFlags(&rec.a, PROF_EVENT_FLAGS));
        HIP_CHECK(hipEventCreateWithFlags(&rec.b, PROF_EVENT_FLAGS));
        rec.wbytes = weight_stream_bytes(W, N, K);
        rec.flops = 2.0 * M * N * K;
        ev_a = rec.a; ev_b = rec.b;
    }
    GemmKArgs g{};
    g.A = reinterpret_cast<const half8 *>(A); g.a_inv_scale = a_inv_scale; g.W = W;
    g.P = P; g.ldp = ldp; g.plane_stride = plane_stride;
    g.M = M; g.N = N; g.Mb = Mb; g.Nb = Nb; g.Kb = Kb; g.steps_per_chunk = p.steps;
    g.n_tiles = p.n_tiles; g.S = p.S; g.m_tiles = p.m_tiles;
#define GEMM_LAUNCH(NBV, ROT, SC, WFV) do { \
        if (p.m_tiles > 1) { \
            if (g_prof_on) hipExtLaunchKernelGGL((gemm_tiled<NBV, 4, ROT, SC, WFV, 1>), grid, block, lds, stream(), ev_a, ev_b, 0, g); \
            else hipLaunchKernelGGL((gemm_tiled<NBV, 4, ROT, SC, WFV, 1>), grid, block, lds, stream(), g); \
        } else if (p.nw == 8) { \
            if (g_prof_on) hipExtLaunchKernelGGL((gemm_tiled<NBV, 8, ROT, SC, WFV>), grid, block, lds, stream(), ev_a, ev_b, 0, g); \
            else hipLaunchKernelGGL((gemm_tiled<NBV, 8, ROT, SC, WFV>), grid, block, lds, stream(), g); \
        } else { \
            if (g_prof_on) hipExtLaunchKernelGGL((gemm_tiled<NBV, 4, ROT, SC, WFV>), grid, block, lds, stream(), ev_a, ev_b, 0, g); \
            else hipLaunchKernelGGL((gemm_tiled<NBV, 4, ROT, SC, WFV>), grid, block, lds, stream(), g); \
        } } while (0)
#define GEMM_PICK_SC(NBV, ROT, WFV) do { if (a_inv_scale) GEMM_LAUNCH(NBV, ROT, 1, WFV); else GEMM_LAUNCH(NBV, ROT, 0, WFV); } while (0)
#define GEMM_PICK_ROT(NBV, WFV) do { if (p.rotate) GEMM_PICK_SC(NBV, 1, WFV); else GEMM_PICK_SC(NBV, 0, WFV); } while (0)
#define GEMM_PICK_NB(WFV) do { if (p.nb == 2) GEMM_PICK_ROT(2, WFV); else GEMM_PICK_ROT(1, WFV); } while (0)
    if (W.fmt == 0) GEMM_PICK_NB(0); else if (W.fmt == 1) GEMM_PICK_NB(1); else GEMM_PICK_NB(2);
#undef GEMM_PICK_NB
#undef GEMM_PICK_ROT
#undef GEMM_PICK_SC
#undef GEMM_LAUNCH
    HIP_CHECK(hipGetLastError());
    if (g_prof_on) g_prof.push_back(rec);
}

// Bytes of weight data one launch has to stream for an [N, K] operand: 2 per F16 weight, 34 per 32 Q8_0 weights.
double weight_stream_bytes(const WeightOp &W, int N, int K)
{
    const double nk = (double)N * K;
    if (W.fmt == 0) return 2.0 * nk;
    if (W.fmt == 1) { const double nq = (double)(W.nbq * 32 < N ? W.nbq * 32 : N); return nq * K * 34.0 / 32.0 + (N - nq) * K * 2.0; }
    const double kq = (double)(W.kbq * 64 < K ? W.kbq * 64 : K);
    return (double)N * kq * 34.0 / 32.0 + (double)N * (K - kq) * 2.0;
}

void launch_rows_to_f16(const float *X, int ldx, half_t *out_tiled, float *inv_scale, int M, int K)
{
    hipLaunchKernelGGL(rows_to_f16_scaled, dim3(M), dim3(256), 0, stream(), X, ldx, out_tiled, inv_scale, K, tiled_kb(K));
    HIP_CHECK(hipGetLastError());
}

void launch_reduce_planes(const float *P, int S, size_t plane_stride, int ldp, const float *row_scale, float *C, int M, int N)
{
    const size_t n = (size_t)M * N;
    hipLaunchKernelGGL(reduce_planes, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream(),
                       P, S, plane_stride, ldp, row_scale, C, M, N);
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

void launch_tile_q8(const uint8_t *blocks, int rows, int cols, uint8_t *q_tiles, half_t *d_tiles, int Kb_dst,
                    int row_off, int k_off, int transpose)
{
    if (rows <= 0 || cols < 32) return;
    if ((cols & 31) || (row_off & 31) || (!transpose && (k_off & 31))) {
        fprintf(stderr, "[fast_hip] tile_q8: offsets and width must be multiples of 32\n");
        abort();
    }
    const size_t n = (size_t)rows * (cols / 32);
    hipLaunchKernelGGL(tile_q8, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream(),
                       blocks, rows, cols / 32, q_tiles, d_tiles, Kb_dst, row_off, k_off, transpose);
    HIP_CHECK(hipGetLastError());
}

void launch_untile_q8(const uint8_t *q_tiles, const half_t *d_tiles, int fmt, int Kb, int row_off, int k_off, int transpose,
                      int rows, int cols, half_t *dst)
{
    const size_t n = (size_t)rows * cols;
    if (!n) return;
    hipLaunchKernelGGL(untile_q8, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream(),
                       q_tiles, d_tiles, fmt, Kb, row_off, k_off, transpose, rows, cols, dst);
    HIP_CHECK(hipGetLastError());
}

int gemm_profiling() { return g_prof_on; }
namespace {
int g_half_planes = 1;
// one workgroup (a wave) per 32-row block of a tiled F16 matrix: the largest sum of |w| over one of its rows
__global__ __launch_bounds__(64) void k_tiled_row_l1(const half8 *__restrict__ W, int N, int Kb, float *__restrict__ out)
{
    const int lane = threadIdx.x;
    const half8 *p = W + (size_t)blockIdx.x * Kb * 256 + lane;
    float s = 0.f;
    for (int kt = 0; kt < Kb; kt++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const half8 v = p[(size_t)kt * 256 + j * 64];
#pragma unroll
            for (int e = 0; e < 8; e++) s += fabsf((float)v[e]);
        }
    if ((int)blockIdx.x * 32 + (lane & 31) >= N) s = 0.f; // rows of the last block past the matrix hold anything
    s += __shfl_xor(s, 32, 64);                           // the two column halves of a row
#pragma unroll
    for (int o = 1; o < 32; o <<= 1) s = fmaxf(s, __shfl_xor(s, o, 64));
    if (lane == 0) atomicMax(reinterpret_cast<int *>(out), __float_as_int(s));   // sums are >= 0: integer order is float order
}
// the same for a Q8_0 operand (FMT 1: one scale per lane and tile; 2: one per column of the tile), of the values d * q
template <int FMT>
__global__ __launch_bounds__(64) void k_q8_row_l1(const uint8_t *__restrict__ q, const half_t *__restrict__ d, int N, int Kb, float *__restrict__ out)
{
    const int lane = threadIdx.x;
    float s = 0.f;
    for (int kt = 0; kt < Kb; kt++) {
        const size_t tile = (size_t)blockIdx.x * Kb + kt;
        const uint4v *qp = reinterpret_cast<const uint4v *>(q) + tile * 128 + lane;
        const uint4v r[2] = {qp[0], qp[64]};
        const half_t *sc = d + tile * 64 + (FMT == 1 ? lane : (lane >> 5) * 32);
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int w = 0; w < 4; w++)
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const int v = (int)(int8_t)((r[h][w] >> (8 * b)) & 0xffu);
                    const int je = (2 * h + (w >> 1)) * 8 + (w & 1) * 4 + b;      // (j, e) of the byte, as load_w_q8_cols numbers them
                    s += fabsf((float)v) * (float)(FMT == 1 ? sc[0] : sc[je]);
                }
    }
    if ((int)blockIdx.x * 32 + (lane & 31) >= N) s = 0.f;
    s += __shfl_xor(s, 32, 64);
#pragma unroll
    for (int o = 1; o < 32; o <<= 1) s = fmaxf(s, __shfl_xor(s, o, 64));
    if (lane == 0) atomicMax(reinterpret_cast<int *>(out), __float_as_int(s));
}
}  // namespace

float weight_max_row_l1(const WeightOp &W, int N, int K)
{
    if (W.fmt == 0) return tiled_max_row_l1(W.w16, N, K);
    // operands that are Q8_0 throughout (no F16 row blocks or K steps behind them)
    if ((W.fmt == 1 && W.nbq != tiled_rb(N)) || (W.fmt == 2 && W.kbq != tiled_kb(K))) return 0.f;
    float *slot = (float *)scratch(SCR_MISC, sizeof(float));
    HIP_CHECK(hipMemsetAsync(slot, 0, sizeof(float), stream()));
    if (W.fmt == 1) hipLaunchKernelGGL(k_q8_row_l1<1>, dim3(tiled_rb(N)), dim3(64), 0, stream(), W.q, W.d, N, tiled_kb(K), slot);
    else hipLaunchKernelGGL(k_q8_row_l1<2>, dim3(tiled_rb(N)), dim3(64), 0, stream(), W.q, W.d, N, tiled_kb(K), slot);
    float v = 0.f;
    HIP_CHECK(hipMemcpyAsync(&v, slot, sizeof(float), hipMemcpyDeviceToHost, stream()));
    HIP_CHECK(hipStreamSynchronize(stream()));
    return v;
}

float tiled_max_row_l1(const half_t *W_tiled, int N, int K)
{
    float *slot = (float *)scratch(SCR_MISC, sizeof(float));
    HIP_CHECK(hipMemsetAsync(slot, 0, sizeof(float), stream()));
    hipLaunchKernelGGL(k_tiled_row_l1, dim3(tiled_rb(N)), dim3(64), 0, stream(), reinterpret_cast<const half8 *>(W_tiled), N, tiled_kb(K), slot);
    float v = 0.f;
    HIP_CHECK(hipMemcpyAsync(&v, slot, sizeof(float), hipMemcpyDeviceToHost, stream()));
    HIP_CHECK(hipStreamSynchronize(stream()));
    return v;
}

float half_plane_scale(float max_row_l1)
{
    // |chunk sum| < 8192 * max_row_l1; the largest power of two s with 8192 * max_row_l1 * s <= 32768 (half the fp16 range)
    if (!(max_row_l1 > 0.f) || !(max_row_l1 < 1e30f)) return 1.0f;
    int e;
    frexpf(4.0f / max_row_l1, &e);                        // 4 / l1 = f * 2^e, f in [0.5, 1)
    int pw = e - 1;
    pw = pw > 24 ? 24 : (pw < -100 ? -100 : pw);
    return ldexpf(1.0f, pw);
}
void set_gemm_half_planes(int on) { g_half_planes = on ? 1 : 0; }
int gemm_half_planes_enabled() { return g_half_planes; }

void set_gemm_ring(int on) { g_ring = on; }
void set_gemm_ring_wide(int on) { g_ring_wide = on; }
int gemm_ring_wide_mode() { return g_ring_wide; }
int gemm_ring_enabled() { return g_ring; }

// Which kernel multiplies an [M, K] activation block with an [N, K] weight.  Measured on MI355X (Qwen3-4B shapes):
// the 128 x 256 LDS-tiled kernel wins for F16 weights once there is about one block per CU (2048 rows: 490-650
// against 300 TFLOP/s for the weight-streaming kernel).  With Q8_0 weights the streaming kernel, whose waves overlap
// each other's unpacking and MFMAs, is ahead of the large-M kernel unpacking tiles into LDS itself (400-470 against
// 340-460 TFLOP/s), but from 1024 rows on it pays to dequantise the operand once into an F16 image (3 bytes of extra
// HBM traffic per weight) and run the large-M kernel on that instead of unpacking every tile again for each 64 rows
// of activations: 4 x 512 rows, 112.9 ms per step against 123 ms (streaming) and 125 ms (Q8_0 inside the large-M kernel).
int g_big_policy = 0;                                     // 0 measured rule, 1 always, -1 never, 2 always and Q8_0 tiles stay quantised
bool use_big_gemm(int M, int N, int K, int fmt)
{
    if (g_big_policy) return g_big_policy > 0;
    const long blocks = (long)((M + 127) / 128) * ((N + 255) / 256);
    const int cus = num_cus() > 0 ? num_cus() : 256;
    const bool long_k = fmt == 0 && blocks * 8 <= cus && K >= 65536;      // few blocks, cut into many K chunks (big_gemm_chunks)
    if (M >= 1024) return blocks >= 160 || long_k;        // either format (Q8_0 through its F16 image)
    // 640 rows, F16 (Gemma3-1B shapes): 135 blocks 24 us against 31 on the streaming kernel, 270 blocks ahead as well;
    // 25-30 blocks of short K lose by a factor of two to four
    return fmt == 0 && M >= 512 && (blocks >= 128 || long_k);
}

// The operand as plain F16 tiles: W itself when it is F16, else an image in the library's scratch arena (valid until
// the next call).
WeightOp f16_image_of(const WeightOp &W, int N, int K, void *keep, bool f16_part_only)
{
    if (W.fmt == 0 || g_big_policy == 2) return W;        // policy 2: the large-M kernel unpacks the Q8_0 tiles into LDS itself
    const int Nb = tiled_rb(N), Kb = tiled_kb(K);
    const size_t tiles = (size_t)Nb * Kb;
    half8 *img = keep ? (half8 *)keep : (half8 *)scratch(SCR_WF16, tiles * 256 * sizeof(half8));
    size_t todo = tiles;
    if (f16_part_only) todo = !W.w16 ? 0 : W.fmt == 1 ? (size_t)(Nb - W.nbq) * Kb : (size_t)Nb * (Kb - W.kbq);
    if (todo) {
        hipLaunchKernelGGL(q8_operand_to_f16, dim3((unsigned)((todo + 3) / 4)), dim3(256), 0, stream(), W, Nb, Kb, img, f16_part_only ? 1 : 0);
        HIP_CHECK(hipGetLastError());
    }
    return weight_f16(reinterpret_cast<const half_t *>(img));
}
bool large_m_unpacks_q8() { return g_big_policy == 2; }

bool gemm_prof_begin(double wbytes, double flops, hipEvent_t *a, hipEvent_t *b)
{
    if (!g_prof_on) return false;
    ProfRec rec{};
    HIP_CHECK(hipEventCreateWithFlags(&rec.a, PROF_EVENT_FLAGS));
    HIP_CHECK(hipEventCreateWithFlags(&rec.b, PROF_EVENT_FLAGS));
    rec.wbytes = wbytes; rec.flops = flops;
    g_prof.push_back(rec);
    *a = rec.a; *b = rec.b;
    return true;
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
        launch_gemm(a16, nullptr, Wt, P, Nout, plane, M, Nout, Kred, p);
        launch_reduce_planes(P, p.S, plane, Nout, inv, C, M, Nout);
    }
}

}  // namespace

namespace lmhip {

const half_t *tiled_weight_of(MetalBuf *W, int N, int K) { return tiled_copy_of(W, N, K, 0); }

void launch_rows_to_f16_split(const float *A, half_t *a16, float *inv, int M, int K)
{
    const bool vec = K % 4 == 0 && ((uintptr_t)A & 15) == 0;
    if (vec && K <= 8192) hipLaunchKernelGGL(rows_to_f16_split_vec<1>, dim3(M), dim3(1024), 0, stream(), A, K, a16, inv, M, K, tiled_kb(K));
    else if (vec && K <= 16384) hipLaunchKernelGGL(rows_to_f16_split_vec<2>, dim3(M), dim3(1024), 0, stream(), A, K, a16, inv, M, K, tiled_kb(K));
    else hipLaunchKernelGGL(rows_to_f16_split, dim3(M), dim3(256), 0, stream(), A, K, a16, inv, M, K, tiled_kb(K));
}

void launch_reduce_planes_split(const float *P, int S, size_t plane_stride, int ldp, const float *inv, float *C, int M, int N)
{
    const size_t n = (size_t)M * N;
    hipLaunchKernelGGL(reduce_planes_split, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream(), P, S, plane_stride, ldp, inv, C, M, N);
}

// C[M, N] fp32 = A[M, K] fp32 * W^T, W an F16 [N, K] weight buffer, with A split into value and residual rows
void gemm_f32a_exact(const float *A, MetalBuf *W, float *C, int M, int N, int K)
{
    const half_t *Wt = tiled_copy_of(W, N, K, 0);
    const int M2 = 2 * M;
    half_t *a16 = (half_t *)scratch(SCR_A16, tiled_elems(M2, K) * sizeof(half_t));
    float *inv = (float *)scratch(SCR_SCALE, (size_t)M2 * sizeof(float));
    launch_rows_to_f16_split(A, a16, inv, M, K);
    GemmPlan p = plan_gemm(M2, N, K);
    const size_t plane = (size_t)M2 * N;
    float *P = (float *)scratch(SCR_PARTIAL, plane * p.S * sizeof(float));
    launch_gemm(a16, nullptr, Wt, P, N, plane, M2, N, K, p);
    launch_reduce_planes_split(P, p.S, plane, N, inv, C, M, N);
    HIP_CHECK(hipGetLastError());
}

}  // namespace lmhip

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

void hip_gemm_force_large_m(int policy) { g_big_policy = policy; }
void hip_gemm_ring(int on) { lmhip::set_gemm_ring(on); }
void hip_gemm_ring_wide(int on) { lmhip::set_gemm_ring_wide(on); }
void hip_gemm_half_planes(int on) { lmhip::set_gemm_half_planes(on); }
void hip_gemm_large_m_split(int mode) { set_big_gemm_split(mode); }
void hip_gemm_large_m_block(int mode) { set_big_gemm_block(mode); }

void hip_gemm_profile_enable(int on)
{
    HIP_CHECK(hipStreamSynchronize(stream()));
    for (auto &r : g_prof) { hipEventDestroy(r.a); hipEventDestroy(r.b); }
    g_prof.clear();
    g_prof_on = on;
}

int hip_gemm_profile_read(double *total_ms, double *total_weight_bytes)
{
    return hip_gemm_profile_read2(total_ms, total_weight_bytes, nullptr);
}

int hip_gemm_profile_read2(double *total_ms, double *total_weight_bytes, double *total_flops)
{
    HIP_CHECK(hipStreamSynchronize(stream()));
    double ms = 0, wb = 0, fl = 0;
    for (auto &r : g_prof) {
        float t = 0;
        HIP_CHECK(hipEventElapsedTime(&t, r.a, r.b));
        ms += t;
        wb += r.wbytes;
        fl += r.flops;
    }
    if (total_ms) *total_ms = ms;
    if (total_weight_bytes) *total_weight_bytes = wb;
    if (total_flops) *total_flops = fl;
    return (int)g_prof.size();
}

// Times `iters` launches of the GEMM alone on synthetic tiled operands of the given shape
// (HIP events on the library's stream).  nb / S = 0 let the planner choose; otherwise they force the
// tile height and the K split.  wf = weight format (0 F16, 1 Q8_0 row scales, 2 Q8_0 column scales).
// Returns the average milliseconds per launch.
double hip_gemm_time_shape(int M, int N, int K, int nb, int wf, int S, int iters, int *used_nb, int *used_S)
{
    const bool read_only = nb == -1;                       // the weight loads of gemm_ring alone (ring_weights_only)
    if (read_only) nb = 0;
    g_force_nb = nb == 128 ? 0 : nb; g_force_S = S;
    const int wide_was = g_ring_wide;
    if (read_only) g_ring_wide = 0;                        // ring_weights_only walks gemm_ring's grid of two row blocks per workgroup
    GemmPlan p = plan_gemm(M, N, K, 0, wf);
    g_force_nb = 0; g_force_S = 0; g_ring_wide = wide_was;
    if (used_nb) *used_nb = p.nb;
    if (used_S) *used_S = p.S;
    void *A = nullptr, *W = nullptr, *D = nullptr, *P = nullptr, *inv = nullptr;
    const size_t tiles = (size_t)tiled_rb(N) * tiled_kb(K);
    const size_t ab = tiled_elems(M, K) * 2, wb = wf ? tiles * 2048 : tiles * 4096, db = tiles * 128;
    const size_t pb = (size_t)(nb == 128 ? (S > 0 ? S : 1) : p.S) * M * N * 4;
    // rotate through enough distinct weight images that no launch finds its weights in a cache
    const int nbuf = (int)((size_t)1200 * 1024 * 1024 / wb) + 1;
    HIP_CHECK(hipMalloc(&A, ab)); HIP_CHECK(hipMalloc(&W, wb * nbuf)); HIP_CHECK(hipMalloc(&D, db * nbuf));
    HIP_CHECK(hipMalloc(&P, pb)); HIP_CHECK(hipMalloc(&inv, (size_t)M * 4));
    if (wf == 0) {                                         // F16 tiles: random values (Q8_0 tiles keep a constant pattern)
        hipLaunchKernelGGL(fill_random_f16, dim3((unsigned)((ab / 2 + 255) / 256)), dim3(256), 0, stream(), (half_t *)A, ab / 2, 1u);
        hipLaunchKernelGGL(fill_random_f16, dim3((unsigned)((wb * nbuf / 2 + 255) / 256)), dim3(256), 0, stream(), (half_t *)W, wb * nbuf / 2, 2u);
    } else {
        HIP_CHECK(hipMemsetAsync(A, 0x11, ab, stream())); HIP_CHECK(hipMemsetAsync(W, 0x11, wb * nbuf, stream()));
    }
    HIP_CHECK(hipMemsetAsync(D, 0x11, db * nbuf, stream()));
    HIP_CHECK(hipMemsetAsync(inv, 0, (size_t)M * 4, stream()));
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0)); HIP_CHECK(hipEventCreate(&e1));
    const int saved = g_prof_on;
    g_prof_on = 0;
    auto op = [&](int i) {
        WeightOp w{};
        w.fmt = wf;
        if (wf == 0) w.w16 = (half_t *)((char *)W + (size_t)(i % nbuf) * wb);
        else { w.q = (uint8_t *)W + (size_t)(i % nbuf) * wb; w.d = (half_t *)((char *)D + (size_t)(i % nbuf) * db);
               w.nbq = tiled_rb(N); w.kbq = tiled_kb(K); }
        return w;
    };
    const bool big = nb == 128;                            // nb = 128 selects the large-M kernel (one launch, 128-row blocks)
    auto run = [&](int i) {
        if (read_only && p.ring) {
            GemmKArgs g{};
            g.W = op(i); g.P = (float *)P; g.Nb = tiled_rb(N); g.Kb = tiled_kb(K); g.steps_per_chunk = p.steps; g.n_tiles = p.n_tiles; g.S = p.S;
            hipLaunchKernelGGL((ring_weights_only<2>), dim3((unsigned)(p.n_tiles * p.S)), dim3(512), 0, stream(), g);
        } else if (big) launch_gemm_big((half_t *)A, (float *)inv, op(i), (float *)P, N, M, N, K, S > 0 ? S : 1, (size_t)M * N);
        else launch_gemm((half_t *)A, nullptr, op(i), (float *)P, N, (size_t)M * N, M, N, K, p);
    };
    for (int i = 0; i < 3; i++) run(i);
    HIP_CHECK(hipEventRecord(e0, stream()));
    for (int i = 0; i < iters; i++) run(i);
    HIP_CHECK(hipEventRecord(e1, stream()));
    HIP_CHECK(hipStreamSynchronize(stream()));
    g_prof_on = saved;
    float ms = 0;
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    hipEventDestroy(e0); hipEventDestroy(e1);
    hipFree(A); hipFree(W); hipFree(D); hipFree(P); hipFree(inv);
    return (double)ms / iters;
}

}  // extern "C"
