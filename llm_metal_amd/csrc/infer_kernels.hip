// The inference enqueues of the reference's dispatch ABI (src/nn/fast_metal.h:19-80) as HIP kernels with the
// reference's buffer layouts: the matrix-vector products of a decode step (F16 rows, Q8_0 blocks, a batch of up to 32
// vectors), the single-vector RMSNorm / per-head RMSNorm / RoPE / KV-cache store, and attention of one query per head
// over the cache.  All activations fp32.
//
// The products are pure weight streaming (2 flop per weight), so the kernels are shaped for HBM: one wave per weight
// row (four rows per wave when there are enough rows), 16-byte (F16) or 8-byte (Q8_0) loads per lane with several in
// flight, the vector(s) held in LDS once per workgroup, fp32 accumulation.  Q8_0 blocks are 34 bytes and therefore
// never aligned; the weight is re-laid once into a split image (all int8 codes, row-major, then all fp16 scales), kept
// with the buffer until something writes it, and the product streams that image.
#include "backend.h"
#include "devutil.h"
#include "gemm.h"
#include <hip/hip_ext.h>

using namespace lmhip;

namespace {

constexpr int TB = 256;
#define LAUNCH(kern, grid, block, lds, ...) do { \
    hipLaunchKernelGGL(kern, grid, block, lds, stream(), __VA_ARGS__); HIP_CHECK(hipGetLastError()); } while (0)

typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(TB) void k_zero(float *p, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i < n) p[i] = 0.f;
}

// a product over an empty reduction
void zero_result(MetalBuf *y, size_t n)
{
    LAUNCH(k_zero, dim3((unsigned)((n + TB - 1) / TB)), dim3(TB), 0, dptr_as<float>(y), n);
    mark_written(y);
}

// ---------------------------------------------------------------- Q8_0 split image

// blocks [n_blocks] of {fp16 d; int8 q[32]} -> q [n_blocks * 32], d [n_blocks]; thread per code
__global__ __launch_bounds__(TB) void k_q8_split(const uint8_t *__restrict__ blocks, int8_t *__restrict__ q,
                                                 uint16_t *__restrict__ d, size_t n_blocks)
{
    const size_t idx = (size_t)blockIdx.x * TB + threadIdx.x;
    if (idx >= n_blocks * 32) return;
    const size_t b = idx >> 5;
    const int j = (int)(idx & 31);
    const uint8_t *blk = blocks + b * 34;
    q[idx] = (int8_t)blk[2 + j];
    if (j == 0) d[b] = (uint16_t)(blk[0] | (blk[1] << 8));
}

inline size_t q8_scale_offset(size_t n_blocks) { return (n_blocks * 32 + 255) & ~(size_t)255; }

// Split image of a Q8_0 weight held in W (rows x nb blocks).  Cached with the buffer (slot 2 of its
// derived images) while the buffer is device-resident and unwritten; otherwise rebuilt in scratch.
const int8_t *q8_split_of(MetalBuf *W, int rows, int nb, const half_t **scales)
{
    const size_t n_blocks = (size_t)rows * nb, soff = q8_scale_offset(n_blocks), bytes = soff + n_blocks * 2;
    const bool cacheable = W->owns && !W->host && !W->parent;
    uint8_t *img;
    bool build = true;
    if (!cacheable) {
        img = (uint8_t *)scratch(SCR_MISC, bytes);
    } else {
        MetalBuf::Tiled &c = W->tiled[2];
        if (c.dev && (c.rows != rows || c.cols != nb)) {
            HIP_CHECK(hipStreamSynchronize(stream()));
            HIP_CHECK(hipFree(c.dev));
            c.dev = nullptr;
        }
        if (!c.dev) HIP_CHECK(hipMalloc(&c.dev, bytes));
        else if (c.version == W->version) build = false;
        c.rows = rows; c.cols = nb; c.version = W->version;
        img = (uint8_t *)c.dev;
    }
    if (build)
        LAUNCH(k_q8_split, dim3((unsigned)((n_blocks * 32 + TB - 1) / TB)), dim3(TB), 0, dptr_as<uint8_t>(W), (int8_t *)img,
               (uint16_t *)(img + soff), n_blocks);
    *scales = (const half_t *)(img + soff);
    return (const int8_t *)img;
}

// ---------------------------------------------------------------- matrix-vector products

// y[row] = sum_c W[row, c] x[c].  FMT 0: W F16 row-major.  FMT 1: W int8 codes row-major with one fp16 scale per
// 32 columns.  Requires cols % 8 == 0 and 16-byte aligned W and x.
// Workgroup = 4 waves; wave w owns rows (4 blockIdx.x + w) R .. + R - 1; a lane owns 8 consecutive columns of every
// 512-column step.  The weights of U steps (all R rows) are one register stage; the next stage is loaded before the
// current one is used, and the first before x is staged into LDS (XLDS; without it, for rows longer than the LDS
// budget, every lane reads its x values from global memory with the weights).  Q8_0: codes are biased to unsigned
// (q + 128, one v_cvt_f32_ubyte each) and the bias is taken out with the lane's sum of x, once per step for all rows.
// GLU (1 SiLU, 2 GELU; R = 2): the matrix is [gate; up] with `rows` rows each; a wave takes gate row i and up row i and
// writes act(gate . x) * (up . x), the gated product the FFN forms next, in place of the two sums.
// NORM (with XLDS): the vector is RMSNorm(v; g) of v = xr + br (br may be null), which every workgroup forms for itself
// while its first weights are on their way: v g goes to LDS, the sum of squares through one block reduction, and the
// factor rsqrt(mean + eps) onto the finished sums; workgroup 0 also writes v to x_out (not xr: the others still read it).
// residual_add + rms_norm of shaders/q8_kernels.metal:133-158, 369-375 without a launch of their own.
// REPS (NORM only): row groups a wave takes one after the other, so that fewer workgroups form the vector.
template <int FMT, int R, int U, int XLDS, int GLU = 0, int NORM = 0, int REPS = 1>
__global__ __launch_bounds__(TB) void k_matvec(const void *__restrict__ Wp, const half_t *__restrict__ scales,
                                               const float *__restrict__ x, float *__restrict__ y, int rows, int cols, NormIn nin)
{
    static_assert(GLU == 0 || R == 2, "the gated variant pairs two rows");
    static_assert(NORM == 0 || XLDS == 1, "the normed vector is staged in LDS");
    extern __shared__ float xs[];                               // [cols] when XLDS
    __shared__ float red[16];
    struct Stage {
        half8   w16[FMT == 0 ? R : 1][U];
        uint2v  w8[FMT == 1 ? R : 1][U];
        float   dsc[FMT == 1 ? R : 1][U];
        float4v x0[XLDS ? 1 : U], x1[XLDS ? 1 : U];
    };
    static_assert(REPS == 1 || NORM == 1, "row groups in turn only where the vector is formed in the kernel");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int row0 = ((blockIdx.x * REPS) * 4 + wave) * (GLU ? 1 : R);
    size_t roff[R];                                             // element offset of each row (clamped: extra rows are not stored)
    float acc[R];
    auto set_rows = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            roff[r] = GLU ? ((size_t)r * rows + min(row0, rows - 1)) * cols : (size_t)min(row0 + r, rows - 1) * cols;
            acc[r] = 0.f;
        }
    };
    set_rows();

    auto load = [&](Stage &g, int c) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int cu = min(c + 512 * u, cols - 8);          // clamped: loads stay unconditional
#pragma unroll
            for (int r = 0; r < R; r++) {
                const size_t e = roff[r] + cu;
                if (FMT == 0) g.w16[r][u] = __builtin_nontemporal_load(reinterpret_cast<const half8 *>((const half_t *)Wp + e));
                else {
                    g.w8[r][u] = __builtin_nontemporal_load(reinterpret_cast<const uint2v *>((const int8_t *)Wp + e));
                    g.dsc[r][u] = (float)scales[e >> 5];
                }
            }
            if (!XLDS) {
                g.x0[u] = *reinterpret_cast<const float4v *>(&x[cu]);
                g.x1[u] = *reinterpret_cast<const float4v *>(&x[cu + 4]);
            }
        }
    };
    auto use = [&](const Stage &g, int c) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int cu = min(c + 512 * u, cols - 8);
            const float live = (c + 512 * u < cols) ? 1.f : 0.f;
            float4v x0, x1;
            if (XLDS) { x0 = *reinterpret_cast<const float4v *>(&xs[cu]); x1 = *reinterpret_cast<const float4v *>(&xs[cu + 4]); }
            else { x0 = g.x0[u]; x1 = g.x1[u]; }
            float xv[8];
#pragma unroll
            for (int e = 0; e < 4; e++) { xv[e] = x0[e] * live; xv[4 + e] = x1[e] * live; }
            float xsum = 0.f;
            if (FMT == 1) {
#pragma unroll
                for (int e = 0; e < 8; e++) xsum += xv[e];
                xsum *= 128.f;
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (FMT == 0) {
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[r] = fmaf((float)g.w16[r][u][e], xv[e], acc[r]);
                } else {
                    const uint32_t lo = g.w8[r][u][0] ^ 0x80808080u, hi = g.w8[r][u][1] ^ 0x80808080u;
                    float p = -xsum;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        p = fmaf((float)((lo >> (8 * e)) & 255u), xv[e], p);
                        p = fmaf((float)((hi >> (8 * e)) & 255u), xv[4 + e], p);
                    }
                    acc[r] = fmaf(g.dsc[r][u], p, acc[r]);
                }
            }
        }
    };

    Stage cur;
    load(cur, lane * 8);
    float norm_inv = 1.f;
    if (NORM) {
        float ss = 0.f;
        for (int i0 = tid * 4; i0 < cols; i0 += TB * 16) {      // four groups of a thread requested together
            float4v v[4], b[4], gg[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int i = min(i0 + u * TB * 4, cols - 4);
                v[u] = *reinterpret_cast<const float4v *>(&nin.xr[i]);
                if (nin.br) b[u] = *reinterpret_cast<const float4v *>(&nin.br[i]);
                gg[u] = *reinterpret_cast<const float4v *>(&nin.g[i]);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int i = i0 + u * TB * 4;
                if (i >= cols) break;
                if (nin.br) v[u] += b[u];
                ss += v[u][0] * v[u][0] + v[u][1] * v[u][1] + v[u][2] * v[u][2] + v[u][3] * v[u][3];
                *reinterpret_cast<float4v *>(&xs[i]) = v[u] * gg[u];
                if (blockIdx.x == 0 && nin.x_out) *reinterpret_cast<float4v *>(&nin.x_out[i]) = v[u];
            }
        }
        norm_inv = rsqrtf(block_sum(ss, red) / (float)cols + nin.eps);      // its barriers also publish xs
    } else if (XLDS) {
        for (int i = tid * 4; i < cols; i += TB * 4)
            *reinterpret_cast<float4v *>(&xs[i]) = *reinterpret_cast<const float4v *>(&x[i]);
        __syncthreads();
    }
#pragma unroll 1
    for (int rep = 0; rep < REPS; rep++) {
        if (rep) {                                              // the next group of rows, with the same vector
            row0 += 4 * (GLU ? 1 : R);
            set_rows();
            load(cur, lane * 8);
        }
        for (int c = lane * 8; c < cols; c += 512 * U) {
            Stage nxt;
            load(nxt, c + 512 * U);
            use(cur, c);
            cur = nxt;
        }
        if (GLU) {
            const float g = wave_sum(acc[0]) * norm_inv, u = wave_sum(acc[R - 1]) * norm_inv;
            if (lane == 0 && row0 < rows)                       // the expressions of silu_mul / gelu_mul
                y[row0] = (GLU == 1 ? g / (1.0f + expf(-g)) : 0.5f * g * (1.0f + tanhf(gelu_inner(g)))) * u;
        } else {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float s = wave_sum(acc[r]) * norm_inv;
                if (lane == 0 && row0 + r < rows) y[row0 + r] = s;
            }
        }
    }
}

// Any cols / alignment: one wave per row, lanes stride single elements.
__global__ __launch_bounds__(TB) void k_matvec_any(const half_t *__restrict__ W, const float *__restrict__ X,
                                                   float *__restrict__ Y, int rows, int cols, int B)
{
    const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const half_t *w = W + (size_t)row * cols;
    for (int b = 0; b < B; b++) {
        const float *x = X + (size_t)b * cols;
        float s = 0.f;
        for (int i = lane; i < cols; i += 64) s = fmaf((float)w[i], x[i], s);
        s = wave_sum(s);
        if (lane == 0) Y[(size_t)b * rows + row] = s;
    }
}

// Rows per wave grow with the matrix so that mid-sized weights (a few thousand rows) still put 16 waves on every CU.
template <int FMT>
void launch_matvec(const void *W, const half_t *scales, const float *x, float *y, int rows, int cols)
{
    // x goes through LDS only where a workgroup covers 16 rows: with fewer, refilling it costs more than it saves
    const size_t lds = (size_t)cols * 4;
    // with the GEMM profile enabled (hip_gemm_profile_enable) every launch is bracketed by events and counted there
    hipEvent_t ev_a = nullptr, ev_b = nullptr;
    const bool prof = gemm_prof_begin((double)rows * cols * (FMT == 0 ? 2.0 : 34.0 / 32.0), 2.0 * rows * cols, &ev_a, &ev_b);
#define MATVEC_LAUNCH(R_, U_, XL_, RPW_, L_) do { \
    const dim3 grid((rows + RPW_ - 1) / RPW_); \
    if (prof) hipExtLaunchKernelGGL((k_matvec<FMT, R_, U_, XL_>), grid, dim3(TB), L_, stream(), ev_a, ev_b, 0, W, scales, x, y, rows, cols, NormIn{}); \
    else hipLaunchKernelGGL((k_matvec<FMT, R_, U_, XL_>), grid, dim3(TB), L_, stream(), W, scales, x, y, rows, cols, NormIn{}); \
    HIP_CHECK(hipGetLastError()); } while (0)
    if (rows >= 32768 && lds <= 40 * 1024) MATVEC_LAUNCH(4, 2, 1, 16, lds);
    else if (rows >= 32768) MATVEC_LAUNCH(4, 2, 0, 16, 0);
    else if (rows >= 8192) MATVEC_LAUNCH(2, 2, 0, 8, 0);
    else MATVEC_LAUNCH(1, 4, 0, 4, 0);
#undef MATVEC_LAUNCH
}

// [gate; up] x with the gate applied (see k_matvec): y[i] = act(gate_i . x) * (up_i . x), i < rows.
template <int FMT>
void launch_matvec_glu(const void *W, const half_t *scales, const float *x, float *y, int rows, int cols, int gelu)
{
    hipEvent_t ev_a = nullptr, ev_b = nullptr;
    const bool prof = gemm_prof_begin(2.0 * rows * cols * (FMT == 0 ? 2.0 : 34.0 / 32.0), 4.0 * rows * cols, &ev_a, &ev_b);
    const dim3 grid((rows + 3) / 4);
#define GLU_LAUNCH(G_) do { \
    if (prof) hipExtLaunchKernelGGL((k_matvec<FMT, 2, 2, 0, G_>), grid, dim3(TB), 0, stream(), ev_a, ev_b, 0, W, scales, x, y, rows, cols, NormIn{}); \
    else hipLaunchKernelGGL((k_matvec<FMT, 2, 2, 0, G_>), grid, dim3(TB), 0, stream(), W, scales, x, y, rows, cols, NormIn{}); \
    HIP_CHECK(hipGetLastError()); } while (0)
    if (gelu) GLU_LAUNCH(2); else GLU_LAUNCH(1);
#undef GLU_LAUNCH
}

// Either product over RMSNorm(xr + br; g), formed by the kernel itself (NORM): glu 0 plain rows, 1 SiLU, 2 GELU pairs.
template <int FMT>
void launch_matvec_norm(const void *W, const half_t *scales, const NormIn &nin, float *y, int rows, int cols, int glu)
{
    hipEvent_t ev_a = nullptr, ev_b = nullptr;
    const double mats = glu ? 2.0 : 1.0;
    const bool prof = gemm_prof_begin(mats * rows * cols * (FMT == 0 ? 2.0 : 34.0 / 32.0), 2.0 * mats * rows * cols, &ev_a, &ev_b);
    const size_t lds = (size_t)cols * 4;
#define NORM_LAUNCH(G_, RPW_, REPS_) do { \
    const dim3 grid((rows + RPW_ * REPS_ - 1) / (RPW_ * REPS_)); \
    if (prof) hipExtLaunchKernelGGL((k_matvec<FMT, 2, 2, 1, G_, 1, REPS_>), grid, dim3(TB), lds, stream(), ev_a, ev_b, 0, W, scales, nullptr, y, rows, cols, nin); \
    else hipLaunchKernelGGL((k_matvec<FMT, 2, 2, 1, G_, 1, REPS_>), grid, dim3(TB), lds, stream(), W, scales, nullptr, y, rows, cols, nin); \
    HIP_CHECK(hipGetLastError()); } while (0)
    // measured at 9728 x 2560 pairs and 6144 x 2560 rows: two row groups per wave for the pairs (2432 workgroups forming
    // the vector cost what the norm's own launch did), one for the rows (384 workgroups leave CUs idle)
    if (glu == 0) NORM_LAUNCH(0, 8, 1); else if (glu == 1) NORM_LAUNCH(1, 4, 2); else NORM_LAUNCH(2, 4, 2);
#undef NORM_LAUNCH
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// ---------------------------------------------------------------- single-vector row ops

// rms_norm, shaders/q8_kernels.metal:133-158 (one workgroup per vector).  out may alias x.
__global__ __launch_bounds__(TB) void k_rms_norm1(const float *x, const float *__restrict__ gamma, float *out, int dim, float eps)
{
    __shared__ float sm[16];
    const size_t off = (size_t)blockIdx.x * dim;
    float ss = 0.f;
    for (int i = threadIdx.x; i < dim; i += TB) { const float v = x[off + i]; ss += v * v; }
    ss = block_sum(ss, sm);
    const float inv = rsqrtf(ss / (float)dim + eps);
    for (int i = threadIdx.x; i < dim; i += TB) out[off + i] = x[off + i] * inv * gamma[i];
}

// rope, shaders/q8_kernels.metal:195-231: half-split pairs (d, d + hd/2) of every q and k head at one position.
__global__ __launch_bounds__(TB) void k_rope1(float *q, float *k, int Hq, int Hkv, int hd, int pos, float theta)
{
    const int half = hd / 2, q_pairs = Hq * half, total = q_pairs + Hkv * half;
    int idx = blockIdx.x * TB + threadIdx.x;
    if (idx >= total) return;
    float *base = q;
    if (idx >= q_pairs) { idx -= q_pairs; base = k; }
    const int d = idx % half;
    float *vec = base + (size_t)(idx / half) * hd;
    const float freq = 1.0f / powf(theta, (float)(2 * d) / (float)hd);
    float s, c;
    sincosf((float)pos * freq, &s, &c);
    const float x0 = vec[d], x1 = vec[d + half];
    vec[d] = x0 * c - x1 * s;
    vec[d + half] = x0 * s + x1 * c;
}

// kv_cache_store, shaders/q8_kernels.metal:237-256: caches are [Hkv, max_seq, hd].
__global__ __launch_bounds__(TB) void k_kv_store(const float *__restrict__ k, const float *__restrict__ v,
                                                 float *__restrict__ kc, float *__restrict__ vc, int Hkv, int max_seq,
                                                 int hd, int pos)
{
    const int idx = blockIdx.x * TB + threadIdx.x;
    if (idx >= Hkv * hd) return;
    const size_t ci = ((size_t)(idx / hd) * max_seq + pos) * hd + idx % hd;
    kc[ci] = k[idx];
    vc[ci] = v[idx];
}

// ---------------------------------------------------------------- attention of one query per head over the cache

constexpr int SL = 256;      // keys per workgroup

// attention, shaders/q8_kernels.metal:262-331, restructured for a GPU with 256 CUs: a workgroup serves `gpw` query
// heads that share a KV head (all G of the group when the context is long, so that the cache is read once; one when
// it is short and the launch is bound by latency, not bytes) over a slice of SL keys; with more than one slice the
// workgroups leave (max, sum, unnormalised output) per query head and k_attn_combine merges them.
// VEC: floats of V per thread in the weighted sum (4 when hd % 4 == 0).
// LDS: q [gpw][hd], scores [gpw][SL], ml [2][gpw], red [4 * 1024].  hd <= 256.
// FUSED: Q is the raw q part of the Q|K|V product; the workgroup finishes its query heads itself (into LDS only) and, when
// its slice holds the newest key, writes that key's and value's cache rows before it reads the cache (every workgroup
// that needs them writes the same values, so no workgroup waits for another).

// One head of the Q|K|V product finished by one wave (lane i owns the rotary pairs i and i + 64 of up to 256 values):
// kind 0 q (LoRA, norm, RoPE), 1 k (norm, RoPE), 2 v (LoRA).  per_head_rms_norm, rope, add_scaled of
// shaders/q8_kernels.metal:165-231, 378-384.
__device__ __forceinline__ void finish_head(const HeadPost &a, int kind, int h, int hd, int lane, float *dst)
{
    const int half = hd / 2;
    const float *vec = a.qkv + (size_t)(kind == 0 ? h : (kind == 1 ? a.Hq + h : a.Hq + a.Hkv + h)) * hd;
    float x0[2] = {0.f, 0.f}, x1[2] = {0.f, 0.f};
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int i = lane + 64 * u;
        if (i < half) {
            x0[u] = vec[i]; x1[u] = vec[i + half];
            if (a.R && kind != 1) {
                const float *B = (kind == 0 ? a.Bq : a.Bv) + (size_t)h * hd * a.R;
                const float *t = kind == 0 ? a.t : a.t + a.R;
                float d0 = 0.f, d1 = 0.f;
                for (int r = 0; r < a.R; r++) { d0 = fmaf(B[(size_t)i * a.R + r], t[r], d0); d1 = fmaf(B[(size_t)(i + half) * a.R + r], t[r], d1); }
                x0[u] = fmaf(a.sc, d0, x0[u]); x1[u] = fmaf(a.sc, d1, x1[u]);
            }
            ss += x0[u] * x0[u] + x1[u] * x1[u];
        }
    }
    if (kind != 2) {
        const float *g = kind == 0 ? a.g_q : a.g_k;
        if (g) {
            const float inv = rsqrtf(wave_sum(ss) / (float)hd + a.eps);
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int i = lane + 64 * u;
                if (i < half) { x0[u] *= inv * g[i]; x1[u] *= inv * g[i + half]; }
            }
        }
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int i = lane + 64 * u;
            if (i < half) {
                const float2 c = a.rope[i];
                const float cs = c.x, sn = c.y;
                const float r0 = x0[u] * cs - x1[u] * sn, r1 = x0[u] * sn + x1[u] * cs;
                x0[u] = r0; x1[u] = r1;
            }
        }
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int i = lane + 64 * u;
        if (i < half) { dst[i] = x0[u]; dst[i + half] = x1[u]; }
    }
}

template <int VEC, bool FUSED>
__global__ __launch_bounds__(TB) void k_attn_decode(const float *__restrict__ Q, const float *Kc, const float *Vc,
                                                    float *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                                                    int n_attend, int hd, int max_seq, int G, int gpw, float scale, int nsplit,
                                                    HeadPost hp)
{
    extern __shared__ float sm[];
    float *qs = sm, *sc = qs + gpw * hd, *ml = sc + gpw * SL, *red = ml + 2 * gpw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int head_groups = FUSED ? (int)gridDim.x - hp.pf_wgs : (int)gridDim.x;
    if (FUSED && (int)blockIdx.x >= head_groups) {       // a workgroup that only asks for the next product's weights
        if (blockIdx.y == 0 && blockIdx.z == 0) request_bytes_ahead(hp.pf_base, hp.pf_bytes, blockIdx.x - head_groups, hp.pf_wgs);
        return;
    }
    const int hq0 = blockIdx.x * gpw, hkv = hq0 / G, split = blockIdx.y;
    const int j0 = split * SL, nj = min(SL, n_attend - j0);
    // blockIdx.z: one of several sequences decoded in lock step (FUSED only), each with its own product row, adapter
    // terms, caches and output; slice results are kept per (sequence, query head)
    const int z = blockIdx.z, Hq_all = head_groups * gpw;
    if (FUSED) {
        hp.qkv += (size_t)z * hp.qkv_step; hp.kc += (size_t)z * hp.cache_step; hp.vc += (size_t)z * hp.cache_step;
        if (hp.R) hp.t += (size_t)z * hp.t_step;
        Kc = hp.kc; Vc = hp.vc;
        out += (size_t)z * Hq_all * hd;
    }
    const int hqz0 = z * Hq_all + hq0;                    // first (sequence, query head) of this workgroup
    const float *kbase = Kc + ((size_t)hkv * max_seq + j0) * hd;
    const float *vbase = Vc + ((size_t)hkv * max_seq + j0) * hd;

    if (FUSED) {
        for (int g = wave; g < gpw; g += 4) finish_head(hp, 0, hq0 + g, hd, lane, qs + g * hd);
        if (j0 <= hp.pos && hp.pos < j0 + SL) {           // the waves after those that had a query head (or all in turn)
            const size_t row = ((size_t)hkv * max_seq + hp.pos) * hd;
            if (wave == (gpw & 3)) finish_head(hp, 1, hkv, hd, lane, hp.kc + row);
            if (wave == ((gpw + 1) & 3)) finish_head(hp, 2, hkv, hd, lane, hp.vc + row);
        }
    } else {
        for (int i = tid; i < gpw * hd; i += TB) qs[i] = Q[(size_t)hq0 * hd + i];
    }
    __syncthreads();                                      // also orders the cache rows written above before the reads below

    // scores: a wave takes KT keys at a time (their loads are in flight together: a trip costs one memory round trip,
    // and a slice of 64 keys is two trips instead of four), lanes over the head dimension, four query heads per pass
    // over the keys
    constexpr int KT = 8;                                 // (2.341 -> 2.321 ms per token at 16-80 keys; 16: 2.335)
    for (int g0 = 0; g0 < gpw; g0 += 4) {
        int gq[4];
#pragma unroll
        for (int u = 0; u < 4; u++) gq[u] = min(g0 + u, gpw - 1);
        for (int jj = wave * KT; jj < nj; jj += 4 * KT) {
            const float *kp[KT];
#pragma unroll
            for (int t = 0; t < KT; t++) kp[t] = kbase + (size_t)min(jj + t, nj - 1) * hd;
            float p[KT][4];
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int u = 0; u < 4; u++) p[t][u] = 0.f;
            for (int d = lane; d < hd; d += 64) {
                float kv[KT], qv[4];
#pragma unroll
                for (int t = 0; t < KT; t++) kv[t] = kp[t][d];
#pragma unroll
                for (int u = 0; u < 4; u++) qv[u] = qs[gq[u] * hd + d];
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int u = 0; u < 4; u++) p[t][u] = fmaf(qv[u], kv[t], p[t][u]);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (g0 + u >= gpw) break;                                   // uniform
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    const float s = wave_sum(p[t][u]);
                    if (lane == 0 && jj + t < nj) sc[(g0 + u) * SL + jj + t] = s * scale;
                }
            }
        }
    }
    __syncthreads();

    // softmax statistics of the slice: one wave per query head, no barriers
    for (int g = wave; g < gpw; g += 4) {
        float m = -3.0e38f;
        for (int j = lane; j < nj; j += 64) m = fmaxf(m, sc[g * SL + j]);
        m = wave_max(m);
        float l = 0.f;
        for (int j = lane; j < nj; j += 64) { const float e = __expf(sc[g * SL + j] - m); sc[g * SL + j] = e; l += e; }
        l = wave_sum(l);
        if (lane == 0) { ml[g] = m; ml[gpw + g] = l; }
    }
    __syncthreads();

    // weighted value sum: thread = (part of the keys, VEC consecutive d); parts are added through LDS
    const int dpt = hd / VEC;                                               // threads along d
    const int parts = max(1, TB / dpt), part = tid / dpt, d = (tid % dpt) * VEC;
    const bool active = part < parts;
    typedef float vecf __attribute__((ext_vector_type(VEC)));
    constexpr int PT = 8;
    for (int g0 = 0; g0 < gpw; g0 += 4) {
        int gq[4];
#pragma unroll
        for (int u = 0; u < 4; u++) gq[u] = min(g0 + u, gpw - 1);
        float o[4][VEC];
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int e = 0; e < VEC; e++) o[u][e] = 0.f;
        if (active)
            for (int jj = part; jj < nj; jj += PT * parts) {                   // PT independent loads per trip
                float v[PT][VEC];
                int jt[PT];
#pragma unroll
                for (int t = 0; t < PT; t++) {
                    jt[t] = min(jj + t * parts, nj - 1);
                    const float live = (jj + t * parts < nj) ? 1.f : 0.f;
                    if (VEC == 1) v[t][0] = vbase[(size_t)jt[t] * hd + d] * live;
                    else {
                        const vecf vv = *reinterpret_cast<const vecf *>(&vbase[(size_t)jt[t] * hd + d]);
#pragma unroll
                        for (int e = 0; e < VEC; e++) v[t][e] = vv[e] * live;
                    }
                }
#pragma unroll
                for (int t = 0; t < PT; t++)
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const float w = sc[gq[u] * SL + jt[t]];
#pragma unroll
                        for (int e = 0; e < VEC; e++) o[u][e] = fmaf(w, v[t][e], o[u][e]);
                    }
            }
        if (active) {
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int e = 0; e < VEC; e++) red[(part * 4 + u) * hd + d + e] = o[u][e];
        }
        __syncthreads();
        // thread t < hd finishes element t of every head of this pass
        if (tid < hd) {
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (g0 + u >= gpw) continue;
                float s = 0.f;
                for (int pp = 0; pp < parts; pp++) s += red[(pp * 4 + u) * hd + tid];
                if (nsplit == 1) out[(size_t)(hq0 + g0 + u) * hd + tid] = s / ml[gpw + g0 + u];
                else part_o[((size_t)(hqz0 + g0 + u) * nsplit + split) * hd + tid] = s;
            }
        }
        __syncthreads();
    }
    if (nsplit > 1 && tid < gpw) {
        const int hq = hqz0 + tid;
        part_ml[((size_t)hq * nsplit + split) * 2] = ml[tid];
        part_ml[((size_t)hq * nsplit + split) * 2 + 1] = ml[gpw + tid];
    }
}

// merge of the slices of one query head: grid = Hq (times the sequences of a batch), block = hd threads (<= 256)
__global__ __launch_bounds__(TB) void k_attn_combine(const float *__restrict__ part_o, const float *__restrict__ part_ml,
                                                     float *__restrict__ out, int hd, int nsplit)
{
    const int hq = blockIdx.x, d = threadIdx.x;
    if (d >= hd) return;
    const float *mlp = part_ml + (size_t)hq * nsplit * 2;
    float m = -3.0e38f;
    for (int s = 0; s < nsplit; s++) m = fmaxf(m, mlp[2 * s]);
    float l = 0.f, o = 0.f;
    for (int s = 0; s < nsplit; s++) {
        const float w = __expf(mlp[2 * s] - m);
        l = fmaf(mlp[2 * s + 1], w, l);
        o = fmaf(part_o[((size_t)hq * nsplit + s) * hd + d], w, o);
    }
    out[(size_t)hq * hd + d] = o / l;
}

// byte offset into a buffer, checked against its size
float *at_offset(MetalBuf *b, size_t off, size_t need, const char *fn)
{
    if (!b || off + need > b->size || (off & 3)) {
        fprintf(stderr, "[fast_hip] %s: offset %zu + %zu bytes outside the buffer (%zu) or unaligned; launch skipped\n", fn, off,
                need, b ? b->size : (size_t)0);
        return nullptr;
    }
    return (float *)((char *)dptr(b) + off);
}

void per_head_rms_norm(float *vec, MetalBuf *gamma, int n_heads, int hd, float eps, const char *fn)
{
    REQUIRE_BYTES(gamma, (size_t)hd * 4, fn);
    if (n_heads <= 0 || hd <= 0) return;
    LAUNCH(k_rms_norm1, dim3(n_heads), dim3(TB), 0, vec, dptr_as<float>(gamma), vec, hd, eps);
}

void rope1(float *q, float *k, int Hq, int Hkv, int hd, int pos, float theta)
{
    const int total = (Hq + Hkv) * (hd / 2);
    if (total <= 0) return;
    LAUNCH(k_rope1, dim3((total + TB - 1) / TB), dim3(TB), 0, q, k, Hq, Hkv, hd, pos, theta);
}

void kv_store(const float *k, const float *v, MetalBuf *kc, MetalBuf *vc, int Hkv, int max_seq, int hd, int pos, const char *fn)
{
    REQUIRE_BYTES(kc, (size_t)Hkv * max_seq * hd * 4, fn);
    REQUIRE_BYTES(vc, (size_t)Hkv * max_seq * hd * 4, fn);
    if (pos < 0 || pos >= max_seq) { fprintf(stderr, "[fast_hip] %s: position %d outside the cache (%d); launch skipped\n", fn, pos, max_seq); return; }
    if (Hkv * hd <= 0) return;
    LAUNCH(k_kv_store, dim3((Hkv * hd + TB - 1) / TB), dim3(TB), 0, k, v, dptr_as<float>(kc), dptr_as<float>(vc), Hkv, max_seq, hd, pos);
    mark_written(kc); mark_written(vc);
}

// floats of slice results the attention over n_attend keys leaves for its merge kernel: per (query head, slice) hd sums and
// (max, sum of exponentials); none for a single slice
size_t attention_partial_floats(int Hq, int hd, int n_attend, int copies = 1)
{
    const int nsplit = (n_attend + SL - 1) / SL;
    return nsplit > 1 ? (size_t)copies * Hq * nsplit * (hd + 2) : 0;
}

// The launches of one attention over device pointers whose shapes the caller has checked.  `partials` holds
// attention_partial_floats(...) floats (unused when that is 0).  copies > 1 (only with hp): that many sequences at the
// same position in one launch, their operands hp's steps apart and their outputs Hq * hd floats apart.
void attention_launch(const float *Q, const float *Kc, const float *Vc, float *out, float *partials, int n_attend, int hd, int max_seq,
                      int Hq, int G, const HeadPost *hp, int copies = 1)
{
    const int nsplit = (n_attend + SL - 1) / SL;
    // short contexts are bound by latency: one query head per workgroup; long ones by cache bytes: the whole group
    const int gpw = n_attend <= 128 ? 1 : G;
    const size_t lds = ((size_t)gpw * hd + (size_t)gpw * SL + 2 * gpw + 4 * 1024) * 4;
    float *po = nsplit > 1 ? partials : nullptr, *pml = nsplit > 1 ? partials + (size_t)copies * Hq * nsplit * hd : nullptr;
    const float scale = 1.0f / sqrtf((float)hd);
    const bool vec4 = hd % 4 == 0 && (((uintptr_t)Vc) & 15) == 0;
    HeadPost post{};
    if (hp) post = *hp;
    if ((Hq / gpw) * nsplit * copies > 128 || !post.pf_base || !post.pf_bytes) post.pf_wgs = 0;      // no spare CUs, or nothing to ask for
    const dim3 grid(Hq / gpw + post.pf_wgs, nsplit, copies);
    const HeadPost none{};
#define ATTN_LAUNCH(V_, F_) LAUNCH((k_attn_decode<V_, F_>), grid, dim3(TB), lds, Q, Kc, Vc, out, po, pml, \
                                   n_attend, hd, max_seq, G, gpw, scale, nsplit, F_ ? post : none)
    if (hp) { if (vec4) ATTN_LAUNCH(4, true); else ATTN_LAUNCH(1, true); }
    else { if (vec4) ATTN_LAUNCH(4, false); else ATTN_LAUNCH(1, false); }
#undef ATTN_LAUNCH
    if (nsplit > 1) LAUNCH(k_attn_combine, dim3(Hq * copies), dim3(TB), 0, po, pml, out, hd, nsplit);
}

void attention(const float *Q, MetalBuf *Kc, MetalBuf *Vc, float *out, int n_attend, int hd, int max_seq, int Hq, int G, const char *fn,
               const HeadPost *hp = nullptr, int copies = 1)
{
    if (Hq <= 0 || n_attend <= 0) return;
    if (G <= 0 || Hq % G) { fprintf(stderr, "[fast_hip] %s: %d query heads are not a multiple of the group ratio %d; launch skipped\n", fn, Hq, G); return; }
    const int Hkv = Hq / G;
    REQUIRE_BYTES(Kc, (size_t)copies * Hkv * max_seq * hd * 4, fn);
    REQUIRE_BYTES(Vc, (size_t)copies * Hkv * max_seq * hd * 4, fn);
    if (n_attend > max_seq) { fprintf(stderr, "[fast_hip] %s: n_attend %d exceeds the cache (%d); launch skipped\n", fn, n_attend, max_seq); return; }
    if (hd > 256 || G > 16) { fprintf(stderr, "[fast_hip] %s: head_dim %d / group ratio %d not supported (<= 256 / <= 16); launch skipped\n", fn, hd, G); return; }
    const size_t pf = attention_partial_floats(Hq, hd, n_attend, copies);
    float *partials = pf ? (float *)scratch(SCR_MISC, pf * sizeof(float)) : nullptr;
    attention_launch(Q, dptr_as<float>(Kc), dptr_as<float>(Vc), out, partials, n_attend, hd, max_seq, Hq, G, hp, copies);
}

// ---- the attention once more for callers that cannot allocate ------------------------------------------------
// Slice results go to a fixed array in the code object's own data segment instead of the grow-only arena.  Each
// device the library runs on holds its own copy of the array at its own address until the process ends.  In host
// code the array's NAME is a stand-in, not a device address: only the pointer hipGetSymbolAddress returns for the
// current device may be handed to a kernel.
constexpr int NA_MAX_HQ = 64, NA_MAX_HD = 256, NA_MAX_KEYS = 8192, NA_MAX_DEVICES = 16;
constexpr size_t NA_FLOATS = (size_t)NA_MAX_HQ * (NA_MAX_KEYS / SL) * (NA_MAX_HD + 2);      // 2.0 MiB
static __device__ __align__(256) float attn_partials_static[NA_FLOATS];
float *g_na_ptr[NA_MAX_DEVICES];                           // per device; null until noalloc_setup ran with that device current

}  // namespace

namespace lmhip {

// Resolves the fixed partials array on the current device (once per device).  Called from fast_metal_init and, for a
// device that became current later, from the first no-allocation call on it.  0, or -1 with a message.
int noalloc_setup()
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= NA_MAX_DEVICES) {
        fprintf(stderr, "[fast_hip] noalloc_setup: no current device below %d (%s)\n", NA_MAX_DEVICES, hipGetErrorString(e));
        return -1;
    }
    if (g_na_ptr[dev]) return 0;
    float *p = nullptr;
    e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(attn_partials_static));
    if (e != hipSuccess || !p) {
        fprintf(stderr, "[fast_hip] noalloc_setup: hipGetSymbolAddress failed on device %d (%s)\n", dev, hipGetErrorString(e));
        return -1;
    }
    g_na_ptr[dev] = p;
    return 0;
}

}  // namespace lmhip

extern "C" {

// q8_matvec, shaders/q8_kernels.metal:10-42; dispatch src/nn/fast_metal.m:253-270.  W: rows x nb Q8_0 blocks.
void metal_enqueue_q8_matvec(MetalBuf *W, MetalBuf *x, MetalBuf *y, int rows, int nb)
{
    REQUIRE_BYTES(W, (size_t)rows * nb * 34, "q8_matvec");
    REQUIRE_BYTES(x, (size_t)nb * 32 * 4, "q8_matvec");
    REQUIRE_BYTES(y, (size_t)rows * 4, "q8_matvec");
    if (rows <= 0) return;
    if (nb <= 0) { zero_result(y, (size_t)rows); return; }
    if (!aligned16(dptr(x))) { fprintf(stderr, "[fast_hip] q8_matvec: x must be 16-byte aligned; launch skipped\n"); return; }
    const half_t *scales = nullptr;
    const int8_t *q = q8_split_of(W, rows, nb, &scales);
    launch_matvec<1>(q, scales, dptr_as<float>(x), dptr_as<float>(y), rows, nb * 32);
    mark_written(y);
}

// f16_matvec, shaders/q8_kernels.metal:97-127; dispatch src/nn/fast_metal.m:272-289.
void metal_enqueue_f16_matvec(MetalBuf *W, MetalBuf *x, MetalBuf *y, int rows, int cols)
{
    REQUIRE_BYTES(W, (size_t)rows * cols * 2, "f16_matvec");
    REQUIRE_BYTES(x, (size_t)cols * 4, "f16_matvec");
    REQUIRE_BYTES(y, (size_t)rows * 4, "f16_matvec");
    if (rows <= 0) return;
    if (cols <= 0) { zero_result(y, (size_t)rows); return; }
    if (cols % 8 || !aligned16(dptr(W)) || !aligned16(dptr(x)))
        LAUNCH(k_matvec_any, dim3((rows + 3) / 4), dim3(TB), 0, dptr_as<half_t>(W), dptr_as<float>(x), dptr_as<float>(y), rows, cols, 1);
    else launch_matvec<0>(dptr(W), nullptr, dptr_as<float>(x), dptr_as<float>(y), rows, cols);
    mark_written(y);
}

// f16_batch_matvec, shaders/q8_kernels.metal:49-91; dispatch src/nn/fast_metal.m:291-307.  Y[B, rows] = X[B, cols] W^T.
// The reference keeps 32 accumulators per lane and is undefined beyond; this one takes any B.  From two vectors on the
// product runs on the matrix cores over the tiled image of W, each fp32 vector split into two fp16 rows (value and
// rounding residual, each with its own power-of-two scale), which keeps 22 bits of every x.
void metal_enqueue_f16_batch_matvec(MetalBuf *W, MetalBuf *X, MetalBuf *Y, int rows, int cols, int B)
{
    if (B <= 0 || rows <= 0) return;
    REQUIRE_BYTES(W, (size_t)rows * cols * 2, "f16_batch_matvec");
    REQUIRE_BYTES(X, (size_t)B * cols * 4, "f16_batch_matvec");
    REQUIRE_BYTES(Y, (size_t)B * rows * 4, "f16_batch_matvec");
    if (cols <= 0) { zero_result(Y, (size_t)B * rows); return; }
    if (B == 1) { metal_enqueue_f16_matvec(W, X, Y, rows, cols); return; }
    gemm_f32a_exact(dptr_as<float>(X), W, dptr_as<float>(Y), B, rows, cols);
    mark_written(Y);
}

// rms_norm of one vector, dispatch src/nn/fast_metal.m:309-324
void metal_enqueue_rms_norm(MetalBuf *x, MetalBuf *gamma, MetalBuf *out, int dim, float eps)
{
    REQUIRE_BYTES(x, (size_t)dim * 4, "rms_norm");
    REQUIRE_BYTES(out, (size_t)dim * 4, "rms_norm");
    REQUIRE_BYTES(gamma, (size_t)dim * 4, "rms_norm");
    if (dim <= 0) return;
    LAUNCH(k_rms_norm1, dim3(1), dim3(TB), 0, dptr_as<float>(x), dptr_as<float>(gamma), dptr_as<float>(out), dim, eps);
    mark_written(out);
}

// per_head_rms_norm, shaders/q8_kernels.metal:165-189; dispatch src/nn/fast_metal.m:343-357, 468-483.  In place.
void metal_enqueue_per_head_rms_norm(MetalBuf *vec, MetalBuf *gamma, int n_heads, int head_dim, float eps)
{
    metal_enqueue_per_head_rms_norm_off(vec, 0, gamma, n_heads, head_dim, eps);
}

void metal_enqueue_per_head_rms_norm_off(MetalBuf *vec, size_t vec_off, MetalBuf *gamma, int n_heads, int head_dim, float eps)
{
    float *v = at_offset(vec, vec_off, (size_t)n_heads * head_dim * 4, "per_head_rms_norm");
    if (!v) return;
    per_head_rms_norm(v, gamma, n_heads, head_dim, eps, "per_head_rms_norm");
    mark_written(vec);
}

// rope, shaders/q8_kernels.metal:195-231; dispatch src/nn/fast_metal.m:359-379, 485-506.  In place on q and k.
void metal_enqueue_rope(MetalBuf *q, MetalBuf *k, int Hq, int Hkv, int hd, int pos, float theta)
{
    metal_enqueue_rope_off(q, 0, k, 0, Hq, Hkv, hd, pos, theta);
}

void metal_enqueue_rope_off(MetalBuf *q, size_t q_off, MetalBuf *k, size_t k_off, int Hq, int Hkv, int hd, int pos, float theta)
{
    float *qp = at_offset(q, q_off, (size_t)Hq * hd * 4, "rope");
    float *kp = at_offset(k, k_off, (size_t)Hkv * hd * 4, "rope");
    if (!qp || !kp) return;
    rope1(qp, kp, Hq, Hkv, hd, pos, theta);
    mark_written(q); mark_written(k);
}

// kv_cache_store, shaders/q8_kernels.metal:237-256; dispatch src/nn/fast_metal.m:381-402, 508-530.
void metal_enqueue_kv_cache_store(MetalBuf *k, MetalBuf *v, MetalBuf *k_cache, MetalBuf *v_cache, int Hkv, int max_seq, int hd, int pos)
{
    metal_enqueue_kv_cache_store_off(k, 0, v, 0, k_cache, v_cache, Hkv, max_seq, hd, pos);
}

void metal_enqueue_kv_cache_store_off(MetalBuf *k, size_t k_off, MetalBuf *v, size_t v_off, MetalBuf *k_cache, MetalBuf *v_cache,
                                      int Hkv, int max_seq, int hd, int pos)
{
    const float *kp = at_offset(k, k_off, (size_t)Hkv * hd * 4, "kv_cache_store");
    const float *vp = at_offset(v, v_off, (size_t)Hkv * hd * 4, "kv_cache_store");
    if (!kp || !vp) return;
    kv_store(kp, vp, k_cache, v_cache, Hkv, max_seq, hd, pos, "kv_cache_store");
}

// attention, shaders/q8_kernels.metal:262-331; dispatch src/nn/fast_metal.m:404-425, 532-556.
// Q, out: [Hq * hd]; caches [Hq / group_ratio, max_seq, hd]; attends keys 0 .. n_attend - 1.
void metal_enqueue_attention(MetalBuf *Q, MetalBuf *Kc, MetalBuf *Vc, MetalBuf *out, int n_attend, int hd, int max_seq, int Hq,
                             int group_ratio)
{
    metal_enqueue_attention_off(Q, 0, Kc, Vc, out, 0, n_attend, hd, max_seq, Hq, group_ratio);
}

void metal_enqueue_attention_off(MetalBuf *Q, size_t q_off, MetalBuf *Kc, MetalBuf *Vc, MetalBuf *out, size_t out_off, int n_attend,
                                 int hd, int max_seq, int Hq, int group_ratio)
{
    const float *qp = at_offset(Q, q_off, (size_t)Hq * hd * 4, "attention");
    float *op = at_offset(out, out_off, (size_t)Hq * hd * 4, "attention");
    if (!qp || !op) return;
    attention(qp, Kc, Vc, op, n_attend, hd, max_seq, Hq, group_ratio, "attention");
    mark_written(out);
}

// metal_enqueue_attention over plain device pointers, allocating nothing.  Q, out: [Hq * hd] fp32; caches
// [Hq / group_ratio, max_seq, hd] fp32; attends keys 0 .. n_attend - 1.  Same kernels and the same results as
// metal_enqueue_attention; the slice results of contexts beyond 256 keys go to the fixed per-device array above, which
// every call on a device shares and which keeps the last call's contents (every element a call reads it has written
// first, so nothing needs clearing).  Returns 0, or -1 with a message when a limit is exceeded (nothing launched).
int hip_attention_noalloc(const float *Q, const float *Kc, const float *Vc, float *out, int n_attend, int hd, int max_seq,
                          int Hq, int group_ratio)
{
    if (!initialized()) { fprintf(stderr, "[fast_hip] attention_noalloc before fast_metal_init\n"); return -1; }
    if (!Q || !Kc || !Vc || !out || Hq <= 0 || hd <= 0 || n_attend <= 0 || group_ratio <= 0 || Hq % group_ratio || n_attend > max_seq) {
        fprintf(stderr, "[fast_hip] attention_noalloc: bad arguments (Hq %d, group ratio %d, head_dim %d, n_attend %d, max_seq %d)\n",
                Hq, group_ratio, hd, n_attend, max_seq);
        return -1;
    }
    if (Hq > NA_MAX_HQ || hd > NA_MAX_HD || group_ratio > 16 || n_attend > NA_MAX_KEYS) {
        fprintf(stderr, "[fast_hip] attention_noalloc: at most %d query heads, head_dim %d, group ratio 16 and %d keys (got %d, %d, %d, %d)\n",
                NA_MAX_HQ, NA_MAX_HD, NA_MAX_KEYS, Hq, hd, group_ratio, n_attend);
        return -1;
    }
    if (attention_partial_floats(Hq, hd, n_attend) > NA_FLOATS) return -1;      // cannot happen within the limits above
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= NA_MAX_DEVICES) return -1;
    if (!g_na_ptr[dev] && noalloc_setup() != 0) return -1;
    attention_launch(Q, Kc, Vc, out, g_na_ptr[dev], n_attend, hd, max_seq, Hq, group_ratio, nullptr);
    return 0;
}

// Microbenchmark of the matrix-vector kernels alone: average ms per launch over `iters` launches that rotate through
// more than 1 GB of distinct weights, so that no launch finds its weights in a cache.  fmt 0: F16 rows (B vectors,
// fmt 1: the split Q8_0 image.  B must be 1 (batches run on the GEMM, see hip_gemm_time_shape).
double hip_matvec_time_shape(int rows, int cols, int fmt, int B, int iters)
{
    if (rows <= 0 || cols <= 0 || cols % 32 || B != 1 || iters <= 0) return -1.0;
    const size_t wb = ((fmt == 1 ? q8_scale_offset((size_t)rows * (cols / 32)) + (size_t)rows * (cols / 32) * 2
                                 : (size_t)rows * cols * 2) + 255) & ~(size_t)255;
    const int nbuf = (int)((size_t)1200 * 1024 * 1024 / wb) + 1;
    void *W = nullptr, *X = nullptr, *Y = nullptr;
    HIP_CHECK(hipMalloc(&W, wb * nbuf)); HIP_CHECK(hipMalloc(&X, (size_t)B * cols * 4)); HIP_CHECK(hipMalloc(&Y, (size_t)B * rows * 4));
    HIP_CHECK(hipMemsetAsync(W, 0x11, wb * nbuf, stream()));
    HIP_CHECK(hipMemsetAsync(X, 0, (size_t)B * cols * 4, stream()));
    auto run = [&](int i) {
        const char *w = (const char *)W + (size_t)(i % nbuf) * wb;
        if (fmt == 1)
            launch_matvec<1>(w, (const half_t *)(w + q8_scale_offset((size_t)rows * (cols / 32))), (const float *)X, (float *)Y,
                             rows, cols);
        else launch_matvec<0>(w, nullptr, (const float *)X, (float *)Y, rows, cols);
    };
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0)); HIP_CHECK(hipEventCreate(&e1));
    for (int i = 0; i < 3; i++) run(i);
    HIP_CHECK(hipEventRecord(e0, stream()));
    for (int i = 0; i < iters; i++) run(i + 3);
    HIP_CHECK(hipEventRecord(e1, stream()));
    HIP_CHECK(hipStreamSynchronize(stream()));
    float ms = 0;
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    hipEventDestroy(e0); hipEventDestroy(e1);
    hipFree(W); hipFree(X); hipFree(Y);
    return (double)ms / iters;
}

}  // extern "C"

namespace lmhip {

// The gate|up product of the FFN with the gate applied in its epilogue: W = [gate; up] ([2 * rows, cols], F16 rows or
// Q8_0 blocks), y[i] = act(gate_i . x) * (up_i . x).  What metal_enqueue_*_matvec followed by metal_enqueue_silu_mul /
// gelu_mul computes (src/nn/fast_inference.c:441-452), in one launch and without the [2 * rows] intermediate.
void matvec_glu(MetalBuf *W, MetalBuf *x, MetalBuf *y, int rows, int cols, int q8, int gelu)
{
    if (rows <= 0 || cols <= 0 || (cols & 31) || !aligned16(dptr(W)) || !aligned16(dptr(x))) {
        fprintf(stderr, "[fast_hip] matvec_glu: unsupported shape %d x %d\n", rows, cols); abort();
    }
    REQUIRE_BYTES(x, (size_t)cols * 4, "matvec_glu");
    REQUIRE_BYTES(y, (size_t)rows * 4, "matvec_glu");
    if (q8) {
        REQUIRE_BYTES(W, (size_t)2 * rows * (cols / 32) * 34, "matvec_glu");
        const half_t *scales = nullptr;
        const int8_t *q = q8_split_of(W, 2 * rows, cols / 32, &scales);
        launch_matvec_glu<1>(q, scales, dptr_as<float>(x), dptr_as<float>(y), rows, cols, gelu);
    } else {
        REQUIRE_BYTES(W, (size_t)2 * rows * cols * 2, "matvec_glu");
        launch_matvec_glu<0>(dptr(W), nullptr, dptr_as<float>(x), dptr_as<float>(y), rows, cols, gelu);
    }
    mark_written(y);
}

// The same products (glu 0: y[i] = W_i . ln for `rows` rows) over ln = RMSNorm(xr + br; g), the sum and the norm formed
// inside the launch: what k_add_norm followed by a matrix-vector product computes, src/nn/fast_inference.c:386-398,
// 437-452.  nin.x_out receives xr + br and must not be xr.
void matvec_norm(MetalBuf *W, const NormIn &nin, MetalBuf *y, int rows, int cols, int q8, int glu)
{
    if (rows <= 0 || cols <= 0 || (cols & 31) || cols > 12288 || !aligned16(dptr(W)) || !nin.xr || !nin.g || nin.x_out == nin.xr ||
        !aligned16(nin.xr) || !aligned16(nin.g) || (nin.br && !aligned16(nin.br)) || (nin.x_out && !aligned16(nin.x_out))) {
        fprintf(stderr, "[fast_hip] matvec_norm: unsupported shape %d x %d or operands\n", rows, cols); abort();
    }
    const int wrows = glu ? 2 * rows : rows;
    REQUIRE_BYTES(y, (size_t)rows * 4, "matvec_norm");
    if (q8) {
        REQUIRE_BYTES(W, (size_t)wrows * (cols / 32) * 34, "matvec_norm");
        const half_t *scales = nullptr;
        const int8_t *q = q8_split_of(W, wrows, cols / 32, &scales);
        launch_matvec_norm<1>(q, scales, nin, dptr_as<float>(y), rows, cols, glu);
    } else {
        REQUIRE_BYTES(W, (size_t)wrows * cols * 2, "matvec_norm");
        launch_matvec_norm<0>(dptr(W), nullptr, nin, dptr_as<float>(y), rows, cols, glu);
    }
    mark_written(y);
}

void attention_decode_fused(const HeadPost &hp, MetalBuf *Kc, MetalBuf *Vc, float *out, int hd, int max_seq, int copies)
{
    if (hp.Hkv <= 0 || hp.Hq % hp.Hkv || (hd & 1) || hp.pos < 0 || hp.pos >= max_seq || copies < 1 || copies > 65535 ||
        (copies > 1 && (hp.cache_step != (size_t)hp.Hkv * max_seq * hd || hp.qkv_step < (size_t)(hp.Hq + 2 * hp.Hkv) * hd))) {
        fprintf(stderr, "[fast_hip] attention_decode_fused: unsupported shape\n"); abort();
    }
    attention(hp.qkv, Kc, Vc, out, hp.pos + 1, hd, max_seq, hp.Hq, hp.Hq / hp.Hkv, "attention_decode_fused", &hp, copies);
    mark_written(Kc); mark_written(Vc);
}

}  // namespace lmhip
