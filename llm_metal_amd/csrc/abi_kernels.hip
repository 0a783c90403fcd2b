// The training enqueues of the reference's dispatch ABI (src/nn/fast_metal.h:36-188)
// as HIP kernels with the reference's buffer layouts and per-kernel arithmetic
// (shaders/q8_kernels.metal).  All activations fp32.  Row reductions use wave64
// shuffles and are exact sums for every row length (the reference's LDS tree
// drops elements when its group size is not a power of two).  Every elementwise
// kernel bounds-checks (the reference launches some of them past the end).
#include "backend.h"
#include "devutil.h"
#include "gemm.h"

using namespace lmhip;

namespace {

constexpr int TB = 256;
inline unsigned blocks_for(size_t n) { return (unsigned)((n + TB - 1) / TB); }

// ---------------------------------------------------------------- row ops

// rms_norm, shaders/q8_kernels.metal:133-158.  One workgroup per row; out may alias x.
__global__ __launch_bounds__(TB) void k_rms_norm(const float *x, const float *__restrict__ gamma, float *out,
                                                 int dim, float eps)
{
    __shared__ float sm[16];
    const size_t off = (size_t)blockIdx.x * dim;
    float ss = 0.f;
    for (int i = threadIdx.x; i < dim; i += TB) { float v = x[off + i]; ss += v * v; }
    ss = block_sum(ss, sm);
    const float inv = rsqrtf(ss / (float)dim + eps);
    for (int i = threadIdx.x; i < dim; i += TB) out[off + i] = x[off + i] * inv * gamma[i];
}

// Short rows (per-head QK norm, dim <= 256): one wave per row, four rows per workgroup.
__global__ __launch_bounds__(TB) void k_rms_norm_wave(const float *x, const float *__restrict__ gamma, float *out,
                                                      int dim, float eps, int rows)
{
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= rows) return;
    const size_t off = (size_t)row * dim;
    float ss = 0.f;
    for (int i = lane; i < dim; i += 64) { float v = x[off + i]; ss += v * v; }
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss / (float)dim + eps);
    for (int i = lane; i < dim; i += 64) out[off + i] = x[off + i] * inv * gamma[i];
}

// rms_norm_train_backward, shaders/q8_kernels.metal:584-625.  dx may alias dy.
__global__ __launch_bounds__(TB) void k_rms_norm_bwd(const float *__restrict__ x, const float *dy,
                                                     const float *__restrict__ gamma, float *dx, int dim, float eps)
{
    __shared__ float sm[16];
    const size_t off = (size_t)blockIdx.x * dim;
    float ss = 0.f, dot = 0.f;
    for (int i = threadIdx.x; i < dim; i += TB) {
        float v = x[off + i];
        ss += v * v;
        dot += dy[off + i] * gamma[i] * v;
    }
    ss = block_sum(ss, sm);
    dot = block_sum(dot, sm);
    const float inv = rsqrtf(ss / (float)dim + eps);
    const float coeff = dot * inv * inv / (float)dim;
    for (int i = threadIdx.x; i < dim; i += TB)
        dx[off + i] = (gamma[i] * dy[off + i] - coeff * x[off + i]) * inv;
}

__global__ __launch_bounds__(TB) void k_rms_norm_bwd_wave(const float *__restrict__ x, const float *dy,
                                                          const float *__restrict__ gamma, float *dx,
                                                          int dim, float eps, int rows)
{
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= rows) return;
    const size_t off = (size_t)row * dim;
    float ss = 0.f, dot = 0.f;
    for (int i = lane; i < dim; i += 64) {
        float v = x[off + i];
        ss += v * v;
        dot += dy[off + i] * gamma[i] * v;
    }
    ss = wave_sum(ss);
    dot = wave_sum(dot);
    const float inv = rsqrtf(ss / (float)dim + eps);
    const float coeff = dot * inv * inv / (float)dim;
    for (int i = lane; i < dim; i += 64)
        dx[off + i] = (gamma[i] * dy[off + i] - coeff * x[off + i]) * inv;
}

// softmax_ce_train, shaders/q8_kernels.metal:646-690 (dlogits unscaled).
__global__ __launch_bounds__(1024) void k_softmax_ce(const float *__restrict__ logits, const uint32_t *__restrict__ targets,
                                                     float *__restrict__ losses, float *__restrict__ dlogits, int V)
{
    __shared__ float sm[16];
    const size_t off = (size_t)blockIdx.x * V;
    const uint32_t tgt = targets[blockIdx.x];
    float mx = -1e30f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) mx = fmaxf(mx, logits[off + i]);
    mx = block_max(mx, sm);
    float sum = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) sum += expf(logits[off + i] - mx);
    sum = block_sum(sum, sm);
    const float lse = logf(sum) + mx;
    if (threadIdx.x == 0) losses[blockIdx.x] = lse - logits[off + tgt];
    for (int i = threadIdx.x; i < V; i += blockDim.x)
        dlogits[off + i] = expf(logits[off + i] - lse) - ((uint32_t)i == tgt ? 1.0f : 0.0f);
}

// grpo_policy_grad, shaders/q8_kernels.metal:698-761.
__global__ __launch_bounds__(1024) void k_grpo_policy_grad(const float *__restrict__ logits, const uint32_t *__restrict__ actions,
                                                           const float *__restrict__ old_lp, const float *__restrict__ advs,
                                                           float *__restrict__ new_lp, float *__restrict__ dlogits,
                                                           int V, float clip_eps)
{
    __shared__ float sm[16];
    const size_t off = (size_t)blockIdx.x * V;
    const uint32_t act = actions[blockIdx.x];
    float mx = -1e30f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) mx = fmaxf(mx, logits[off + i]);
    mx = block_max(mx, sm);
    float sum = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) sum += expf(logits[off + i] - mx);
    sum = block_sum(sum, sm);
    const float lse = logf(sum) + mx;
    const float lp = logits[off + act] - lse;
    if (threadIdx.x == 0) new_lp[blockIdx.x] = lp;
    const float ratio = expf(lp - old_lp[blockIdx.x]);
    const float clipped = fminf(fmaxf(ratio, 1.0f - clip_eps), 1.0f + clip_eps);
    const float adv = advs[blockIdx.x];
    float w;
    if (adv >= 0) w = (ratio <= clipped) ? -adv : 0.0f;
    else          w = (ratio >= clipped) ? -adv : 0.0f;
    for (int i = threadIdx.x; i < V; i += blockDim.x)
        dlogits[off + i] = w * ratio * (expf(logits[off + i] - lse) - ((uint32_t)i == act ? 1.0f : 0.0f));
}

// ---------------------------------------------------------------- layout ops

// transpose_heads_fwd/_rev, shaders/q8_kernels.metal:438-474: [N, H*D] <-> [H, N, D]
__global__ void k_transpose_heads(const float *__restrict__ src, float *__restrict__ dst, int N, int H, int D, int rev)
{
    const size_t idx = (size_t)blockIdx.x * TB + threadIdx.x;
    if (idx >= (size_t)N * H * D) return;
    const int d = idx % D;
    const size_t t = idx / D;
    // idx enumerates the [N, H, D] order
    const int h = t % H, n = (int)(t / H);
    const size_t hnd = ((size_t)h * N + n) * D + d;
    if (rev) dst[idx] = src[hnd]; else dst[hnd] = src[idx];
}

// repeat_kv, shaders/q8_kernels.metal:476-492
__global__ void k_repeat_kv(const float *__restrict__ src, float *__restrict__ dst, size_t ND, int n_q, int ratio)
{
    const size_t idx = (size_t)blockIdx.x * TB + threadIdx.x;
    if (idx >= ND * n_q) return;
    const size_t hq = idx / ND, rem = idx % ND;
    dst[idx] = src[(hq / ratio) * ND + rem];
}

// repeat_kv_bwd, shaders/q8_kernels.metal:973-992
__global__ void k_repeat_kv_bwd(const float *__restrict__ dexp, float *__restrict__ dkv, size_t ND, int n_kv, int ratio)
{
    const size_t idx = (size_t)blockIdx.x * TB + threadIdx.x;
    if (idx >= ND * n_kv) return;
    const size_t hkv = idx / ND, rem = idx % ND;
    float s = 0.f;
    for (int g = 0; g < ratio; g++) s += dexp[(hkv * ratio + g) * ND + rem];
    dkv[idx] = s;
}

// rope_train / rope_train_bwd, shaders/q8_kernels.metal:495-538, 997-1038.
// One thread per (head, position, pair) over q then k; sign = +1 forward, -1 inverse.
__global__ void k_rope_train(float *q, float *k, int Hq, int Hkv, int hd, int N, float theta, float sign)
{
    const int half = hd / 2;
    const size_t q_total = (size_t)Hq * N * half, total = q_total + (size_t)Hkv * N * half;
    size_t idx = (size_t)blockIdx.x * TB + threadIdx.x;
    if (idx >= total) return;
    float *base = q;
    if (idx >= q_total) { idx -= q_total; base = k; }
    const int d = idx % half;
    const size_t t = idx / half;
    const int pos = t % N;
    float *vec = base + t * hd;                         // t = head * N + pos
    const float freq = 1.0f / powf(theta, (float)(2 * d) / (float)hd);
    const float ang = (float)pos * freq;
    float s, c;
    sincosf(ang, &s, &c);
    s *= sign;
    const float x0 = vec[d], x1 = vec[d + half];
    vec[d] = x0 * c - x1 * s;
    vec[d + half] = x0 * s + x1 * c;
}

// ---------------------------------------------------------------- attention (probs-saving form)

// attn_train_fwd, shaders/q8_kernels.metal:769-851: one wave per (head, query).
// Lane j owns keys j, j+64, ...; scores live in LDS (N <= 4096 as in the reference).
__global__ __launch_bounds__(64) void k_attn_train_fwd(const float *__restrict__ Q, const float *__restrict__ K,
                                                       const float *__restrict__ V, float *__restrict__ out,
                                                       float *__restrict__ probs, int N, int D, float scale)
{
    extern __shared__ float sc[];                        // [N] scores then probs, [D] query
    float *qs = sc + N;
    const int h = blockIdx.x, i = blockIdx.y, lane = threadIdx.x;
    const size_t ND = (size_t)N * D;
    const float *q = Q + h * ND + (size_t)i * D;
    for (int d = lane; d < D; d += 64) qs[d] = q[d];
    __syncthreads();
    float mx = -1e30f;
    for (int j = lane; j <= i; j += 64) {
        const float *kr = K + h * ND + (size_t)j * D;
        float dot = 0.f;
        for (int d = 0; d < D; d++) dot += qs[d] * kr[d];
        dot *= scale;
        sc[j] = dot;
        mx = fmaxf(mx, dot);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int j = lane; j <= i; j += 64) { float e = expf(sc[j] - mx); sc[j] = e; sum += e; }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
    float *pr = probs + ((size_t)h * N + i) * N;
    for (int j = lane; j < N; j += 64) {
        const float p = (j <= i) ? sc[j] * inv : 0.f;
        sc[j] = p;
        pr[j] = p;
    }
    __syncthreads();
    for (int d = lane; d < D; d += 64) {
        float acc = 0.f;
        for (int j = 0; j <= i; j++) acc += sc[j] * V[h * ND + (size_t)j * D + d];
        out[h * ND + (size_t)i * D + d] = acc;
    }
}

// attn_bwd_dq, shaders/q8_kernels.metal:857-925
__global__ __launch_bounds__(64) void k_attn_bwd_dq(const float *__restrict__ dO, const float *__restrict__ probs,
                                                    const float *__restrict__ V, const float *__restrict__ K,
                                                    float *__restrict__ dscore, float *__restrict__ dQ,
                                                    int N, int D, float scale)
{
    extern __shared__ float dr[];                        // [N] d_raw then ds, [D] dO row
    float *dos = dr + N;
    const int h = blockIdx.x, i = blockIdx.y, lane = threadIdx.x;
    const size_t ND = (size_t)N * D;
    const float *pr = probs + ((size_t)h * N + i) * N;
    for (int d = lane; d < D; d += 64) dos[d] = dO[h * ND + (size_t)i * D + d];
    __syncthreads();
    float dp = 0.f;
    for (int j = lane; j <= i; j += 64) {
        const float *vr = V + h * ND + (size_t)j * D;
        float dot = 0.f;
        for (int d = 0; d < D; d++) dot += dos[d] * vr[d];
        dr[j] = dot;
        dp += pr[j] * dot;
    }
    dp = wave_sum(dp);
    float *ds = dscore + ((size_t)h * N + i) * N;
    for (int j = lane; j < N; j += 64) {
        const float v = (j <= i) ? pr[j] * (dr[j] - dp) * scale : 0.f;
        dr[j] = v;
        ds[j] = v;
    }
    __syncthreads();
    for (int d = lane; d < D; d += 64) {
        float acc = 0.f;
        for (int j = 0; j <= i; j++) acc += dr[j] * K[h * ND + (size_t)j * D + d];
        dQ[h * ND + (size_t)i * D + d] = acc;
    }
}

// attn_bwd_dkv, shaders/q8_kernels.metal:931-968: one wave per (head, key j)
__global__ __launch_bounds__(64) void k_attn_bwd_dkv(const float *__restrict__ dscore, const float *__restrict__ Q,
                                                     const float *__restrict__ probs, const float *__restrict__ dO,
                                                     float *__restrict__ dK, float *__restrict__ dV, int N, int D)
{
    const int h = blockIdx.x, j = blockIdx.y, lane = threadIdx.x;
    const size_t ND = (size_t)N * D, NN = (size_t)N * N;
    for (int d = lane; d < D; d += 64) {
        float dk = 0.f, dv = 0.f;
        for (int i = j; i < N; i++) {
            const float ds = dscore[h * NN + (size_t)i * N + j];
            const float p = probs[h * NN + (size_t)i * N + j];
            dk += ds * Q[h * ND + (size_t)i * D + d];
            dv += p * dO[h * ND + (size_t)i * D + d];
        }
        dK[h * ND + (size_t)j * D + d] = dk;
        dV[h * ND + (size_t)j * D + d] = dv;
    }
}

// ---------------------------------------------------------------- elementwise

__global__ void k_silu_mul(float *gate, const float *__restrict__ up, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n) return;
    const float g = gate[i];
    gate[i] = (g / (1.0f + expf(-g))) * up[i];
}

__global__ void k_gelu_mul(float *gate, const float *__restrict__ up, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n) return;
    const float g = gate[i];
    gate[i] = 0.5f * g * (1.0f + tanhf(gelu_inner(g))) * up[i];
}

__global__ void k_silu_mul_bwd(const float *dout, const float *__restrict__ gate, const float *__restrict__ up,
                               float *dgate, float *dup, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n) return;
    const float g = gate[i], u = up[i], dy = dout[i];
    const float sig = 1.0f / (1.0f + expf(-g));
    dgate[i] = dy * u * (sig * (1.0f + g * (1.0f - sig)));
    dup[i] = dy * (g * sig);
}

__global__ void k_gelu_mul_bwd(const float *dout, const float *__restrict__ gate, const float *__restrict__ up,
                               float *dgate, float *dup, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n) return;
    const float g = gate[i], u = up[i], dy = dout[i];
    const float t = tanhf(gelu_inner(g));
    const float gelu = 0.5f * g * (1.0f + t);
    const float grad = 0.5f * (1.0f + t) + 0.5f * g * (1.0f - t * t) * 0.7978845608f * (1.0f + 3.0f * 0.044715f * g * g);
    dgate[i] = dy * u * grad;
    dup[i] = dy * gelu;
}

__global__ void k_residual_add(float *x, const float *__restrict__ y, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i < n) x[i] += y[i];
}
__global__ void k_scale(float *x, float a, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i < n) x[i] *= a;
}
__global__ void k_add_scaled(float *y, const float *__restrict__ x, float a, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i < n) y[i] += a * x[i];
}
__global__ void k_clamp(float *x, float mx, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i < n) x[i] = fminf(fmaxf(x[i], -mx), mx);
}
__global__ void k_copy(const float *__restrict__ s, float *__restrict__ d, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i < n) d[i] = s[i];
}

// ---------------------------------------------------------------- small fp32 products (LoRA)

// C[M,N] = sum_k opA(m,k) * opB(k,n): strides select the three orientations of
// float_matmul / _tn / _nt (shaders/q8_kernels.metal:1043-1152).  16x16 tiles.
__global__ __launch_bounds__(256) void k_float_matmul(const float *__restrict__ A, size_t a_sm, size_t a_sk,
                                                      const float *__restrict__ B, size_t b_sk, size_t b_sn,
                                                      float *__restrict__ C, int M, int N, int K)
{
    __shared__ float tA[16][17], tB[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int row = blockIdx.y * 16 + ty, col = blockIdx.x * 16 + tx;
    float s = 0.f;
    for (int t = 0; t < K; t += 16) {
        tA[ty][tx] = (row < M && t + tx < K) ? A[row * a_sm + (size_t)(t + tx) * a_sk] : 0.f;
        tB[ty][tx] = (col < N && t + ty < K) ? B[(size_t)(t + ty) * b_sk + col * b_sn] : 0.f;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; k++) s += tA[ty][k] * tB[k][tx];
        __syncthreads();
    }
    if (row < M && col < N) C[(size_t)row * N + col] = s;
}

// The F16 update rules below are separate fp32 operations (multiply, add, one rounding to F16);
// a fused multiply-add would change results at rounding ties.
#pragma clang fp contract(off)

// f16_sgd_fused / f16_grad_accum, shaders/q8_kernels.metal:1097-1125, 1164-1190:
// T[M,N] (F16) = half(float(T) + alpha * sum_k dY[k,M] X[k,N])
__global__ __launch_bounds__(256) void k_f16_rank_update(half_t *__restrict__ T, const float *__restrict__ dY,
                                                         const float *__restrict__ X, int M, int K, int N, float alpha)
{
    __shared__ float tA[16][17], tB[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int row = blockIdx.y * 16 + ty, col = blockIdx.x * 16 + tx;
    float s = 0.f;
    for (int t = 0; t < K; t += 16) {
        tA[ty][tx] = (row < M && t + tx < K) ? dY[(size_t)(t + tx) * M + row] : 0.f;
        tB[ty][tx] = (col < N && t + ty < K) ? X[(size_t)(t + ty) * N + col] : 0.f;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; k++) s += tA[ty][k] * tB[k][tx];
        __syncthreads();
    }
    if (row < M && col < N) {
        const size_t idx = (size_t)row * N + col;
        T[idx] = f2h(h2f(T[idx]) + alpha * s);
    }
}

// f16_sgd_apply, shaders/q8_kernels.metal:1195-1206
__global__ void k_f16_sgd_apply(half_t *__restrict__ W, half_t *__restrict__ G, size_t n, float lr)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n) return;
    W[i] = f2h(h2f(W[i]) - lr * h2f(G[i]));
    G[i] = (half_t)0;
}

#define LAUNCH(kern, grid, block, lds, ...) do { \
    hipLaunchKernelGGL(kern, grid, block, lds, stream(), __VA_ARGS__); HIP_CHECK(hipGetLastError()); } while (0)

}  // namespace

extern "C" {

void metal_enqueue_rms_norm_batched(MetalBuf *x, MetalBuf *gamma, MetalBuf *out, int dim, float eps, int B)
{
    REQUIRE_BYTES(x, (size_t)B * dim * 4, "rms_norm_batched");
    REQUIRE_BYTES(out, (size_t)B * dim * 4, "rms_norm_batched");
    REQUIRE_BYTES(gamma, (size_t)dim * 4, "rms_norm_batched");
    if (B <= 0) return;
    if (dim <= 256) LAUNCH(k_rms_norm_wave, dim3((B + 3) / 4), dim3(TB), 0, dptr_as<float>(x), dptr_as<float>(gamma),
                           dptr_as<float>(out), dim, eps, B);
    else LAUNCH(k_rms_norm, dim3(B), dim3(TB), 0, dptr_as<float>(x), dptr_as<float>(gamma), dptr_as<float>(out), dim, eps);
    mark_written(out);
}

void metal_enqueue_rms_norm_backward(MetalBuf *x, MetalBuf *dy, MetalBuf *gamma, MetalBuf *dx, int batch, int dim, float eps)
{
    REQUIRE_BYTES(x, (size_t)batch * dim * 4, "rms_norm_backward");
    REQUIRE_BYTES(dy, (size_t)batch * dim * 4, "rms_norm_backward");
    REQUIRE_BYTES(dx, (size_t)batch * dim * 4, "rms_norm_backward");
    REQUIRE_BYTES(gamma, (size_t)dim * 4, "rms_norm_backward");
    if (batch <= 0) return;
    if (dim <= 256) LAUNCH(k_rms_norm_bwd_wave, dim3((batch + 3) / 4), dim3(TB), 0, dptr_as<float>(x), dptr_as<float>(dy),
                           dptr_as<float>(gamma), dptr_as<float>(dx), dim, eps, batch);
    else LAUNCH(k_rms_norm_bwd, dim3(batch), dim3(TB), 0, dptr_as<float>(x), dptr_as<float>(dy), dptr_as<float>(gamma),
                dptr_as<float>(dx), dim, eps);
    mark_written(dx);
}

void metal_enqueue_softmax_ce(MetalBuf *logits, MetalBuf *targets, MetalBuf *losses, MetalBuf *dlogits, int batch, int V)
{
    REQUIRE_BYTES(logits, (size_t)batch * V * 4, "softmax_ce");
    REQUIRE_BYTES(dlogits, (size_t)batch * V * 4, "softmax_ce");
    REQUIRE_BYTES(targets, (size_t)batch * 4, "softmax_ce");
    REQUIRE_BYTES(losses, (size_t)batch * 4, "softmax_ce");
    if (batch <= 0) return;
    LAUNCH(k_softmax_ce, dim3(batch), dim3(V >= 4096 ? 1024 : 256), 0, dptr_as<float>(logits), dptr_as<uint32_t>(targets),
           dptr_as<float>(losses), dptr_as<float>(dlogits), V);
    mark_written(losses); mark_written(dlogits);
}

void metal_enqueue_grpo_policy_grad(MetalBuf *logits, MetalBuf *actions, MetalBuf *old_lp, MetalBuf *advs,
                                    MetalBuf *new_lp, MetalBuf *dlogits, int N, int V, float clip_eps)
{
    REQUIRE_BYTES(logits, (size_t)N * V * 4, "grpo_policy_grad");
    REQUIRE_BYTES(dlogits, (size_t)N * V * 4, "grpo_policy_grad");
    REQUIRE_BYTES(actions, (size_t)N * 4, "grpo_policy_grad");
    REQUIRE_BYTES(old_lp, (size_t)N * 4, "grpo_policy_grad");
    REQUIRE_BYTES(advs, (size_t)N * 4, "grpo_policy_grad");
    REQUIRE_BYTES(new_lp, (size_t)N * 4, "grpo_policy_grad");
    if (N <= 0) return;
    LAUNCH(k_grpo_policy_grad, dim3(N), dim3(V >= 4096 ? 1024 : 256), 0, dptr_as<float>(logits), dptr_as<uint32_t>(actions),
           dptr_as<float>(old_lp), dptr_as<float>(advs), dptr_as<float>(new_lp), dptr_as<float>(dlogits), V, clip_eps);
    mark_written(new_lp); mark_written(dlogits);
}

static void transpose_heads(MetalBuf *src, MetalBuf *dst, int N, int H, int D, int rev, const char *fn)
{
    const size_t n = (size_t)N * H * D;
    REQUIRE_BYTES(src, n * 4, fn);
    REQUIRE_BYTES(dst, n * 4, fn);
    if (!n) return;
    LAUNCH(k_transpose_heads, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(src), dptr_as<float>(dst), N, H, D, rev);
    mark_written(dst);
}
void metal_enqueue_transpose_heads_fwd(MetalBuf *src, MetalBuf *dst, int N, int H, int D) { transpose_heads(src, dst, N, H, D, 0, "transpose_heads_fwd"); }
void metal_enqueue_transpose_heads_rev(MetalBuf *src, MetalBuf *dst, int N, int H, int D) { transpose_heads(src, dst, N, H, D, 1, "transpose_heads_rev"); }

void metal_enqueue_repeat_kv(MetalBuf *src, MetalBuf *dst, int n_kv, int N, int D, int ratio)
{
    const size_t ND = (size_t)N * D;
    REQUIRE_BYTES(src, ND * n_kv * 4, "repeat_kv");
    REQUIRE_BYTES(dst, ND * n_kv * ratio * 4, "repeat_kv");
    if (!ND || n_kv * ratio <= 0) return;
    LAUNCH(k_repeat_kv, dim3(blocks_for(ND * n_kv * ratio)), dim3(TB), 0, dptr_as<float>(src), dptr_as<float>(dst), ND, n_kv * ratio, ratio);
    mark_written(dst);
}

void metal_enqueue_repeat_kv_bwd(MetalBuf *dexp, MetalBuf *dkv, int n_kv, int N, int D, int ratio)
{
    const size_t ND = (size_t)N * D;
    REQUIRE_BYTES(dexp, ND * n_kv * ratio * 4, "repeat_kv_bwd");
    REQUIRE_BYTES(dkv, ND * n_kv * 4, "repeat_kv_bwd");
    if (!ND || n_kv <= 0) return;
    LAUNCH(k_repeat_kv_bwd, dim3(blocks_for(ND * n_kv)), dim3(TB), 0, dptr_as<float>(dexp), dptr_as<float>(dkv), ND, n_kv, ratio);
    mark_written(dkv);
}

static void rope(MetalBuf *q, MetalBuf *k, int Hq, int Hkv, int hd, int N, float theta, float sign, const char *fn)
{
    REQUIRE_BYTES(q, (size_t)Hq * N * hd * 4, fn);
    REQUIRE_BYTES(k, (size_t)Hkv * N * hd * 4, fn);
    const size_t total = (size_t)(Hq + Hkv) * N * (hd / 2);
    if (!total) return;
    LAUNCH(k_rope_train, dim3(blocks_for(total)), dim3(TB), 0, dptr_as<float>(q), dptr_as<float>(k), Hq, Hkv, hd, N, theta, sign);
    mark_written(q); mark_written(k);
}
void metal_enqueue_rope_train(MetalBuf *q, MetalBuf *k, int Hq, int Hkv, int hd, int N, float theta) { rope(q, k, Hq, Hkv, hd, N, theta, 1.0f, "rope_train"); }
void metal_enqueue_rope_train_bwd(MetalBuf *q, MetalBuf *k, int Hq, int Hkv, int hd, int N, float theta) { rope(q, k, Hq, Hkv, hd, N, theta, -1.0f, "rope_train_bwd"); }

void metal_enqueue_attn_train_fwd(MetalBuf *Q, MetalBuf *K, MetalBuf *V, MetalBuf *out, MetalBuf *probs,
                                  int H, int N, int D, float scale)
{
    const size_t hnd = (size_t)H * N * D * 4;
    REQUIRE_BYTES(Q, hnd, "attn_train_fwd"); REQUIRE_BYTES(K, hnd, "attn_train_fwd"); REQUIRE_BYTES(V, hnd, "attn_train_fwd");
    REQUIRE_BYTES(out, hnd, "attn_train_fwd"); REQUIRE_BYTES(probs, (size_t)H * N * N * 4, "attn_train_fwd");
    if (H <= 0 || N <= 0) return;
    if (N > 4096) { fprintf(stderr, "[fast_hip] attn_train_fwd: N=%d exceeds 4096\n", N); return; }
    LAUNCH(k_attn_train_fwd, dim3(H, N), dim3(64), (size_t)(N + D) * 4, dptr_as<float>(Q), dptr_as<float>(K), dptr_as<float>(V),
           dptr_as<float>(out), dptr_as<float>(probs), N, D, scale);
    mark_written(out); mark_written(probs);
}

void metal_enqueue_attn_bwd_dq(MetalBuf *d_out, MetalBuf *probs, MetalBuf *V, MetalBuf *K, MetalBuf *d_score, MetalBuf *dQ,
                               int H, int N, int D, float scale)
{
    const size_t hnd = (size_t)H * N * D * 4, hnn = (size_t)H * N * N * 4;
    REQUIRE_BYTES(d_out, hnd, "attn_bwd_dq"); REQUIRE_BYTES(V, hnd, "attn_bwd_dq"); REQUIRE_BYTES(K, hnd, "attn_bwd_dq");
    REQUIRE_BYTES(dQ, hnd, "attn_bwd_dq"); REQUIRE_BYTES(probs, hnn, "attn_bwd_dq"); REQUIRE_BYTES(d_score, hnn, "attn_bwd_dq");
    if (H <= 0 || N <= 0) return;
    if (N > 4096) { fprintf(stderr, "[fast_hip] attn_bwd_dq: N=%d exceeds 4096\n", N); return; }
    LAUNCH(k_attn_bwd_dq, dim3(H, N), dim3(64), (size_t)(N + D) * 4, dptr_as<float>(d_out), dptr_as<float>(probs), dptr_as<float>(V),
           dptr_as<float>(K), dptr_as<float>(d_score), dptr_as<float>(dQ), N, D, scale);
    mark_written(d_score); mark_written(dQ);
}

void metal_enqueue_attn_bwd_dkv(MetalBuf *d_score, MetalBuf *Q, MetalBuf *probs, MetalBuf *d_out, MetalBuf *dK, MetalBuf *dV,
                                int H, int N, int D)
{
    const size_t hnd = (size_t)H * N * D * 4, hnn = (size_t)H * N * N * 4;
    REQUIRE_BYTES(d_out, hnd, "attn_bwd_dkv"); REQUIRE_BYTES(Q, hnd, "attn_bwd_dkv"); REQUIRE_BYTES(dK, hnd, "attn_bwd_dkv");
    REQUIRE_BYTES(dV, hnd, "attn_bwd_dkv"); REQUIRE_BYTES(probs, hnn, "attn_bwd_dkv"); REQUIRE_BYTES(d_score, hnn, "attn_bwd_dkv");
    if (H <= 0 || N <= 0) return;
    LAUNCH(k_attn_bwd_dkv, dim3(H, N), dim3(64), 0, dptr_as<float>(d_score), dptr_as<float>(Q), dptr_as<float>(probs),
           dptr_as<float>(d_out), dptr_as<float>(dK), dptr_as<float>(dV), N, D);
    mark_written(dK); mark_written(dV);
}

#define EW_GUARD(fn, n) if ((n) <= 0) return

void metal_enqueue_silu_mul(MetalBuf *gate, MetalBuf *up, int n)
{
    EW_GUARD("silu_mul", n);
    REQUIRE_BYTES(gate, (size_t)n * 4, "silu_mul"); REQUIRE_BYTES(up, (size_t)n * 4, "silu_mul");
    LAUNCH(k_silu_mul, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(gate), dptr_as<float>(up), (size_t)n);
    mark_written(gate);
}
void metal_enqueue_gelu_mul(MetalBuf *gate, MetalBuf *up, int n)
{
    EW_GUARD("gelu_mul", n);
    REQUIRE_BYTES(gate, (size_t)n * 4, "gelu_mul"); REQUIRE_BYTES(up, (size_t)n * 4, "gelu_mul");
    LAUNCH(k_gelu_mul, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(gate), dptr_as<float>(up), (size_t)n);
    mark_written(gate);
}
void metal_enqueue_silu_mul_backward(MetalBuf *dout, MetalBuf *gate, MetalBuf *up, MetalBuf *dgate, MetalBuf *dup, int n)
{
    EW_GUARD("silu_mul_backward", n);
    REQUIRE_BYTES(dout, (size_t)n * 4, "silu_mul_backward"); REQUIRE_BYTES(gate, (size_t)n * 4, "silu_mul_backward");
    REQUIRE_BYTES(up, (size_t)n * 4, "silu_mul_backward"); REQUIRE_BYTES(dgate, (size_t)n * 4, "silu_mul_backward");
    REQUIRE_BYTES(dup, (size_t)n * 4, "silu_mul_backward");
    LAUNCH(k_silu_mul_bwd, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(dout), dptr_as<float>(gate), dptr_as<float>(up),
           dptr_as<float>(dgate), dptr_as<float>(dup), (size_t)n);
    mark_written(dgate); mark_written(dup);
}
void metal_enqueue_gelu_mul_backward(MetalBuf *dout, MetalBuf *gate, MetalBuf *up, MetalBuf *dgate, MetalBuf *dup, int n)
{
    EW_GUARD("gelu_mul_backward", n);
    REQUIRE_BYTES(dout, (size_t)n * 4, "gelu_mul_backward"); REQUIRE_BYTES(gate, (size_t)n * 4, "gelu_mul_backward");
    REQUIRE_BYTES(up, (size_t)n * 4, "gelu_mul_backward"); REQUIRE_BYTES(dgate, (size_t)n * 4, "gelu_mul_backward");
    REQUIRE_BYTES(dup, (size_t)n * 4, "gelu_mul_backward");
    LAUNCH(k_gelu_mul_bwd, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(dout), dptr_as<float>(gate), dptr_as<float>(up),
           dptr_as<float>(dgate), dptr_as<float>(dup), (size_t)n);
    mark_written(dgate); mark_written(dup);
}
void metal_enqueue_residual_add(MetalBuf *x, MetalBuf *y, int n)
{
    EW_GUARD("residual_add", n);
    REQUIRE_BYTES(x, (size_t)n * 4, "residual_add"); REQUIRE_BYTES(y, (size_t)n * 4, "residual_add");
    LAUNCH(k_residual_add, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(x), dptr_as<float>(y), (size_t)n);
    mark_written(x);
}
void metal_enqueue_scale(MetalBuf *x, float alpha, int n)
{
    EW_GUARD("scale", n);
    REQUIRE_BYTES(x, (size_t)n * 4, "scale");
    LAUNCH(k_scale, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(x), alpha, (size_t)n);
    mark_written(x);
}
void metal_enqueue_add_scaled(MetalBuf *y, MetalBuf *x, float alpha, int n)
{
    EW_GUARD("add_scaled", n);
    REQUIRE_BYTES(x, (size_t)n * 4, "add_scaled"); REQUIRE_BYTES(y, (size_t)n * 4, "add_scaled");
    LAUNCH(k_add_scaled, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(y), dptr_as<float>(x), alpha, (size_t)n);
    mark_written(y);
}
void metal_enqueue_clamp(MetalBuf *x, float max_val, int n)
{
    EW_GUARD("clamp", n);
    REQUIRE_BYTES(x, (size_t)n * 4, "clamp");
    LAUNCH(k_clamp, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(x), max_val, (size_t)n);
    mark_written(x);
}
void metal_enqueue_copy(MetalBuf *src, MetalBuf *dst, int n)
{
    EW_GUARD("copy", n);
    REQUIRE_BYTES(src, (size_t)n * 4, "copy"); REQUIRE_BYTES(dst, (size_t)n * 4, "copy");
    LAUNCH(k_copy, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<float>(src), dptr_as<float>(dst), (size_t)n);
    mark_written(dst);
}

void metal_enqueue_float_matmul(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K)
{
    REQUIRE_BYTES(A, (size_t)M * K * 4, "float_matmul"); REQUIRE_BYTES(W, (size_t)N * K * 4, "float_matmul");
    REQUIRE_BYTES(C, (size_t)M * N * 4, "float_matmul");
    if (M <= 0 || N <= 0) return;
    LAUNCH(k_float_matmul, dim3((N + 15) / 16, (M + 15) / 16), dim3(256), 0, dptr_as<float>(A), (size_t)K, (size_t)1,
           dptr_as<float>(W), (size_t)1, (size_t)K, dptr_as<float>(C), M, N, K);
    mark_written(C);
}
void metal_enqueue_float_matmul_tn(MetalBuf *A, MetalBuf *B, MetalBuf *C, int M, int N, int K)
{
    REQUIRE_BYTES(A, (size_t)K * M * 4, "float_matmul_tn"); REQUIRE_BYTES(B, (size_t)K * N * 4, "float_matmul_tn");
    REQUIRE_BYTES(C, (size_t)M * N * 4, "float_matmul_tn");
    if (M <= 0 || N <= 0) return;
    LAUNCH(k_float_matmul, dim3((N + 15) / 16, (M + 15) / 16), dim3(256), 0, dptr_as<float>(A), (size_t)1, (size_t)M,
           dptr_as<float>(B), (size_t)N, (size_t)1, dptr_as<float>(C), M, N, K);
    mark_written(C);
}
// C[M,K] = A[M,N] W[N,K]: output width K, reduction N
void metal_enqueue_float_matmul_nt(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K)
{
    REQUIRE_BYTES(A, (size_t)M * N * 4, "float_matmul_nt"); REQUIRE_BYTES(W, (size_t)N * K * 4, "float_matmul_nt");
    REQUIRE_BYTES(C, (size_t)M * K * 4, "float_matmul_nt");
    if (M <= 0 || K <= 0) return;
    LAUNCH(k_float_matmul, dim3((K + 15) / 16, (M + 15) / 16), dim3(256), 0, dptr_as<float>(A), (size_t)N, (size_t)1,
           dptr_as<float>(W), (size_t)K, (size_t)1, dptr_as<float>(C), M, K, N);
    mark_written(C);
}

void metal_enqueue_f16_sgd_fused(MetalBuf *W, MetalBuf *dY, MetalBuf *X, int M, int K, int N, float lr)
{
    REQUIRE_BYTES(W, (size_t)M * N * 2, "f16_sgd_fused"); REQUIRE_BYTES(dY, (size_t)K * M * 4, "f16_sgd_fused");
    REQUIRE_BYTES(X, (size_t)K * N * 4, "f16_sgd_fused");
    if (M <= 0 || N <= 0) return;
    LAUNCH(k_f16_rank_update, dim3((N + 15) / 16, (M + 15) / 16), dim3(256), 0, dptr_as<half_t>(W), dptr_as<float>(dY),
           dptr_as<float>(X), M, K, N, -lr);
    mark_written(W);
}
void metal_enqueue_f16_grad_accum(MetalBuf *G, MetalBuf *dY, MetalBuf *X, int M, int K, int N)
{
    REQUIRE_BYTES(G, (size_t)M * N * 2, "f16_grad_accum"); REQUIRE_BYTES(dY, (size_t)K * M * 4, "f16_grad_accum");
    REQUIRE_BYTES(X, (size_t)K * N * 4, "f16_grad_accum");
    if (M <= 0 || N <= 0) return;
    LAUNCH(k_f16_rank_update, dim3((N + 15) / 16, (M + 15) / 16), dim3(256), 0, dptr_as<half_t>(G), dptr_as<float>(dY),
           dptr_as<float>(X), M, K, N, 1.0f);
    mark_written(G);
}
void metal_enqueue_f16_sgd_apply(MetalBuf *W, MetalBuf *G, int n, float lr)
{
    EW_GUARD("f16_sgd_apply", n);
    REQUIRE_BYTES(W, (size_t)n * 2, "f16_sgd_apply"); REQUIRE_BYTES(G, (size_t)n * 2, "f16_sgd_apply");
    LAUNCH(k_f16_sgd_apply, dim3(blocks_for(n)), dim3(TB), 0, dptr_as<half_t>(W), dptr_as<half_t>(G), (size_t)n, lr);
    mark_written(W); mark_written(G);
}

}  // extern "C"
