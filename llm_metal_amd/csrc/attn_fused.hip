// Head-block attention kernels for short sequences (seq <= 64, head_dim <= 128):
// one workgroup owns one (sequence, query head) and keeps Q, K, V of that head in
// LDS, so the QKV epilogue (plane sum, LoRA term, per-head RMSNorm, RoPE) and the
// attention itself are ONE launch, and the four 64 x 64 x hd products run on the
// matrix cores in fp32 (v_mfma_f32_32x32x2_f32: no rounding of the operands).
//
// Same arithmetic as k_qkv_post + k_attn_fwd (fused_kernels.hip), which remain
// the general path: add_scaled / rms_norm / rope_train / attn_train_fwd of
// src/nn/fast_sft.c:638-689 and shaders/q8_kernels.metal:495-538, 769-851.
#include "fused.h"
#include "planes.h"

namespace lmhip {
namespace {

#define LAUNCH(kern, grid, block, lds, ...) do { \
    hipLaunchKernelGGL(kern, grid, block, lds, stream(), __VA_ARGS__); HIP_CHECK(hipGetLastError()); } while (0)

constexpr int MAXR = 16;                                  // LoRA rank limit of this path

// x[c] += sc * sum_r t[r] * bw[c][r]
__device__ __forceinline__ void lora_add(float4 &x, const float *t, const float (&bw)[4][MAXR], int R, float sc)
{
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
    for (int r = 0; r < MAXR; r++) {
        if (r < R) { const float tr = t[r]; a0 += tr * bw[0][r]; a1 += tr * bw[1][r]; a2 += tr * bw[2][r]; a3 += tr * bw[3][r]; }
    }
    x.x += sc * a0; x.y += sc * a1; x.z += sc * a2; x.w += sc * a3;
}

__device__ __forceinline__ void load_b_rows(float (&bw)[4][MAXR], const float *B, int row0, int R)
{
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < MAXR; r++) bw[c][r] = (r < R) ? B[(size_t)(row0 + c) * R + r] : 0.f;
}

// Sum over the HV lanes that share a row (HV a power of two <= 32, groups aligned inside the wave).
template <int HV>
__device__ __forceinline__ float group_sum(float v)
{
#pragma unroll
    for (int o = HV / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

// RMSNorm over the head (gamma g) followed by half-split RoPE at position pos; the lane holds
// elements 4v..4v+3 of the head, its partner (lane ^ HV/2) the other half of each rotation pair.
template <int HV>
__device__ __forceinline__ float4 head_norm_rope(float4 x, int v, const float *g, float eps, const float2 *rope, int pos)
{
    constexpr int HD = 4 * HV, HALF = HD / 2;
    const float ss = group_sum<HV>(sumsq4(x));
    const float inv = rsqrtf(ss / (float)HD + eps);
    const float4 gg = ld4(g + 4 * v);
    const float4 n = make_float4(x.x * inv * gg.x, x.y * inv * gg.y, x.z * inv * gg.z, x.w * inv * gg.w);
    float4 o;                                              // the partner's normalised values
    o.x = __shfl_xor(n.x, HV / 2, WAVE); o.y = __shfl_xor(n.y, HV / 2, WAVE);
    o.z = __shfl_xor(n.z, HV / 2, WAVE); o.w = __shfl_xor(n.w, HV / 2, WAVE);
    const bool first = v < HV / 2;
    const int d = first ? 4 * v : 4 * v - HALF;
    const float4 t0 = ld4(reinterpret_cast<const float *>(rope + (size_t)pos * HALF + d));       // (cos, sin) x 2
    const float4 t1 = ld4(reinterpret_cast<const float *>(rope + (size_t)pos * HALF + d + 2));
    // first half:  n0 cos - n1 sin  with n0 = own, n1 = partner;  second half: n0 sin + n1 cos with n0 = partner, n1 = own
    float4 r;
    if (first) { r.x = n.x * t0.x - o.x * t0.y; r.y = n.y * t0.z - o.y * t0.w; r.z = n.z * t1.x - o.z * t1.y; r.w = n.w * t1.z - o.w * t1.w; }
    else       { r.x = o.x * t0.y + n.x * t0.x; r.y = o.y * t0.w + n.y * t0.z; r.z = o.z * t1.y + n.z * t1.x; r.w = o.w * t1.w + n.w * t1.z; }
    return r;
}

__device__ __forceinline__ void st_lds4(float *p, float4 v) { p[0] = v.x; p[1] = v.y; p[2] = v.z; p[3] = v.w; }

// grid (Hq, batch), block 256, dynamic LDS: 3 x 64 x (hd + 1) + seq x 2R floats.
template <int HV>
__global__ __launch_bounds__(256) void k_attn_fused_fwd(AttnFusedFwdArgs A)
{
    extern __shared__ float lds[];
    const QkvPostArgs &a = A.q;
    constexpr int HD = 4 * HV, LD = HD + 1, RPP = 256 / HV, LP = 65;
    const int N = a.seq, R = a.R, h = blockIdx.x, b = blockIdx.y;
    const int ratio = a.Hq / a.Hkv, hk = h / ratio;
    const int qd = a.Hq * HD, kd = a.Hkv * HD;
    float *Qs = lds, *Ks = Qs + 64 * LD, *Vs = Ks + 64 * LD, *Ts = Vs + 64 * LD;      // Ts: [N][2R] = tq | tv
    float *Ps = Qs;                                        // [64][65] scores / probabilities, after Q is consumed
    const int tid = threadIdx.x, v = tid % HV, rr = tid / HV, lane = tid & 63, wave = tid >> 6;
    const int l31 = lane & 31, hh = lane >> 5;
    const size_t r0 = (size_t)b * N;
    const bool writer = (h % ratio) == 0;                  // one query head per KV group saves K and V

    // LoRA mids t = x A^T: the last 2R columns of the fused QKV product
    if (R > 0) {
        const int per = 2 * R / 4;
        for (int idx = tid; idx < N * per; idx += 256) {
            const int i = idx / per, c = idx % per;
            const float4 t = planes_at4(a.qkv, r0 + i, qd + 2 * kd + 4 * c);
            st_lds4(Ts + i * 2 * R + 4 * c, t);
            if (h == 0) {
                if (4 * c < R) st4(a.tq + (r0 + i) * R + 4 * c, t);
                else           st4(a.tv + (r0 + i) * R + 4 * c - R, t);
            }
        }
    }
    // rows past the sequence read as zero in the matrix products
    for (int idx = tid; idx < (64 - N) * LD; idx += 256) { Qs[N * LD + idx] = 0.f; Ks[N * LD + idx] = 0.f; Vs[N * LD + idx] = 0.f; }
    __syncthreads();

    float bw[4][MAXR];
    // ---- Q: planes + LoRA, save, norm, RoPE, save
    if (R > 0) load_b_rows(bw, a.Bq, h * HD + 4 * v, R);
    for (int i = rr; i < N; i += RPP) {                    // the HV lanes of a row group share i: shuffles stay convergent
        float4 x = planes_at4(a.qkv, r0 + i, h * HD + 4 * v);
        if (R > 0) lora_add(x, Ts + i * 2 * R, bw, R, a.sc);
        st4(a.q_pre + (r0 + i) * qd + h * HD + 4 * v, x);
        const float4 f = head_norm_rope<HV>(x, v, a.g_q, a.eps, a.rope, i);
        st4(a.q_fin + (r0 + i) * qd + h * HD + 4 * v, f);
        st_lds4(Qs + i * LD + 4 * v, f);
    }
    // ---- K: planes, save, norm, RoPE, save
    for (int i = rr; i < N; i += RPP) {
        const float4 x = planes_at4(a.qkv, r0 + i, qd + hk * HD + 4 * v);
        const float4 f = head_norm_rope<HV>(x, v, a.g_k, a.eps, a.rope, i);
        if (writer) { st4(a.k_pre + (r0 + i) * kd + hk * HD + 4 * v, x); st4(a.k_fin + (r0 + i) * kd + hk * HD + 4 * v, f); }
        st_lds4(Ks + i * LD + 4 * v, f);
    }
    // ---- V: planes + LoRA, save
    if (R > 0) load_b_rows(bw, a.Bv, hk * HD + 4 * v, R);
    for (int i = rr; i < N; i += RPP) {
        float4 x = planes_at4(a.qkv, r0 + i, qd + kd + hk * HD + 4 * v);
        if (R > 0) lora_add(x, Ts + i * 2 * R + R, bw, R, a.sc);
        if (writer) st4(a.v_out + (r0 + i) * kd + hk * HD + 4 * v, x);
        st_lds4(Vs + i * LD + 4 * v, x);
    }
    __syncthreads();

    // ---- S = scale * Q K^T on 32 x 32 tiles: waves 0, 1, 2 take (0,0), (1,0), (1,1); (0,1) is above the diagonal
    float16v acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
    const int ti = wave >= 1 ? 1 : 0, tj = wave == 2 ? 1 : 0;
    if (wave < 3 && 32 * ti < N) {
        const float *qa = Qs + (32 * ti + l31) * LD + hh, *kb = Ks + (32 * tj + l31) * LD + hh;
#pragma unroll 8
        for (int kk = 0; kk < HD / 2; kk++)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[2 * kk], kb[2 * kk], acc, 0, 0, 0);
    }
    __syncthreads();                                       // every wave has read its Q rows: Ps may overwrite them
    if (wave < 3) {
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int i = 32 * ti + 8 * (e >> 2) + 4 * hh + (e & 3), j = 32 * tj + l31;
            Ps[i * LP + j] = acc[e] * A.scale;
        }
    }
    __syncthreads();

    // ---- causal softmax, four lanes per row; probabilities saved (attn_train_fwd keeps them for the backward)
    {
        const int i = tid >> 2, part = tid & 3;
        float e[16];
        float mx = -1e30f;
#pragma unroll
        for (int c = 0; c < 16; c++) { const int j = part * 16 + c; e[c] = (j <= i) ? Ps[i * LP + j] : -1e30f; mx = fmaxf(mx, e[c]); }
        mx = fmaxf(mx, __shfl_xor(mx, 1, WAVE)); mx = fmaxf(mx, __shfl_xor(mx, 2, WAVE));
        float sum = 0.f;
#pragma unroll
        for (int c = 0; c < 16; c++) { const int j = part * 16 + c; e[c] = (j <= i) ? expf(e[c] - mx) : 0.f; sum += e[c]; }
        sum += __shfl_xor(sum, 1, WAVE); sum += __shfl_xor(sum, 2, WAVE);
        const float inv = 1.0f / sum;
        float *pr = A.probs + (((size_t)b * a.Hq + h) * N + i) * N;
#pragma unroll
        for (int c = 0; c < 16; c++) {
            const int j = part * 16 + c;
            const float p = e[c] * inv;
            Ps[i * LP + j] = p;
            if (i < N && j < N) pr[j] = p;
        }
    }
    __syncthreads();

    // ---- O = P V: tiles (ti, td), td < hd/32, dealt round-robin to the waves; K runs to the diagonal block only
    const int Kb = tiled_kb(qd);
    constexpr int TD = HD / 32 > 0 ? HD / 32 : 1;
    for (int t = wave; t < 2 * TD; t += 4) {
        const int oi = t / TD, td = t % TD;
        if (32 * oi >= N) continue;
#pragma unroll
        for (int e = 0; e < 16; e++) acc[e] = 0.f;
        const float *pa = Ps + (32 * oi + l31) * LP + hh, *vb = Vs + hh * LD + 32 * td + l31;
        const int ksteps = 16 * (oi + 1);
        for (int kk = 0; kk < ksteps; kk++)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[2 * kk], vb[2 * kk * LD], acc, 0, 0, 0);
        const int d = 32 * td + l31;
        if (d < HD) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int i = 32 * oi + 8 * (e >> 2) + 4 * hh + (e & 3);
                if (i < N) A.out16[tiled_index((int)(r0 + i), h * HD + d, Kb)] = f2h(acc[e]);
            }
        }
    }
    if (h == a.Hq - 1)                                     // zero the K padding of the operand rows once
        for (int idx = tid; idx < N * (Kb * 64 - qd); idx += 256) {
            const int i = idx / (Kb * 64 - qd), c = qd + idx % (Kb * 64 - qd);
            A.out16[tiled_index((int)(r0 + i), c, Kb)] = (half_t)0;
        }
}

}  // namespace

bool attn_fused_fwd_supported(const QkvPostArgs &a)
{
    return a.seq <= 64 && (a.hd == 32 || a.hd == 64 || a.hd == 128) && a.R <= MAXR && (a.R % 4) == 0 && a.Hq % a.Hkv == 0 &&
           a.qkv.ld % 4 == 0;
}

void launch_attn_fused_fwd(const AttnFusedFwdArgs &A)
{
    const QkvPostArgs &a = A.q;
    if (!attn_fused_fwd_supported(a)) { fprintf(stderr, "[fast_hip] attn_fused_fwd: unsupported shape\n"); abort(); }
    const size_t lds = ((size_t)3 * 64 * (a.hd + 1) + (size_t)a.seq * 2 * a.R) * sizeof(float);
    const dim3 grid(a.Hq, A.batch);
#define FUSED_FWD(HV) do { \
        static bool attr_set = false; \
        if (!attr_set) { HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_attn_fused_fwd<HV>), \
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024)); attr_set = true; } \
        LAUNCH(k_attn_fused_fwd<HV>, grid, dim3(256), lds, A); } while (0)
    if (a.hd == 128) FUSED_FWD(32); else if (a.hd == 64) FUSED_FWD(16); else FUSED_FWD(8);
#undef FUSED_FWD
}

}  // namespace lmhip
