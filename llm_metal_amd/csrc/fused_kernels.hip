// Fused row / head kernels of the SFT step.  Each one sits between two
// weight-streaming GEMMs: it sums the producer GEMM's K-split partial planes on
// load, does the reference's per-row arithmetic in fp32 (shaders/q8_kernels.metal,
// cited per kernel) and writes what the next GEMM reads as a scaled fp16 row in
// the GEMM's tiled layout.  One launch here replaces between 3 and 12 dispatches
// of the reference's forward_to_logits / sft_backward_ex (src/nn/fast_sft.c:616-982).
//
// With 64..160 rows per step these kernels are latency bound, not bandwidth
// bound: a row gets one 1024-thread workgroup, every thread keeps its few float4
// of the row in registers between the reductions, and all plane loads of a
// thread are independent so they are in flight together.
#include "fused.h"
#include "planes.h"
#include "kargs.h"

namespace lmhip {
namespace {

constexpr int TB = 256;
constexpr int RB = 1024;                                  // threads of a row workgroup
constexpr int MAXV = 3;                                   // float4 per thread: rows up to 12288 wide
constexpr int MANY_ROWS = 512;                            // rows from which a row kernel takes 256 threads per row instead of 1024
constexpr int MAXV_ROW = MAXV;                            // (the name the row kernels with their own MAXV parameter use)

// four consecutive elements (k % 4 == 0) of row `row` of a tiled fp16 operand
__device__ __forceinline__ void st_tiled4(half_t *out, size_t row, int k, int Kb, float4 v, float s)
{
    half4 h = {f2h(v.x * s), f2h(v.y * s), f2h(v.z * s), f2h(v.w * s)};
    *reinterpret_cast<half4 *>(out + tiled_a_index((int)row, k, Kb)) = h;
}

// zero the K padding [n, Kb*64) of a tiled row
__device__ __forceinline__ void zero_tiled_pad(half_t *out, size_t row, int n, int Kb)
{
    for (int i = n + threadIdx.x; i < Kb * 64; i += blockDim.x) out[tiled_a_index((int)row, i, Kb)] = (half_t)0;
}

// Row `row` of a tiled fp16 operand [*, n] from fp32 values in LDS, scaled by s.
__device__ __forceinline__ void write_f16_tiled(const float *vals, int n, half_t *out, size_t row, float s)
{
    const int Kb = tiled_kb(n);
    for (int c = threadIdx.x; c < Kb * 8; c += blockDim.x) {
        half8 hv;
#pragma unroll
        for (int e = 0; e < 8; e++) { const int i = c * 8 + e; hv[e] = (i < n) ? f2h(vals[i] * s) : (half_t)0; }
        *reinterpret_cast<half8 *>(out + tiled_a_index((int)row, c * 8, Kb)) = hv;
    }
}

// ------------------------------------------------------------------ forward rows
// x = (gathered embedding | x_prev) [+ branch | + RN(branch; g_branch)];  ln = RN(x; g_norm).
// rms_norm: shaders/q8_kernels.metal:133-158; residual_add :369-375; the Gemma3
// ordering (norm the branch, then add) is src/nn/fast_sft.c:698-705, 732-736.
// MAXV: float4 per thread (1 for rows up to 4096 wide, which leaves registers for 20 planes of the branch in flight).
// GROUPED: the branch planes carry a factor per group of planes.
// NT: threads per row.  1024 when a step has few rows (one row's loads all in flight at once); 256 from a few hundred
// rows on, where eight resident workgroups per CU hide each other's reductions and barriers.
template <int MAXV, bool GROUPED, int NT = RB>
__global__ __launch_bounds__(NT) void k_norm_rows(KARGS24)
{
    KARGS_HOT(NormRowsArgs, a);                           // rows_launched, D, pf
    __shared__ float sm[32];
    if (blockIdx.x >= a.rows_launched) {                  // workgroups beyond the rows fetch weights; they are the last
        prefetch_weight_tiles<NT>(a.pf, blockIdx.x - a.rows_launched);      // to finish and have nothing to wait for
        return;
    }
    kargs_rest(a);
    const size_t r = xcd_block_row(blockIdx.x, a.rows_launched);
    const int D = a.D, nv = D >> 2;
    float4 x[MAXV], b[MAXV];
    const bool gather = a.x_prev == nullptr;
    const uint32_t tok = gather ? a.tokens[r] : 0u;
    const bool padded = gather && a.zero_rows && tok == ZERO_ROW_TOKEN;      // zero rows past the end of a sequence
    const float *base = gather ? a.emb + (size_t)(padded ? 0u : tok) * D : a.x_prev + r * D;
    size_t rows[MAXV]; int cols[MAXV]; bool ok[MAXV];
#pragma unroll
    for (int t = 0; t < MAXV; t++) {
        const int v = threadIdx.x + t * NT;
        x[t] = b[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        rows[t] = r; cols[t] = 4 * v; ok[t] = v < nv;
        if (v < nv && !padded) x[t] = ld4(base + 4 * v);
    }
    // one value per thread: the norm weights are requested with the row, not after the reductions they do not depend on
    // (a round trip each); with more values per thread the registers are worth more
    constexpr bool AHEAD = MAXV == 1;
    float4 gn[MAXV], gb[MAXV];
    if constexpr (AHEAD) {
        const int v = threadIdx.x;
        gn[0] = gb[0] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v < nv && a.g_norm) gn[0] = ld4(a.g_norm + 4 * v);
        if (v < nv && a.branch.S > 0 && a.g_branch) gb[0] = ld4(a.g_branch + 4 * v);
    }
    if (a.branch.S > 0) // (many rows: a plane per round trip and 48 registers, so that eight workgroups fit a CU: 25.5 -> 22.7 us at 2048 x 2560)
    planes_at4_multi<MAXV, (MAXV == 1 ? 20 : NT == RB ? 6 : 1), GROUPED>(a.branch, rows, cols, ok, b);
    if (gather && a.emb_scale != 1.0f) {
#pragma unroll
        for (int t = 0; t < MAXV; t++) { x[t].x *= a.emb_scale; x[t].y *= a.emb_scale; x[t].z *= a.emb_scale; x[t].w *= a.emb_scale; }
    }
    if (a.branch.S > 0) {
        float inv = 1.0f;
        if (a.g_branch) {
            float ss = 0.f;
#pragma unroll
            for (int t = 0; t < MAXV; t++) ss += sumsq4(b[t]);
            ss = block_sum(ss, sm);
            inv = rsqrtf(ss / (float)D + a.eps);
        }
#pragma unroll
        for (int t = 0; t < MAXV; t++) {
            const int v = threadIdx.x + t * NT;
            if (v >= nv) continue;
            if (a.g_branch) {
                if (a.branch_raw_out) st4(a.branch_raw_out + r * D + 4 * v, b[t]);
                float4 g;
                if constexpr (AHEAD) g = gb[t]; else g = ld4(a.g_branch + 4 * v);
                x[t].x += b[t].x * inv * g.x; x[t].y += b[t].y * inv * g.y;
                x[t].z += b[t].z * inv * g.z; x[t].w += b[t].w * inv * g.w;
            } else {
                x[t].x += b[t].x; x[t].y += b[t].y; x[t].z += b[t].z; x[t].w += b[t].w;
            }
        }
    }
    if (a.x_out) {
#pragma unroll
        for (int t = 0; t < MAXV; t++) { const int v = threadIdx.x + t * NT; if (v < nv) st4(a.x_out + r * D + 4 * v, x[t]); }
    }
    if (!a.g_norm) return;
    float ss = 0.f;
#pragma unroll
    for (int t = 0; t < MAXV; t++) ss += sumsq4(x[t]);
    float amax = 0.f, inv;
    if constexpr (AHEAD) {
        // the norm weights are here already: the row maximum of x g, which the factor 1 / rms scales like every entry,
        // goes through the same pair of barriers as the sum of squares
        float mxg = 0.f;
#pragma unroll
        for (int t = 0; t < MAXV; t++)
            mxg = fmaxf(mxg, amax4(make_float4(x[t].x * gn[t].x, x[t].y * gn[t].y, x[t].z * gn[t].z, x[t].w * gn[t].w)));
        block_sum_max(ss, mxg, sm);
        inv = rsqrtf(ss / (float)D + a.eps);
        amax = mxg * inv;
#pragma unroll
        for (int t = 0; t < MAXV; t++) {
            const float4 g = gn[t];
            x[t].x = x[t].x * inv * g.x; x[t].y = x[t].y * inv * g.y; x[t].z = x[t].z * inv * g.z; x[t].w = x[t].w * inv * g.w;
        }
    } else {
        ss = block_sum(ss, sm);
        inv = rsqrtf(ss / (float)D + a.eps);
#pragma unroll
        for (int t = 0; t < MAXV; t++) {
            const int v = threadIdx.x + t * NT;
            if (v >= nv) continue;
            const float4 g = ld4(a.g_norm + 4 * v);
            x[t].x = x[t].x * inv * g.x; x[t].y = x[t].y * inv * g.y; x[t].z = x[t].z * inv * g.z; x[t].w = x[t].w * inv * g.w;
            amax = fmaxf(amax, amax4(x[t]));
        }
        amax = block_max(amax, sm);
    }
    const float s = row_scale_for(amax);
    const int Kb = tiled_kb(D);
#pragma unroll
    for (int t = 0; t < MAXV; t++) { const int v = threadIdx.x + t * NT; if (v < nv) st_tiled4(a.ln16, r, 4 * v, Kb, x[t], s); }
    zero_tiled_pad(a.ln16, r, D, Kb);
    if (threadIdx.x == 0) a.inv_scale[r] = 1.0f / s;
}

// cos/sin of pos * theta^(-2d/hd), exactly as rope_train forms them
// (shaders/q8_kernels.metal:527-530): table[pos][d] = (cos, sin), d < hd/2.
__global__ void k_rope_table(float2 *tab, int seq, int half, int hd, float theta)
{
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= seq * half) return;
    const int pos = idx / half, d = idx % half;
    const float freq = 1.0f / powf(theta, (float)(2 * d) / (float)hd);
    float s, c;
    sincosf((float)pos * freq, &s, &c);
    tab[idx] = make_float2(c, s);
}

// ------------------------------------------------------------------ QKV epilogue
// One wave per (row, head): sums the fused QKV GEMM planes, adds the LoRA term
// sc * (x A^T) B^T (add_scaled, src/nn/fast_sft.c:639-644, 651-656), saves the
// pre-norm head, applies the per-head RMSNorm (src/nn/fast_sft.c:668-669) and the
// half-split RoPE (rope_train, shaders/q8_kernels.metal:495-538).  Works on the
// [rows][H*hd] layout, so the reference's three head transposes, repeat_kv and
// five buffer copies disappear.  A lane owns the pairs (d, d + hd/2).
constexpr int MAXP = 4;                                   // pairs per lane: hd <= 512
// NP: pairs per lane compiled in (1 serves head_dim <= 128); RK: the LoRA rank compiled in (16), 0 for none, -1 for any.
// The kernel runs once per wave, so what is compiled out is code it does not have to fetch.
template <int NP, int RK>
__global__ __launch_bounds__(TB) void k_qkv_post(QkvPostArgs a)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int HT = a.Hq + 2 * a.Hkv;
    const size_t task = (size_t)blockIdx.x * 4 + wave;
    if (task >= (size_t)a.rows * HT) return;            // whole wave leaves together; no block barrier below
    const size_t row = task / HT;
    const int slot = (int)(task % HT);
    const int hd = a.hd, half = hd / 2, qd = a.Hq * hd, kd = a.Hkv * hd;
    const int kind = slot < a.Hq ? 0 : (slot < a.Hq + a.Hkv ? 1 : 2);     // 0 q, 1 k, 2 v
    const int h = kind == 0 ? slot : (kind == 1 ? slot - a.Hq : slot - a.Hq - a.Hkv);
    const int col0 = kind == 0 ? h * hd : (kind == 1 ? qd + h * hd : qd + kd + h * hd);
    const int t0 = qd + 2 * kd + (kind == 2 ? a.R : 0);
    const bool lora = RK != 0 && a.R > 0 && kind != 1;
    const float *B = kind == 0 ? a.Bq : a.Bv;

    // what the epilogue needs and nothing computed here decides -- the norm weights, the rotation, the rows of B --
    // is requested before the planes, so that all of it is one round trip
    const int pos = (int)(row % a.seq);
    float g0[NP], g1[NP]; float2 cs[NP];
    if (kind != 2) {
        const float *g = kind == 0 ? a.g_q : a.g_k;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int d = min(lane + 64 * p, half - 1);
            g0[p] = g[d]; g1[p] = g[d + half]; cs[p] = a.rope[(size_t)pos * half + d];
        }
    }
    constexpr bool B_AHEAD = NP == 1 && RK == 16;          // (more pairs per lane would hold too many registers)
    float4 bw0[4], bw1[4];
    if constexpr (B_AHEAD) {
#pragma unroll
        for (int i = 0; i < 4; i++) bw0[i] = bw1[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (lora && lane < half) {
            const float *b0 = B + (size_t)(h * hd + lane) * a.R, *b1 = b0 + (size_t)half * a.R;
#pragma unroll
            for (int i = 0; i < 4; i++) { bw0[i] = ld4(b0 + 4 * i); bw1[i] = ld4(b1 + 4 * i); }
        }
    }
    // everything this lane reads from the planes in one go: positions p (first half of the head), NP + p (second
    // half) and 2 NP (the lane's entry of x A^T)
    float x0[NP], x1[NP], tval;
    {
        int cols[2 * NP + 1]; bool ok[2 * NP + 1]; float got[2 * NP + 1];
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int d = lane + 64 * p;
            cols[p] = col0 + d; cols[NP + p] = col0 + d + half; ok[p] = ok[NP + p] = d < half;
        }
        cols[2 * NP] = t0 + lane; ok[2 * NP] = lora && lane < a.R;
        planes_at_multi<2 * NP + 1, 5>(a.qkv, row, cols, ok, got);
#pragma unroll
        for (int p = 0; p < NP; p++) { x0[p] = got[p]; x1[p] = got[NP + p]; }
        tval = got[2 * NP];
    }
    if (lora && h == 0 && lane < a.R) (kind == 0 ? a.tq : a.tv)[row * a.R + lane] = tval;

    float ss = 0.f;
#pragma unroll
    for (int p = 0; p < NP; p++) {
        const int d = lane + 64 * p;
        if (lora && 64 * p < half) {                          // uniform branch: the broadcasts stay convergent
            float acc0 = 0.f, acc1 = 0.f;
            const float *b0 = B + (size_t)(h * hd + (d < half ? d : 0)) * a.R;
            const float *b1 = b0 + (size_t)half * a.R;
            if constexpr (RK == 16) {                          // t through scalar registers, whole rows of B as 16-byte loads
                float4 w0[4], w1[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    if constexpr (B_AHEAD) { w0[i] = bw0[i]; w1[i] = bw1[i]; }
                    else { w0[i] = w1[i] = make_float4(0.f, 0.f, 0.f, 0.f); if (d < half) { w0[i] = ld4(b0 + 4 * i); w1[i] = ld4(b1 + 4 * i); } }
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float t0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tval), 4 * i));
                    const float t1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tval), 4 * i + 1));
                    const float t2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tval), 4 * i + 2));
                    const float t3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tval), 4 * i + 3));
                    acc0 += t0 * w0[i].x; acc0 += t1 * w0[i].y; acc0 += t2 * w0[i].z; acc0 += t3 * w0[i].w;
                    acc1 += t0 * w1[i].x; acc1 += t1 * w1[i].y; acc1 += t2 * w1[i].z; acc1 += t3 * w1[i].w;
                }
            } else if constexpr (RK == 0) {
            } else if ((a.R & 3) == 0) {
                for (int r4 = 0; r4 < a.R; r4 += 4) {
                    float4 w0 = make_float4(0.f, 0.f, 0.f, 0.f), w1 = w0;
                    if (d < half) { w0 = ld4(b0 + r4); w1 = ld4(b1 + r4); }
                    const float t0 = __shfl(tval, r4, WAVE), t1 = __shfl(tval, r4 + 1, WAVE);
                    const float t2 = __shfl(tval, r4 + 2, WAVE), t3 = __shfl(tval, r4 + 3, WAVE);
                    acc0 += t0 * w0.x; acc0 += t1 * w0.y; acc0 += t2 * w0.z; acc0 += t3 * w0.w;
                    acc1 += t0 * w1.x; acc1 += t1 * w1.y; acc1 += t2 * w1.z; acc1 += t3 * w1.w;
                }
            } else {
                for (int r = 0; r < a.R; r++) {
                    const float t = __shfl(tval, r, WAVE);
                    if (d < half) { acc0 += t * b0[r]; acc1 += t * b1[r]; }
                }
            }
            x0[p] += a.sc * acc0;
            x1[p] += a.sc * acc1;
        }
        ss += x0[p] * x0[p] + x1[p] * x1[p];
    }
    if (kind == 2) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int d = lane + 64 * p;
            if (d < half) {
                a.v_out[row * kd + h * hd + d] = x0[p]; a.v_out[row * kd + h * hd + d + half] = x1[p];
                if (a.vT) {
                    const int ldt = attn_ldt(a.seq), ps = (int)(row % a.seq);
                    float *t = a.vT + ((row / a.seq * a.Hkv + h) * hd) * (size_t)ldt;
                    t[attn_t_index(d, ps, ldt)] = x0[p]; t[attn_t_index(d + half, ps, ldt)] = x1[p];
                }
            }
        }
        return;
    }
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss / (float)hd + a.eps);
    float *pre = kind == 0 ? a.q_pre : a.k_pre, *fin = kind == 0 ? a.q_fin : a.k_fin;
    const int W = kind == 0 ? qd : kd;
#pragma unroll
    for (int p = 0; p < NP; p++) {
        const int d = lane + 64 * p;
        if (d >= half) continue;
        const size_t o = row * W + h * hd + d;
        pre[o] = x0[p];
        pre[o + half] = x1[p];
        const float n0 = x0[p] * inv * g0[p], n1 = x1[p] * inv * g1[p];
        const float f0 = n0 * cs[p].x - n1 * cs[p].y, f1 = n0 * cs[p].y + n1 * cs[p].x;
        fin[o] = f0;
        fin[o + half] = f1;
        if (kind == 1 && a.kT) {
            const int ldt = attn_ldt(a.seq);
            float *t = a.kT + ((row / a.seq * a.Hkv + h) * hd) * (size_t)ldt;
            t[attn_t_index(d, pos, ldt)] = f0; t[attn_t_index(d + half, pos, ldt)] = f1;
        }
    }
}

// ------------------------------------------------------------------ attention
// attn_train_fwd, shaders/q8_kernels.metal:769-851, on [rows][H*hd] activations
// with the KV head picked as h / ratio (repeat_kv, :476-492) and one wave per
// (head, query, sequence).  Output goes straight to the O-projection's fp16 operand.
__global__ __launch_bounds__(64) void k_attn_fwd(AttnFwdArgs a)
{
    extern __shared__ float sc[];                        // [seq] scores/probs, [hd] query
    const int N = a.seq, hd = a.hd;
    float *qs = sc + N;
    const int h = blockIdx.x, i = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
    const int qd = a.Hq * hd, kd = a.Hkv * hd, hk = h / (a.Hq / a.Hkv);
    const size_t r0 = (size_t)b * N;
    const float *q = a.q + (r0 + i) * qd + h * hd;
    for (int d = lane; d < hd; d += 64) qs[d] = q[d];
    __syncthreads();
    const int lo = (a.window > 0 && i >= a.window) ? i - a.window + 1 : 0;      // first key the query sees
    float mx = -1e30f;
    for (int j = lo + lane; j <= i; j += 64) {
        const float4 *kr = reinterpret_cast<const float4 *>(a.k + (r0 + j) * kd + hk * hd);
        float dot = 0.f;
#pragma unroll 8
        for (int d4 = 0; d4 < hd / 4; d4++) {
            const float4 kv = kr[d4];
            dot += qs[4 * d4] * kv.x + qs[4 * d4 + 1] * kv.y + qs[4 * d4 + 2] * kv.z + qs[4 * d4 + 3] * kv.w;
        }
        dot *= a.scale;
        sc[j] = dot;
        mx = fmaxf(mx, dot);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int j = lo + lane; j <= i; j += 64) { const float e = expf(sc[j] - mx); sc[j] = e; sum += e; }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
    float *pr = a.probs + (((size_t)b * a.Hq + h) * N + i) * N;
    for (int j = lane; j < N; j += 64) {
        const float p = (j >= lo && j <= i) ? sc[j] * inv : 0.f;
        sc[j] = p;
        pr[j] = p;
    }
    __syncthreads();
    const int Kb = tiled_kb(qd);
    for (int d = lane; d < hd; d += 64) {
        float acc = 0.f;
#pragma unroll 8
        for (int j = lo; j <= i; j++) acc += sc[j] * a.v[(r0 + j) * kd + hk * hd + d];
        a.out16[tiled_a_index((int)(r0 + i), h * hd + d, Kb)] = f2h(acc);
    }
    if (h == a.Hq - 1)                                    // zero the K padding of this row once
        for (int c = qd + lane; c < Kb * 64; c += 64) a.out16[tiled_a_index((int)(r0 + i), c, Kb)] = (half_t)0;
}

// attn_bwd_dq, shaders/q8_kernels.metal:857-925.  Also leaves the plane-summed dO
// row in dO_red for the dK/dV kernel.
__global__ __launch_bounds__(64) void k_attn_bwd_dq(AttnBwdArgs a)
{
    extern __shared__ float dr[];                        // [seq] d_raw/ds, [hd] dO row
    const int N = a.seq, hd = a.hd;
    float *dos = dr + N;
    const int h = blockIdx.x, i = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
    const int qd = a.Hq * hd, kd = a.Hkv * hd, hk = h / (a.Hq / a.Hkv);
    const size_t r0 = (size_t)b * N;
    for (int d = lane; d < hd; d += 64) {
        const float v = planes_at(a.dO, r0 + i, h * hd + d);
        dos[d] = v;
        a.dO_red[(r0 + i) * qd + h * hd + d] = v;
    }
    __syncthreads();
    const float *pr = a.probs + (((size_t)b * a.Hq + h) * N + i) * N;
    float dp = 0.f;
    for (int j = lane; j <= i; j += 64) {
        const float4 *vr = reinterpret_cast<const float4 *>(a.v + (r0 + j) * kd + hk * hd);
        float dot = 0.f;
#pragma unroll 8
        for (int d4 = 0; d4 < hd / 4; d4++) {
            const float4 vv = vr[d4];
            dot += dos[4 * d4] * vv.x + dos[4 * d4 + 1] * vv.y + dos[4 * d4 + 2] * vv.z + dos[4 * d4 + 3] * vv.w;
        }
        dr[j] = dot;
        dp += pr[j] * dot;
    }
    dp = wave_sum(dp);
    float *ds = a.dscore + (((size_t)b * a.Hq + h) * N + i) * N;
    for (int j = lane; j < N; j += 64) {
        const float v = (j <= i) ? pr[j] * (dr[j] - dp) * a.scale : 0.f;
        dr[j] = v;
        ds[j] = v;
    }
    __syncthreads();
    for (int d = lane; d < hd; d += 64) {
        float acc = 0.f;
#pragma unroll 8
        for (int j = 0; j <= i; j++) acc += dr[j] * a.k[(r0 + j) * kd + hk * hd + d];
        a.dq[(r0 + i) * qd + h * hd + d] = acc;
    }
}

// attn_bwd_dkv + repeat_kv_bwd, shaders/q8_kernels.metal:931-992: one workgroup per
// (kv head, key j, sequence).  The column j of dS and P for every query head of the group
// is first gathered into LDS (one round of independent loads), then the four waves split
// the (head, query) pairs and stream the matching q / dO rows; partial rows meet in LDS.
__global__ __launch_bounds__(TB) void k_attn_bwd_dkv(AttnBwdArgs a)
{
    extern __shared__ float lds[];                       // [ratio*N] ds column, [ratio*N] p column, [4][2][hd] partials
    const int N = a.seq, hd = a.hd, ratio = a.Hq / a.Hkv;
    const int hk = blockIdx.x, j = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int qd = a.Hq * hd, kd = a.Hkv * hd;
    const size_t r0 = (size_t)b * N;
    float *dsc = lds, *pc = lds + ratio * N, *part = lds + 2 * ratio * N;
    const int npair = ratio * (N - j);                   // pairs (g, i) with i >= j
    for (int t = threadIdx.x; t < npair; t += TB) {
        const int g = t / (N - j), i = j + t % (N - j);
        const size_t o = (((size_t)b * a.Hq + hk * ratio + g) * N + i) * N + j;
        dsc[t] = a.dscore[o];
        pc[t] = a.probs[o];
    }
    __syncthreads();
    for (int d0 = 0; d0 < hd; d0 += 64) {
        const int d = d0 + lane;
        float dk = 0.f, dv = 0.f;
        if (d < hd) {
#pragma unroll 8
            for (int t = wave; t < npair; t += 4) {
                const int g = t / (N - j), i = j + t % (N - j);
                const size_t o = (r0 + i) * qd + (hk * ratio + g) * hd + d;
                dk += dsc[t] * a.q[o];
                dv += pc[t] * a.dO_red[o];
            }
            part[(wave * 2 + 0) * hd + d] = dk;
            part[(wave * 2 + 1) * hd + d] = dv;
        }
    }
    __syncthreads();
    for (int d = threadIdx.x; d < 2 * hd; d += TB) {
        const int which = d / hd, dd = d % hd;
        const float s = part[(0 * 2 + which) * hd + dd] + part[(1 * 2 + which) * hd + dd]
                      + part[(2 * 2 + which) * hd + dd] + part[(3 * 2 + which) * hd + dd];
        (which ? a.dv : a.dk)[(r0 + j) * kd + hk * hd + dd] = s;
    }
}

// ------------------------------------------------------------------ QKV backward rows
// Per row: inverse RoPE (rope_train_bwd, shaders/q8_kernels.metal:997-1038), QK-norm
// backward (rms_norm_train_backward :584-625 on rows of hd), dh = sc * dq B
// (float_matmul_nt + scale, src/nn/fast_sft.c:950-951, 964-965), then the whole
// row [dq | dk | dv | dh_q | dh_v] as one scaled fp16 operand so that a single GEMM
// against [Wq; Wk; Wv; A_q; A_v]^T yields dq Wq + dk Wk + dv Wv + dh_q A_q + dh_v A_v
// (src/nn/fast_sft.c:953-971).
// NP, RK: pairs per lane and LoRA rank compiled in, as in k_qkv_post.  NT: threads per row (1024, or 256 from a few
// hundred rows on, as in k_norm_rows).
// dk or dv of (row, KV head hk, column d) from the shares the one-launch attention backward leaves
// ([query block][Hq][rows_total][hd]): the query heads of the group, and the query blocks that see the key
// U elements of a thread at once (element u: shares[u], KV head hk[u], column d[u]; skipped unless on[u]): the loads of all
// of them are issued before the first sum, one memory round trip per four query heads of the group for all U.
template <int U>
__device__ __forceinline__ void kv_share_sums(const QkvBwdArgs &a, const float *const (&shares)[U], size_t row, int pos, const int (&hk)[U],
                                              const int (&d)[U], const bool (&on)[U], float (&s)[U])
{
    const int ratio = a.Hq / a.Hkv, nqb = (a.seq + 31) >> 5;
    const size_t st_h = (size_t)a.rows_total * a.hd, st_qb = st_h * a.Hq;
    const int qb0 = pos >> 5;
    const float *p[U];
#pragma unroll
    for (int u = 0; u < U; u++) { p[u] = shares[u] + ((size_t)hk[u] * ratio * a.rows_total + row) * a.hd + d[u]; s[u] = 0.f; }
    for (int g0 = 0; g0 < ratio; g0 += 4) {
        float v[U][2][4];
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int q = 0; q < 2; q++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const bool ok = on[u] && qb0 + q < nqb && g0 + g < ratio;
                    v[u][q][g] = ok ? p[u][(size_t)(qb0 + q) * st_qb + (size_t)(g0 + g) * st_h] : 0.f;
                }
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int q = 0; q < 2; q++)
#pragma unroll
                for (int g = 0; g < 4; g++) s[u] += v[u][q][g];
    }
}

template <int NP, int RK, int NT = RB>
__global__ __launch_bounds__(NT) void k_qkv_bwd_rows(QkvBwdArgs a)
{
    extern __shared__ float buf[];                       // [qd + 2kd + 2R] then [NT / 64 waves][32] partials
    __shared__ float sm[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (blockIdx.x >= a.rows_launched) {                  // workgroups beyond the rows fetch weights
        prefetch_weight_tiles<NT>(a.pf, blockIdx.x - a.rows_launched);
        return;
    }
    const size_t row = xcd_block_row(blockIdx.x, a.rows_launched);
    const int hd = a.hd, half = hd / 2, qd = a.Hq * hd, kd = a.Hkv * hd, R = a.R;
    const int n = qd + 2 * kd + 2 * R;
    float *dhp = buf + n;
    const int pos = (int)(row % a.seq);
    // A wave takes the (q or k) heads wave, wave + 16, wave + 32, ... three at a time: the loads of all three are
    // issued before the first reduction, so their latency is paid once per trip instead of once per head.
    constexpr int SU = 3;
    const int nslots = a.Hq + a.Hkv;
    float g0[SU][NP], g1[SU][NP], p0[SU][NP], p1[SU][NP], w0[SU][NP], w1[SU][NP];
    float2 cs[NP];
    float amax = 0.f;                                      // over what this thread puts into the row's final values
    // the loads of one trip; with `defer_shares` the dk values of a K head are left for take_shares()
    auto load_trip = [&](int s0, bool defer_shares) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int d = lane + 64 * p;
            cs[p] = d < half ? a.rope[(size_t)pos * half + d] : make_float2(1.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < SU; u++) {
            const int slot = min(s0 + (NT / 64) * u, nslots - 1);      // clamped: the extra work is not stored
            const int isk = slot >= a.Hq, h = isk ? slot - a.Hq : slot;
            const int W = isk ? kd : qd;
            const float *gin = (isk ? a.dk : a.dq) + row * W + h * hd;
            const float *xp = (isk ? a.k_pre : a.q_pre) + row * W + h * hd;
            const float *g = isk ? a.g_k : a.g_q;
            const bool shares = isk && a.dkp;                          // uniform per wave
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const int d = lane + 64 * p;
                g0[u][p] = g1[u][p] = p0[u][p] = p1[u][p] = w0[u][p] = w1[u][p] = 0.f;
                if (d < half) {
                    if (shares) { if (!defer_shares) { g0[u][p] = buf[qd + h * hd + d]; g1[u][p] = buf[qd + h * hd + d + half]; } }
                    else { g0[u][p] = gin[d]; g1[u][p] = gin[d + half]; }
                    p0[u][p] = xp[d]; p1[u][p] = xp[d + half];
                    w0[u][p] = g[d]; w1[u][p] = g[d + half];
                }
            }
        }
    };
    auto take_shares = [&](int s0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < SU; u++) {
            const int slot = min(s0 + (NT / 64) * u, nslots - 1);
            if (slot < a.Hq) continue;
            const int h = slot - a.Hq;
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const int d = lane + 64 * p;
                if (d < half) { g0[u][p] = buf[qd + h * hd + d]; g1[u][p] = buf[qd + h * hd + d + half]; }
            }
        }
    };
    auto finish_trip = [&](int s0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < SU; u++) {
            const int slot = s0 + (NT / 64) * u;
            float y0[NP], y1[NP];
            float ss = 0.f, dot = 0.f;
#pragma unroll
            for (int p = 0; p < NP; p++) {
                y0[p] = g0[u][p] * cs[p].x + g1[u][p] * cs[p].y;
                y1[p] = -g0[u][p] * cs[p].y + g1[u][p] * cs[p].x;
                ss += p0[u][p] * p0[u][p] + p1[u][p] * p1[u][p];
                dot += y0[p] * w0[u][p] * p0[u][p] + y1[p] * w1[u][p] * p1[u][p];
            }
            ss = wave_sum(ss);
            dot = wave_sum(dot);
            if (slot >= nslots) continue;                              // uniform per wave
            const int isk = slot >= a.Hq, h = isk ? slot - a.Hq : slot;
            const float inv = rsqrtf(ss / (float)hd + a.eps);
            const float coeff = dot * inv * inv / (float)hd;
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const int d = lane + 64 * p;
                if (d >= half) continue;
                const float d0 = (w0[u][p] * y0[p] - coeff * p0[u][p]) * inv;
                const float d1 = (w1[u][p] * y1[p] - coeff * p1[u][p]) * inv;
                const int c0 = (isk ? qd : 0) + h * hd + d;
                buf[c0] = d0;
                buf[c0 + half] = d1;
                amax = fmaxf(amax, fmaxf(fabsf(d0), fabsf(d1)));
                if (!isk) { a.dq_f[row * qd + h * hd + d] = d0; a.dq_f[row * qd + h * hd + d + half] = d1; }
            }
        }
    };
    constexpr int TRIP = (NT / 64) * SU;
    const bool first = wave < nslots;
    if (first) load_trip(wave, true);
    if (a.dkp) {
        // dk and dv arrive as shares: their sums are formed by all threads while the loads of the first trip are on
        // their way, SHU elements of a thread per round trip.  dk waits in its place in the row (the wave that owns a
        // head reads it there before it writes the head's result), dv is final.
        constexpr int SHU = NP == 1 ? 2 : 1;               // (wide heads: the first trip's values leave no registers for two)
        for (int c0 = threadIdx.x; c0 < 2 * kd; c0 += SHU * NT) {
            const float *sh[SHU]; int hk[SHU], dd[SHU], cc[SHU]; bool on[SHU], isv[SHU]; float v[SHU];
#pragma unroll
            for (int u = 0; u < SHU; u++) {
                const int c = c0 + u * NT;
                on[u] = c < 2 * kd; isv[u] = c >= kd; cc[u] = on[u] ? (isv[u] ? c - kd : c) : 0;
                sh[u] = isv[u] ? a.dvp : a.dkp; hk[u] = cc[u] / hd; dd[u] = cc[u] % hd;
            }
            kv_share_sums<SHU>(a, sh, row, pos, hk, dd, on, v);
#pragma unroll
            for (int u = 0; u < SHU; u++) {
                if (!on[u]) continue;
                buf[qd + c0 + u * NT] = v[u];
                if (isv[u]) { a.dv_f[row * kd + cc[u]] = v[u]; amax = fmaxf(amax, fabsf(v[u])); }
            }
        }
        __syncthreads();
        if (first) take_shares(wave);
    }
    if (first) finish_trip(wave);
    for (int s0 = wave + TRIP; s0 < nslots; s0 += TRIP) { load_trip(s0, false); finish_trip(s0); }
    if (!a.dvp)
        for (int c = threadIdx.x; c < kd; c += NT) { const float v = a.dv[row * kd + c]; buf[qd + kd + c] = v; amax = fmaxf(amax, fabsf(v)); }
    __syncthreads();
    // dh[r] = sc * sum_c d[c] * B[c][r].  Rank 16 (the common case): four threads share a row of B (16 floats, one
    // float4 each) and 256 such groups split the columns, so a thread keeps 4 + 4 sums and a wave reduces over its 16
    // groups in four shuffle steps; other ranks: a thread walks whole rows of B.
    if (RK != 0 && R > 0) {
        if constexpr (RK == 16) {
            const int sub = threadIdx.x & 3;
            float aq[4] = {0.f, 0.f, 0.f, 0.f}, av[4] = {0.f, 0.f, 0.f, 0.f};
            // two plain loops (q columns, then v columns), so that the loads of B of eight trips can be in flight at once:
            // every workgroup reads all of B, and what bounds it is how much of that one CU keeps in flight
            if (a.Bq16 && NT == RB) {                      // (uniform; decided outside the loops so that each keeps its loads in flight)
                // fp16 copies, a row per workgroup of 1024 threads: the fp32 loop's shape with 8-byte loads
                typedef _Float16 half4v __attribute__((ext_vector_type(4)));
#pragma unroll 8
                for (int c = threadIdx.x >> 2; c < qd; c += NT / 4) {
                    const float x = buf[c];
                    const half4v w = *reinterpret_cast<const half4v *>(a.Bq16 + (size_t)c * 16 + 4 * sub);
                    aq[0] += x * (float)w[0]; aq[1] += x * (float)w[1]; aq[2] += x * (float)w[2]; aq[3] += x * (float)w[3];
                }
#pragma unroll 4
                for (int c = threadIdx.x >> 2; c < kd; c += NT / 4) {
                    const float x = buf[qd + kd + c];
                    const half4v w = *reinterpret_cast<const half4v *>(a.Bv16 + (size_t)c * 16 + 4 * sub);
                    av[0] += x * (float)w[0]; av[1] += x * (float)w[1]; av[2] += x * (float)w[2]; av[3] += x * (float)w[3];
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
#pragma unroll
                    for (int o = 4; o < 64; o <<= 1) { aq[e] += __shfl_xor(aq[e], o, WAVE); av[e] += __shfl_xor(av[e], o, WAVE); }
                }
                if (lane < 4) {
#pragma unroll
                    for (int e = 0; e < 4; e++) { dhp[wave * 32 + 4 * lane + e] = aq[e]; dhp[wave * 32 + 16 + 4 * lane + e] = av[e]; }
                }
            } else if (a.Bq16) {                           // 256 threads per row (many rows): the loads dominate, see below
                // fp16 copies: two threads share a row of B (8 halves = 16 bytes each): half as many load instructions for
                // half the bytes (a thread of a 256-thread workgroup walks 32 rows of B_q)
                const int sub2 = threadIdx.x & 1;
                float q8s[8], v8s[8];
#pragma unroll
                for (int e = 0; e < 8; e++) q8s[e] = v8s[e] = 0.f;
#pragma unroll 8
                for (int c = threadIdx.x >> 1; c < qd; c += NT / 2) {
                    const float x = buf[c];
                    const half8 w = *reinterpret_cast<const half8 *>(a.Bq16 + (size_t)c * 16 + 8 * sub2);
#pragma unroll
                    for (int e = 0; e < 8; e++) q8s[e] += x * h2f(w[e]);
                }
#pragma unroll 2
                for (int c = threadIdx.x >> 1; c < kd; c += NT / 2) {
                    const float x = buf[qd + kd + c];
                    const half8 w = *reinterpret_cast<const half8 *>(a.Bv16 + (size_t)c * 16 + 8 * sub2);
#pragma unroll
                    for (int e = 0; e < 8; e++) v8s[e] += x * h2f(w[e]);
                }
#pragma unroll
                for (int e = 0; e < 8; e++) {
#pragma unroll
                    for (int o = 2; o < 64; o <<= 1) { q8s[e] += __shfl_xor(q8s[e], o, WAVE); v8s[e] += __shfl_xor(v8s[e], o, WAVE); }
                }
                if (lane < 2) {
#pragma unroll
                    for (int e = 0; e < 8; e++) { dhp[wave * 32 + 8 * lane + e] = q8s[e]; dhp[wave * 32 + 16 + 8 * lane + e] = v8s[e]; }
                }
            } else {
#pragma unroll 8
                for (int c = threadIdx.x >> 2; c < qd; c += NT / 4) {
                    const float x = buf[c];
                    const float4 w = ld4(a.Bq + (size_t)c * 16 + 4 * sub);
                    aq[0] += x * w.x; aq[1] += x * w.y; aq[2] += x * w.z; aq[3] += x * w.w;
                }
#pragma unroll 4
                for (int c = threadIdx.x >> 2; c < kd; c += NT / 4) {
                    const float x = buf[qd + kd + c];
                    const float4 w = ld4(a.Bv + (size_t)c * 16 + 4 * sub);
                    av[0] += x * w.x; av[1] += x * w.y; av[2] += x * w.z; av[3] += x * w.w;
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
#pragma unroll
                    for (int o = 4; o < 64; o <<= 1) { aq[e] += __shfl_xor(aq[e], o, WAVE); av[e] += __shfl_xor(av[e], o, WAVE); }
                }
                if (lane < 4) {
#pragma unroll
                    for (int e = 0; e < 4; e++) { dhp[wave * 32 + 4 * lane + e] = aq[e]; dhp[wave * 32 + 16 + 4 * lane + e] = av[e]; }
                }
            }
        } else {
        float acc[32];
#pragma unroll
        for (int r = 0; r < 32; r++) acc[r] = 0.f;
#pragma unroll 4
        for (int c = threadIdx.x; c < qd + kd; c += NT) {
            const int isv = c >= qd;
            const float x = buf[isv ? c + kd : c];
            const float *Br = isv ? a.Bv + (size_t)(c - qd) * R : a.Bq + (size_t)c * R;
            float bv[16];
            if ((R & 3) == 0) {
#pragma unroll
                for (int r4 = 0; r4 < 16; r4 += 4) {
                    float4 w = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (r4 < R) w = ld4(Br + r4);
                    bv[r4] = w.x; bv[r4 + 1] = w.y; bv[r4 + 2] = w.z; bv[r4 + 3] = w.w;
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; r++) bv[r] = (r < R) ? Br[r] : 0.f;
            }
#pragma unroll
            for (int r = 0; r < 16; r++) { if (isv) acc[16 + r] += x * bv[r]; else acc[r] += x * bv[r]; }
        }
#pragma unroll
        for (int r = 0; r < 32; r++) acc[r] = wave_sum(acc[r]);
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < 32; r++) dhp[wave * 32 + r] = acc[r];
        }
        }
        __syncthreads();
        if (threadIdx.x < 2 * R) {
            const int isv = threadIdx.x >= R, rr = isv ? threadIdx.x - R : threadIdx.x;
            float s = 0.f;
            for (int w = 0; w < NT / 64; w++) s += dhp[w * 32 + (isv ? 16 : 0) + rr];
            s *= a.sc;
            buf[qd + 2 * kd + threadIdx.x] = s;
            a.dh[row * 2 * R + threadIdx.x] = s;
            amax = fmaxf(amax, fabsf(s));
        }
        __syncthreads();
    }
    amax = block_max(amax, sm);                           // (every entry of the row was written by a thread that also took it into its maximum)
    const float s = row_scale_for(amax);
    write_f16_tiled(buf, n, a.out16, row, s);
    if (threadIdx.x == 0) a.inv_scale[row] = 1.0f / s;
}

// ------------------------------------------------------------------ LoRA gradients
// dB = sc * dY^T t, dA = dh^T ln1 (float_matmul_tn + scale, src/nn/fast_sft.c:948-952,
// 962-966): one thread per gradient element, looping over the rows.  Each
// workgroup also leaves the sum of squares of what it wrote (for the global norm).
__global__ __launch_bounds__(TB) void k_lora_grads(LoraGradArgs a)
{
    __shared__ float sm[16];
    {                                                     // blockIdx.y = layer
        const size_t L = blockIdx.y;
        a.dq_f += L * a.st_dq; a.dv_f += L * a.st_dv; a.tq += L * a.st_t; a.tv += L * a.st_t; a.dh += L * a.st_dh;
        a.ln16 += L * a.st_ln16; a.ln_inv_scale += L * a.st_lninv; a.grad += L * a.st_grad; a.sq_slots += L * a.st_slots;
    }
    const size_t idx = (size_t)blockIdx.x * TB + threadIdx.x;
    const size_t nA = (size_t)a.R * a.D, nBq = (size_t)a.qd * a.R, nBv = (size_t)a.kd * a.R;
    float gval = 0.f;
    if (idx < 2 * nA + nBq + nBv) {
        size_t o = idx;
        int which;                                        // 0 dA_q, 1 dB_q, 2 dA_v, 3 dB_v
        if (o < nA) which = 0;
        else if ((o -= nA) < nBq) which = 1;
        else if ((o -= nBq) < nA) which = 2;
        else { o -= nA; which = 3; }
        float s = 0.f;
        if (which == 0 || which == 2) {
            const int r = (int)(o / a.D), d = (int)(o % a.D);
            const int hc = (which == 2 ? a.R : 0) + r;
            const int Kb = tiled_kb(a.D);
#pragma unroll 8
            for (int i = 0; i < a.rows; i++)
                s += a.dh[(size_t)i * 2 * a.R + hc] * (h2f(a.ln16[tiled_a_index(i, d, Kb)]) * a.ln_inv_scale[i]);
        } else {
            const int c = (int)(o / a.R), r = (int)(o % a.R);
            const float *dy = which == 1 ? a.dq_f : a.dv_f;
            const float *t = which == 1 ? a.tq : a.tv;
            const int W = which == 1 ? a.qd : a.kd;
#pragma unroll 8
            for (int i = 0; i < a.rows; i++) s += dy[(size_t)i * W + c] * t[(size_t)i * a.R + r];
            s *= a.sc;
        }
        a.grad[idx] = s;
        gval = s;
    }
    const float sq = block_sum(gval * gval, sm);
    if (threadIdx.x == 0) a.sq_slots[blockIdx.x] = sq;
}

// The same for rank R (16), laid out for coalesced reads: a thread owns one column of dY and forms the R entries of
// its row of dB (or one column d of the input and the 2R entries dA_q[:, d], dA_v[:, d]), looping over the rows with the
// R (2R) factors of a row coming from LDS.  Every sum runs over the rows in the same order as above, so the results are
// the same; only the partial sums of squares are grouped differently.  grid.x = lora_grad_blocks(), block 256.
template <int R>
__global__ __launch_bounds__(256) void k_lora_grads_rank(LoraGradArgs a)
{
    __shared__ float ts[64 * 2 * R];
    __shared__ float sm[16];
    {                                                     // blockIdx.y = layer
        const size_t L = blockIdx.y;
        a.dq_f += L * a.st_dq; a.dv_f += L * a.st_dv; a.tq += L * a.st_t; a.tv += L * a.st_t; a.dh += L * a.st_dh;
        a.ln16 += L * a.st_ln16; a.ln_inv_scale += L * a.st_lninv; a.grad += L * a.st_grad; a.sq_slots += L * a.st_slots;
    }
    const int nbq = (a.qd + 255) / 256, nbv = (a.kd + 255) / 256;
    const int bx = blockIdx.x, tid = threadIdx.x;
    const size_t nA = (size_t)R * a.D, nBq = (size_t)a.qd * R;
    float sq = 0.f;
    if (bx < nbq + nbv) {                                 // dB_q, dB_v
        const bool isv = bx >= nbq;
        const int c = (isv ? bx - nbq : bx) * 256 + tid, W = isv ? a.kd : a.qd;
        const float *dy = isv ? a.dv_f : a.dq_f, *t = isv ? a.tv : a.tq;
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = 0.f;
        for (int i0 = 0; i0 < a.rows; i0 += 64) {
            const int nr = min(64, a.rows - i0);
            __syncthreads();
            for (int e = tid; e < nr * R; e += 256) ts[e] = t[(size_t)i0 * R + e];
            __syncthreads();
            if (c < W) {
#pragma unroll 8
                for (int i = 0; i < nr; i++) {
                    const float y = dy[(size_t)(i0 + i) * W + c];
#pragma unroll
                    for (int r = 0; r < R; r++) acc[r] += y * ts[i * R + r];
                }
            }
        }
        if (c < W) {
            float *out = a.grad + (isv ? 2 * nA + nBq : nA) + (size_t)c * R;
#pragma unroll
            for (int r = 0; r < R; r += 4) {
                const float4 gv = make_float4(acc[r] * a.sc, acc[r + 1] * a.sc, acc[r + 2] * a.sc, acc[r + 3] * a.sc);
                st4(out + r, gv);
                sq += sumsq4(gv);
            }
        }
    } else {                                              // dA_q, dA_v
        const int d = (bx - nbq - nbv) * 256 + tid, Kb = tiled_kb(a.D);
        float aq[R], av[R];
#pragma unroll
        for (int r = 0; r < R; r++) aq[r] = av[r] = 0.f;
        for (int i0 = 0; i0 < a.rows; i0 += 64) {
            const int nr = min(64, a.rows - i0);
            __syncthreads();
            for (int e = tid; e < nr * 2 * R; e += 256) ts[e] = a.dh[(size_t)i0 * 2 * R + e];
            __syncthreads();
            if (d < a.D) {
#pragma unroll 4
                for (int i = 0; i < nr; i++) {
                    const float x = h2f(a.ln16[tiled_a_index(i0 + i, d, Kb)]) * a.ln_inv_scale[i0 + i];
#pragma unroll
                    for (int r = 0; r < R; r++) { aq[r] += ts[i * 2 * R + r] * x; av[r] += ts[i * 2 * R + R + r] * x; }
                }
            }
        }
        if (d < a.D) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                a.grad[(size_t)r * a.D + d] = aq[r];
                a.grad[nA + nBq + (size_t)r * a.D + d] = av[r];
                sq += aq[r] * aq[r] + av[r] * av[r];
            }
        }
    }
    sq = block_sum(sq, sm);
    if (tid == 0) a.sq_slots[bx] = sq;
}

// ------------------------------------------------------------------ gated FFN rows
__device__ __forceinline__ float act_fwd(float g, int gelu)
{
    return gelu ? 0.5f * g * (1.0f + tanhf(gelu_inner(g))) : g / (1.0f + expf(-g));
}

// silu_mul / gelu_mul, shaders/q8_kernels.metal:337-362, with the gate/up saves of
// src/nn/fast_sft.c:715-718.
template <int NT, int MV, int NB, int WPE>                 // threads per row, float4 per thread (4 NT MV >= IS), planes per batch of loads, waves per SIMD to fit
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void k_glu_fwd(GluArgs a)
{
    __shared__ float sm[16];
    const size_t r = xcd_block_row(blockIdx.x, gridDim.x);
    const int IS = a.IS, nv = IS >> 2;
    float4 act[MV];
    float amax = 0.f;
    // the gate and up values of all the thread's columns in one go: positions t (gate) and MV + t (up)
    float4 gu[2 * MV];
    {
        size_t rows[2 * MV]; int cols[2 * MV]; bool ok[2 * MV];
#pragma unroll
        for (int t = 0; t < MV; t++) {
            const int v = threadIdx.x + t * NT;
            rows[t] = rows[MV + t] = r; cols[t] = 4 * v; cols[MV + t] = IS + 4 * v; ok[t] = ok[MV + t] = v < nv;
        }
        planes_at4_multi<2 * MV, NB>(a.in, rows, cols, ok, gu);
    }
#pragma unroll
    for (int t = 0; t < MV; t++) {
        const int v = threadIdx.x + t * NT;
        act[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v < nv) {
            const float4 g = gu[t], u = gu[MV + t];
            if (!a.in_place) {                                // in place: the product wrote [gate | up] where they are kept
                st4(a.gate_pre + r * a.ld_gu + 4 * v, g);
                st4(a.up_val + r * a.ld_gu + 4 * v, u);
            }
            act[t] = make_float4(act_fwd(g.x, a.gelu) * u.x, act_fwd(g.y, a.gelu) * u.y,
                                 act_fwd(g.z, a.gelu) * u.z, act_fwd(g.w, a.gelu) * u.w);
            amax = fmaxf(amax, amax4(act[t]));
        }
    }
    amax = block_max(amax, sm);
    const float s = row_scale_for(amax);
    const int Kb = tiled_kb(IS);
#pragma unroll
    for (int t = 0; t < MV; t++) { const int v = threadIdx.x + t * NT; if (v < nv) st_tiled4(a.out16, r, 4 * v, Kb, act[t], s); }
    zero_tiled_pad(a.out16, r, IS, Kb);
    if (threadIdx.x == 0) a.inv_scale[r] = 1.0f / s;
}

// The same with the columns of a row split among workgroups (grid (rows, groups), block 256): group c covers the
// columns [c * sg.cols, (c + 1) * sg.cols) and scales them by a factor of its own, inv_scale[row * groups + c].  The
// GEMM that reads the operand cuts K into chunks that do not straddle groups, so every plane of its result belongs to
// one factor.  64 rows then occupy the whole GPU instead of 64 CUs.
constexpr int MAXC = 2;                                   // float4 per thread of a column-group workgroup
constexpr int GC_MAX = 512;                               // its threads: 256 for groups of up to 2048 columns, 512 up to 4096
template <int GELU, int GC>                               // compile-time: the kernel's code stays one straight run
__global__ __launch_bounds__(GC) void k_glu_fwd_cols(KARGS16)
{
    KARGS_HOT(GluArgs, a);                                // in, gate_pre, IS, sg.cols
    __shared__ float sm[16];
    const size_t r = blockIdx.x;
    const int IS = a.IS, c0 = blockIdx.y * a.sg.cols, width = min(IS, c0 + a.sg.cols) - c0, nv = width >> 2;
    float4 act[MAXC], gu[2 * MAXC];
    float amax = 0.f;
    {
        size_t rows[2 * MAXC]; int cols[2 * MAXC]; bool ok[2 * MAXC];
#pragma unroll
        for (int t = 0; t < MAXC; t++) {
            const int v = threadIdx.x + t * GC;
            rows[t] = rows[MAXC + t] = r; cols[t] = c0 + 4 * v; cols[MAXC + t] = IS + c0 + 4 * v; ok[t] = ok[MAXC + t] = v < nv;
        }
        kargs_rest(a);                                    // asked for beside the planes
        planes_at4_multi<2 * MAXC, 3>(a.in, rows, cols, ok, gu);
    }
#pragma unroll
    for (int t = 0; t < MAXC; t++) {
        const int v = threadIdx.x + t * GC;
        act[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v < nv) {
            const float4 g = gu[t], u = gu[MAXC + t];
            if (!a.in_place) {
                st4(a.gate_pre + r * a.ld_gu + c0 + 4 * v, g);
                st4(a.up_val + r * a.ld_gu + c0 + 4 * v, u);
            }
            act[t] = make_float4(act_fwd(g.x, GELU) * u.x, act_fwd(g.y, GELU) * u.y,
                                 act_fwd(g.z, GELU) * u.z, act_fwd(g.w, GELU) * u.w);
            amax = fmaxf(amax, amax4(act[t]));
        }
    }
    amax = block_max(amax, sm);
    const float s = row_scale_for(amax);
    const int Kb = tiled_kb(IS);
#pragma unroll
    for (int t = 0; t < MAXC; t++) { const int v = threadIdx.x + t * GC; if (v < nv) st_tiled4(a.out16, r, c0 + 4 * v, Kb, act[t], s); }
    if (c0 + width == IS) zero_tiled_pad(a.out16, r, IS, Kb);
    if (threadIdx.x == 0) a.inv_scale[r * a.sg.groups + blockIdx.y] = 1.0f / s;
}

__device__ __forceinline__ void act_bwd(float dy, float g, float u, int gelu, float &dg, float &du)
{
    if (gelu) {                                           // gelu_mul_backward, shaders/q8_kernels.metal:561-580
        const float t = tanhf(gelu_inner(g));
        const float grad = 0.5f * (1.0f + t) + 0.5f * g * (1.0f - t * t) * 0.7978845608f * (1.0f + 3.0f * 0.044715f * g * g);
        dg = dy * u * grad;
        du = dy * (0.5f * g * (1.0f + t));
    } else {                                              // silu_mul_backward, :540-556
        const float sig = 1.0f / (1.0f + expf(-g));
        dg = dy * u * (sig * (1.0f + g * (1.0f - sig)));
        du = dy * (g * sig);
    }
}

template <int NT, int MV, int NB, int WPE>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void k_glu_bwd(GluArgs a)
{
    __shared__ float sm[16];
    const size_t r = xcd_block_row(blockIdx.x, gridDim.x);
    const int IS = a.IS, nv = IS >> 2;
    float4 dg[MV], du[MV];
    float amax = 0.f;
    float4 dys[MV], gs[MV], us[MV];
    {
        size_t rows[MV]; int cols[MV]; bool ok[MV];
#pragma unroll
        for (int t = 0; t < MV; t++) {
            const int v = threadIdx.x + t * NT;
            rows[t] = r; cols[t] = 4 * v; ok[t] = v < nv;
            gs[t] = us[t] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (v < nv) { gs[t] = ld4(a.gate_pre + r * a.ld_gu + 4 * v); us[t] = ld4(a.up_val + r * a.ld_gu + 4 * v); }
        }
        planes_at4_multi<MV, NB>(a.in, rows, cols, ok, dys);
    }
#pragma unroll
    for (int t = 0; t < MV; t++) {
        const int v = threadIdx.x + t * NT;
        dg[t] = du[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v < nv) {
            const float4 dy = dys[t], g = gs[t], u = us[t];
            act_bwd(dy.x, g.x, u.x, a.gelu, dg[t].x, du[t].x);
            act_bwd(dy.y, g.y, u.y, a.gelu, dg[t].y, du[t].y);
            act_bwd(dy.z, g.z, u.z, a.gelu, dg[t].z, du[t].z);
            act_bwd(dy.w, g.w, u.w, a.gelu, dg[t].w, du[t].w);
            amax = fmaxf(amax, fmaxf(amax4(dg[t]), amax4(du[t])));
        }
    }
    amax = block_max(amax, sm);
    const float s = row_scale_for(amax);
    const int Kb = tiled_kb(2 * IS);
#pragma unroll
    for (int t = 0; t < MV; t++) {
        const int v = threadIdx.x + t * NT;
        if (v < nv) { st_tiled4(a.out16, r, 4 * v, Kb, dg[t], s); st_tiled4(a.out16, r, IS + 4 * v, Kb, du[t], s); }
    }
    zero_tiled_pad(a.out16, r, 2 * IS, Kb);
    if (threadIdx.x == 0) a.inv_scale[r] = 1.0f / s;
}

// The same with the columns of the output row [dgate | dup] split among workgroups (grid (rows, groups), block GC), as
// in k_glu_fwd_cols.  A group may lie in either half or straddle the middle, so a thread computes the half its output
// column belongs to; the inputs of a column are then read twice in all, by different workgroups.
template <int GELU, int GC>
__global__ __launch_bounds__(GC) void k_glu_bwd_cols(KARGS16)
{
    KARGS_HOT(GluArgs, a);                                // in, gate_pre, IS, sg.cols; up_val = gate_pre + IS and ld_gu = 2 IS (checked by the launcher)
    __shared__ float sm[16];
    const size_t r = blockIdx.x;
    const int IS = a.IS, c0 = blockIdx.y * a.sg.cols, width = min(2 * IS, c0 + a.sg.cols) - c0, nv = width >> 2;
    float4 o[MAXC], dys[MAXC], gs[MAXC], us[MAXC];
    float amax = 0.f;
    {
        size_t rows[MAXC]; int cols[MAXC]; bool ok[MAXC];
#pragma unroll
        for (int t = 0; t < MAXC; t++) {
            const int v = threadIdx.x + t * GC, j = c0 + 4 * v;
            rows[t] = r; cols[t] = j < IS ? j : j - IS; ok[t] = v < nv;
            gs[t] = us[t] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (v < nv) { gs[t] = ld4(a.gate_pre + r * (size_t)(2 * IS) + cols[t]); us[t] = ld4(a.gate_pre + r * (size_t)(2 * IS) + IS + cols[t]); }
        }
        kargs_rest(a);
        planes_at4_multi<MAXC, 5>(a.in, rows, cols, ok, dys);
    }
#pragma unroll
    for (int t = 0; t < MAXC; t++) {
        const int v = threadIdx.x + t * GC, j = c0 + 4 * v;
        o[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v < nv) {
            float4 dg, du;
            act_bwd(dys[t].x, gs[t].x, us[t].x, GELU, dg.x, du.x);
            act_bwd(dys[t].y, gs[t].y, us[t].y, GELU, dg.y, du.y);
            act_bwd(dys[t].z, gs[t].z, us[t].z, GELU, dg.z, du.z);
            act_bwd(dys[t].w, gs[t].w, us[t].w, GELU, dg.w, du.w);
            const bool first = j < IS;
            o[t] = make_float4(first ? dg.x : du.x, first ? dg.y : du.y, first ? dg.z : du.z, first ? dg.w : du.w);
            amax = fmaxf(amax, amax4(o[t]));
        }
    }
    amax = block_max(amax, sm);
    const float s = row_scale_for(amax);
    const int Kb = tiled_kb(2 * IS);
#pragma unroll
    for (int t = 0; t < MAXC; t++) { const int v = threadIdx.x + t * GC; if (v < nv) st_tiled4(a.out16, r, c0 + 4 * v, Kb, o[t], s); }
    if (c0 + width == 2 * IS) zero_tiled_pad(a.out16, r, 2 * IS, Kb);
    if (threadIdx.x == 0) a.inv_scale[r * a.sg.groups + blockIdx.y] = 1.0f / s;
}

// ------------------------------------------------------------------ backward rows
// dx_out = dx_prev + RNB(x_saved, sum(dy planes); g), clamped (rms_norm_train_backward,
// shaders/q8_kernels.metal:584-625; residual_add; clamp_tensor :1155-1161;
// src/nn/fast_sft.c:870-874, 975-980).  The operand of the next dX GEMM is dx_out
// itself (Qwen3) or RNB(branch_raw, dx_out; g_branch) (Gemma3's post-norms,
// src/nn/fast_sft.c:798-802, 877-881).
template <int MAXV, bool GROUPED, int NT = RB>
__global__ __launch_bounds__(NT) void k_norm_bwd_rows(KARGS24)
{
    KARGS_HOT(NormBwdArgs, a);                            // rows_launched, D, pf
    __shared__ float sm[32];
    if (blockIdx.x >= a.rows_launched) {                  // these set the kernel's duration: nothing to wait for
        prefetch_weight_tiles<NT>(a.pf, blockIdx.x - a.rows_launched);
        return;
    }
    kargs_rest(a);
    const size_t r = xcd_block_row(blockIdx.x, a.rows_launched);
    const int D = a.D, nv = D >> 2;
    float4 dy[MAXV], x[MAXV], g[MAXV];
    float ss = 0.f, dot = 0.f;
    size_t rows[MAXV]; int cols[MAXV]; bool ok[MAXV];
#pragma unroll
    for (int t = 0; t < MAXV; t++) {
        const int v = threadIdx.x + t * NT;
        x[t] = g[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        rows[t] = r; cols[t] = 4 * v; ok[t] = v < nv;
        if (v < nv) x[t] = ld4(a.x_saved + r * D + 4 * v);
    }
    // one value per thread: the norm weights and the gradient to add to are requested with the row, not after the planes
    // and the reduction (a round trip each); with more values per thread the registers are worth more
    constexpr bool AHEAD = MAXV == 1;
    float4 dprev[MAXV], xb[MAXV], gb[MAXV];
    if constexpr (AHEAD) {
        const int v = threadIdx.x;
        dprev[0] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v < nv) g[0] = ld4(a.g + 4 * v);
        if (v < nv && a.dx_prev) dprev[0] = ld4(a.dx_prev + r * D + 4 * v);
        xb[0] = gb[0] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v < nv && a.d16 && a.branch_raw) { xb[0] = ld4(a.branch_raw + r * D + 4 * v); gb[0] = ld4(a.g_branch + 4 * v); }
    }
    planes_at4_multi<MAXV, (MAXV == 1 ? 20 : NT == RB ? 4 : 3), GROUPED>(a.dy, rows, cols, ok, dy);      // (many rows: 92 registers instead of 108)
    if constexpr (!AHEAD) {
#pragma unroll
        for (int t = 0; t < MAXV; t++) { const int v = threadIdx.x + t * NT; if (v < nv) g[t] = ld4(a.g + 4 * v); }
    }
#pragma unroll
    for (int t = 0; t < MAXV; t++) {
        ss += sumsq4(x[t]);
        dot += dy[t].x * g[t].x * x[t].x + dy[t].y * g[t].y * x[t].y + dy[t].z * g[t].z * x[t].z + dy[t].w * g[t].w * x[t].w;
    }
    block_sum2(ss, dot, sm);
    const float inv = rsqrtf(ss / (float)D + a.eps);
    const float coeff = dot * inv * inv / (float)D;
    float4 dx[MAXV];
#pragma unroll
    for (int t = 0; t < MAXV; t++) {
        const int v = threadIdx.x + t * NT;
        dx[t] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v >= nv) continue;
        dx[t] = make_float4((g[t].x * dy[t].x - coeff * x[t].x) * inv, (g[t].y * dy[t].y - coeff * x[t].y) * inv,
                            (g[t].z * dy[t].z - coeff * x[t].z) * inv, (g[t].w * dy[t].w - coeff * x[t].w) * inv);
        if (a.dx_prev) {
            float4 p;
            if constexpr (AHEAD) p = dprev[t]; else p = ld4(a.dx_prev + r * D + 4 * v);
            dx[t].x += p.x; dx[t].y += p.y; dx[t].z += p.z; dx[t].w += p.w;
        }
        if (a.clamp > 0.f) {
            dx[t].x = fminf(fmaxf(dx[t].x, -a.clamp), a.clamp); dx[t].y = fminf(fmaxf(dx[t].y, -a.clamp), a.clamp);
            dx[t].z = fminf(fmaxf(dx[t].z, -a.clamp), a.clamp); dx[t].w = fminf(fmaxf(dx[t].w, -a.clamp), a.clamp);
        }
        st4(a.dx_out + r * D + 4 * v, dx[t]);
    }
    if (!a.d16) return;
    float amax = 0.f;
    if (a.branch_raw) {
        float ssb = 0.f, dotb = 0.f;
#pragma unroll
        for (int t = 0; t < MAXV; t++) {
            const int v = threadIdx.x + t * NT;
            if (v >= nv) continue;
            if constexpr (AHEAD) { x[t] = xb[t]; g[t] = gb[t]; }
            else { x[t] = ld4(a.branch_raw + r * D + 4 * v); g[t] = ld4(a.g_branch + 4 * v); }
            ssb += sumsq4(x[t]);
            dotb += dx[t].x * g[t].x * x[t].x + dx[t].y * g[t].y * x[t].y + dx[t].z * g[t].z * x[t].z + dx[t].w * g[t].w * x[t].w;
        }
        block_sum2(ssb, dotb, sm);
        const float invb = rsqrtf(ssb / (float)D + a.eps);
        const float cb = dotb * invb * invb / (float)D;
#pragma unroll
        for (int t = 0; t < MAXV; t++) {
            const int v = threadIdx.x + t * NT;
            if (v >= nv) continue;
            dx[t] = make_float4((g[t].x * dx[t].x - cb * x[t].x) * invb, (g[t].y * dx[t].y - cb * x[t].y) * invb,
                                (g[t].z * dx[t].z - cb * x[t].z) * invb, (g[t].w * dx[t].w - cb * x[t].w) * invb);
        }
    }
#pragma unroll
    for (int t = 0; t < MAXV; t++) amax = fmaxf(amax, amax4(dx[t]));
    amax = block_max(amax, sm);
    const float s = row_scale_for(amax);
    const int Kb = tiled_kb(D);
#pragma unroll
    for (int t = 0; t < MAXV; t++) { const int v = threadIdx.x + t * NT; if (v < nv) st_tiled4(a.d16, r, 4 * v, Kb, dx[t], s); }
    zero_tiled_pad(a.d16, r, D, Kb);
    if (threadIdx.x == 0) a.inv_scale[r] = 1.0f / s;
}

// ------------------------------------------------------------------ loss rows
// softmax_ce_train + scale(1/BN), shaders/q8_kernels.metal:646-690 and
// src/nn/fast_sft.c:754-760.  The gradient is written once, as the lm_head dX GEMM's
// fp16 operand: (softmax - onehot) * 1024 with row factor (1/BN) / 1024.  With a.grpo the row
// factor carries the policy-gradient weight instead (src/nn/fast_grpo.c:437-452).
// A row of logits (150 k to 260 k floats) is cut into CE_CHUNKS pieces so that rows x CE_CHUNKS workgroups
// share the work: the first launch leaves every piece's maximum and sum of exponentials, the second combines
// them into the row's log-sum-exp and writes its piece of the gradient.
__device__ __forceinline__ void ce_chunk_range(int V, int chunk, int &c_beg, int &c_end)
{
    const int groups = tiled_kb(V) * 8;                   // 8-column groups of the tiled fp16 row, K padding included
    const int per = (groups + CE_CHUNKS - 1) / CE_CHUNKS;
    c_beg = min(chunk * per, groups);
    c_end = min(c_beg + per, groups);
}

__global__ __launch_bounds__(256) void k_ce_partial(CeArgs a)
{
    __shared__ float sm[16];
    const size_t r = blockIdx.y;
    const int chunk = blockIdx.x, V = a.V;
    const float *lg = a.logits + r * V;
    int c_beg, c_end;
    ce_chunk_range(V, chunk, c_beg, c_end);
    const int e_beg = min(c_beg * 8, V), e_end = min(c_end * 8, V);     // V % 4 == 0 is checked by the launcher
    // one pass over the piece: every thread keeps a running maximum and the sum of exponentials relative to it, rescaled
    // when the maximum moves; the threads' pairs are then brought to the piece's maximum
    float tm = -1e30f, ts = 0.f;
#pragma unroll 4
    for (int i = e_beg + 4 * threadIdx.x; i < e_end; i += 4 * 256) {
        const float4 x = ld4(lg + i);
        const float m4 = fmaxf(fmaxf(x.x, x.y), fmaxf(x.z, x.w));
        if (m4 > tm) { ts *= expf(tm - m4); tm = m4; }
        ts += expf(x.x - tm) + expf(x.y - tm) + expf(x.z - tm) + expf(x.w - tm);
    }
    const float mx = block_max(tm, sm);
    const float sum = block_sum(ts * expf(tm - mx), sm);   // a thread without elements: 0 * exp(-1e30 - mx) = 0
    if (threadIdx.x == 0) a.partials[r * CE_CHUNKS + chunk] = make_float2(mx, sum);
}

__global__ __launch_bounds__(256) void k_ce_rows(CeArgs a)
{
    const size_t r = blockIdx.y;
    const int chunk = blockIdx.x, V = a.V;
    const float *lg = a.logits + r * V;
    const uint32_t tgt = a.targets[r];
    float mx = -1e30f;
    float2 part[CE_CHUNKS];
#pragma unroll
    for (int c = 0; c < CE_CHUNKS; c++) { part[c] = a.partials[r * CE_CHUNKS + c]; mx = fmaxf(mx, part[c].x); }
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < CE_CHUNKS; c++) sum += part[c].y * expf(part[c].x - mx);      // empty pieces: 0 * exp(-1e30 - mx) = 0
    const float lse = logf(sum) + mx;
    if (chunk == 0 && threadIdx.x == 0) {
        // coefficient of (softmax - onehot): 1/BN for the cross-entropy; w * ratio * dl_scale for the
        // PPO-clip policy gradient (grpo_policy_grad, shaders/q8_kernels.metal:741-760)
        float coef = 1.0f / (float)a.rows_total;
        if (a.grpo) {
            const float new_lp = lg[tgt] - lse;
            const float ratio = expf(new_lp - a.old_lp[r]);
            const float clipped = fminf(fmaxf(ratio, 1.0f - a.clip_eps), 1.0f + a.clip_eps);
            const float adv = a.advs[r];
            const float w = (adv >= 0.f) ? ((ratio <= clipped) ? -adv : 0.f) : ((ratio >= clipped) ? -adv : 0.f);
            coef = w * ratio * a.dl_scale;
            a.new_lp[r] = new_lp;
        } else {
            a.losses[r] = lse - lg[tgt];
        }
        a.inv_scale[r] = coef * (1.0f / 1024.0f);
    }
    int c_beg, c_end;
    ce_chunk_range(V, chunk, c_beg, c_end);
    const int Kb = tiled_kb(V);
    // four groups of eight logits per thread and trip, all eight loads issued before the first exponential
    constexpr int U = 4;
    for (int cb = c_beg + threadIdx.x; cb < c_end; cb += 256 * U) {
        float4 lo4[U], hi4[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = cb + 256 * u;
            // V % 4 == 0 (checked by the launcher): the eight logits are two aligned 16-byte loads, each inside the row or not
            lo4[u] = (c < c_end && c * 8 < V) ? ld4(lg + c * 8) : make_float4(0.f, 0.f, 0.f, 0.f);
            hi4[u] = (c < c_end && c * 8 + 4 < V) ? ld4(lg + c * 8 + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = cb + 256 * u;
            if (c >= c_end) break;
            const float x[8] = {lo4[u].x, lo4[u].y, lo4[u].z, lo4[u].w, hi4[u].x, hi4[u].y, hi4[u].z, hi4[u].w};
            half8 hv;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int i = c * 8 + e;
                hv[e] = (i < V) ? f2h((expf(x[e] - lse) - ((uint32_t)i == tgt ? 1.0f : 0.0f)) * 1024.0f) : (half_t)0;
            }
            *reinterpret_cast<half8 *>(a.dl16 + tiled_a_index((int)r, c * 8, Kb)) = hv;
        }
    }
}

// The second launch for many rows: a workgroup takes eight consecutive rows of one piece, thread t row t & 7, so that the
// eight 16-byte groups that share a 128-byte line of the tiled gradient (the same columns of eight rows) are written by
// eight neighbouring lanes as one line; a row is still read in runs of 256 bytes (eight groups) per wave.
__global__ __launch_bounds__(256) void k_ce_rows8(CeArgs a, int rows)
{
    __shared__ float s_lse[8];
    __shared__ uint32_t s_tgt[8];
    const int chunk = blockIdx.x, V = a.V, sub = threadIdx.x & 7;
    const size_t r = (size_t)blockIdx.y * 8 + sub;
    if (threadIdx.x < 8 && r < (size_t)rows) {
        const float *lg = a.logits + r * V;
        const uint32_t tgt = a.targets[r];
        float mx = -1e30f;
        float2 part[CE_CHUNKS];
#pragma unroll
        for (int c = 0; c < CE_CHUNKS; c++) { part[c] = a.partials[r * CE_CHUNKS + c]; mx = fmaxf(mx, part[c].x); }
        float sum = 0.f;
#pragma unroll
        for (int c = 0; c < CE_CHUNKS; c++) sum += part[c].y * expf(part[c].x - mx);
        const float lse = logf(sum) + mx;
        s_lse[sub] = lse; s_tgt[sub] = tgt;
        if (chunk == 0) {                                  // as in k_ce_rows
            float coef = 1.0f / (float)a.rows_total;
            if (a.grpo) {
                const float new_lp = lg[tgt] - lse;
                const float ratio = expf(new_lp - a.old_lp[r]);
                const float clipped = fminf(fmaxf(ratio, 1.0f - a.clip_eps), 1.0f + a.clip_eps);
                const float adv = a.advs[r];
                const float w = (adv >= 0.f) ? ((ratio <= clipped) ? -adv : 0.f) : ((ratio >= clipped) ? -adv : 0.f);
                coef = w * ratio * a.dl_scale;
                a.new_lp[r] = new_lp;
            } else {
                a.losses[r] = lse - lg[tgt];
            }
            a.inv_scale[r] = coef * (1.0f / 1024.0f);
        }
    }
    __syncthreads();
    if (r >= (size_t)rows) return;
    const float lse = s_lse[sub];
    const uint32_t tgt = s_tgt[sub];
    const float *lg = a.logits + r * V;
    // pieces of whole tiles (eight groups), not the first launch's pieces: a wave then writes both column halves of its
    // rows, 256 contiguous bytes per slice of a tile
    const int Kb = tiled_kb(V), tiles_per = (Kb + CE_CHUNKS - 1) / CE_CHUNKS;
    const int c_beg = min(chunk * tiles_per, Kb) * 8, c_end = min((chunk + 1) * tiles_per, Kb) * 8;
    constexpr int U = 4;
    for (int cb = c_beg + (threadIdx.x >> 3); cb < c_end; cb += 32 * U) {
        float4 lo4[U], hi4[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = cb + 32 * u;
            lo4[u] = (c < c_end && c * 8 < V) ? ld4(lg + c * 8) : make_float4(0.f, 0.f, 0.f, 0.f);
            hi4[u] = (c < c_end && c * 8 + 4 < V) ? ld4(lg + c * 8 + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = cb + 32 * u;
            if (c >= c_end) break;
            const float x[8] = {lo4[u].x, lo4[u].y, lo4[u].z, lo4[u].w, hi4[u].x, hi4[u].y, hi4[u].z, hi4[u].w};
            half8 hv;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int i = c * 8 + e;
                hv[e] = (i < V) ? f2h((expf(x[e] - lse) - ((uint32_t)i == tgt ? 1.0f : 0.0f)) * 1024.0f) : (half_t)0;
            }
            *reinterpret_cast<half8 *>(a.dl16 + tiled_a_index((int)r, c * 8, Kb)) = hv;
        }
    }
}

// ------------------------------------------------------------------ optimiser
// clip_grad_norm + adamw_update, src/nn/fast_sft.c:1045-1107, in one pass over the
// flat LoRA arena: the global norm comes from the per-workgroup sums of squares
// (double accumulator, as the reference), gradients are rescaled in place when
// the norm exceeds max_norm, and the fp16 images of A_q / A_v inside the fused
// QKV weight (and its transpose) are refreshed for the next step's GEMMs.
__global__ __launch_bounds__(1024) void k_grad_norm(const float *__restrict__ slots, int n, float *out)
{
    __shared__ double sd[16];
    double s = 0.0;
    for (int i = threadIdx.x; i < n; i += blockDim.x) s += (double)slots[i];
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, WAVE);
    if ((threadIdx.x & 63) == 0) sd[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int i = 0; i < (int)(blockDim.x >> 6); i++) t += sd[i];
        out[0] = (float)sqrt(t);
    }
}

__device__ __forceinline__ void shadow_store(const AdamArgs &a, size_t idx, float pv)
{
    if (a.p16) a.p16[idx] = f2h(pv);
    const size_t L = idx / a.layer_size;
    size_t o = idx % a.layer_size;
    const size_t nA = (size_t)a.R * a.D, nBq = (size_t)a.qd * a.R;
    int rbase;
    if (o < nA) rbase = 0;
    else if (o >= nA + nBq && o < 2 * nA + nBq) { o -= nA + nBq; rbase = a.R; }
    else return;
    const int r = (int)(o / a.D), d = (int)(o % a.D);
    const int rowx = a.a_row0 + rbase + r;
    const half_t hv = f2h(pv);
    a.wqkv[L * a.wqkv_layer_stride + tiled_index(rowx, d, tiled_kb(a.D))] = hv;
    a.wqkvT[L * a.wqkvT_layer_stride + tiled_index(d, rowx, a.kbT)] = hv;
}

__global__ __launch_bounds__(TB) void k_adamw(AdamArgs a)
{
    const float lr = a.hyper[0], bc1 = a.hyper[1], bc2 = a.hyper[2];
    const float norm = a.grad_norm_out[0];
    const float gscale = (norm > a.max_norm) ? a.max_norm / norm : 1.0f;
    const bool clip = norm > a.max_norm;
    for (size_t i = (size_t)blockIdx.x * TB + threadIdx.x; i < a.n; i += (size_t)gridDim.x * TB) {
        float g = a.g[i];
        if (clip) { g *= gscale; a.g[i] = g; }
        const float m = a.b1 * a.m[i] + (1.0f - a.b1) * g;
        const float v = a.b2 * a.v[i] + (1.0f - a.b2) * g * g;
        a.m[i] = m;
        a.v[i] = v;
        const float mh = m / bc1, vh = v / bc2;
        float p = a.p[i];
        p -= lr * (mh / (sqrtf(vh) + a.eps) + a.wd * p);
        a.p[i] = p;
        shadow_store(a, i, p);
    }
}

__global__ __launch_bounds__(TB) void k_lora_shadow(AdamArgs a)
{
    for (size_t i = (size_t)blockIdx.x * TB + threadIdx.x; i < a.n; i += (size_t)gridDim.x * TB)
        shadow_store(a, i, a.p[i]);
}

__global__ void k_fill_f32(float *p, float v, size_t n)
{
    const size_t i = (size_t)blockIdx.x * TB + threadIdx.x;
    if (i < n) p[i] = v;
}

#define LAUNCH(kern, grid, block, lds, ...) do { \
    hipLaunchKernelGGL(kern, grid, block, lds, stream(), __VA_ARGS__); HIP_CHECK(hipGetLastError()); } while (0)
// a kernel declared with KARGS<NQ> (kargs.h): its argument struct travels as NQ scalar words
#define LAUNCHK(NQ, kern, grid, block, lds, args) do { \
    launch_kargs<NQ>(kern, grid, block, lds, stream(), args); HIP_CHECK(hipGetLastError()); } while (0)

void require(bool ok, const char *what)
{
    if (!ok) { fprintf(stderr, "[fast_hip] unsupported shape: %s\n", what); abort(); }
}

}  // namespace

void launch_norm_rows(const NormRowsArgs &a, int rows)
{
    require(a.D > 0 && a.D % 4 == 0 && a.D <= 4 * RB * MAXV, "norm_rows: hidden size must be a multiple of 4, <= 12288");
    require(a.branch.S == 0 || a.branch.ld % 4 == 0, "norm_rows: plane row length must be a multiple of 4");
    require((a.emb != nullptr) != (a.x_prev != nullptr), "norm_rows: the row is either gathered (emb) or read (x_prev)");
    const bool grouped = a.branch.S > 0 && a.branch.scale_groups != 0;
    NormRowsArgs b = a;
    b.rows_launched = rows;
    const dim3 grid(rows + (a.pf.base ? a.pf.wgs : 0));
    if (rows >= MANY_ROWS && !grouped && !a.pf.base && a.D <= 4 * TB * MAXV_ROW) { LAUNCHK(24, (k_norm_rows<MAXV_ROW, false, TB>), grid, dim3(TB), 0, b); return; }
    if (a.D <= 4 * RB) { if (grouped) LAUNCHK(24, (k_norm_rows<1, true>), grid, dim3(RB), 0, b); else LAUNCHK(24, (k_norm_rows<1, false>), grid, dim3(RB), 0, b); }
    else { if (grouped) LAUNCHK(24, (k_norm_rows<MAXV_ROW, true>), grid, dim3(RB), 0, b); else LAUNCHK(24, (k_norm_rows<MAXV_ROW, false>), grid, dim3(RB), 0, b); }
}

void launch_rope_table(float2 *tab, int seq, int hd, float theta)
{
    const int n = seq * (hd / 2);
    LAUNCH(k_rope_table, dim3((n + 255) / 256), dim3(256), 0, tab, seq, hd / 2, hd, theta);
}

void launch_qkv_post(const QkvPostArgs &a, int rows)
{
    require(a.hd % 2 == 0 && a.hd <= 2 * 64 * MAXP && a.R <= 64 && a.Hq % a.Hkv == 0, "qkv_post: head_dim <= 512, rank <= 64");
    require(!a.qkv.scale_groups, "qkv_post: input planes with grouped row factors are not supported");
    const size_t tasks = (size_t)rows * (a.Hq + 2 * a.Hkv);
    QkvPostArgs b = a;
    b.rows = rows;
    const dim3 grid((unsigned)((tasks + 3) / 4));
    if (a.hd <= 128) {
        if (a.R == 16) LAUNCH((k_qkv_post<1, 16>), grid, dim3(TB), 0, b);
        else if (a.R == 0) LAUNCH((k_qkv_post<1, 0>), grid, dim3(TB), 0, b);
        else LAUNCH((k_qkv_post<1, -1>), grid, dim3(TB), 0, b);
    } else {
        if (a.R == 16) LAUNCH((k_qkv_post<MAXP, 16>), grid, dim3(TB), 0, b);
        else if (a.R == 0) LAUNCH((k_qkv_post<MAXP, 0>), grid, dim3(TB), 0, b);
        else LAUNCH((k_qkv_post<MAXP, -1>), grid, dim3(TB), 0, b);
    }
}

void launch_attn_fwd(const AttnFwdArgs &a)
{
    require(a.hd % 4 == 0 && a.seq <= 4096, "attn_fwd: head_dim % 4, seq <= 4096");
    LAUNCH(k_attn_fwd, dim3(a.Hq, a.seq, a.batch), dim3(64), (size_t)(a.seq + a.hd) * 4, a);
}

void launch_attn_bwd(const AttnBwdArgs &a)
{
    require(a.hd % 4 == 0 && a.seq <= 4096, "attn_bwd: head_dim % 4, seq <= 4096");
    LAUNCH(k_attn_bwd_dq, dim3(a.Hq, a.seq, a.batch), dim3(64), (size_t)(a.seq + a.hd) * 4, a);
    const size_t dkv_lds = ((size_t)2 * (a.Hq / a.Hkv) * a.seq + 8 * a.hd) * 4;
    require(dkv_lds <= 64 * 1024, "attn_bwd: (Hq/Hkv) * seq too large for the dK/dV kernel");
    LAUNCH(k_attn_bwd_dkv, dim3(a.Hkv, a.seq, a.batch), dim3(TB), dkv_lds, a);
}

void launch_qkv_bwd(const QkvBwdArgs &a, int rows)
{
    const size_t n = (size_t)(a.Hq + 2 * a.Hkv) * a.hd + 2 * a.R + 16 * 32;
    require(a.hd <= 2 * 64 * MAXP && n * 4 <= 64 * 1024 && a.R <= 16, "qkv_bwd: row of dq|dk|dv must fit 64 KB of LDS, rank <= 16");
    QkvBwdArgs b = a;
    b.rows_launched = rows;
    const dim3 grid(rows + (a.pf.base ? a.pf.wgs : 0));
    if (rows >= MANY_ROWS && a.R == 16 && a.hd <= 128 && !a.pf.base) { LAUNCH((k_qkv_bwd_rows<1, 16, TB>), grid, dim3(TB), n * 4, b); return; }
    if (rows >= MANY_ROWS && a.R == 0 && !a.pf.base) {      // full-parameter mode: a handful of heads, no adapter projection
        if (a.hd <= 128) LAUNCH((k_qkv_bwd_rows<1, 0, TB>), grid, dim3(TB), n * 4, b);
        else LAUNCH((k_qkv_bwd_rows<MAXP, 0, TB>), grid, dim3(TB), n * 4, b);
        return;
    }
    if (a.hd <= 128) {
        if (a.R == 16) LAUNCH((k_qkv_bwd_rows<1, 16>), grid, dim3(RB), n * 4, b);
        else if (a.R == 0) LAUNCH((k_qkv_bwd_rows<1, 0>), grid, dim3(RB), n * 4, b);
        else LAUNCH((k_qkv_bwd_rows<1, -1>), grid, dim3(RB), n * 4, b);
    } else {
        if (a.R == 16) LAUNCH((k_qkv_bwd_rows<MAXP, 16>), grid, dim3(RB), n * 4, b);
        else if (a.R == 0) LAUNCH((k_qkv_bwd_rows<MAXP, 0>), grid, dim3(RB), n * 4, b);
        else LAUNCH((k_qkv_bwd_rows<MAXP, -1>), grid, dim3(RB), n * 4, b);
    }
}

int lora_grad_blocks(int D, int qd, int kd, int R)
{
    if (R == 16) return (qd + 255) / 256 + (kd + 255) / 256 + (D + 255) / 256;      // k_lora_grads_rank
    const size_t n = (size_t)2 * R * D + (size_t)qd * R + (size_t)kd * R;
    return (int)((n + TB - 1) / TB);
}

void launch_lora_grads(const LoraGradArgs &a)
{
    const dim3 grid(lora_grad_blocks(a.D, a.qd, a.kd, a.R), a.layers > 0 ? a.layers : 1);
    if (a.R == 16) LAUNCH(k_lora_grads_rank<16>, grid, dim3(256), 0, a);
    else LAUNCH(k_lora_grads, grid, dim3(TB), 0, a);
}

void launch_glu_fwd(const GluArgs &a, int rows)
{
    require(a.IS % 4 == 0 && a.IS <= 4 * RB * MAXV && a.in.ld % 4 == 0, "glu_fwd: FFN width must be a multiple of 4, <= 12288");
    require(!a.in.scale_groups, "glu_fwd: input planes with grouped row factors are not supported");
    require(!a.in_place || (a.in.S == 1 && !a.in.row_scale && a.in.p == a.gate_pre && (size_t)a.in.ld == a.ld_gu),
            "glu_fwd: in place needs the product's one finished plane to be the kept [gate | up] array");
    if (a.sg.cols) {
        require(a.sg.cols % 64 == 0 && a.sg.cols <= 4 * GC_MAX * MAXC && (long)a.sg.cols * a.sg.groups >= a.IS && (long)a.sg.cols * (a.sg.groups - 1) < a.IS,
                "glu_fwd: column groups do not fit the row");
        if (a.sg.cols <= 4 * 256 * MAXC) {
            if (a.gelu) LAUNCHK(16, (k_glu_fwd_cols<1, 256>), dim3(rows, a.sg.groups), dim3(256), 0, a);
            else LAUNCHK(16, (k_glu_fwd_cols<0, 256>), dim3(rows, a.sg.groups), dim3(256), 0, a);
        } else {
            if (a.gelu) LAUNCHK(16, (k_glu_fwd_cols<1, 512>), dim3(rows, a.sg.groups), dim3(512), 0, a);
            else LAUNCHK(16, (k_glu_fwd_cols<0, 512>), dim3(rows, a.sg.groups), dim3(512), 0, a);
        }
        return;
    }
    // many rows: one plane per batch of loads keeps the kernel within 64 registers, so that two workgroups share a CU and
    // one's loads run under the other's arithmetic and stores (2048 x 9728: 53.9 -> 38.7 us forward, 75.7 -> 59.7 backward)
    if (rows >= MANY_ROWS) { LAUNCH((k_glu_fwd<RB, MAXV, 1, 8>), dim3(rows), dim3(RB), 0, a); return; }
    LAUNCH((k_glu_fwd<RB, MAXV, 3, 4>), dim3(rows), dim3(RB), 0, a);
}
void launch_glu_bwd(const GluArgs &a, int rows)
{
    require(a.IS % 4 == 0 && a.IS <= 4 * RB * MAXV && a.in.ld % 4 == 0, "glu_bwd: FFN width must be a multiple of 4, <= 12288");
    require(!a.in.scale_groups, "glu_bwd: input planes with grouped row factors are not supported");
    if (a.sg.cols) {
        require(a.sg.cols % 64 == 0 && a.sg.cols <= 4 * GC_MAX * MAXC && (long)a.sg.cols * a.sg.groups >= 2 * a.IS && (long)a.sg.cols * (a.sg.groups - 1) < 2 * a.IS,
                "glu_bwd: column groups do not fit the row");
        require(a.ld_gu == (size_t)2 * a.IS && a.up_val == a.gate_pre + a.IS, "glu_bwd: gate and up are kept as one [rows][2 IS] array");
        if (a.sg.cols <= 4 * 256 * MAXC) {
            if (a.gelu) LAUNCHK(16, (k_glu_bwd_cols<1, 256>), dim3(rows, a.sg.groups), dim3(256), 0, a);
            else LAUNCHK(16, (k_glu_bwd_cols<0, 256>), dim3(rows, a.sg.groups), dim3(256), 0, a);
        } else {
            if (a.gelu) LAUNCHK(16, (k_glu_bwd_cols<1, 512>), dim3(rows, a.sg.groups), dim3(512), 0, a);
            else LAUNCHK(16, (k_glu_bwd_cols<0, 512>), dim3(rows, a.sg.groups), dim3(512), 0, a);
        }
        return;
    }
    if (rows >= MANY_ROWS) { LAUNCH((k_glu_bwd<RB, MAXV, 1, 8>), dim3(rows), dim3(RB), 0, a); return; }
    LAUNCH((k_glu_bwd<RB, MAXV, 5, 4>), dim3(rows), dim3(RB), 0, a);
}

void launch_norm_bwd_rows(const NormBwdArgs &a, int rows)
{
    require(a.D > 0 && a.D % 4 == 0 && a.D <= 4 * RB * MAXV && a.dy.ld % 4 == 0, "norm_bwd_rows: hidden size must be a multiple of 4, <= 12288");
    const bool grouped = a.dy.scale_groups != 0;
    NormBwdArgs b = a;
    b.rows_launched = rows;
    const dim3 grid(rows + (a.pf.base ? a.pf.wgs : 0));
    if (rows >= MANY_ROWS && !grouped && !a.pf.base && a.D <= 4 * TB * MAXV_ROW) { LAUNCHK(24, (k_norm_bwd_rows<MAXV_ROW, false, TB>), grid, dim3(TB), 0, b); return; }
    if (a.D <= 4 * RB) { if (grouped) LAUNCHK(24, (k_norm_bwd_rows<1, true>), grid, dim3(RB), 0, b); else LAUNCHK(24, (k_norm_bwd_rows<1, false>), grid, dim3(RB), 0, b); }
    else { if (grouped) LAUNCHK(24, (k_norm_bwd_rows<MAXV_ROW, true>), grid, dim3(RB), 0, b); else LAUNCHK(24, (k_norm_bwd_rows<MAXV_ROW, false>), grid, dim3(RB), 0, b); }
}

void launch_ce_rows(const CeArgs &a, int rows)
{
    require(a.V % 4 == 0, "ce_rows: vocabulary size must be a multiple of 4");
    require(a.partials != nullptr, "ce_rows: partials scratch missing");
    LAUNCH(k_ce_partial, dim3(CE_CHUNKS, rows), dim3(256), 0, a);
    if (rows >= MANY_ROWS) LAUNCH(k_ce_rows8, dim3(CE_CHUNKS, (rows + 7) / 8), dim3(256), 0, a, rows);
    else LAUNCH(k_ce_rows, dim3(CE_CHUNKS, rows), dim3(256), 0, a);
}

void launch_adamw(const AdamArgs &a)
{
    if (!a.n) return;
    LAUNCH(k_grad_norm, dim3(1), dim3(1024), 0, a.sq_slots, a.n_slots, a.grad_norm_out);
    size_t blocks = (a.n + TB - 1) / TB;
    if (blocks > 4096) blocks = 4096;
    LAUNCH(k_adamw, dim3((unsigned)blocks), dim3(TB), 0, a);
}

void launch_lora_shadow(const float *p, size_t n, half_t *wqkv, size_t wqkv_layer_stride, half_t *wqkvT,
                        size_t wqkvT_layer_stride, int D, int qd, int kd, int R, size_t layer_size, int a_row0, int kbT, half_t *p16)
{
    if (!n) return;
    AdamArgs a{};
    a.p16 = p16;
    a.p = const_cast<float *>(p); a.n = n; a.wqkv = wqkv; a.wqkv_layer_stride = wqkv_layer_stride;
    a.wqkvT = wqkvT; a.wqkvT_layer_stride = wqkvT_layer_stride;
    a.D = D; a.qd = qd; a.kd = kd; a.R = R; a.layer_size = layer_size; a.a_row0 = a_row0; a.kbT = kbT;
    size_t blocks = (n + TB - 1) / TB;
    if (blocks > 4096) blocks = 4096;
    LAUNCH(k_lora_shadow, dim3((unsigned)blocks), dim3(TB), 0, a);
}

void launch_fill_f32(float *p, float v, size_t n)
{
    if (!n) return;
    LAUNCH(k_fill_f32, dim3((unsigned)((n + TB - 1) / TB)), dim3(TB), 0, p, v, n);
}

}  // namespace lmhip
