// Device helpers shared by the row kernels: reading a GEMM result that is still
// split into K-chunk planes, and 16-byte loads/stores.
#pragma once
#include "fused.h"

namespace lmhip {

__device__ __forceinline__ float planes_at(const Planes &P, size_t row, int col)
{
    float s = 0.f;
    const float *p = P.p + row * P.ld + col;
    if (P.scale_groups) {
        for (int i = 0; i < P.S; i++) s += p[(size_t)i * P.stride] * P.row_scale[row * P.scale_groups + (i >> P.group_shift)];
        return s;
    }
    for (int i = 0; i < P.S; i++) s += p[(size_t)i * P.stride];
    return P.row_scale ? s * P.row_scale[row] : s;
}

// Sum of the planes at four consecutive columns (col % 4 == 0, ld % 4 == 0), added in plane order.
// The loads of up to eight planes are issued together, so their latency is paid once.
__device__ __forceinline__ float4 planes_at4(const Planes &P, size_t row, int col)
{
    const float *p = P.p + row * P.ld + col;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (P.scale_groups) {
        for (int i = 0; i < P.S; i++) {
            const float4 v = *reinterpret_cast<const float4 *>(p + (size_t)i * P.stride);
            const float f = P.row_scale[row * P.scale_groups + (i >> P.group_shift)];
            s.x += v.x * f; s.y += v.y * f; s.z += v.z * f; s.w += v.w * f;
        }
        return s;
    }
    for (int i0 = 0; i0 < P.S; i0 += 8) {
        float4 v[8];
#pragma unroll
        for (int i = 0; i < 8; i++)
            v[i] = (i0 + i < P.S) ? *reinterpret_cast<const float4 *>(p + (size_t)(i0 + i) * P.stride) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < 8; i++) { s.x += v[i].x; s.y += v[i].y; s.z += v[i].z; s.w += v[i].w; }
    }
    if (P.row_scale) { const float f = P.row_scale[row]; s.x *= f; s.y *= f; s.z *= f; s.w *= f; }
    return s;
}

// The same for T positions of one thread at once: the loads of NB planes at all T positions are issued together, so the
// thread pays ceil(S / NB) memory round trips for all of them, where one call of planes_at4 per position pays at least
// one each (its loop over the planes has a run-time bound, which keeps the compiler from overlapping two calls).
// Position t is read only when ok[t]; the sums are formed in plane order, exactly as planes_at4 forms them.
// GROUPED: the planes carry a factor per group of planes (Planes::scale_groups != 0); all T positions must then lie in
// row[0], and row[0] must be the same for the whole wave.
// Planes of halves (Planes::half_unscale != 0) are read 8 bytes at a time and summed in fp32 the same way, NBH planes per
// round trip (twice NB holds the same number of registers).
template <int T, int NB, bool GROUPED = false, int NBH = NB>
__device__ __forceinline__ void planes_at4_multi(const Planes &P, const size_t (&row)[T], const int (&col)[T], const bool (&ok)[T], float4 (&s)[T])
{
    // the rows' factors are requested before the planes (after the sums they would cost a round trip of their own)
    float rs[T];
#pragma unroll
    for (int t = 0; t < T; t++) rs[t] = (!GROUPED && P.row_scale && ok[t]) ? P.row_scale[row[t]] : 1.0f;
    if (P.half_unscale != 0.f) {                          // uniform
        typedef _Float16 half4v __attribute__((ext_vector_type(4)));
        const half_t *ph[T];
#pragma unroll
        for (int t = 0; t < T; t++) { ph[t] = reinterpret_cast<const half_t *>(P.p) + row[t] * P.ld + col[t]; s[t] = make_float4(0.f, 0.f, 0.f, 0.f); }
        auto hbatch = [&](int i0) __attribute__((always_inline)) {
            half4v v[T][NBH];
#pragma unroll
            for (int i = 0; i < NBH; i++)
#pragma unroll
                for (int t = 0; t < T; t++) {
                    v[t][i] = half4v{(_Float16)0, (_Float16)0, (_Float16)0, (_Float16)0};
                    if (ok[t] && i0 + i < P.S) v[t][i] = *reinterpret_cast<const half4v *>(ph[t] + (size_t)(i0 + i) * P.stride);
                }
            if (GROUPED) {
                static_assert(NBH <= 64, "one lane per plane of a batch");
                const int li = threadIdx.x & 63;
                const float fl = (li < NBH && i0 + li < P.S) ? P.row_scale[row[0] * P.scale_groups + ((i0 + li) >> P.group_shift)] : 0.f;
#pragma unroll
                for (int i = 0; i < NBH; i++) {
                    const float f = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fl), i));
#pragma unroll
                    for (int t = 0; t < T; t++) {
                        s[t].x += (float)v[t][i][0] * f; s[t].y += (float)v[t][i][1] * f; s[t].z += (float)v[t][i][2] * f; s[t].w += (float)v[t][i][3] * f;
                    }
                }
                return;
            }
#pragma unroll
            for (int t = 0; t < T; t++)
#pragma unroll
                for (int i = 0; i < NBH; i++) { s[t].x += (float)v[t][i][0]; s[t].y += (float)v[t][i][1]; s[t].z += (float)v[t][i][2]; s[t].w += (float)v[t][i][3]; }
        };
        for (int i0 = 0; i0 < P.S; i0 += NBH) hbatch(i0);
#pragma unroll
        for (int t = 0; t < T; t++) {
            const float f = P.half_unscale * rs[t];
            s[t].x *= f; s[t].y *= f; s[t].z *= f; s[t].w *= f;
        }
        return;
    }
    const float *p[T];
#pragma unroll
    for (int t = 0; t < T; t++) { p[t] = P.p + row[t] * P.ld + col[t]; s[t] = make_float4(0.f, 0.f, 0.f, 0.f); }
    // (a loop, not unrolled: these kernels run their code once, and what they gain from straight-line batches they lose
    // again fetching the longer code)
    auto batch = [&](int i0) __attribute__((always_inline)) {
        float4 v[T][NB];
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (int t = 0; t < T; t++)
                v[t][i] = (ok[t] && i0 + i < P.S) ? *reinterpret_cast<const float4 *>(p[t] + (size_t)(i0 + i) * P.stride) : make_float4(0.f, 0.f, 0.f, 0.f);
        if (GROUPED) {                                    // a factor per plane, fetched with the planes
            // lane i of every wave fetches the factor of plane i0 + i (one load, in flight with the planes); the
            // values then reach all lanes through scalar registers
            static_assert(NB <= 64, "one lane per plane of a batch");
            const int li = threadIdx.x & 63;
            const float fl = (li < NB && i0 + li < P.S) ? P.row_scale[row[0] * P.scale_groups + ((i0 + li) >> P.group_shift)] : 0.f;
            float f[NB];
#pragma unroll
            for (int i = 0; i < NB; i++) f[i] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fl), i));
#pragma unroll
            for (int t = 0; t < T; t++)
#pragma unroll
                for (int i = 0; i < NB; i++) {
                    s[t].x += v[t][i].x * f[i]; s[t].y += v[t][i].y * f[i]; s[t].z += v[t][i].z * f[i]; s[t].w += v[t][i].w * f[i];
                }
            return;
        }
#pragma unroll
        for (int t = 0; t < T; t++)
#pragma unroll
            for (int i = 0; i < NB; i++) { s[t].x += v[t][i].x; s[t].y += v[t][i].y; s[t].z += v[t][i].z; s[t].w += v[t][i].w; }
    };
    for (int i0 = 0; i0 < P.S; i0 += NB) batch(i0);
    if (!GROUPED && P.row_scale) {
#pragma unroll
        for (int t = 0; t < T; t++)
            if (ok[t]) { const float f = rs[t]; s[t].x *= f; s[t].y *= f; s[t].z *= f; s[t].w *= f; }
    }
}

// Single values instead of groups of four (planes without grouped factors only).
template <int T, int NB>
__device__ __forceinline__ void planes_at_multi(const Planes &P, size_t row, const int (&col)[T], const bool (&ok)[T], float (&s)[T])
{
    const float *p[T];
    const float rs = P.row_scale ? P.row_scale[row] : 1.0f;   // requested before the planes, not after their sums
#pragma unroll
    for (int t = 0; t < T; t++) { p[t] = P.p + row * P.ld + col[t]; s[t] = 0.f; }
    auto batch = [&](int i0) __attribute__((always_inline)) {
        float v[T][NB];
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (int t = 0; t < T; t++) v[t][i] = (ok[t] && i0 + i < P.S) ? p[t][(size_t)(i0 + i) * P.stride] : 0.f;
#pragma unroll
        for (int t = 0; t < T; t++)
#pragma unroll
            for (int i = 0; i < NB; i++) s[t] += v[t][i];
    };
    for (int i0 = 0; i0 < P.S; i0 += NB) batch(i0);
    if (P.row_scale) {
#pragma unroll
        for (int t = 0; t < T; t++) s[t] *= rs;
    }
}

// Workgroup `pw` of pf.wgs prefetching workgroups of THREADS threads.  A 4 KB tile is one 16-byte load for each of 256
// threads, so the workgroup takes THREADS / 256 tiles at a time; the loads of a thread are issued eight at a time before
// the first is waited for.
template <int THREADS>
__device__ __forceinline__ void prefetch_weight_tiles(const WeightPrefetch &pf, int pw)
{
    constexpr int TPR = THREADS / 256;                   // tiles per round
    const int total = pf.n_tiles * pf.S, q = threadIdx.x >> 8, t16 = (threadIdx.x & 255) * 16;
    const int per_g = (pf.depth * pf.nb + TPR - 1) / TPR;  // loads of a thread per workgroup of the product
    unsigned sink = 0u;
    for (int j0 = 0; j0 < pf.per_wg * per_g; j0 += 8) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            v[u] = make_uint4(0u, 0u, 0u, 0u);
            const int j = (j0 + u) / per_g, e = (j0 + u) % per_g;
            const int g = pw + pf.wgs * j;               // a workgroup of the product
            const int ts = e * TPR + q, w = ts / pf.nb, b = ts % pf.nb;
            if (j0 + u < pf.per_wg * per_g && g < total && w < pf.depth) {
                const int x = g % pf.n_tiles, y = g / pf.n_tiles;
                const int kb_beg = y * pf.steps, nsteps = min(pf.Kb, kb_beg + pf.steps) - kb_beg;
                if (pf.rotate & 2) {
                    // Q8_0 tiles (2 KB of int8 each, K steps of a row block side by side; Kb even): a 4 KB load takes the
                    // pair of K steps that holds step kb_beg + 2 w
                    const int kt = (kb_beg + 2 * w) & ~1;
                    if (2 * w < nsteps && kt < pf.Kb) {
                        const size_t tile = (size_t)min(x * pf.nb + b, pf.Nb - 1) * pf.Kb + kt;
                        v[u] = *reinterpret_cast<const uint4 *>(pf.base + tile * 2048 + t16);
                    }
                } else {
                    const int rot = pf.rotate ? (int)((x * 7u + y * 3u) % (unsigned)nsteps) : 0;
                    int kk = w + rot;
                    if (kk >= nsteps) kk -= nsteps;
                    if (w < nsteps) {
                        const size_t tile = (size_t)min(x * pf.nb + b, pf.Nb - 1) * pf.Kb + kb_beg + kk;
                        v[u] = *reinterpret_cast<const uint4 *>(pf.base + tile * 4096 + t16);
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 8; u++) sink ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    asm volatile("" :: "v"(sink));                        // the loads have a use, and nothing is stored
}

// Row of workgroup `id` in a one-workgroup-per-row kernel over `rows` rows.  Workgroup ids go to the eight XCDs in
// turn, and such a kernel writes its row of a tiled fp16 operand as 16-byte pieces 512 bytes apart, which only fill
// whole memory lines together with the other 31 rows of the 32-row block.  So within every run of 256 ids XCD x gets
// the 32 rows of one block, one after the other: the pieces meet in that XCD's L2 instead of reaching memory as
// partial lines from eight L2s.  Rows beyond the last whole run of 256 keep their id.
__device__ __forceinline__ int xcd_block_row(int id, int rows)
{
    if (id >= (rows & ~255)) return id;
    const int in = id & 255;
    return (id & ~255) + ((in & 7) << 5) + (in >> 3);
}

__device__ __forceinline__ float4 ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ void st4(float *p, float4 v) { *reinterpret_cast<float4 *>(p) = v; }
__device__ __forceinline__ float amax4(float4 v) { return fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))); }
__device__ __forceinline__ float sumsq4(float4 v) { return v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w; }


}  // namespace lmhip
