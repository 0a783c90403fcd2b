// Device-side helpers shared by the kernels: wave64 / workgroup reductions,
// F16 <-> fp32 conversion with explicit rounding, vector types.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float    float16v __attribute__((ext_vector_type(16)));
typedef float    float4v __attribute__((ext_vector_type(4)));

#define WAVE 64

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// Workgroup reductions for blocks of up to 1024 threads (16 waves).  `smem`
// must hold 16 floats; every thread gets the result.  Two barriers per call,
// so the same `smem` may be reused by the next call.
__device__ __forceinline__ float block_sum(float v, float *smem)
{
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nw; i++) r += smem[i];
    __syncthreads();
    return r;
}

// Two sums for one pair of barriers; `smem` must hold 32 floats.  Each sum is formed in the order block_sum forms it.
__device__ __forceinline__ void block_sum2(float &a, float &b, float *smem)
{
    a = wave_sum(a); b = wave_sum(b);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (lane == 0) { smem[w] = a; smem[16 + w] = b; }
    __syncthreads();
    float ra = 0.f, rb = 0.f;
    for (int i = 0; i < nw; i++) { ra += smem[i]; rb += smem[16 + i]; }
    __syncthreads();
    a = ra; b = rb;
}

// A sum and a maximum for one pair of barriers; `smem` must hold 32 floats.  The sum is formed in the order block_sum forms it.
__device__ __forceinline__ void block_sum_max(float &a, float &m, float *smem)
{
    a = wave_sum(a); m = wave_max(m);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (lane == 0) { smem[w] = a; smem[16 + w] = m; }
    __syncthreads();
    float ra = 0.f, rm = smem[16];
    for (int i = 0; i < nw; i++) { ra += smem[i]; rm = fmaxf(rm, smem[16 + i]); }
    __syncthreads();
    a = ra; m = rm;
}

__device__ __forceinline__ float block_max(float v, float *smem)
{
    v = wave_max(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float r = smem[0];
    for (int i = 1; i < nw; i++) r = fmaxf(r, smem[i]);
    __syncthreads();
    return r;
}

// Power-of-two scale s such that amax * s lies in [2^12, 2^13): the fp16 image of
// a row then keeps 11 significant bits for everything within 2^-26 of the row
// maximum and cannot overflow.  Exact to undo (inv = 1/s is a power of two).
__device__ __forceinline__ float row_scale_for(float amax)
{
    if (!(amax > 0.f) || !(amax < 3.0e38f)) return 1.0f;
    int e;
    frexpf(amax, &e);                 // amax = f * 2^e, f in [0.5, 1)
    int p = 13 - e;
    p = p > 120 ? 120 : (p < -120 ? -120 : p);
    return ldexpf(1.0f, p);
}

// Argument of the tanh in the GELU approximation, clamped as the reference clamps it (gelu_mul,
// shaders/q8_kernels.metal:349-362).
__device__ __forceinline__ float gelu_inner(float g)
{
    const float in = 0.7978845608f * (g + 0.044715f * g * g * g);
    return fminf(fmaxf(in, -15.0f), 15.0f);
}

__device__ __forceinline__ half_t f2h(float x) { return (half_t)x; }      // v_cvt_f16_f32: round to nearest even
__device__ __forceinline__ float  h2f(half_t x) { return (float)x; }

// Workgroup `wg` of `nwgs` reads its share of [base, base + bytes) with 16-byte loads, eight in flight per thread, and
// throws the values away: what a launch with spare CUs does for the weights of the product that follows it (the data then
// waits in the memory-side cache).  bytes % 16 == 0; block of 256 threads or more.
__device__ __forceinline__ void request_bytes_ahead(const char *base, size_t bytes, int wg, int nwgs)
{
    const size_t row = (size_t)blockDim.x * 16;
    const size_t per = ((bytes + nwgs - 1) / nwgs + row - 1) / row * row;
    const size_t beg = (size_t)wg * per, end = bytes < beg + per ? bytes : beg + per;
    unsigned sink = 0u;
    for (size_t o = beg + (size_t)threadIdx.x * 16; o < end; o += 8 * row) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = (o + u * row < end) ? *reinterpret_cast<const uint4 *>(base + o + u * row) : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int u = 0; u < 8; u++) sink ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    asm volatile("" :: "v"(sink));
}
