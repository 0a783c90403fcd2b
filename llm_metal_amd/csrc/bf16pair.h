// An fp32 value as two bf16 values for the matrix cores: x = hi + lo, hi the upper 16 bits of x and lo those of x - hi.
// A product of two such operands is three v_mfma_f32_32x32x16_bf16 (hi*hi + lo*hi + hi*lo), accumulated in fp32: 16
// mantissa bits and the whole fp32 exponent range of every operand.
#pragma once
#include "devutil.h"

namespace lmhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// upper halves of two floats in one dword: (lo16 = bf16 of a, hi16 = bf16 of b), truncating
__device__ __forceinline__ uint32_t pack_hi(float a, float b) { return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u); }
// what the truncation to bf16 leaves behind (exact in fp32)
__device__ __forceinline__ float rest(float a) { return a - __uint_as_float(__float_as_uint(a) & 0xffff0000u); }

// eight consecutive reduction values of a lane as matrix-core operands
struct HL { bf16x8 hi, lo; };
__device__ __forceinline__ HL split8(const float (&x)[8])
{
    u32x4 h, l;
#pragma unroll
    for (int i = 0; i < 4; i++) { h[i] = pack_hi(x[2 * i], x[2 * i + 1]); l[i] = pack_hi(rest(x[2 * i]), rest(x[2 * i + 1])); }
    return HL{__builtin_bit_cast(bf16x8, h), __builtin_bit_cast(bf16x8, l)};
}
__device__ __forceinline__ HL split8(const float4 &p, const float4 &q)
{
    const float x[8] = {p.x, p.y, p.z, p.w, q.x, q.y, q.z, q.w};
    return split8(x);
}

}  // namespace lmhip
