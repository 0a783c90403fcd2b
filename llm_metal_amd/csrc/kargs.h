// Kernel arguments as scalars.  A kernel that takes its argument struct by value reads it from the kernarg segment with
// scalar loads when its first waves start -- memory the host wrote a moment ago, 1.3 to 1.9 us away -- before it can form
// its first address.  gfx950's command processor can instead put the first 14 dwords of a kernel's arguments into SGPRs
// while the dispatch is being set up (compiler option -mllvm -amdgpu-kernarg-preload-count=16), but only for arguments
// that are scalars, not for a struct.  So the hot kernels take their struct as a row of 64-bit words (KARGS<n> in the
// signature, kargs_unpack in the body, launch_kargs on the host): the struct's first 56 bytes arrive preloaded, the rest
// by scalar loads as before.  A struct is therefore ordered with what its kernel needs for its first loads in front:
// whatever else it touches before those loads are issued costs the full wait again.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <string.h>
#include <utility>

#define KARGS8  uint64_t k0, uint64_t k1, uint64_t k2, uint64_t k3, uint64_t k4, uint64_t k5, uint64_t k6, uint64_t k7
#define KARGS16 KARGS8, uint64_t k8, uint64_t k9, uint64_t k10, uint64_t k11, uint64_t k12, uint64_t k13, uint64_t k14, uint64_t k15
#define KARGS24 KARGS16, uint64_t k16, uint64_t k17, uint64_t k18, uint64_t k19, uint64_t k20, uint64_t k21, uint64_t k22, uint64_t k23
#define KARGS32 KARGS24, uint64_t k24, uint64_t k25, uint64_t k26, uint64_t k27, uint64_t k28, uint64_t k29, uint64_t k30, uint64_t k31
#define KARGS40 KARGS32, uint64_t k32, uint64_t k33, uint64_t k34, uint64_t k35, uint64_t k36, uint64_t k37, uint64_t k38, uint64_t k39
#define KARGS48 KARGS40, uint64_t k40, uint64_t k41, uint64_t k42, uint64_t k43, uint64_t k44, uint64_t k45, uint64_t k46, uint64_t k47
#define KLIST8  k0, k1, k2, k3, k4, k5, k6, k7
#define KLIST16 KLIST8, k8, k9, k10, k11, k12, k13, k14, k15
#define KLIST24 KLIST16, k16, k17, k18, k19, k20, k21, k22, k23
#define KLIST32 KLIST24, k24, k25, k26, k27, k28, k29, k30, k31
#define KLIST40 KLIST32, k32, k33, k34, k35, k36, k37, k38, k39
#define KLIST48 KLIST40, k40, k41, k42, k43, k44, k45, k46, k47

namespace lmhip {

// the struct back from its words (NQ words >= sizeof(A)); all indices are constants, so this is register renaming
template <typename A, int NQ>
__device__ __forceinline__ A kargs_unpack(const uint64_t (&w)[NQ])
{
    static_assert(sizeof(A) <= NQ * sizeof(uint64_t), "the kernel's signature has too few words for its argument struct");
    A a;
    __builtin_memcpy(&a, w, sizeof(A));
    return a;
}

// The same in two steps, for kernels that must not wait for the whole struct before their first loads: KARGS_HOT fills the
// struct's first 56 bytes (the preloaded words k0 .. k6) and leaves the rest unset; kargs_rest() reads the rest from the
// kernarg segment where it is called -- after the first loads have been issued, behind a scheduling barrier, so that its
// wait runs beside theirs.  Between the two only the struct's leading members may be used.
constexpr int KARGS_HOT_BYTES = 56;
#define KARGS_HOT(Type, name) Type name; do { const uint64_t hot_words_[7] = {k0, k1, k2, k3, k4, k5, k6}; \
    static_assert(sizeof(Type) >= lmhip::KARGS_HOT_BYTES, "argument struct shorter than the preloaded part"); \
    __builtin_memcpy(&name, hot_words_, lmhip::KARGS_HOT_BYTES); } while (0)
template <typename A>
__device__ __forceinline__ void kargs_rest(A &a)
{
    typedef __attribute__((address_space(4))) const uint32_t karg_word;
    __builtin_amdgcn_sched_barrier(0);
    karg_word *ka = (karg_word *)((__attribute__((address_space(4))) const char *)__builtin_amdgcn_kernarg_segment_ptr() + KARGS_HOT_BYTES);
    constexpr int NW = (sizeof(A) - KARGS_HOT_BYTES + 3) / 4;
    uint32_t w[NW];
#pragma unroll
    for (int i = 0; i < NW; i++) w[i] = ka[i];
    __builtin_memcpy(reinterpret_cast<char *>(&a) + KARGS_HOT_BYTES, w, sizeof(A) - KARGS_HOT_BYTES);
}

template <int NQ, typename K, typename A, size_t... I>
inline void launch_kargs_seq(K kern, dim3 grid, dim3 block, size_t lds, hipStream_t st, hipEvent_t ev_a, hipEvent_t ev_b, const A &a,
                             std::index_sequence<I...>)
{
    static_assert(sizeof(A) <= NQ * sizeof(uint64_t), "too few words for the argument struct");
    uint64_t w[NQ] = {};
    memcpy(w, &a, sizeof(A));
    if (ev_a || ev_b) hipExtLaunchKernelGGL(kern, grid, block, lds, st, ev_a, ev_b, 0, w[I]...);
    else hipLaunchKernelGGL(kern, grid, block, lds, st, w[I]...);
}
// launches a kernel declared with KARGS<NQ>; ev_a / ev_b (or null) ride on the dispatch as with hipExtLaunchKernelGGL
template <int NQ, typename K, typename A>
inline void launch_kargs(K kern, dim3 grid, dim3 block, size_t lds, hipStream_t st, const A &a, hipEvent_t ev_a = nullptr, hipEvent_t ev_b = nullptr)
{
    launch_kargs_seq<NQ>(kern, grid, block, lds, st, ev_a, ev_b, a, std::make_index_sequence<NQ>());
}

}  // namespace lmhip
