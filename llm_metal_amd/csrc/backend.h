// Internal header of the HIP backend: buffer handle layout, the library's one
// stream, scratch arenas and launch-time checks shared by the translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include "../../include/fast_hip.h"

struct MetalBuf {
    void   *dev;          // address kernels use (HBM, or the device view of pinned host memory)
    void   *host;         // pinned host allocation once metal_buf_ptr has been called, else NULL
    size_t  size;
    int     owns;         // 0 for views
    MetalBuf *parent;     // views: the buffer whose allocation this window lies in
    size_t  parent_off;
    // lazily built images of a weight held in this buffer: [0], [1] tiled F16 (as is, transposed) for
    // metal_enqueue_f16_matmul / _nt; [2] Q8_0 split into codes and scales for metal_enqueue_q8_matvec
    struct Tiled { void *dev; int rows, cols; uint64_t version; } tiled[3];
    uint64_t version;     // bumped by every enqueue that writes this buffer
};

namespace lmhip {

hipStream_t stream();
int  initialized();
int  num_cus();
void die(const char *what, hipError_t e, const char *file, int line);

// Grow-only device scratch, one arena per purpose; contents are only valid
// within the enqueue that asked for them.
enum ScratchSlot { SCR_A16 = 0, SCR_SCALE, SCR_PARTIAL, SCR_MISC, SCR_WF16, SCR_COUNT };   // SCR_WF16: F16 image of a Q8_0 weight
void *scratch(ScratchSlot slot, size_t bytes);
// infer_kernels.hip: resolves, for the current device, the fixed array behind hip_attention_noalloc (0 / -1)
int noalloc_setup();

// Device address of a buffer; views resolve through their parent so that they
// follow it when metal_buf_ptr migrates the allocation to host memory.
inline void *dptr(const MetalBuf *b) { return b->parent ? (void *)((char *)b->parent->dev + b->parent_off) : b->dev; }
template <typename T> inline T *dptr_as(const MetalBuf *b) { return (T *)dptr(b); }

inline void mark_written(MetalBuf *b) { if (b) { b->version++; if (b->parent) b->parent->version++; } }

// What the generation pipeline does to the Q|K|V product before the attention (src/nn/fast_inference.c:402-427): LoRA
// terms on q and v, per-head RMSNorm and RoPE on q and k, k and v into row `pos` of the caches.
struct HeadPost {
    const float *qkv;                    // [Hq*hd | Hkv*hd | Hkv*hd], left as it is
    const float *g_q, *g_k;              // per-head norm gammas or NULL
    float *kc, *vc;                      // caches [Hkv, max_seq, hd]
    const float *t, *Bq, *Bv;            // adapters: t [2R], B_q [Hq*hd, R], B_v [Hkv*hd, R]; R == 0: none
    int Hq, Hkv, R, pos;
    const float2 *rope;                  // (cos, sin) of the hd/2 rotary pairs at position pos
    float eps, sc;
    size_t qkv_step, cache_step, t_step; // floats from one sequence's qkv / caches / t to the next when several are decoded at once
    // weights of the product that follows, requested ahead by pf_wgs extra workgroups while the few attention workgroups
    // run (pf_wgs == 0: none)
    const char *pf_base; size_t pf_bytes; int pf_wgs;
};
// infer_kernels.hip: that and the attention over the cache rows 0 .. pos in one launch (out [Hq*hd]); with copies > 1
// for that many sequences at position pos, whose caches lie cache_step floats apart inside Kc and Vc (out [copies, Hq*hd])
void attention_decode_fused(const HeadPost &hp, MetalBuf *Kc, MetalBuf *Vc, float *out, int hd, int max_seq, int copies = 1);

// infer_kernels.hip: y[i] = act(gate_i . x) * (up_i . x) for W = [gate; up] of 2 * rows rows (F16, or Q8_0 blocks when q8)
void matvec_glu(MetalBuf *W, MetalBuf *x, MetalBuf *y, int rows, int cols, int q8, int gelu);
// The vector of a product as the sum and norm before it left it: RMSNorm(xr + br; g) with br optional; xr + br goes to
// x_out (another buffer than xr) when that is given.
struct NormIn {
    const float *xr, *br, *g;
    float *x_out;
    float eps;
};
// infer_kernels.hip: y = W . RMSNorm(xr + br; g) (glu 0), or the gated pair product of matvec_glu over it (1 SiLU, 2 GELU)
void matvec_norm(MetalBuf *W, const NormIn &nin, MetalBuf *y, int rows, int cols, int q8, int glu);

}  // namespace lmhip

#define LMHIP_API extern "C" __attribute__((visibility("default")))
#define HIP_CHECK(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) lmhip::die(#expr, e_, __FILE__, __LINE__); } while (0)

// Host-side guard against launching on operands smaller than the kernel will touch.
#define REQUIRE_BYTES(buf, bytes, fn) do { \
    if (!(buf) || (buf)->size < (size_t)(bytes)) { \
        fprintf(stderr, "[fast_hip] %s: buffer %s too small (%zu < %zu bytes); launch skipped\n", \
                fn, #buf, (buf) ? (buf)->size : (size_t)0, (size_t)(bytes)); \
        return; } } while (0)
