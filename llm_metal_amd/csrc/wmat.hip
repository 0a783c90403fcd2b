// Weight container: F16 and Q8_0 matrices in HBM, built on the device.
// Host API of the reference's src/nn/wmat.{h,c}; the conversions the reference
// runs on one CPU core (wmat_create_f16 :63-75, quantize_row_q8 :19-44) run as
// kernels over an uploaded fp32 staging copy, with bit-identical results.
#include "backend.h"
#include "devutil.h"
#include "../../include/sft_hip.h"
#include <string.h>

using namespace lmhip;

namespace {

__global__ void k_f32_to_f16(const float *__restrict__ src, half_t *__restrict__ dst, size_t n)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = f2h(src[i]);
}

// One thread per 32-value block.  Every fp32 operation below is a single
// correctly rounded IEEE operation, as in the C reference.
__global__ void k_q8_quantize(const float *__restrict__ src, uint8_t *__restrict__ dst, int rows, int cols, int nb)
{
    const size_t blk = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (blk >= (size_t)rows * nb) return;
    const size_t r = blk / nb, b = blk % nb;
    const float *sp = src + r * cols + b * 32;
    float v[32];
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 32; j++) { v[j] = sp[j]; amax = fmaxf(amax, fabsf(v[j])); }
    const float scale = __fdiv_rn(amax, 127.0f);
    const half_t d = f2h(scale);
    uint8_t *o = dst + blk * 34;
    const uint16_t bits = __builtin_bit_cast(uint16_t, d);
    o[0] = (uint8_t)(bits & 0xff);
    o[1] = (uint8_t)(bits >> 8);
    if (scale != 0.0f) {
        const float inv = __fdiv_rn(1.0f, scale);
#pragma unroll
        for (int j = 0; j < 32; j++) {
            int q = (int)roundf(__fmul_rn(v[j], inv));
            q = q < -128 ? -128 : (q > 127 ? 127 : q);
            o[2 + j] = (uint8_t)(int8_t)q;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 32; j++) o[2 + j] = 0;
    }
}

template <typename OutT>
__global__ void k_q8_dequant(const uint8_t *__restrict__ src, OutT *__restrict__ dst, int rows, int cols, int nb)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;      // one thread per element of the blocked part
    if (idx >= (size_t)rows * nb * 32) return;
    const size_t blk = idx / 32;
    const int j = idx % 32;
    const size_t r = blk / nb, b = blk % nb;
    const uint8_t *p = src + blk * 34;
    const uint16_t bits = (uint16_t)(p[0] | (p[1] << 8));
    const float d = h2f(__builtin_bit_cast(half_t, bits));
    const float val = __fmul_rn(d, (float)(int8_t)p[2 + j]);
    dst[r * cols + b * 32 + j] = (OutT)val;
}

}  // namespace

extern "C" {

void hip_enqueue_f32_to_f16(MetalBuf *src, MetalBuf *dst, size_t n)
{
    REQUIRE_BYTES(src, n * 4, "f32_to_f16");
    REQUIRE_BYTES(dst, n * 2, "f32_to_f16");
    if (!n) return;
    size_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(k_f32_to_f16, dim3((unsigned)blocks), dim3(256), 0, stream(), dptr_as<float>(src), dptr_as<half_t>(dst), n);
    HIP_CHECK(hipGetLastError());
    mark_written(dst);
}

void hip_enqueue_q8_quantize(MetalBuf *src, MetalBuf *dst, int rows, int cols)
{
    const int nb = cols / 32;
    REQUIRE_BYTES(src, (size_t)rows * cols * 4, "q8_quantize");
    REQUIRE_BYTES(dst, (size_t)rows * nb * 34, "q8_quantize");
    const size_t nblk = (size_t)rows * nb;
    if (!nblk) return;
    hipLaunchKernelGGL(k_q8_quantize, dim3((unsigned)((nblk + 127) / 128)), dim3(128), 0, stream(),
                       dptr_as<float>(src), dptr_as<uint8_t>(dst), rows, cols, nb);
    HIP_CHECK(hipGetLastError());
    mark_written(dst);
}

void hip_enqueue_q8_dequant(MetalBuf *src, MetalBuf *dst, int rows, int cols)
{
    const int nb = cols / 32;
    REQUIRE_BYTES(src, (size_t)rows * nb * 34, "q8_dequant");
    REQUIRE_BYTES(dst, (size_t)rows * cols * 4, "q8_dequant");
    const size_t n = (size_t)rows * nb * 32;
    if (!n) return;
    hipLaunchKernelGGL(k_q8_dequant<float>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream(),
                       dptr_as<uint8_t>(src), dptr_as<float>(dst), rows, cols, nb);
    HIP_CHECK(hipGetLastError());
    mark_written(dst);
}

void hip_enqueue_q8_to_f16(MetalBuf *src, MetalBuf *dst, int rows, int cols)
{
    const int nb = cols / 32;
    REQUIRE_BYTES(src, (size_t)rows * nb * 34, "q8_to_f16");
    REQUIRE_BYTES(dst, (size_t)rows * cols * 2, "q8_to_f16");
    const size_t n = (size_t)rows * nb * 32;
    if (!n) return;
    hipLaunchKernelGGL(k_q8_dequant<half_t>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream(),
                       dptr_as<uint8_t>(src), dptr_as<half_t>(dst), rows, cols, nb);
    HIP_CHECK(hipGetLastError());
    mark_written(dst);
}

// ---- src/nn/wmat.h:58-78 ----

static WMat *wmat_from_f32(const float *src, int rows, int cols, int use_fp16)
{
    WMat *w = (WMat *)calloc(1, sizeof(WMat));
    w->rows = rows;
    w->cols = cols;
    const size_t n = (size_t)rows * cols;
    MetalBuf *stage = metal_buf_from_data(src, n * sizeof(float));
    if (use_fp16) {
        w->nb = 0;
        w->mbuf = metal_buf_create(n * 2);
        hip_enqueue_f32_to_f16(stage, w->mbuf, n);
    } else {
        w->nb = cols / 32;                                  // truncating, src/nn/wmat.c:53
        w->mbuf = metal_buf_create((size_t)rows * w->nb * 34);
        hip_enqueue_q8_quantize(stage, w->mbuf, rows, cols);
    }
    metal_buf_free(stage);                                  // synchronises the stream first
    return w;
}

WMat *wmat_create_f16(const float *src, int rows, int cols) { return wmat_from_f32(src, rows, cols, 1); }
WMat *wmat_create_q8(const float *src, int rows, int cols) { return wmat_from_f32(src, rows, cols, 0); }
WMat *wmat_convert(const float *data, int rows, int cols, int use_fp16) { return wmat_from_f32(data, rows, cols, use_fp16); }

void wmat_free(WMat *w)
{
    if (!w) return;
    metal_buf_free(w->mbuf);
    free(w);
}

MetalBuf *norm_upload(const float *gamma, int dim) { return metal_buf_from_data(gamma, (size_t)dim * sizeof(float)); }

LayerW *layers_convert_upload(const LayerWeightRef *refs, int n_layers, int use_fp16)
{
    LayerW *layers = (LayerW *)calloc(n_layers, sizeof(LayerW));
    for (int i = 0; i < n_layers; i++) {
        const LayerWeightRef *r = &refs[i];
        LayerW *lw = &layers[i];
        lw->q_proj = wmat_from_f32(r->q_proj.data, r->q_proj.rows, r->q_proj.cols, use_fp16);
        lw->k_proj = wmat_from_f32(r->k_proj.data, r->k_proj.rows, r->k_proj.cols, use_fp16);
        lw->v_proj = wmat_from_f32(r->v_proj.data, r->v_proj.rows, r->v_proj.cols, use_fp16);
        lw->o_proj = wmat_from_f32(r->o_proj.data, r->o_proj.rows, r->o_proj.cols, use_fp16);
        lw->gate_proj = wmat_from_f32(r->gate_proj.data, r->gate_proj.rows, r->gate_proj.cols, use_fp16);
        lw->up_proj = wmat_from_f32(r->up_proj.data, r->up_proj.rows, r->up_proj.cols, use_fp16);
        lw->down_proj = wmat_from_f32(r->down_proj.data, r->down_proj.rows, r->down_proj.cols, use_fp16);
        lw->input_norm_g = norm_upload(r->input_norm_g, r->d_model);
        lw->post_attn_norm_g = norm_upload(r->post_attn_norm_g, r->d_model);
        if (r->pre_ff_norm_g) lw->pre_ff_norm_g = norm_upload(r->pre_ff_norm_g, r->d_model);
        if (r->post_ff_norm_g) lw->post_ff_norm_g = norm_upload(r->post_ff_norm_g, r->d_model);
        if (r->q_norm_g) lw->q_norm_g = norm_upload(r->q_norm_g, r->head_dim);
        if (r->k_norm_g) lw->k_norm_g = norm_upload(r->k_norm_g, r->head_dim);
    }
    return layers;
}

void layers_free(LayerW *layers, int n_layers)
{
    if (!layers) return;
    for (int i = 0; i < n_layers; i++) {
        LayerW *lw = &layers[i];
        wmat_free(lw->q_proj); wmat_free(lw->k_proj); wmat_free(lw->v_proj); wmat_free(lw->o_proj);
        wmat_free(lw->gate_proj); wmat_free(lw->up_proj); wmat_free(lw->down_proj);
        metal_buf_free(lw->input_norm_g); metal_buf_free(lw->post_attn_norm_g);
        metal_buf_free(lw->pre_ff_norm_g); metal_buf_free(lw->post_ff_norm_g);
        metal_buf_free(lw->q_norm_g); metal_buf_free(lw->k_norm_g);
    }
    free(layers);
}

}  // extern "C"
