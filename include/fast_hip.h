/*
 * fast_hip.h — C ABI of the MI355X (gfx950) backend for llm.metal's fast
 * training pipelines.
 *
 * This is the drop-in boundary: it exports the symbols the reference's
 * src/nn/fast_metal.h declares (same names, argument order and meaning as the
 * reference CALL SITES use them), implemented by hand-written HIP kernels on
 * one in-order stream.  Reference callers (src/nn/wmat.c, fast_sft.c,
 * fast_grpo.c) link against this library instead of fast_metal.m.
 *
 * Conventions kept from the reference (src/nn/fast_metal.m):
 *   - fast_metal_init returns 0 / -1 and is reference counted (:69-76,171);
 *     every other function is void and silent;
 *   - enqueues execute in program order, each seeing the previous one's
 *     writes (:231-233); metal_flush blocks until everything has run (:235-249);
 *   - in == out aliasing is allowed where the reference relies on it
 *     (rms_norm, rms_norm_backward, silu/gelu_mul_backward with dgate == dout).
 * Differences forced by a discrete GPU are listed at metal_buf_ptr.
 *
 * All 49 symbols of src/nn/fast_metal.h are exported: init / shutdown, the
 * buffer functions, flush, the 26 training enqueues and the 16 inference
 * enqueues (:20-80, declared further down).
 */
#ifndef FAST_HIP_H
#define FAST_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* src/nn/fast_metal.h:8-9.  Fails (-1, message on stderr) when no gfx950
 * device is present; there is no CPU fallback. */
int  fast_metal_init(void);
void fast_metal_shutdown(void);

/* src/nn/fast_metal.h:12-17 */
typedef struct MetalBuf MetalBuf;
MetalBuf *metal_buf_create(size_t size);                    /* uninitialised device memory */
MetalBuf *metal_buf_from_data(const void *data, size_t sz); /* copies; caller keeps `data` */
void      metal_buf_free(MetalBuf *b);                      /* NULL is a no-op */
/* Returns a CPU pointer valid for the buffer's lifetime and coherent at
 * metal_flush boundaries, as the reference's shared-storage buffers are.
 * On first use the buffer MIGRATES to pinned, device-mapped host memory and
 * stays there: kernels then reach it over the host link.  Meant for the small
 * CPU-touched buffers (inputs, targets, losses, GRPO actions); for bulk data
 * use metal_buf_read / metal_buf_write, which leave the buffer in HBM. */
void     *metal_buf_ptr(MetalBuf *b);

/* Extensions (no counterpart in the reference): explicit staging that keeps
 * the buffer in HBM.  Both order themselves after all enqueued work. */
void   metal_buf_read(MetalBuf *b, size_t offset, void *dst, size_t n);
void   metal_buf_write(MetalBuf *b, size_t offset, const void *src, size_t n);
size_t metal_buf_size(MetalBuf *b);
/* Extension: the address kernels use for the buffer (device memory, or the device view of pinned host memory once
 * metal_buf_ptr was called).  For callers that pass plain device pointers to hip_attention_noalloc. */
void *hip_buf_device_ptr(MetalBuf *b);
/* free and total bytes of the current device's memory (hipMemGetInfo): lets a caller see that a call allocated nothing */
void hip_mem_info(size_t *free_bytes, size_t *total_bytes);
/* Non-owning window [offset, offset+size) of another buffer. */
MetalBuf *metal_buf_view(MetalBuf *parent, size_t offset, size_t size);

/* src/nn/fast_metal.h:83 */
void metal_flush(void);

/* ---- enqueues shared with inference (src/nn/fast_metal.h:36-61) ---- */
void metal_enqueue_rms_norm_batched(MetalBuf *x, MetalBuf *gamma, MetalBuf *out,
                                    int dim, float eps, int B);
void metal_enqueue_silu_mul(MetalBuf *gate, MetalBuf *up, int n);
void metal_enqueue_gelu_mul(MetalBuf *gate, MetalBuf *up, int n);
void metal_enqueue_residual_add(MetalBuf *x, MetalBuf *y, int n);

/* ---- inference enqueues (src/nn/fast_metal.h:19-80): one decode step, all activations fp32 ---- */
/* y[rows] = W x, W = rows x nb Q8_0 blocks of 34 bytes (src/nn/fast_metal.h:20-21).  The first call on a weight
 * builds an aligned image of it (all codes, then all scales: its size again in HBM), kept until the buffer is written. */
void metal_enqueue_q8_matvec(MetalBuf *W, MetalBuf *x, MetalBuf *y, int rows, int nb);
/* y[rows] = W x, W F16 [rows, cols] (src/nn/fast_metal.h:24-25) */
void metal_enqueue_f16_matvec(MetalBuf *W, MetalBuf *x, MetalBuf *y, int rows, int cols);
/* Y[B, rows] = X[B, cols] W^T (src/nn/fast_metal.h:28-29); any B (the reference's kernel holds at most 32) */
void metal_enqueue_f16_batch_matvec(MetalBuf *W, MetalBuf *X, MetalBuf *Y, int rows, int cols, int B);
/* out = gamma * x / sqrt(mean(x^2) + eps) for one vector (src/nn/fast_metal.h:33-34); out may alias x */
void metal_enqueue_rms_norm(MetalBuf *x, MetalBuf *gamma, MetalBuf *out, int dim, float eps);
/* in-place RMSNorm of each of n_heads vectors of head_dim with a shared gamma (src/nn/fast_metal.h:39-40) */
void metal_enqueue_per_head_rms_norm(MetalBuf *vec, MetalBuf *gamma, int n_heads, int head_dim, float eps);
/* half-split rotary embedding of q [Hq*hd] and k [Hkv*hd] at position pos (src/nn/fast_metal.h:43-44) */
void metal_enqueue_rope(MetalBuf *q, MetalBuf *k, int Hq, int Hkv, int hd, int pos, float theta);
/* caches [Hkv, max_seq, hd]: row pos of every head := k, v (src/nn/fast_metal.h:47-49) */
void metal_enqueue_kv_cache_store(MetalBuf *k, MetalBuf *v, MetalBuf *k_cache, MetalBuf *v_cache,
                                  int Hkv, int max_seq, int hd, int pos);
/* out[h] = softmax(q[h] K[h / group_ratio, 0..n_attend)^T / sqrt(hd)) V (src/nn/fast_metal.h:52-54); hd <= 256,
 * group_ratio <= 16; the reference holds the scores of at most 4096 keys, this one any n_attend <= max_seq */
void metal_enqueue_attention(MetalBuf *Q, MetalBuf *Kc, MetalBuf *Vc, MetalBuf *attn_out, int n_attend, int hd,
                             int max_seq, int Hq, int group_ratio);
/* the same four with byte offsets into the per-item buffers (src/nn/fast_metal.h:66-80); offsets are multiples of 4 */
void metal_enqueue_per_head_rms_norm_off(MetalBuf *vec, size_t vec_off, MetalBuf *gamma, int n_heads, int head_dim, float eps);
void metal_enqueue_rope_off(MetalBuf *q, size_t q_off, MetalBuf *k, size_t k_off, int Hq, int Hkv, int hd, int pos, float theta);
void metal_enqueue_kv_cache_store_off(MetalBuf *k, size_t k_off, MetalBuf *v, size_t v_off, MetalBuf *k_cache,
                                      MetalBuf *v_cache, int Hkv, int max_seq, int hd, int pos);
void metal_enqueue_attention_off(MetalBuf *Q, size_t q_off, MetalBuf *Kc, MetalBuf *Vc, MetalBuf *attn_out, size_t out_off,
                                 int n_attend, int hd, int max_seq, int Hq, int group_ratio);

/* ---- training enqueues (src/nn/fast_metal.h:88-188) ----
 * Argument ORDER follows the reference's implementation and call sites
 * (src/nn/fast_metal.m:562-594, src/nn/fast_sft.c:638): the first buffer is the
 * fp32 activation, the second the F16 weight, whatever the header names say. */

/* C[M,N] fp32 = A[M,K] fp32 * W[N,K]^T, W F16 row-major. */
void metal_enqueue_f16_matmul(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K);
/* C[M,K] fp32 = A[M,N] fp32 * W[N,K], W F16 row-major. */
void metal_enqueue_f16_matmul_nt(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K);
void metal_enqueue_transpose_heads_fwd(MetalBuf *src, MetalBuf *dst, int seq_len, int n_heads, int head_dim);
void metal_enqueue_transpose_heads_rev(MetalBuf *src, MetalBuf *dst, int seq_len, int n_heads, int head_dim);
void metal_enqueue_repeat_kv(MetalBuf *src, MetalBuf *dst, int n_kv, int seq_len, int head_dim, int group_ratio);
void metal_enqueue_rope_train(MetalBuf *q, MetalBuf *k, int Hq, int Hkv, int hd, int seq_len, float theta);
void metal_enqueue_silu_mul_backward(MetalBuf *dout, MetalBuf *gate, MetalBuf *up,
                                     MetalBuf *dgate, MetalBuf *dup, int n);
void metal_enqueue_gelu_mul_backward(MetalBuf *dout, MetalBuf *gate, MetalBuf *up,
                                     MetalBuf *dgate, MetalBuf *dup, int n);
void metal_enqueue_rms_norm_backward(MetalBuf *x, MetalBuf *dy, MetalBuf *gamma, MetalBuf *dx,
                                     int batch, int dim, float eps);
void metal_enqueue_scale(MetalBuf *x, float alpha, int n);
void metal_enqueue_add_scaled(MetalBuf *y, MetalBuf *x, float alpha, int n);
void metal_enqueue_softmax_ce(MetalBuf *logits, MetalBuf *targets, MetalBuf *losses,
                              MetalBuf *dlogits, int batch, int vocab_size);
void metal_enqueue_attn_train_fwd(MetalBuf *Q, MetalBuf *K, MetalBuf *V, MetalBuf *out, MetalBuf *probs,
                                  int H, int N, int D, float scale);
void metal_enqueue_attn_bwd_dq(MetalBuf *d_out, MetalBuf *probs, MetalBuf *V, MetalBuf *K,
                               MetalBuf *d_score, MetalBuf *dQ, int H, int N, int D, float scale);
void metal_enqueue_attn_bwd_dkv(MetalBuf *d_score, MetalBuf *Q, MetalBuf *probs, MetalBuf *d_out,
                                MetalBuf *dK, MetalBuf *dV, int H, int N, int D);
void metal_enqueue_repeat_kv_bwd(MetalBuf *d_expanded, MetalBuf *d_kv,
                                 int n_kv, int seq_len, int head_dim, int group_ratio);
void metal_enqueue_rope_train_bwd(MetalBuf *q, MetalBuf *k, int Hq, int Hkv, int hd, int seq_len, float theta);
/* fp32 LoRA products: C[M,N] = A[M,K] W[N,K]^T;  C[M,N] = A[K,M]^T B[K,N];  C[M,K] = A[M,N] W[N,K]. */
void metal_enqueue_float_matmul(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K);
void metal_enqueue_float_matmul_tn(MetalBuf *A, MetalBuf *B, MetalBuf *C, int M, int N, int K);
void metal_enqueue_float_matmul_nt(MetalBuf *A, MetalBuf *W, MetalBuf *C, int M, int N, int K);
void metal_enqueue_copy(MetalBuf *src, MetalBuf *dst, int n);
void metal_enqueue_clamp(MetalBuf *x, float max_val, int n);
/* W[M,N] F16 -= lr * dY[K,M]^T X[K,N] */
void metal_enqueue_f16_sgd_fused(MetalBuf *W, MetalBuf *dY, MetalBuf *X, int M, int K, int N, float lr);
void metal_enqueue_grpo_policy_grad(MetalBuf *logits, MetalBuf *actions, MetalBuf *old_lp, MetalBuf *advs,
                                    MetalBuf *new_lp, MetalBuf *dlogits, int N, int V, float clip_eps);
/* G[M,N] F16 += dY[K,M]^T X[K,N], one rounding per call */
void metal_enqueue_f16_grad_accum(MetalBuf *G, MetalBuf *dY, MetalBuf *X, int M, int K, int N);
void metal_enqueue_f16_sgd_apply(MetalBuf *W, MetalBuf *G, int n, float lr);

/* ---- extensions used by the weight container ---- */
/* dst F16 [n] = round-to-nearest-even(src fp32 [n]); wmat_create_f16, src/nn/wmat.c:63-75 */
void hip_enqueue_f32_to_f16(MetalBuf *src, MetalBuf *dst, size_t n);
/* dst Q8_0 blocks (34 B each) from src fp32 [rows, cols]; quantize_row_q8, src/nn/wmat.c:19-44 */
void hip_enqueue_q8_quantize(MetalBuf *src, MetalBuf *dst, int rows, int cols);
/* dst fp32 [rows, cols] = float(scale) * code; src/data/gguf.c:225-253 */
void hip_enqueue_q8_dequant(MetalBuf *src, MetalBuf *dst, int rows, int cols);
/* dst F16 [rows, cols] = half(float(scale) * code): the values the dequant-fused GEMM multiplies with */
void hip_enqueue_q8_to_f16(MetalBuf *src, MetalBuf *dst, int rows, int cols);

/* 0: choose the GEMM kernel by the measured rule; 1: always the LDS-tiled large-M kernel (Q8_0 operands through an
 * F16 image made once per product); 2: always the large-M kernel with Q8_0 tiles kept quantised and unpacked into LDS
 * by the kernel itself; -1: never (always the weight-streaming kernel). */
void hip_gemm_force_large_m(int policy);
/* Products of up to 64 activation rows: 1 (default) = the kernel whose workgroups stream their operands into an LDS ring
 * (gemm_ring: one or two workgroups per CU, 4 to 6 K chunks; Q8_0 tiles travel quantised, 1.06 bytes per weight, and are
 * unpacked to fp16 from LDS), 0 = the kernel with one K step per wave in registers (gemm_tiled: 13 to 19 K chunks, Q8_0
 * unpacked in registers), which every product of more rows takes.  Same results up to the order of the sums. */
void hip_gemm_ring(int on);
/* gemm_ring with four weight row blocks per workgroup (1.5 instead of 2 bytes into LDS per F16 weight byte; Q8_0 tiles
 * likewise quantised up to LDS) for the products of 33 to 64 rows that have enough row tiles to give every CU such a
 * workgroup: 1 = on, 0 = off, 2 = for every product of 33 to 64 rows whatever its size (tests). */
void hip_gemm_ring_wide(int on);
/* 1 (default): a LoRA training state of at most 64 rows (frozen F16 or Q8_0 weights) stores the K-split planes of five of its eight
 * products per layer (gate|up and down forward; down, gate|up and O backward) as halves: every chunk sum, formed in fp32,
 * leaves times a power of two derived from the weight matrix (8192 times its largest row sum of |w| stays below the fp16
 * maximum) and is summed in fp32 again by the kernel that consumes the planes.  Half the plane bytes, 11 significant
 * bits per chunk sum.  0: fp32 planes everywhere.  Read when a product is launched. */
void hip_gemm_half_planes(int on);
/* K chunks of the large-M kernel on F16 tiles (each chunk writes a plane, the consumer adds them): 1 = by the measured
 * rule (three chunks when the 128 x 256 output blocks leave a third of the CUs idle and K >= 4096), 0 = never, n > 1 =
 * always n. */
void hip_gemm_large_m_split(int mode);
/* Output block of the large-M kernel on F16 tiles: 0 = by the measured rule (256 x 256 where that leaves at least 0.8
 * as much of the GPU on useful work as 128 x 256 does, counting partial rounds of blocks and partial tiles), 1 = always
 * 128 x 256, 2 = always 256 x 256. */
void hip_gemm_large_m_block(int mode);
/* A training state with frozen Q8_0 weights whose products run on the large-M kernel keeps the F16 image of every
 * weight it has used (made once instead of once per product) while they fit this many MB per state (default 65536;
 * the 4B model needs 16 GB); weights beyond that, or all with 0, get an image per product. */
void hip_gemm_image_budget_mb(int mb);
/* Training attention without the [seq, seq] probability matrices in memory (running softmax in the forward, the
 * probabilities formed again in the backward): -1 = for head_dim 64 / 128 when ceil(seq / 128) * query heads * batch
 * is at least 128 or the sequence is longer than 1024 (default, the measured rule), 0 = never, 1 = whenever the head
 * size allows.  Read when a training state is created. */
void hip_attention_flash(int mode);
/* 1 (default): for sequences of at most 64 positions the attention backward is one launch (dQ, and dK / dV as shares per
 * query block and query head that the next kernel sums); 0: dQ, then dK / dV, as for longer sequences */
void hip_attention_backward_one_launch(int on);
/* Timing aid for benchmarks: when enabled, every GEMM launch is bracketed by HIP events on the
 * library's stream.  hip_gemm_profile_read (after metal_flush) returns the number of launches recorded
 * since the last enable and adds up their durations (ms) and weight bytes; _read2 also their flops. */
void hip_gemm_profile_enable(int on);
int  hip_gemm_profile_read(double *total_ms, double *total_weight_bytes);
int  hip_gemm_profile_read2(double *total_ms, double *total_weight_bytes, double *total_flops);
/* Microbenchmark of the GEMM alone at one shape (M rows, N x K weight) on synthetic operands,
 * rotating through > 1 GB of distinct weight images.  nb / S = 0: planner's choice, else forced
 * tile height (1, 2; 128 = the large-M kernel; -1 = no product at all, only the weight loads of gemm_ring on its grid) and K split (for the large-M kernel: K chunks, F16 tiles only).  wf: weight format, 0 F16, 1 Q8_0 with row scales (forward image),
 * 2 Q8_0 with column scales (transposed image).  Returns average ms per launch. */
double hip_gemm_time_shape(int M, int N, int K, int nb, int wf, int S, int iters, int *used_nb, int *used_S);

/* metal_enqueue_attention once more, ALLOCATING NOTHING.  No counterpart in the reference: it is for callers that cannot
 * call hipMalloc -- code under HIP graph capture, tight serving loops, harnesses that forbid allocation.  Plain device
 * pointers: Q, out [Hq * hd] fp32; caches [Hq / group_ratio, max_seq, hd] fp32; keys 0 .. n_attend - 1 are attended.
 * Same kernels on the library's stream, results identical to metal_enqueue_attention.  The slice results that contexts
 * beyond 256 keys need go to a fixed 2 MiB array that each device holds until the process ends, which bounds the call:
 * Hq <= 64, hd <= 256, group_ratio <= 16, n_attend <= 8192; anything larger returns -1 with a message and launches
 * nothing (0 otherwise).  Every call on a GPU shares that GPU's array: calls that overlap on one GPU race. */
int hip_attention_noalloc(const float *Q, const float *Kc, const float *Vc, float *out, int n_attend, int hd, int max_seq,
                          int Hq, int group_ratio);

/* The same for the matrix-vector kernels of the decode step: rows x cols weight, fmt 0 F16 or 1 Q8_0 (split image),
 * B = 1; cols a multiple of 32.  Returns average ms per launch, -1 for bad arguments. */
double hip_matvec_time_shape(int rows, int cols, int fmt, int B, int iters);

#ifdef __cplusplus
}
#endif
#endif /* FAST_HIP_H */
