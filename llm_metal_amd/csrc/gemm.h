// Internal interface of the weight-streaming GEMM (gemm.hip) and of the tiled
// fp16 operand layout it reads.
#pragma once
#include "backend.h"
#include "devutil.h"

struct SFTState;

namespace lmhip {

// ---- tiled fp16 operand layout ------------------------------------------------
// A matrix [R, K] is cut into tiles of 32 rows x 64 columns (4 KB).  Inside a
// tile the order is [j = 0..3][lane = 0..63][e = 0..7] with
//     row = lane & 31,   col = (lane >> 5) * 32 + 8 * j + e,
// i.e. exactly the registers lane `lane` feeds to the j-th v_mfma_f32_32x32x16_f16
// of a 64-wide K step (the K order inside a step is permuted the same way for
// both operands, which a dot product does not see).  Tiles are stored
// [row block][K block].  One wave-wide 16-byte load therefore reads 1 KB of
// contiguous memory.  R is padded to 32 and K to 64; padding must hold zeros
// in K (rows beyond R may hold anything: their outputs are never stored).
__host__ __device__ inline int tiled_kb(int K) { return (K + 63) >> 6; }
__host__ __device__ inline int tiled_rb(int R) { return (R + 31) >> 5; }
__host__ __device__ inline size_t tiled_elems(int R, int K) { return (size_t)tiled_rb(R) * tiled_kb(K) * 2048; }
__host__ __device__ inline size_t tiled_index(int r, int k, int Kb)
{
    const int c = k & 63;
    const size_t tile = (size_t)(r >> 5) * Kb + (k >> 6);
    return ((tile * 4 + ((c & 31) >> 3)) * 64 + ((c >> 5) << 5) + (r & 31)) * 8 + (c & 7);
}

// Activation operands (the GEMM's first operand, written a row at a time by the row kernels) use the same tiles with the
// two 16-byte vectors of a row inside a 1 KB slice side by side: [j][row][column half][e], so lane `lane` of the MFMA
// finds its vector at slot a_lane(lane) of the slice.  A wave-wide load still reads the slice's 1 KB whole; a row
// kernel's stores come in runs of 32 bytes instead of 16, half as many write requests for the lines that eight rows
// share (the 2048-row step: 53.83 -> 53.57 ms).  Weight operands keep tiled_index.
__host__ __device__ inline int a_lane(int lane) { return ((lane & 31) << 1) | (lane >> 5); }
__host__ __device__ inline size_t tiled_a_index(int r, int k, int Kb)
{
    const int c = k & 63;
    const size_t tile = (size_t)(r >> 5) * Kb + (k >> 6);
    return ((tile * 4 + ((c & 31) >> 3)) * 64 + ((r & 31) << 1) + (c >> 5)) * 8 + (c & 7);
}

// Weight operand of the GEMM.  fmt 0: F16 tiles in w16.  fmt 1 / 2: Q8_0 (GGML blocks of 32 int8 with
// one fp16 scale, src/nn/wmat.c:9-44) re-laid for the kernel: `q` holds the int8 of a 32 x 64 tile as
// [2][64 lanes][16 bytes] (lane, j, e as in the F16 tile, j = 2 * half + byte / 8), `d` 64 scales per tile.
//   fmt 1: scales belong to (row, 32-column block): d[tile][lane] is the one scale of that lane's 32 weights;
//          row blocks from nbq on are F16 tiles in w16 (row block index - nbq).
//   fmt 2: the transposed image of a Q8_0 matrix: scales belong to (column, 32-row block), d[tile][column];
//          K steps from kbq on are F16 tiles in w16 ([row block][Kb - kbq]).
struct WeightOp {
    const half_t *w16;
    const uint8_t *q;
    const half_t *d;
    int fmt, nbq, kbq;
};
inline WeightOp weight_f16(const half_t *w) { return WeightOp{w, nullptr, nullptr, 0, 0, 0}; }

// A training state's own forward images and norm gammas of one layer, nothing copied (sft.hip): what a generation
// state made from the training state reads.  qkv holds the rows Q | K | V (any adapter rows behind them are not part
// of the product), gu the rows gate | up.  The gammas are windows on the training state's arenas and belong to it.
struct BorrowedLayer {
    WeightOp qkv, o, gu, down;
    struct ::MetalBuf *g_in, *g_post_attn, *g_pre_ff, *g_post_ff, *g_q, *g_k;
};
void sft_borrow_layer(::SFTState *s, int L, BorrowedLayer *out);
WeightOp sft_borrow_lm_head(::SFTState *s);

struct GemmPlan {
    int nb;        // 32-row weight blocks per wave (1 or 2)
    int nw;        // waves per workgroup (4): they split the workgroup's K chunk
    int S;         // K chunks = partial planes written
    int steps;     // 64-wide K steps per chunk
    int n_tiles, m_tiles;
    int rotate;    // start each workgroup at a different K step of its chunk
    int ring;      // gemm_ring (one 64-row tile of activations; F16 or Q8_0 weights): kg K groups of four waves per workgroup
    int kg;
    int wide;      // ring plans: gemm_ring_wide, four weight row blocks per workgroup (nb = 4), one K group
};

// nbq: Q8_0 row blocks of a fmt-1 operand (an odd count forces one row block per wave); fmt: WeightOp::fmt of the operand
GemmPlan plan_gemm(int M, int N, int K, int nbq = 0, int fmt = 0);
void set_gemm_ring(int on);
int gemm_ring_wide_mode();
void set_gemm_ring_wide(int on);     // 1: products with enough row tiles take gemm_ring_wide; 2: every F16 product of 33 to 64 rows (tests)
int gemm_ring_enabled();            // 1 (default): products of up to 64 rows take gemm_ring (Q8_0 tiles stay quantised up to LDS); 0: gemm_tiled

// P[s][m][n] (s < plan.S, plane s at P + s*plane_stride, row stride ldp) =
//   inv_scale[m] * sum_{k in chunk s} A[m][k] * W[n][k],  A and W in the tiled layout.
// Pass a_inv_scale = null to leave the row factors to the consumer of the planes.
// half_scale != 0 (ring plans only, a_inv_scale null): the planes are written as halves, each chunk sum times half_scale
// (see gemm_ring); plane_stride and ldp then count halves, and only planes_at4_multi reads such planes.
void launch_gemm(const half_t *A_tiled, const float *a_inv_scale, const WeightOp &W,
                 float *P, int ldp, size_t plane_stride, int M, int N, int K, const GemmPlan &p, float half_scale = 0.f);
// Largest sum of |w| over a row of a tiled F16 matrix [N, K]: with operand rows scaled below 8192 (row_scale_for), no
// chunk sum of a product with this matrix exceeds 8192 times it.  Synchronises the stream.
// the same over the values a weight operand of any format multiplies with (0 when the operand mixes Q8_0 and F16 tiles)
float weight_max_row_l1(const WeightOp &W, int N, int K);
float tiled_max_row_l1(const half_t *W_tiled, int N, int K);
// the power of two by which chunk sums of products with a matrix of that row bound are multiplied to leave as halves
float half_plane_scale(float max_row_l1);
void set_gemm_half_planes(int on);
int gemm_half_planes_enabled();     // 1 (default): LoRA training states store the K-split planes of their frozen-weight ring products as halves
inline void launch_gemm(const half_t *A_tiled, const float *a_inv_scale, const half_t *W_tiled,
                        float *P, int ldp, size_t plane_stride, int M, int N, int K, const GemmPlan &p)
{
    launch_gemm(A_tiled, a_inv_scale, weight_f16(W_tiled), P, ldp, plane_stride, M, N, K, p);
}
// non-zero while per-launch GEMM events are being recorded (hip_gemm_profile_enable)
int gemm_profiling();
// when profiling: registers one launch (weight bytes, flops) and hands out the two events to attach to its dispatch
bool gemm_prof_begin(double wbytes, double flops, hipEvent_t *a, hipEvent_t *b);
// bytes of weight data one launch streams for an [N, K] operand (2 per F16 weight, 34 per 32 Q8_0 weights)
double weight_stream_bytes(const WeightOp &W, int N, int K);
// C[m][n] (row stride ldc) = a_inv_scale[m] * sum_k A[m][k] W[n][k] in one launch of 128 x 128 output blocks staged
// through LDS (gemm_big.hip): the path for M of several hundred rows and more, where the product is MFMA bound.
// W as plain F16 tiles: itself when F16, else dequantised once into a scratch image that the next call overwrites
// `keep`: the image goes there (tiled_elems(N, K) halves, the caller's) instead of the scratch arena; with
// f16_part_only only the tiles that are F16 in W are written (the Q8_0 part of `keep` holds its image from before).
WeightOp f16_image_of(const WeightOp &W, int N, int K, void *keep = nullptr, bool f16_part_only = false);
bool large_m_unpacks_q8();                                // the large-M policy that reads Q8_0 tiles itself is in force
// chunks > 1 (F16 tiles only): the K steps are cut into that many chunks, chunk c writing the plane at C + c * plane_stride;
// big_gemm_chunks: what the measured rule picks for a product
int big_gemm_chunks(int M, int N, int K, int fmt);
// the same for any operand: Q8_0 tiles that the 256 x 256 dequant-fused kernel can take are cut into chunks as well
int big_gemm_chunks_for(int M, int N, int K, const WeightOp &W);
void set_big_gemm_split(int mode);     // 1 measured rule, 0 never, n > 1 always n chunks
void set_big_gemm_block(int mode);     // F16 tiles: 0 block shape by the measured rule, 1 always 128 x 256, 2 always 256 x 256
// Returns the number of planes written (fewer than `chunks` when K has too few steps for that many).
int launch_gemm_big(const half_t *A_tiled, const float *a_inv_scale, const WeightOp &W, float *C, int ldc, int M, int N, int K,
                    int chunks = 1, size_t plane_stride = 0);
// true when the large-M kernel is the faster one for this product
bool use_big_gemm(int M, int N, int K, int fmt);
// Q8_0 blocks in the reference's row-major layout ([rows][cols/32] blocks of 34 bytes) -> kernel tiles.
// Element (r, c) goes to tiled (row_off + r, k_off + c) with row scales (fmt 1), or, transposed, to
// (row_off + c, k_off + r) with column scales (fmt 2).  Kb_dst = K blocks per row block of the destination.
// row_off must be a multiple of 32 and k_off of 32 (fmt 1); cols a multiple of 32.
void launch_tile_q8(const uint8_t *blocks, int rows, int cols, uint8_t *q_tiles, half_t *d_tiles, int Kb_dst,
                    int row_off, int k_off, int transpose);

// out (tiled [M, K]) = fp16(X[m][k] * s_m), zero in the K padding; inv_scale[m] = 1/s_m
void launch_rows_to_f16(const float *X, int ldx, half_t *out_tiled, float *inv_scale, int M, int K);
// C[m][n] = row_scale[m] * sum_s P[s][m][n] (row_scale may be null)
// C[M, N] fp32 = A[M, K] fp32 * W^T on the matrix cores with A kept to 22 bits: every row goes in twice, as its fp16
// image and as the fp16 image of the rounding residual.  W: row-major F16 [N, K] buffer (its tiled image is cached).
void gemm_f32a_exact(const float *A, struct ::MetalBuf *W, float *C, int M, int N, int K);
// Its three parts, for callers that fold the first or the last into kernels of their own: the cached tiled image of W;
// rows m and M + m of the tiled operand a16 [2M, K] and their factors inv [2M] from A [M, K]; launch_gemm over
// plan_gemm(2M, N, K) into planes of [2M, N]; C [M, N] from the planes.
const half_t *tiled_weight_of(struct ::MetalBuf *W, int N, int K);
void launch_rows_to_f16_split(const float *A, half_t *a16, float *inv, int M, int K);
void launch_reduce_planes_split(const float *P, int S, size_t plane_stride, int ldp, const float *inv, float *C, int M, int N);
// element (m, n) of such a product: the planes of row m and of row M + m summed, each sum times its row's factor
__device__ __forceinline__ float split_planes_value(const float *__restrict__ P, int S, size_t plane_stride, int ldp,
                                                    const float *__restrict__ inv, int M, int m, int n)
{
    const float *ph = P + (size_t)m * ldp + n, *pl = P + (size_t)(M + m) * ldp + n;
    float hi = 0.f, lo = 0.f;
    int p = 0;
    for (; p + 8 <= S; p += 8) {                          // eight planes' loads in flight; summed in plane order
        float h[8], l[8];
#pragma unroll
        for (int q = 0; q < 8; q++) { h[q] = ph[(p + q) * plane_stride]; l[q] = pl[(p + q) * plane_stride]; }
#pragma unroll
        for (int q = 0; q < 8; q++) { hi += h[q]; lo += l[q]; }
    }
    for (; p < S; p++) { hi += ph[p * plane_stride]; lo += pl[p * plane_stride]; }
    return fmaf(lo, inv[M + m], hi * inv[m]);
}
void launch_reduce_planes(const float *P, int S, size_t plane_stride, int ldp, const float *row_scale, float *C, int M, int N);
// dst (tiled, Kb_dst K blocks) <- src row-major F16 [rows, cols]:
//   element (r, c) goes to tiled(row_off + r, k_off + c), or tiled(row_off + c, k_off + r) when transposed
void launch_tile_f16(const half_t *src, int rows, int cols, half_t *dst_tiled, int Kb_dst,
                     int row_off, int k_off, int transpose);

// dst (row-major F16 [rows, cols]) <- half(d * q) of a window of a Q8_0 tiled operand (fmt 1 or 2), optionally transposed
void launch_untile_q8(const uint8_t *q_tiles, const half_t *d_tiles, int fmt, int Kb, int row_off, int k_off, int transpose,
                      int rows, int cols, half_t *dst);

}  // namespace lmhip
