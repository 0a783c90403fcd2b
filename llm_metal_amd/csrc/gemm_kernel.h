// The weight-streaming GEMM kernel (device code only; included by gemm.hip).
#pragma once
#include "kargs.h"
#include "devutil.h"
#include "gemm.h"

namespace lmhip {

// (ordered for kargs.h: what gemm_ring needs to request its first stages lies in the first 56 bytes)
struct GemmKArgs {
    const half8 *A;
    const half_t *w16_ring;                              // W.w16 once more, for gemm_ring
    int Kb, Nb, Mb, n_tiles, steps_per_chunk, M;
    int N, S, m_tiles;                                   // (m_tiles > 1: the grid is the 1-D one described at gemm_tiled)
    int ldp;
    const float *a_inv_scale;
    WeightOp W;
    float *P; size_t plane_stride;
    float half_scale;                                    // gemm_ring<.., .., 1>: the planes are halves, each sum times this power of two
};

typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

// Eight int8 (two dwords, little endian) -> eight exact fp16 integers.  x ^ 0x80 is q + 128 as an
// unsigned byte; 0x6400 | byte is the fp16 number 1024 + byte; subtracting 1152 leaves q.
__device__ __forceinline__ half8 q8_unpack8(uint32_t lo, uint32_t hi)
{
    lo ^= 0x80808080u; hi ^= 0x80808080u;
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 bits;
    bits[0] = __builtin_amdgcn_perm(0x64646464u, lo, 0x04010400u);
    bits[1] = __builtin_amdgcn_perm(0x64646464u, lo, 0x04030402u);
    bits[2] = __builtin_amdgcn_perm(0x64646464u, hi, 0x04010400u);
    bits[3] = __builtin_amdgcn_perm(0x64646464u, hi, 0x04030402u);
    half8 v = __builtin_bit_cast(half8, bits);
    const half_t off = (half_t)1152.0f;
    return v - off;
}

__device__ __forceinline__ half8 bcast8(half_t d)
{
    half8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = d;
    return v;
}

// Weight registers of one 64-wide K step for row block `nb`: w[j] feeds the j-th MFMA of the step.
// FMT 0: F16 tiles, `kb_stride` K blocks per row block, K block `kt`.
// SHARED: the workgroups of several activation row tiles read the same weight tile through one L2 (gemm_tiled's MTILES),
// so the loads are ordinary ones; a tile that only one workgroup reads is streamed past the caches.
template <int SHARED = 0>
__device__ __forceinline__ void load_w_f16(half8 (&w)[4], const half_t *W16, int nb, int kb_stride, int kt, int lane)
{
    const half8 *p = reinterpret_cast<const half8 *>(W16) + ((size_t)nb * kb_stride + kt) * 256 + lane;
#pragma unroll
    for (int j = 0; j < 4; j++) w[j] = SHARED ? p[j * 64] : __builtin_nontemporal_load(&p[j * 64]);
}

// FMT 1: Q8_0, one scale per (row, 32 columns): the 32 weights of a lane share one scale.
// The products d * q are rounded to fp16 once, which is what a stored F16 image of the
// dequantised weight would hold.
template <int SHARED = 0>
__device__ __forceinline__ void load_w_q8_rows(half8 (&w)[4], const WeightOp &W, int nb, int kb_stride, int kt, int lane)
{
    const size_t tile = (size_t)nb * kb_stride + kt;
    const uint4v *q = reinterpret_cast<const uint4v *>(W.q) + tile * 128 + lane;
    const uint4v r0 = SHARED ? q[0] : __builtin_nontemporal_load(&q[0]), r1 = SHARED ? q[64] : __builtin_nontemporal_load(&q[64]);
    const half8 d = bcast8(SHARED ? W.d[tile * 64 + lane] : __builtin_nontemporal_load(&W.d[tile * 64 + lane]));
    w[0] = q8_unpack8(r0[0], r0[1]) * d;
    w[1] = q8_unpack8(r0[2], r0[3]) * d;
    w[2] = q8_unpack8(r1[0], r1[1]) * d;
    w[3] = q8_unpack8(r1[2], r1[3]) * d;
}

// FMT 2: Q8_0 of the transposed matrix: one scale per (column, 32 rows), so a tile (32 rows) has 64
// column scales and a lane multiplies its weight (j, e) by the scale of column (lane / 32) * 32 + 8 j + e.
template <int SHARED = 0>
__device__ __forceinline__ void load_w_q8_cols(half8 (&w)[4], const WeightOp &W, int nb, int kb_stride, int kt, int lane)
{
    const size_t tile = (size_t)nb * kb_stride + kt;
    const uint4v *q = reinterpret_cast<const uint4v *>(W.q) + tile * 128 + lane;
    const uint4v r0 = SHARED ? q[0] : __builtin_nontemporal_load(&q[0]), r1 = SHARED ? q[64] : __builtin_nontemporal_load(&q[64]);
    const half8 *sc = reinterpret_cast<const half8 *>(W.d + tile * 64 + (lane >> 5) * 32);
    const half8 s0 = sc[0], s1 = sc[1], s2 = sc[2], s3 = sc[3];
    w[0] = q8_unpack8(r0[0], r0[1]) * s0;
    w[1] = q8_unpack8(r0[2], r0[3]) * s1;
    w[2] = q8_unpack8(r1[0], r1[1]) * s2;
    w[3] = q8_unpack8(r1[2], r1[3]) * s3;
}

// First register of the segment that wave w of nw still holds after `rounds` rounds of the accumulator exchange (see the
// end of gemm_tiled): every round halves the segment, the wave whose bit nw >> (round + 1) is set keeps the upper half.
__host__ __device__ constexpr int exchange_seg_lo(int regs, int nw, int w, int rounds)
{
    int lo = 0, len = regs;
    for (int r = 0; r < rounds; r++) { len >>= 1; if (w & (nw >> (r + 1))) lo += len; }
    return lo;
}

// grid: x = ceil(Nb / NB) weight-row tiles, y = S (K chunks), z = ceil(M / 64); block = NW waves of 64.
// Kb = number of 64-wide K steps of the (padded) reduction; Nb, Mb = 32-row blocks of W and A.
//
// Each wave loads one K step (NB weight tiles + 2 activation tiles), waits, issues its MFMAs and
// moves on; there is no register double buffering.  Measured on MI355X, the lower register count
// (four resident workgroups per CU instead of two) hides the load latency better than a second
// register stage does.  ROTATE starts every workgroup at a different step of its chunk: without
// it all workgroups of a chunk ask L2 for the same activation lines at the same moment.
// SCALE: multiply row m of the result by a_inv_scale[m] here (used when the output is final, S == 1);
// otherwise the consumer of the partial planes applies the row factors.
// NW = 4 or 8: the waves of a workgroup split its K chunk and add their accumulators through LDS; each then stores its
// part of the tile.  Eight waves cut K into half as many chunks for the same number of waves in flight: half the planes
// to write and for the consumer to add.
// WF: weight format (WeightOp::fmt).  1: row blocks below W.nbq are Q8_0 tiles, the rest F16 tiles
// (the trainable LoRA rows of the fused QKV weight); the planner keeps W.nbq a multiple of NB, so a
// workgroup is of one kind.  2: K steps below W.kbq are Q8_0 tiles with column scales, the rest F16.
template <int NB, int NW, int ROTATE, int SCALE, int WF, int MTILES = 0>
__global__ __launch_bounds__(NW * 64, 2) void gemm_tiled(GemmKArgs g)
{
    extern __shared__ float red[];                       // [NW][NB*16 regs][64 lanes]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    // Block coordinates: (weight-row tile, K chunk, 64-row tile of the activations).  With one row tile they are the grid's.
    // With several, the workgroups that share a weight tile must meet in one L2 or the weights are streamed from memory
    // once per row tile: the grid is then 1-D, the hardware deals consecutive ids to the eight XCDs in turn, and the ids
    // (8 * (m_tiles * u + z) + xcd), z = 0 .. m_tiles - 1, take the row tiles of weight tile 8 * u + xcd (MTILES = 1).
    int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
    if (MTILES) {                                         // compile-time: the one-tile kernels do not carry this code
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        const int t = (slot / g.m_tiles) * 8 + xcd;
        if (t >= g.n_tiles * g.S) return;                 // padding of the last group of eight; the whole workgroup leaves
        bz = slot % g.m_tiles; bx = t % g.n_tiles; by = t / g.n_tiles;
    }
    const int nb0 = bx * NB, mb0 = bz * 2;
    const int Kb = g.Kb, Nb = g.Nb, M = g.M, N = g.N;
    const int kb_beg = by * g.steps_per_chunk;
    const int nsteps = min(Kb, kb_beg + g.steps_per_chunk) - kb_beg;

    int nbi[NB];                                          // row block of each weight tile (clamped: the extra rows are never stored)
    const half8 *ap[2];
#pragma unroll
    for (int b = 0; b < NB; b++) nbi[b] = min(nb0 + b, Nb - 1);
#pragma unroll
    for (int mb = 0; mb < 2; mb++) ap[mb] = g.A + (size_t)min(mb0 + mb, g.Mb - 1) * Kb * 256 + a_lane(lane);
    const bool q8_rows = WF == 1 && nb0 < g.W.nbq;

    float16v acc[2][NB];
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[mb][b][v] = 0.f;

    // wave w takes the K steps w, w+NW, w+2NW, ... of this workgroup's chunk (rotated)
    const int rot = ROTATE ? (int)(((unsigned)bx * 7u + (unsigned)by * 3u) % (unsigned)nsteps) : 0;
    for (int i = wave; i < nsteps; i += NW) {
        int kk = i + rot;
        if (kk >= nsteps) kk -= nsteps;
        const int kt = kb_beg + kk;
        half8 a[2][4], w[NB][4];
#pragma unroll
        for (int b = 0; b < NB; b++) {
            if (WF == 0) load_w_f16<MTILES>(w[b], g.W.w16, nbi[b], Kb, kt, lane);
            else if (WF == 1) {
                if (q8_rows) load_w_q8_rows<MTILES>(w[b], g.W, nbi[b], Kb, kt, lane);
                else load_w_f16<MTILES>(w[b], g.W.w16, nbi[b] - g.W.nbq, Kb, kt, lane);
            } else {
                if (kt < g.W.kbq) load_w_q8_cols<MTILES>(w[b], g.W, nbi[b], g.W.kbq, kt, lane);
                else load_w_f16<MTILES>(w[b], g.W.w16, nbi[b], Kb - g.W.kbq, kt - g.W.kbq, lane);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int mb = 0; mb < 2; mb++) a[mb][j] = ap[mb][(size_t)kt * 256 + j * 64];
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int b = 0; b < NB; b++)
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
                    acc[mb][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mb][j], w[b][j], acc[mb][b], 0, 0, 0);
    }

    // Add the waves' accumulators through LDS so that every wave ends up with the finished sums of 1 / NW of the tile and
    // stores that part.  The registers are numbered i = (mb * NB + b) * 16 + v.  In round r the waves w and
    // w ^ (NW >> (r + 1)) exchange halves of the segment both still hold (the wave without that bit keeps the lower half),
    // so after log2(NW) rounds wave w holds the sums of [seg_lo(w), seg_lo(w) + REGS / NW); the last round's addition
    // is done on the way to memory.
    static_assert(NW == 4 || NW == 8, "the exchange below is written for four or eight waves");
    constexpr int REGS = 2 * NB * 16, ROUNDS = NW == 4 ? 2 : 3;
#define ACC_AT(i) acc[(i) / (NB * 16)][((i) / 16) % NB][(i) % 16]
    // what wave W gives away in round R: the half of its segment that it does not keep
#define GIVE(W, R) if constexpr ((W) < NW) { if (wave == (W)) { \
        constexpr int half = REGS >> ((R) + 1), bit = NW >> ((R) + 1), lo = exchange_seg_lo(REGS, NW, (W), (R)); \
        constexpr int give_lo = ((W) & bit) ? lo : lo + half; \
        float *mine = red + (size_t)(W) * half * 64; \
        _Pragma("unroll") for (int k = 0; k < half; k++) mine[k * 64 + lane] = ACC_AT(give_lo + k); } }
#define TAKE(W, R) if constexpr ((W) < NW) { if (wave == (W)) { \
        constexpr int half = REGS >> ((R) + 1), bit = NW >> ((R) + 1), keep_lo = exchange_seg_lo(REGS, NW, (W), (R) + 1); \
        const float *theirs = red + (size_t)((W) ^ bit) * half * 64; \
        _Pragma("unroll") for (int k = 0; k < half; k++) ACC_AT(keep_lo + k) += theirs[k * 64 + lane]; } }
#define ALL_WAVES(OP, R) OP(0, R) OP(1, R) OP(2, R) OP(3, R) OP(4, R) OP(5, R) OP(6, R) OP(7, R)
    ALL_WAVES(GIVE, 0)
    __syncthreads();
    ALL_WAVES(TAKE, 0)
    __syncthreads();                                      // all have read before the slots are written again
    if constexpr (ROUNDS == 3) {
        ALL_WAVES(GIVE, 1)
        __syncthreads();
        ALL_WAVES(TAKE, 1)
        __syncthreads();
    }
    ALL_WAVES(GIVE, ROUNDS - 1)
    __syncthreads();
    float *Pp = g.P + (size_t)by * g.plane_stride;
    // D layout of v_mfma_f32_32x32x16: column = lane & 31, row = 8*(v/4) + 4*(lane/32) + v%4.  SCALE: the row factors
    // are fetched here, where the K loop's registers are free (holding them through the loop costs a wave of occupancy).
    // A tile inside the matrix stores without bounds tests: under a test per element the compiler puts each LDS read into
    // the branch of its store, and the sixteen read-wait-store groups run one after the other.
    const bool inside = (mb0 + 2) * 32 <= M && (nb0 + NB) * 32 <= N;
#define PART_STORE(W, R) if constexpr ((W) < NW) { if (wave == (W)) { \
        constexpr int Q = REGS / NW, i0 = exchange_seg_lo(REGS, NW, (W), ROUNDS); \
        const float *theirs = red + (size_t)((W) ^ 1) * Q * 64; \
        float sc[Q], sres[Q]; \
        if (SCALE) { \
            /* all factors requested before the first store (row clamped): a load under the store's condition would make \
               every store wait for the one before it */ \
            _Pragma("unroll") for (int k = 0; k < Q; k++) { \
                const int i = i0 + k, mb = i / (NB * 16), v = i % 16; \
                sc[k] = g.a_inv_scale[min((mb0 + mb) * 32 + 8 * (v >> 2) + 4 * h + (v & 3), M - 1)]; \
            } \
        } \
        _Pragma("unroll") for (int k = 0; k < Q; k++) { \
            sres[k] = ACC_AT(i0 + k) + theirs[k * 64 + lane]; \
            if (SCALE) sres[k] *= sc[k]; \
        } \
        if (inside) { \
            _Pragma("unroll") for (int k = 0; k < Q; k++) { \
                const int i = i0 + k, mb = i / (NB * 16), b = (i / 16) % NB, v = i % 16; \
                const int m = (mb0 + mb) * 32 + 8 * (v >> 2) + 4 * h + (v & 3), n = (nb0 + b) * 32 + r; \
                Pp[(size_t)m * g.ldp + n] = sres[k]; \
            } \
        } else { \
            _Pragma("unroll") for (int k = 0; k < Q; k++) { \
                const int i = i0 + k, mb = i / (NB * 16), b = (i / 16) % NB, v = i % 16; \
                const int m = (mb0 + mb) * 32 + 8 * (v >> 2) + 4 * h + (v & 3), n = (nb0 + b) * 32 + r; \
                if (m < M && n < N) Pp[(size_t)m * g.ldp + n] = sres[k]; \
            } \
        } } }
    ALL_WAVES(PART_STORE, 0)
#undef PART_STORE
#undef ALL_WAVES
#undef TAKE
#undef GIVE
#undef ACC_AT
}

// ---- the same product for one 64-row tile of activations: workgroups that own their loads --------------
// gemm_ring<KG, SCALE>: one workgroup of 4 KG waves per (64 weight rows, K chunk).  Where gemm_tiled puts twelve waves on a
// CU, each with one K step in registers, and then adds the waves' accumulators through LDS (32 KB per workgroup, all
// workgroups of a launch at the same moment), this kernel gives the CU one or two workgroups whose loads go straight
// into LDS (global_load_lds_dwordx4: no registers, so the bytes in flight do not depend on the number of waves) and
// splits the 64 x 64 output among the waves as 2 x 2 quadrants of 32 x 32 times KG groups that take every KG-th K step:
//   * a K step is one 16 KB stage: [weight row block 0 | 1 | activation row block 0 | 1], 4 KB each; wave (q, kg)
//     requests block q of its group's stage (four 1 KB pieces) and multiplies weight block q & 1 with activation block
//     q >> 1: every byte is fetched once per workgroup and read from LDS twice;
//   * the ring holds two rounds of KG stages; round r + 2 is requested when round r has been read;
//   * at the end the KG groups exchange 16 / KG accumulator registers per lane (4 KB per wave instead of 12) and every
//     wave stores its part.
// A workgroup covers a K chunk that four-wave workgroups would cut into three, so a product leaves 4 to 6 planes where it
// left 13 to 19, and the launch runs one workgroup per CU (plan_gemm), which keeps the CUs' shares of the stream equal.
// Weight loads are non-temporal (streamed once), activation loads are not (every workgroup of a chunk reads them).
// The LDS-direct loads are issued as assembly: the compiler cannot tell which LDS bytes a pending load writes and would
// wait for all of them before every LDS read; the waits are written by hand below.
typedef __attribute__((address_space(3))) void lds_void_t;

// HALFP (with SCALE 0): the chunk's sums leave as halves, times g.half_scale -- a power of two that the caller derives from
// the weight matrix so that no sum of 8192-bounded operand values can pass the fp16 maximum; plane_stride and ldp then
// count halves.  Half the bytes to write here and for the consumer to read; 11 significant bits per chunk sum.
//
// WF 1, 2: Q8_0 weights (WeightOp fmt 1 / 2) stay quantised on their way through the ring.  A weight tile's slot of a stage
// then holds the tile's 2 KB of int8 as two 1 KB pieces, and behind them its 64 scales (128 bytes, fetched by eight lanes);
// the waves that multiply the tile read their 32 bytes and their scale(s) from LDS and turn them into fp16 there, with
// the arithmetic of load_w_q8_rows / load_w_q8_cols (the value an F16 image of the dequantised weight holds).  1.06 bytes
// per weight from HBM instead of 2.  The F16 tiles that such an operand carries -- the adapter rows behind a fused Q | K | V
// matrix (fmt 1: row blocks from nbq on), the K steps from kbq on of its transposed image (fmt 2) -- take the F16 way
// through the same slot; which way is uniform per wave and stage.  Every wave issues four loads per round either way (a
// quantised tile's fourth asks for its scales once more), so that one count serves the waits.
template <int KG, int SCALE, int HALFP = 0, int WF = 0>
__global__ __launch_bounds__(256 * KG) void gemm_ring(KARGS24)
{
    static_assert(!(SCALE && HALFP), "final outputs stay fp32");
    static_assert(WF >= 0 && WF <= 2, "weight format");
    const uint64_t kw[24] = {KLIST24};
    const GemmKArgs g = kargs_unpack<GemmKArgs>(kw);
    static_assert(KG == 1 || KG == 2 || KG == 4, "K groups per workgroup");
    constexpr int LOADS_PER_ROUND = 4;                    // LDS-direct loads a wave issues per round: the four 1 KB pieces of its block
    __shared__ half8 ring[2 * KG * 1024];                 // [round parity][K group][block 0..3][slice 0..3][64 lanes]
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int q = wv & 3, kg = wv >> 2, qm = q >> 1, qn = q & 1;
    const int r = lane & 31, h = lane >> 5;
    const int tile = blockIdx.x % g.n_tiles, chunk = blockIdx.x / g.n_tiles;
    const int kb_beg = chunk * g.steps_per_chunk;
    const int nsteps = min(g.Kb, kb_beg + g.steps_per_chunk) - kb_beg;
    const int rounds = (nsteps + KG - 1) / KG;
    // q = 0, 1: weight row blocks 2 tile + q; q = 2, 3: activation row blocks q - 2 (clamped: rows beyond M or N are not stored)
    // the weight row block this wave requests (q < 2) and the one it multiplies (qn); fmt 1: from nbq on they are F16 tiles
    const int wb_req = min(2 * tile + (q & 1), g.Nb - 1), wb_mul = min(2 * tile + qn, g.Nb - 1);
    const bool req_q8_rows = WF == 1 && wb_req < g.W.nbq, mul_q8_rows = WF == 1 && wb_mul < g.W.nbq;
    const half8 *src;
    if (WF == 0) src = q < 2 ? reinterpret_cast<const half8 *>(g.w16_ring) + ((size_t)wb_req * g.Kb + kb_beg) * 256 + lane
                             : g.A + ((size_t)min(q - 2, g.Mb - 1) * g.Kb + kb_beg) * 256 + a_lane(lane);
    else if (WF == 1) src = q < 2 ? reinterpret_cast<const half8 *>(g.W.w16) + ((size_t)max(wb_req - g.W.nbq, 0) * g.Kb + kb_beg) * 256 + lane
                                  : g.A + ((size_t)min(q - 2, g.Mb - 1) * g.Kb + kb_beg) * 256 + a_lane(lane);
    else src = q < 2 ? reinterpret_cast<const half8 *>(g.W.w16) + (size_t)wb_req * (g.Kb - g.W.kbq) * 256 + lane     // (+ the F16 step's index)
                     : g.A + ((size_t)min(q - 2, g.Mb - 1) * g.Kb + kb_beg) * 256 + a_lane(lane);
    const uint32_t base = (uint32_t)(uintptr_t)(lds_void_t *)ring;
    // a quantised tile: int8 at slot + 0 .. 2047, scales at + 2048 .. 2175 (and once more at + 2304)
    auto request_q8 = [&](uint32_t sb, size_t tile_index) __attribute__((always_inline)) {
        const uint8_t *qp = g.W.q + tile_index * 2048 + lane * 16;
        asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(qp), "s"(sb) : "m0", "memory");
        asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(qp + 1024), "s"(sb + 1024u) : "m0", "memory");
        const half_t *dp = g.W.d + tile_index * 64 + (lane & 7) * 8;
        if (lane < 8) {
            asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(dp), "s"(sb + 2048u) : "m0", "memory");
            asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(dp), "s"(sb + 2304u) : "m0", "memory");
        }
    };
    auto request = [&](int round) __attribute__((always_inline)) {
        const int step = min(round * KG + kg, nsteps - 1);    // a group without a step in the last round loads the last step again
        const uint32_t sb = base + (uint32_t)(((round & 1) * KG + kg) * 16384 + q * 4096);
        // at most 32 activation rows: the second activation block does not exist; its slot is never filled, the waves that
        // multiply it work on whatever the LDS holds, and their rows are not stored (this wave's waits then pass at once).
        // A quarter fewer stage bytes: 14-16 % off the launch (lm_head forward 174 -> 147 us at 32 rows)
        if (q == 3 && g.Mb == 1) return;
        if constexpr (WF == 1) {
            if (q < 2 && req_q8_rows) { request_q8(sb, (size_t)wb_req * g.Kb + kb_beg + step); return; }
        }
        if constexpr (WF == 2) {
            if (q < 2) {
                const int kt = kb_beg + step;
                if (kt < g.W.kbq) { request_q8(sb, (size_t)wb_req * g.W.kbq + kt); return; }
#pragma unroll
                for (int j = 0; j < LOADS_PER_ROUND; j++)
                    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(src + (size_t)(kt - g.W.kbq) * 256 + j * 64), "s"(sb + (uint32_t)(j * 1024)) : "m0", "memory");
                return;
            }
        }
#pragma unroll
        for (int j = 0; j < LOADS_PER_ROUND; j++) {
            if (q < 2) asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(src + (size_t)step * 256 + j * 64), "s"(sb + (uint32_t)(j * 1024)) : "m0", "memory");
            else asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(src + (size_t)step * 256 + j * 64), "s"(sb + (uint32_t)(j * 1024)) : "m0", "memory");
        }
    };
    float16v acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.f;
    request(0);
    if (rounds > 1) request(1);
    for (int rd = 0; rd < rounds; rd++) {
        // in flight at this point: this wave's loads of round rd and, if there is one, of round rd + 1; loads retire in
        // order, so all but the LOADS_PER_ROUND newest having retired means round rd has landed
        if (rd + 1 < rounds) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(LOADS_PER_ROUND) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();                     // ... and every other wave's as well
        const half8 *st = ring + ((rd & 1) * KG + kg) * 1024;
        half8 w[4], a[4];
        const int kt_mul = kb_beg + min(rd * KG + kg, nsteps - 1);
        if ((WF == 1 && mul_q8_rows) || (WF == 2 && kt_mul < g.W.kbq)) {
            const uint8_t *sq = reinterpret_cast<const uint8_t *>(st) + qn * 4096;
            const uint4v r0 = *reinterpret_cast<const uint4v *>(sq + lane * 16), r1 = *reinterpret_cast<const uint4v *>(sq + 1024 + lane * 16);
            const half_t *sd = reinterpret_cast<const half_t *>(sq + 2048);
            if (WF == 1) {
                const half8 d = bcast8(sd[lane]);
                w[0] = q8_unpack8(r0[0], r0[1]) * d; w[1] = q8_unpack8(r0[2], r0[3]) * d;
                w[2] = q8_unpack8(r1[0], r1[1]) * d; w[3] = q8_unpack8(r1[2], r1[3]) * d;
            } else {
                const half8 *sc = reinterpret_cast<const half8 *>(sd + (lane >> 5) * 32);
                w[0] = q8_unpack8(r0[0], r0[1]) * sc[0]; w[1] = q8_unpack8(r0[2], r0[3]) * sc[1];
                w[2] = q8_unpack8(r1[0], r1[1]) * sc[2]; w[3] = q8_unpack8(r1[2], r1[3]) * sc[3];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) w[j] = st[(qn * 4 + j) * 64 + lane];
        }
#pragma unroll
        for (int j = 0; j < 4; j++) a[j] = st[((2 + qm) * 4 + j) * 64 + lane];
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();                     // all waves have read the stages of this round: they may be refilled
        if (rd + 2 < rounds) request(rd + 2);
        if (rd * KG + kg < nsteps) {
#pragma unroll
            for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j], w[j], acc, 0, 0, 0);
        }
    }
    // Exchange: wave (q, kg) ends up with registers [kg Q, kg Q + Q) of quadrant q, Q = 16 / KG, summed over the groups.
    constexpr int Q = 16 / KG;
    float res[Q];
#pragma unroll
    for (int k = 0; k < Q; k++) res[k] = acc[kg * Q + k];
    if constexpr (KG > 1) {
        float *ex = reinterpret_cast<float *>(ring);       // [q][owner][giver][Q][64 lanes]; the ring is free (last barrier above)
#pragma unroll
        for (int o = 0; o < KG; o++)
            if (o != kg) {
#pragma unroll
                for (int k = 0; k < Q; k++) ex[(((q * KG + o) * KG + kg) * Q + k) * 64 + lane] = acc[o * Q + k];
            }
        __syncthreads();
#pragma unroll
        for (int gv = 0; gv < KG; gv++)
            if (gv != kg) {
#pragma unroll
                for (int k = 0; k < Q; k++) res[k] += ex[(((q * KG + kg) * KG + gv) * Q + k) * 64 + lane];
            }
    }
    // D layout of v_mfma_f32_32x32x16: column = lane & 31, row = 8 (v / 4) + 4 (lane / 32) + v % 4
    const int n = (tile * 2 + qn) * 32 + r;
    const bool inside = 64 <= g.M && (tile + 1) * 64 <= g.N;
    if constexpr (HALFP) {
        half_t *Ph = reinterpret_cast<half_t *>(g.P) + (size_t)chunk * g.plane_stride;
#pragma unroll
        for (int k = 0; k < Q; k++) {
            const int v = kg * Q + k, m = qm * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
            if (inside || (m < g.M && n < g.N)) Ph[(size_t)m * g.ldp + n] = f2h(res[k] * g.half_scale);
        }
        return;
    }
    float *Pp = g.P + (size_t)chunk * g.plane_stride;
    float sc[Q];
    if (SCALE) {
#pragma unroll
        for (int k = 0; k < Q; k++) { const int v = kg * Q + k; sc[k] = g.a_inv_scale[min(qm * 32 + 8 * (v >> 2) + 4 * h + (v & 3), g.M - 1)]; }
#pragma unroll
        for (int k = 0; k < Q; k++) res[k] *= sc[k];
    }
    if (inside) {
#pragma unroll
        for (int k = 0; k < Q; k++) { const int v = kg * Q + k; Pp[(size_t)(qm * 32 + 8 * (v >> 2) + 4 * h + (v & 3)) * g.ldp + n] = res[k]; }
    } else {
#pragma unroll
        for (int k = 0; k < Q; k++) {
            const int v = kg * Q + k, m = qm * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
            if (m < g.M && n < g.N) Pp[(size_t)m * g.ldp + n] = res[k];
        }
    }
}

// gemm_ring with four weight row blocks per workgroup instead of two and one K group (more than 32 activation rows): a
// stage is four weight tiles and the two activation tiles, 24 KB of LDS, so the bytes a workgroup pulls into LDS per F16
// weight byte are 1.5 instead of 2 (Q8_0: 16.5 KB instead of 24.7 KB per four tiles) -- and it is those stage bytes,
// weights and activation tiles together, that a launch's time follows.  Eight waves: 4 x 2 output quadrants of 32 x 32;
// 48 KB of ring, up to three workgroups per CU; a workgroup walks its K chunk one step per round and every wave stores
// its whole quadrant (no exchange).  Rounds and waits as in gemm_ring.
// WF 0: the 24 pieces of a stage are requested three per wave.  WF 1, 2 (Q8_0 tiles, quantised up to LDS as in gemm_ring):
// waves 0 .. 3 request one weight tile each (four loads: a quantised tile's 2 KB and its scales, twice; or the four
// pieces of an F16 tile that the operand carries), waves 4 .. 7 two pieces each of the activation blocks; the waits count
// per wave.
template <int SCALE, int HALFP, int WF = 0>
__global__ __launch_bounds__(512) void gemm_ring_wide(KARGS24)
{
    static_assert(!(SCALE && HALFP), "final outputs stay fp32");
    static_assert(WF >= 0 && WF <= 2, "weight format");
    const uint64_t kw[24] = {KLIST24};
    const GemmKArgs g = kargs_unpack<GemmKArgs>(kw);
    constexpr int WB = 4, LOADS_PER_ROUND = 3, STAGE = (WB + 2) * 256;      // half8 elements per stage (24 KB)
    __shared__ half8 wring[2 * STAGE];                    // [round parity][weight block 0..3, activation block 0, 1][slice][64 lanes]
    const int lane = threadIdx.x & 63, q = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int qn = q & 3, qm = q >> 2;
    const int r = lane & 31, h = lane >> 5;
    const int tile = blockIdx.x % g.n_tiles, chunk = blockIdx.x / g.n_tiles;
    const int kb_beg = chunk * g.steps_per_chunk;
    const int nsteps = min(g.Kb, kb_beg + g.steps_per_chunk) - kb_beg;
    const uint32_t base = (uint32_t)(uintptr_t)(lds_void_t *)wring;
    // WF 0: wave q requests the pieces 3 q .. 3 q + 2 of a stage: piece p = slice p % 4 of block p / 4 (blocks 0 .. 3: weight
    // row blocks 4 tile + b; 4, 5: activation row blocks; clamped: rows beyond M or N are not stored)
    const half8 *src[LOADS_PER_ROUND];
    uint32_t off[LOADS_PER_ROUND];
    bool is_w[LOADS_PER_ROUND];
#pragma unroll
    for (int i = 0; i < LOADS_PER_ROUND; i++) {
        const int p = q * LOADS_PER_ROUND + i, b = p >> 2, j = p & 3;
        is_w[i] = b < WB;
        src[i] = is_w[i] ? reinterpret_cast<const half8 *>(g.w16_ring) + ((size_t)min(WB * tile + b, g.Nb - 1) * g.Kb + kb_beg) * 256 + j * 64 + lane
                         : g.A + ((size_t)min(b - WB, g.Mb - 1) * g.Kb + kb_beg) * 256 + j * 64 + a_lane(lane);
        off[i] = (uint32_t)(b * 4096 + j * 1024);
    }
    // WF 1, 2: the weight row block wave q < 4 requests, the one this wave multiplies (fmt 1: from nbq on they are F16
    // tiles), and for q >= 4 the two activation pieces (slices 2 (q & 1), + 1 of block (q - 4) / 2)
    const int wb_req = min(WB * tile + qn, g.Nb - 1);     // (q < 4: qn = q; also the block that waves qn and 4 + qn multiply)
    const bool q8_rows = WF == 1 && wb_req < g.W.nbq;
    const half8 *qsrc = nullptr;
    uint32_t qoff = 0;
    if constexpr (WF != 0) {
        if (q < WB) {
            qsrc = WF == 1 ? reinterpret_cast<const half8 *>(g.W.w16) + ((size_t)max(wb_req - g.W.nbq, 0) * g.Kb + kb_beg) * 256 + lane
                           : reinterpret_cast<const half8 *>(g.W.w16) + (size_t)wb_req * (g.Kb - g.W.kbq) * 256 + lane;    // (+ the F16 step's index)
            qoff = (uint32_t)(q * 4096);
        } else {
            const int b = (q - WB) >> 1, s0 = 2 * (q & 1);
            qsrc = g.A + ((size_t)min(b, g.Mb - 1) * g.Kb + kb_beg) * 256 + s0 * 64 + a_lane(lane);
            qoff = (uint32_t)((WB + b) * 4096 + s0 * 1024);
        }
    }
    // a quantised tile: int8 at slot + 0 .. 2047, scales at + 2048 .. 2175 (and once more at + 2304)
    auto request_q8 = [&](uint32_t sb, size_t tile_index) __attribute__((always_inline)) {
        const uint8_t *qp = g.W.q + tile_index * 2048 + lane * 16;
        asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(qp), "s"(sb) : "m0", "memory");
        asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(qp + 1024), "s"(sb + 1024u) : "m0", "memory");
        const half_t *dp = g.W.d + tile_index * 64 + (lane & 7) * 8;
        if (lane < 8) {
            asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(dp), "s"(sb + 2048u) : "m0", "memory");
            asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(dp), "s"(sb + 2304u) : "m0", "memory");
        }
    };
    auto request = [&](int step) __attribute__((always_inline)) {
        const uint32_t sb = base + (uint32_t)((step & 1) * STAGE * 16);
        if constexpr (WF == 0) {
#pragma unroll
            for (int i = 0; i < LOADS_PER_ROUND; i++) {
                if (is_w[i]) asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(src[i] + (size_t)step * 256), "s"(sb + off[i]) : "m0", "memory");
                else asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(src[i] + (size_t)step * 256), "s"(sb + off[i]) : "m0", "memory");
            }
        } else if (q < WB) {
            const int kt = kb_beg + step;
            if (WF == 1 && q8_rows) { request_q8(sb + qoff, (size_t)wb_req * g.Kb + kt); return; }
            if (WF == 2 && kt < g.W.kbq) { request_q8(sb + qoff, (size_t)wb_req * g.W.kbq + kt); return; }
            const half8 *f = WF == 1 ? qsrc + (size_t)step * 256 : qsrc + (size_t)(kt - g.W.kbq) * 256;
#pragma unroll
            for (int j = 0; j < 4; j++)
                asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(f + j * 64), "s"(sb + qoff + (uint32_t)(j * 1024)) : "m0", "memory");
        } else {
#pragma unroll
            for (int j = 0; j < 2; j++)
                asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(qsrc + (size_t)step * 256 + j * 64), "s"(sb + qoff + (uint32_t)(j * 1024)) : "m0", "memory");
        }
    };
    float16v acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.f;
    request(0);
    if (nsteps > 1) request(1);
    for (int rd = 0; rd < nsteps; rd++) {
        // in flight: this wave's loads of step rd and, if there is one, of step rd + 1 (loads retire in order)
        if (rd + 1 < nsteps) {
            if constexpr (WF == 0) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(LOADS_PER_ROUND) : "memory");
            else if (q < WB) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        } else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        const half8 *st = wring + (rd & 1) * STAGE;
        half8 w[4], a[4];
        if ((WF == 1 && q8_rows) || (WF == 2 && kb_beg + rd < g.W.kbq)) {
            const uint8_t *sq = reinterpret_cast<const uint8_t *>(st) + qn * 4096;
            const uint4v r0 = *reinterpret_cast<const uint4v *>(sq + lane * 16), r1 = *reinterpret_cast<const uint4v *>(sq + 1024 + lane * 16);
            const half_t *sd = reinterpret_cast<const half_t *>(sq + 2048);
            if (WF == 1) {
                const half8 d = bcast8(sd[lane]);
                w[0] = q8_unpack8(r0[0], r0[1]) * d; w[1] = q8_unpack8(r0[2], r0[3]) * d;
                w[2] = q8_unpack8(r1[0], r1[1]) * d; w[3] = q8_unpack8(r1[2], r1[3]) * d;
            } else {
                const half8 *sc = reinterpret_cast<const half8 *>(sd + (lane >> 5) * 32);
                w[0] = q8_unpack8(r0[0], r0[1]) * sc[0]; w[1] = q8_unpack8(r0[2], r0[3]) * sc[1];
                w[2] = q8_unpack8(r1[0], r1[1]) * sc[2]; w[3] = q8_unpack8(r1[2], r1[3]) * sc[3];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) w[j] = st[(qn * 4 + j) * 64 + lane];
        }
#pragma unroll
        for (int j = 0; j < 4; j++) a[j] = st[((WB + qm) * 4 + j) * 64 + lane];
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();                     // all waves have read this step's stage: it may be refilled
        if (rd + 2 < nsteps) request(rd + 2);
#pragma unroll
        for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j], w[j], acc, 0, 0, 0);
    }
    // D layout of v_mfma_f32_32x32x16: column = lane & 31, row = 8 (v / 4) + 4 (lane / 32) + v % 4
    const int n = (tile * WB + qn) * 32 + r;
    const bool inside = 64 <= g.M && (tile + 1) * 32 * WB <= g.N;
    if constexpr (HALFP) {
        half_t *Ph = reinterpret_cast<half_t *>(g.P) + (size_t)chunk * g.plane_stride;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = qm * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
            if (inside || (m < g.M && n < g.N)) Ph[(size_t)m * g.ldp + n] = f2h(acc[v] * g.half_scale);
        }
        return;
    }
    float *Pp = g.P + (size_t)chunk * g.plane_stride;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int m = qm * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        float o = acc[v];
        if (SCALE) o *= g.a_inv_scale[min(m, g.M - 1)];
        if (inside || (m < g.M && n < g.N)) Pp[(size_t)m * g.ldp + n] = o;
    }
}

// The weight loads of gemm_ring alone, on the same grid and through the same LDS ring: what a launch needs just to pull its
// weight bytes into LDS (timing reference for the product; nothing is multiplied or stored).
template <int KG>
__global__ __launch_bounds__(256 * KG) void ring_weights_only(GemmKArgs g)
{
    __shared__ half8 ring[2 * KG * 1024];
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int q = wv & 3, kg = wv >> 2;
    const int tile = blockIdx.x % g.n_tiles, chunk = blockIdx.x / g.n_tiles;
    const int kb_beg = chunk * g.steps_per_chunk;
    const int nsteps = min(g.Kb, kb_beg + g.steps_per_chunk) - kb_beg;
    const int rounds = (nsteps + KG - 1) / KG;
    if (q >= 2) return;
    const half8 *src = reinterpret_cast<const half8 *>(g.W.w16) + ((size_t)min(2 * tile + q, g.Nb - 1) * g.Kb + kb_beg) * 256 + lane;
    const uint32_t base = (uint32_t)(uintptr_t)(lds_void_t *)ring;
    auto request = [&](int round) __attribute__((always_inline)) {
        const int step = min(round * KG + kg, nsteps - 1);
        const uint32_t sb = base + (uint32_t)(((round & 1) * KG + kg) * 16384 + q * 4096);
#pragma unroll
        for (int j = 0; j < 4; j++)
            asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(src + (size_t)step * 256 + j * 64), "s"(sb + (uint32_t)(j * 1024)) : "m0", "memory");
    };
    request(0);
    if (rounds > 1) request(1);
    for (int rd = 0; rd < rounds; rd++) {
        if (rd + 1 < rounds) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");    // four loads per round and wave, as in gemm_ring
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (rd + 2 < rounds) request(rd + 2);
    }
    if (ring[lane][0] == (half_t)12345.0f) g.P[0] = 1.f;   // the loads have a use
}

}  // namespace lmhip
