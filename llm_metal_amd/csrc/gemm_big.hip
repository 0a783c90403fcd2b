// Large-M GEMM: C[M, N] = inv_scale[m] * A16[M, K] * W[N, K]^T for M of several hundred rows and more
// (batch * seq = 2048 in the Q8_0 configuration), where a weight tile is reused by enough activation rows
// that the matrix cores, not HBM, bound the product.  Same operands as the weight-streaming kernel
// (gemm.h: tiled fp16 activations with per-row power-of-two factors; F16 or Q8_0 weight tiles), same
// arithmetic (v_mfma_f32_32x32x16_f16, fp32 accumulation), one launch, no K split.
//
// A workgroup of four waves owns a 128 x 256 block of C and walks K in steps of 64.  Per step every wave
// fetches one 32-row block of the activation tile and two of the weight tile from L2/HBM in the MFMA
// register layout, Q8_0 blocks are unpacked to fp16 there (int8 * fp16 scale, once per tile instead of once
// per consumer), and both go to LDS in the same [j][lane][8 halves] order, so a wave reads any row block back
// with conflict-free 16-byte loads.  LDS is double buffered and the operands travel three steps ahead in registers:
// during the MFMAs of step k the loads of step k+3 are issued and step k+1 is written to the other buffer; one
// barrier per step.  That is the kernel for Q8_0 tiles (gemm_big<1>, <2>); F16 tiles take gemm_big_f16 (the same block)
// or gemm_big_f16_256 (a 256 x 256 block) below, whose operands reach LDS without passing through registers, and
// launch_gemm_big chooses between the two block shapes, or gives each a part of the columns.
#include "backend.h"
#include "devutil.h"
#include "gemm.h"
#include "gemm_kernel.h"
#include <hip/hip_ext.h>
#include <algorithm>

namespace lmhip {
namespace {

int g_big_split = 1;                  // 1: K chunks by the measured rule (big_gemm_chunks), 0: never, n > 1: always n
int g_big_block = 0;                  // F16 tiles: 0 block shape by the measured rule, 1 always 128 x 256, 2 always 256 x 256
constexpr int WPW = 2;               // weight row blocks each wave fetches per K step: the block is 128 x (WPW * 128)
constexpr int PF = 3;                // K steps whose operands are in flight in registers ahead of the one being multiplied

// What one thread holds of a K step that is still on its way to LDS: one row block of A and WPW of W, as loaded
// (Q8_0 stays packed until it is written to LDS, so nothing waits on a fresh load).
struct Stage {
    half8 a[4];
    half8 w16[WPW][4];               // F16 tile, or the column scales of a transposed Q8_0 tile
    uint4v q[WPW][2];                // Q8_0 int8
    uint32_t d[WPW];                 // Q8_0 row scale of this lane's weights: the fp16 bits in a register of their own (two halves
                                     // packed into one register would make the pack wait for the load that was just issued)
};

// kind of weight tile (uniform per wave): 0 F16, 1 Q8_0 row scales, 2 Q8_0 column scales
template <int WF>
__device__ __forceinline__ int tile_kind(const GemmKArgs &g, int nb, int kt)
{
    if (WF == 0) return 0;
    if (WF == 1) return nb < g.W.nbq ? 1 : 0;
    return kt < g.W.kbq ? 2 : 0;
}

template <int WF>
__device__ __forceinline__ void fetch(Stage &s, const GemmKArgs &g, int mb, const int (&nb)[WPW], int kt, int lane)
{
    const half8 *ap = g.A + ((size_t)mb * g.Kb + kt) * 256 + a_lane(lane);
#pragma unroll
    for (int j = 0; j < 4; j++) s.a[j] = ap[j * 64];
#pragma unroll
    for (int u = 0; u < WPW; u++) {
        const int kind = tile_kind<WF>(g, nb[u], kt);
        if (kind == 0) {
            if (WF == 0) load_w_f16(s.w16[u], g.W.w16, nb[u], g.Kb, kt, lane);
            else if (WF == 1) load_w_f16(s.w16[u], g.W.w16, nb[u] - g.W.nbq, g.Kb, kt, lane);
            else load_w_f16(s.w16[u], g.W.w16, nb[u], g.Kb - g.W.kbq, kt - g.W.kbq, lane);
        } else {
            const size_t tile = (size_t)nb[u] * (kind == 1 ? g.Kb : g.W.kbq) + kt;
            const uint4v *q = reinterpret_cast<const uint4v *>(g.W.q) + tile * 128 + lane;
            s.q[u][0] = __builtin_nontemporal_load(&q[0]);
            s.q[u][1] = __builtin_nontemporal_load(&q[64]);
            if (kind == 1) s.d[u] = reinterpret_cast<const uint16_t *>(g.W.d)[tile * 64 + lane];
            else {
                const half8 *sc = reinterpret_cast<const half8 *>(g.W.d + tile * 64 + (lane >> 5) * 32);
#pragma unroll
                for (int j = 0; j < 4; j++) s.w16[u][j] = sc[j];
            }
        }
    }
}

// fp16 weight registers of a fetched tile (Q8_0: int8 * scale, rounded once to fp16)
template <int WF>
__device__ __forceinline__ void unpack(half8 (&w)[4], const Stage &s, int u, int kind)
{
    if (kind == 0) {
#pragma unroll
        for (int j = 0; j < 4; j++) w[j] = s.w16[u][j];
        return;
    }
    const half8 q0 = q8_unpack8(s.q[u][0][0], s.q[u][0][1]), q1 = q8_unpack8(s.q[u][0][2], s.q[u][0][3]);
    const half8 q2 = q8_unpack8(s.q[u][1][0], s.q[u][1][1]), q3 = q8_unpack8(s.q[u][1][2], s.q[u][1][3]);
    if (kind == 1) { const half8 d = bcast8(__builtin_bit_cast(half_t, (uint16_t)s.d[u])); w[0] = q0 * d; w[1] = q1 * d; w[2] = q2 * d; w[3] = q3 * d; }
    else { w[0] = q0 * s.w16[u][0]; w[1] = q1 * s.w16[u][1]; w[2] = q2 * s.w16[u][2]; w[3] = q3 * s.w16[u][3]; }
}

// 1-D grid, block 256; LDS 2 x (4 + 4 WPW) row blocks x 4 KB.
// Wave (wm, wn) owns rows [64 wm, +64) and columns [64 WPW wn, +64 WPW) of the block.
//
// Which block a workgroup takes is chosen for the eight L2 caches: the hardware deals consecutive workgroup ids
// to the XCDs in turn, so id % 8 is the XCD.  Each XCD gets every eighth column of blocks, and the 32 workgroups
// that are resident on it together form an 8 x 4 patch (8 row blocks x 4 column blocks).  They walk K in step, so
// an activation slice fetched into that L2 serves 4 workgroups and a weight slice 8, instead of one each.
template <int WF>
__global__ __launch_bounds__(256) void gemm_big(GemmKArgs g)
{
    extern __shared__ half8 tiles[];                      // [buf][A blocks 0-3 | W blocks 0 .. 4 WPW - 1][j][lane]
    constexpr int NBLK = 4 + 4 * WPW, BUF = NBLK * 256, NW = 2 * WPW;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int MT = (g.M + 127) >> 7, NT = (g.N + 128 * WPW - 1) / (128 * WPW);
    const int m_patches = (MT + 7) >> 3;
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3, patch = seq >> 5, in_patch = seq & 31;
    const int mt = (patch % m_patches) * 8 + (in_patch & 7);
    const int nt = ((patch / m_patches) * 4 + (in_patch >> 3)) * 8 + xcd;
    if (mt >= MT || nt >= NT) return;                     // padding of the patch grid; the whole workgroup leaves
    const int nb0 = nt * 4 * WPW, mb0 = mt * 4;
    const int wm = wave >> 1, wn = wave & 1;
    // the row blocks this wave fetches (clamped: rows past the end are computed and never stored)
    const int mb_ld = min(mb0 + wave, g.Mb - 1);
    int nb_ld[WPW];
#pragma unroll
    for (int u = 0; u < WPW; u++) nb_ld[u] = min(nb0 + wave * WPW + u, g.Nb - 1);

    float16v acc[2][NW];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < NW; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    Stage st[PF];                                         // step s travels in st[s % PF]
    auto park = [&](const Stage &s, int kt, half8 *buf) {
#pragma unroll
        for (int j = 0; j < 4; j++) buf[(wave * 4 + j) * 64 + lane] = s.a[j];
#pragma unroll
        for (int u = 0; u < WPW; u++) {
            half8 w[4];
            unpack<WF>(w, s, u, tile_kind<WF>(g, nb_ld[u], kt));
#pragma unroll
            for (int j = 0; j < 4; j++) buf[((4 + wave * WPW + u) * 4 + j) * 64 + lane] = w[j];
        }
    };
    // Every fetch is issued unconditionally (past the end it asks for the last step again): with a fetch under a
    // condition the compiler cannot count how many younger loads are in flight when a stage is parked, and waits for
    // all of them -- the prefetch then hides nothing.
    const int last = g.Kb - 1;
#pragma unroll
    for (int p = 0; p < PF; p++) fetch<WF>(st[p], g, mb_ld, nb_ld, min(p, last), lane);
    park(st[0], 0, tiles);
    __syncthreads();
    // one K step: multiply step kt out of LDS buffer kt & 1 while step kt + 1 is unpacked and parked in the other one
    // and step kt + PF is requested into the slot that step kt left (u = kt % PF, a compile-time constant at every call)
    auto step = [&](int kt, int u) __attribute__((always_inline)) {
        const half8 *cur = tiles + (size_t)(kt & 1) * BUF;
        fetch<WF>(st[u], g, mb_ld, nb_ld, min(kt + PF, last), lane);
        // fp16 image of the next step's weight blocks: plain VALU work with no dependence on this step's MFMAs, placed in
        // the same block of code so that the two interleave (on the last step it unpacks a repeated step and the result
        // lands in the buffer nobody reads any more)
        const Stage &sn = st[(u + 1) % PF];
        half8 wnext[WPW][4];
#pragma unroll
        for (int x = 0; x < WPW; x++) unpack<WF>(wnext[x], sn, x, tile_kind<WF>(g, nb_ld[x], min(kt + 1, last)));
        // operands of K slice j + 1 are read from LDS before the MFMAs of slice j are issued, so the reads run under them
        half8 a[2][2], w[2][NW];
        auto read = [&](int j) {
#pragma unroll
            for (int i = 0; i < 2; i++) a[j & 1][i] = cur[((2 * wm + i) * 4 + j) * 64 + lane];
#pragma unroll
            for (int k = 0; k < NW; k++) w[j & 1][k] = cur[((4 + NW * wn + k) * 4 + j) * 64 + lane];
        };
        read(0);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (j + 1 < 4) read(j + 1);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int k = 0; k < NW; k++)
                    acc[i][k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j & 1][i], w[j & 1][k], acc[i][k], 0, 0, 0);
        }
        half8 *nxt = tiles + (size_t)((kt + 1) & 1) * BUF;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            nxt[(wave * 4 + j) * 64 + lane] = sn.a[j];
#pragma unroll
            for (int x = 0; x < WPW; x++) nxt[((4 + wave * WPW + x) * 4 + j) * 64 + lane] = wnext[x][j];
        }
        // Issue order of the step, one memory instruction in the shadow of each MFMA (a wave is the only one on its SIMD,
        // so whatever is not issued between two MFMAs is paid for on top of them): the 6 LDS reads of slice 0, then per
        // MFMA of slices 0-2 one LDS read of the next slice, the 12 global loads under slices 0-1, the 12 LDS writes
        // under slices 2-3.  Left to itself the scheduler sinks every read to just before its use.
        __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
        for (int i = 0; i < 32; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < 24 && (i & 7) < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (i < 12) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            if (i >= 20) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        __syncthreads();
    };
    const int full = g.Kb / PF * PF;
    for (int kt0 = 0; kt0 < full; kt0 += PF) {
#pragma unroll
        for (int u = 0; u < PF; u++) step(kt0 + u, u);
    }
#pragma unroll
    for (int u = 0; u < PF - 1; u++) if (full + u < g.Kb) step(full + u, u);

    // D layout of v_mfma_f32_32x32x16: column = lane & 31, row = 8*(v/4) + 4*(lane/32) + v%4
    if (mb0 * 32 + 128 <= g.M && (nb0 + 4 * WPW) * 32 <= g.N) {
        // Block inside the matrix: no bounds tests, so the row factors are all requested at once and the stores follow
        // each other without a wait (a store under a condition makes the compiler drain the queue before every one).
        float sc[2][16];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) sc[i][v] = 1.0f;
        if (g.a_inv_scale) {
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    sc[i][v] = g.a_inv_scale[(mb0 + 2 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3)];
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = (mb0 + 2 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                float *row = g.P + (size_t)m * g.ldp + (nb0 + NW * wn) * 32 + r;
#pragma unroll
                for (int k = 0; k < NW; k++) row[k * 32] = acc[i][k][v] * sc[i][v];
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = (mb0 + 2 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
            if (m >= g.M) continue;
            const float sc = g.a_inv_scale ? g.a_inv_scale[m] : 1.0f;
#pragma unroll
            for (int k = 0; k < NW; k++) {
                const int n = (nb0 + NW * wn + k) * 32 + r;
                if (n < g.N) g.P[(size_t)m * g.ldp + n] = acc[i][k][v] * sc;
            }
        }
}


// F16 weight tiles need no unpacking, so their steps go from L2/HBM straight into LDS (global_load_lds_dwordx4: a
// wave-uniform LDS base in M0, lane i's 16 bytes land at base + 16 i -- the [j][lane] order of the tiles) and never
// pass through registers or ds_write.  K goes in half steps of 32 (two of a tile's four 1 KB slices per row block)
// through six 24 KB LDS buffers, distinct objects: half step h is multiplied out of buffer h % 6 while h + 1 .. h + 5
// are in LDS or on their way.  The copies are issued as assembly right after the barrier, so the compiler does not count
// them among its own loads (it cannot tell which LDS bytes a pending copy writes and would wait for all of them before
// every LDS read); the wait before the barrier is written by hand: the barrier that ends half step h - 1 finds h and
// h + 1 in LDS -- every wave has waited for its own copies of them -- so slice 0 of h + 1 is read under the MFMAs of
// slice 1 of h and no half step starts by waiting out an LDS round trip; h + 5 is requested into the buffer h - 1 left.
__global__ __launch_bounds__(256) void gemm_big_f16(GemmKArgs g)
{
    constexpr int HB = 12 * 2 * 64;                       // half8 per buffer: [4 A + 8 W row blocks][2 slices][64 lanes]
    __shared__ half8 lb0[HB], lb1[HB], lb2[HB], lb3[HB], lb4[HB], lb5[HB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int MT = (g.M + 127) >> 7, NT = (g.N + 255) >> 8;
    const int m_patches = (MT + 7) >> 3;
    int mt, nt, chunk = 0;
    if (g.S > 1) {
        const int t = blockIdx.x % (MT * NT);
        chunk = blockIdx.x / (MT * NT); mt = t % MT; nt = t / MT;
    } else {
        const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3, patch = seq >> 5, in_patch = seq & 31;
        mt = (patch % m_patches) * 8 + (in_patch & 7);
        nt = ((patch / m_patches) * 4 + (in_patch >> 3)) * 8 + xcd;
        if (mt >= MT || nt >= NT) return;
    }
    const int nb0 = nt * 8, mb0 = mt * 4;
    const int wm = wave >> 1, wn = wave & 1;
    const int k_beg = chunk * g.steps_per_chunk, nsteps = min(g.Kb, k_beg + g.steps_per_chunk) - k_beg;
    const int nhalf = 2 * nsteps, last = nhalf - 1;
    const half8 *src[3];
    src[0] = g.A + ((size_t)min(mb0 + wave, g.Mb - 1) * g.Kb + k_beg) * 256 + a_lane(lane);
    src[1] = reinterpret_cast<const half8 *>(g.W.w16) + ((size_t)min(nb0 + 2 * wave, g.Nb - 1) * g.Kb + k_beg) * 256 + lane;
    src[2] = reinterpret_cast<const half8 *>(g.W.w16) + ((size_t)min(nb0 + 2 * wave + 1, g.Nb - 1) * g.Kb + k_beg) * 256 + lane;
    const int dst[3] = {wave, 4 + 2 * wave, 5 + 2 * wave};
    float *const Cp = g.P + (size_t)chunk * g.plane_stride;

    float16v acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    typedef __attribute__((address_space(3))) void lds_void;
    uint32_t loff[3][2];
#pragma unroll
    for (int u = 0; u < 3; u++)
#pragma unroll
        for (int j = 0; j < 2; j++) loff[u][j] = __builtin_amdgcn_readfirstlane((uint32_t)((dst[u] * 2 + j) * 64 * 16));
    constexpr int LOADS = 3 * 2, AHEAD = 5, LANDED = 2;   // copies per request and wave; requests in flight after a request; how many of them a barrier needs
    constexpr int WAIT = (AHEAD - LANDED) * LOADS;
    static_assert(WAIT == 18 && AHEAD * LOADS < 64, "the hand-written waits count this wave's LDS-direct loads; vmcnt has six bits");
    auto request = [&](half8 (&buf)[HB], int hs) __attribute__((always_inline)) {
        const size_t o = (size_t)(hs >> 1) * 256 + (hs & 1) * 128;
        const uint32_t base = (uint32_t)(uintptr_t)(lds_void *)buf;
#pragma unroll
        for (int u = 0; u < 3; u++)
#pragma unroll
            for (int j = 0; j < 2; j++)                    // LOADS of these
                asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(src[u] + o + j * 64), "s"(base + loff[u][j]) : "m0");
    };
    half8 a0[2], w0[4];
    auto read = [&](half8 (&a)[2], half8 (&w)[4], const half8 (&cur)[HB], int j) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; i++) a[i] = cur[((2 * wm + i) * 2 + j) * 64 + lane];
#pragma unroll
        for (int k = 0; k < 4; k++) w[k] = cur[((4 + 4 * wn + k) * 2 + j) * 64 + lane];
    };
    auto multiply = [&](const half8 (&a)[2], const half8 (&w)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int k = 0; k < 4; k++) acc[i][k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], w[k], acc[i][k], 0, 0, 0);
    };
    auto step = [&](int hs, const half8 (&cur)[HB], const half8 (&nxt)[HB], half8 (&free_buf)[HB]) __attribute__((always_inline)) {
        request(free_buf, min(hs + 5, last));
        half8 a1[2], w1[4];
        read(a1, w1, cur, 1);
        multiply(a0, w0);
        read(a0, w0, nxt, 0);
        multiply(a1, w1);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < 4 || (i >= 8 && i < 14)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        // In flight here: this wave's copies of half steps hs + 1 .. hs + 5, LOADS each, oldest first.  The barrier must find
        // hs + 1 and hs + 2 in LDS, so all but the newest three requests have to have retired (loads retire in order).
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(WAIT) : "memory");
    };
    request(lb0, 0); request(lb1, min(1, last)); request(lb2, min(2, last)); request(lb3, min(3, last)); request(lb4, min(4, last));
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(WAIT) : "memory");   // five requests out: the first two have landed
    read(a0, w0, lb0, 0);
    const int full = nhalf / 6 * 6;
    for (int h0 = 0; h0 < full; h0 += 6) {
        step(h0, lb0, lb1, lb5);
        step(h0 + 1, lb1, lb2, lb0);
        step(h0 + 2, lb2, lb3, lb1);
        step(h0 + 3, lb3, lb4, lb2);
        step(h0 + 4, lb4, lb5, lb3);
        step(h0 + 5, lb5, lb0, lb4);
    }
    if (full < nhalf) step(full, lb0, lb1, lb5);
    if (full + 1 < nhalf) step(full + 1, lb1, lb2, lb0);
    if (full + 2 < nhalf) step(full + 2, lb2, lb3, lb1);
    if (full + 3 < nhalf) step(full + 3, lb3, lb4, lb2);
    if (full + 4 < nhalf) step(full + 4, lb4, lb5, lb3);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    if (mb0 * 32 + 128 <= g.M && (nb0 + 8) * 32 <= g.N) {
        float sc[2][16];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                sc[i][v] = g.a_inv_scale ? g.a_inv_scale[(mb0 + 2 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3)] : 1.0f;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = (mb0 + 2 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                float *row = Cp + (size_t)m * g.ldp + (nb0 + 4 * wn) * 32 + r;
#pragma unroll
                for (int k = 0; k < 4; k++) row[k * 32] = acc[i][k][v] * sc[i][v];
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = (mb0 + 2 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
            if (m >= g.M) continue;
            const float sc = g.a_inv_scale ? g.a_inv_scale[m] : 1.0f;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int n = (nb0 + 4 * wn + k) * 32 + r;
                if (n < g.N) Cp[(size_t)m * g.ldp + n] = acc[i][k][v] * sc;
            }
        }
}


// The same product on a 256 x 256 block: four waves of 128 x 128 (sixteen accumulator tiles each, in the accumulation
// registers), so that a wave reads 0.5 KB of LDS per MFMA instead of 0.75 and a block fetches half as many operand bytes
// per flop.  K goes in half steps of 32 (two of a tile's four 1 KB slices per row block) through five 32 KB LDS buffers
// (all 160 KB of a CU): half step h is multiplied out of buffer h % 5 while h + 1 .. h + 4 are in LDS or on their way.
// The copies are LDS-direct loads issued as assembly, right after the barrier: the compiler does not count them among
// its own loads (it cannot tell which LDS bytes a pending copy writes and would wait for all of them before every LDS
// read); the wait before the barrier is written by hand.
// 8192 x 8192 x 8192 on random operands: 1 227 TFLOP/s against 1 083 for 128 x 256 (constant operands, which toggle few
// bits and let the GPU hold a higher clock, give 1 667 and 1 387).  There are half as many blocks: launch_gemm_big picks
// the shape that loses less to partial rounds and partial tiles.
__global__ __launch_bounds__(256) void gemm_big_f16_256(GemmKArgs g)
{
    constexpr int HB = 16 * 2 * 64;                       // half8 per buffer: [16 row blocks][2 slices][64 lanes]
    __shared__ half8 lb0[HB], lb1[HB], lb2[HB], lb3[HB], lb4[HB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int MT = (g.M + 255) >> 8, NT = (g.N + 255) >> 8;
    const int m_patches = (MT + 7) >> 3;
    int mt, nt, chunk = 0;
    if (g.S > 1) {
        const int t = blockIdx.x % (MT * NT);
        chunk = blockIdx.x / (MT * NT); mt = t % MT; nt = t / MT;
    } else {
        const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3, patch = seq >> 5, in_patch = seq & 31;
        mt = (patch % m_patches) * 8 + (in_patch & 7);
        nt = ((patch / m_patches) * 4 + (in_patch >> 3)) * 8 + xcd;
        if (mt >= MT || nt >= NT) return;
    }
    const int nb0 = nt * 8, mb0 = mt * 8;
    const int wm = wave >> 1, wn = wave & 1;
    const int k_beg = chunk * g.steps_per_chunk, nsteps = min(g.Kb, k_beg + g.steps_per_chunk) - k_beg;
    const int nhalf = 2 * nsteps, last = nhalf - 1;
    // this wave's share of a half step: both slices of A row blocks w, 4 + w and of W row blocks w, 4 + w
    const half8 *src[4];
    src[0] = g.A + ((size_t)min(mb0 + wave, g.Mb - 1) * g.Kb + k_beg) * 256 + a_lane(lane);
    src[1] = g.A + ((size_t)min(mb0 + 4 + wave, g.Mb - 1) * g.Kb + k_beg) * 256 + a_lane(lane);
    src[2] = reinterpret_cast<const half8 *>(g.W.w16) + ((size_t)min(nb0 + wave, g.Nb - 1) * g.Kb + k_beg) * 256 + lane;
    src[3] = reinterpret_cast<const half8 *>(g.W.w16) + ((size_t)min(nb0 + 4 + wave, g.Nb - 1) * g.Kb + k_beg) * 256 + lane;
    const int dst[4] = {wave, 4 + wave, 8 + wave, 12 + wave};
    float *const Cp = g.P + (size_t)chunk * g.plane_stride;

    float16v acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    typedef __attribute__((address_space(3))) void lds_void;
    uint32_t loff[4][2];                                   // byte offsets inside a buffer of this wave's eight 1 KB pieces
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
        for (int j = 0; j < 2; j++) loff[u][j] = __builtin_amdgcn_readfirstlane((uint32_t)((dst[u] * 2 + j) * 64 * 16));
    auto request = [&](half8 (&buf)[HB], int hs) __attribute__((always_inline)) {
        const size_t o = (size_t)(hs >> 1) * 256 + (hs & 1) * 128;
        const uint32_t base = (uint32_t)(uintptr_t)(lds_void *)buf;
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(src[u] + o + j * 64), "s"(base + loff[u][j]) : "m0");
    };
    constexpr int LOADS = 4 * 2, AHEAD = 4, LANDED = 2;    // copies per request and wave; requests in flight after a request; how many a barrier needs
    constexpr int WAIT = (AHEAD - LANDED) * LOADS;
    static_assert(WAIT == 16 && AHEAD * LOADS < 64, "the hand-written waits count this wave's LDS-direct loads; vmcnt has six bits");
    half8 a0[4], w0[4];                                    // fragments of slice 0 of the half step about to be multiplied
    auto read = [&](half8 (&a)[4], half8 (&w)[4], const half8 (&cur)[HB], int j) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++) a[i] = cur[((4 * wm + i) * 2 + j) * 64 + lane];
#pragma unroll
        for (int k = 0; k < 4; k++) w[k] = cur[((8 + 4 * wn + k) * 2 + j) * 64 + lane];
    };
    auto multiply = [&](const half8 (&a)[4], const half8 (&w)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int k = 0; k < 4; k++) acc[i][k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], w[k], acc[i][k], 0, 0, 0);
    };
    // Half step hs is multiplied out of buffer hs % 5.  The barrier that ends half step hs - 1 has found hs and hs + 1 in
    // LDS (every wave waited for its own copies of them), so slice 0 of hs + 1 is read while slice 1 of hs is multiplied
    // and no half step starts by waiting out an LDS round trip; hs + 4 is requested into the buffer hs - 1 left.
    auto step = [&](int hs, const half8 (&cur)[HB], const half8 (&nxt)[HB], half8 (&free_buf)[HB]) __attribute__((always_inline)) {
        request(free_buf, min(hs + 4, last));
        half8 a1[4], w1[4];
        read(a1, w1, cur, 1);
        multiply(a0, w0);
        read(a0, w0, nxt, 0);
        multiply(a1, w1);
        // issue order: under each MFMA of slice 0 one LDS read of slice 1, under each of slice 1 one of the next slice 0
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
        for (int i = 0; i < 32; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < 6 || (i >= 16 && i < 24)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        // in flight: this wave's copies of hs + 1 .. hs + 4, 8 each (4 pieces x 2 slices); hs + 1 and hs + 2 must have landed
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(WAIT) : "memory");
    };
    request(lb0, 0); request(lb1, min(1, last)); request(lb2, min(2, last)); request(lb3, min(3, last));
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(WAIT) : "memory");   // four requests out: the first two have landed
    read(a0, w0, lb0, 0);
    const int full = nhalf / 5 * 5;
    for (int h0 = 0; h0 < full; h0 += 5) {
        step(h0, lb0, lb1, lb4);
        step(h0 + 1, lb1, lb2, lb0);
        step(h0 + 2, lb2, lb3, lb1);
        step(h0 + 3, lb3, lb4, lb2);
        step(h0 + 4, lb4, lb0, lb3);
    }
    if (full < nhalf) step(full, lb0, lb1, lb4);
    if (full + 1 < nhalf) step(full + 1, lb1, lb2, lb0);
    if (full + 2 < nhalf) step(full + 2, lb2, lb3, lb1);
    if (full + 3 < nhalf) step(full + 3, lb3, lb4, lb2);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    if (mb0 * 32 + 256 <= g.M && (nb0 + 8) * 32 <= g.N) {  // a block inside the matrix: stores without tests, factors first
        float sc[4][16];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                sc[i][v] = g.a_inv_scale ? g.a_inv_scale[(mb0 + 4 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3)] : 1.0f;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = (mb0 + 4 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                float *row = Cp + (size_t)m * g.ldp + (nb0 + 4 * wn) * 32 + r;
#pragma unroll
                for (int k = 0; k < 4; k++) row[k * 32] = acc[i][k][v] * sc[i][v];
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = (mb0 + 4 * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
            if (m >= g.M) continue;
            const float sc = g.a_inv_scale ? g.a_inv_scale[m] : 1.0f;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int n = (nb0 + 4 * wn + k) * 32 + r;
                if (n < g.N) Cp[(size_t)m * g.ldp + n] = acc[i][k][v] * sc;
            }
        }
}

// The 256 x 256 block over Q8_0 weight tiles that stay quantised all the way into LDS: the dequant-fused product for
// many activation rows.  A half step of a weight row block is ONE 1 KB piece (16 int8 per lane: both 8-value slices), its
// 64 fp16 scales another 128 bytes, so a block's half step is 16 KB of activations + 8 KB of weights instead of 32 KB and
// six buffers fit; the copies are LDS-direct loads as in gemm_big_f16_256 (the scales as one dword per lane, lanes 32-63
// fetching the same 128 bytes again into the second half of a 256-byte slot, which keeps every lane active and inside
// the array).  A wave unpacks its fragments on the way from LDS to the MFMA: bytes to exact fp16 integers with
// v_perm_b32, times the scale with packed fp16 multiplies -- the values an F16 image of the dequantised weight holds.
// WF 1: scales per (row, 32 columns), all row blocks of the launch Q8_0 (the caller gives F16 row blocks to another
// launch).  WF 2: the transposed image, scales per (column, 32 rows); K steps from W.kbq on are F16 tiles (the adapter
// rows of the fused QKV weight): at most a step or two at the end of K, multiplied straight from memory after the loop.
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
// BM: rows of the block.  The launcher uses 256 (four waves of 128 x 128); with 128 (four waves of 64 x 128) a wave unpacks
// as many weight fragments for half as many MFMAs, and 192 such blocks took 68 us where the F16 kernel's take 45.
// TAIL (WF 1): the launch has a column block of F16 tiles at its end (only then does the loop carry that case).
template <int WF, int BM, bool TAIL = false>
__global__ __launch_bounds__(256) void gemm_big_q8(GemmKArgs g)
{
    constexpr int AB = BM / 32, MI = BM / 64, AU = BM / 128;  // A row blocks per block; accumulator tile rows and A pieces per wave
    // LDS-direct copies a wave issues per request (2 per A piece; 2 weight pieces + 2 scale pieces, or 4 F16 pieces), requests
    // in flight after a request (six buffers), and how many of them a barrier needs in LDS: the hand-written waits below
    constexpr int Q8_LOADS = 2 * AU + 4, Q8_AHEAD = 5, Q8_LANDED = 2, Q8_WAIT = (Q8_AHEAD - Q8_LANDED) * Q8_LOADS;
    static_assert(Q8_WAIT == (BM == 256 ? 24 : 18) && Q8_AHEAD * Q8_LOADS < 64, "the waits count this wave's LDS-direct loads; vmcnt has six bits");
    constexpr int HB = (2 * AB + 8) * 64;                 // 16-byte units per buffer: A [AB blocks][2 slices][64], Wq [8 blocks][64]
    __shared__ uint4v lb0[HB], lb1[HB], lb2[HB], lb3[HB], lb4[HB], lb5[HB];
    __shared__ half_t scl[6][8][128];                      // scales of the weight row blocks of the half step in buffer i
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int MT = (g.M + BM - 1) / BM, NT = (g.N + 255) >> 8;
    const int m_patches = (MT + 7) >> 3;
    int mt, nt, chunk = 0;
    if (g.S > 1) {
        const int t = blockIdx.x % (MT * NT);
        chunk = blockIdx.x / (MT * NT); mt = t % MT; nt = t / MT;
    } else {
        const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3, patch = seq >> 5, in_patch = seq & 31;
        mt = (patch % m_patches) * 8 + (in_patch & 7);
        nt = ((patch / m_patches) * 4 + (in_patch >> 3)) * 8 + xcd;
        if (mt >= MT || nt >= NT) return;
    }
    const int nb0 = nt * 8, mb0 = mt * AB;
    const int wm = wave >> 1, wn = wave & 1;
    const int k_beg = chunk * g.steps_per_chunk, k_end = min(g.Kb, k_beg + g.steps_per_chunk);
    const int kq_end = WF == 2 ? min(k_end, g.W.kbq) : k_end;              // Q8_0 steps of this chunk: [k_beg, kq_end)
    const int nsteps = kq_end - k_beg, nhalf = 2 * nsteps, last = nhalf - 1;
    const int kstride = WF == 2 ? g.W.kbq : g.Kb;                           // K blocks per row block of the Q8_0 tile arrays
    // A column block from row block W.nbq on holds F16 tiles (WF 1: the adapter rows at the end of the fused QKV weight;
    // W.nbq is a multiple of 8 and at most one row block follows it, the rest of the block lies outside the matrix): its
    // one row block travels as two 1 KB slices per half step in the places of a piece and a scale copy.
    const bool f16_cols = TAIL && WF == 1 && nb0 >= g.W.nbq;
    // this wave's share of a half step: both slices of A row blocks w (, 4 + w); the piece and the scales of W row blocks w, 4 + w
    const uint4v *asrc[AU], *qsrc[2];
    const uint32_t *dsrc[2];
#pragma unroll
    for (int u = 0; u < AU; u++)
        asrc[u] = reinterpret_cast<const uint4v *>(g.A) + ((size_t)min(mb0 + 4 * u + wave, g.Mb - 1) * g.Kb + k_beg) * 256 + a_lane(lane);
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const size_t tile0 = (size_t)min(nb0 + 4 * u + wave, (WF == 1 ? min(g.Nb, g.W.nbq) : g.Nb) - 1) * kstride + k_beg;
        qsrc[u] = reinterpret_cast<const uint4v *>(g.W.q) + tile0 * 128 + lane;
        dsrc[u] = reinterpret_cast<const uint32_t *>(g.W.d + tile0 * 64) + (lane & 31);
    }
    const uint4v *fsrc = f16_cols ? reinterpret_cast<const uint4v *>(g.W.w16) + ((size_t)min(nb0 - g.W.nbq, g.Nb - g.W.nbq - 1) * g.Kb + k_beg) * 256 + lane : nullptr;
    float *const Cp = g.P + (size_t)chunk * g.plane_stride;

    float16v acc[MI][4];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    typedef __attribute__((address_space(3))) void lds_void;
    uint32_t aoff[AU][2], qoff[2], doff[2];                // byte offsets of this wave's pieces inside a buffer / a scale slot
#pragma unroll
    for (int u = 0; u < AU; u++)
#pragma unroll
        for (int j = 0; j < 2; j++) aoff[u][j] = __builtin_amdgcn_readfirstlane((uint32_t)((((4 * u + wave) * 2 + j) * 64) * 16));
#pragma unroll
    for (int u = 0; u < 2; u++) {
        qoff[u] = __builtin_amdgcn_readfirstlane((uint32_t)((2 * AB * 64 + (4 * u + wave) * 64) * 16));
        doff[u] = __builtin_amdgcn_readfirstlane((uint32_t)((4 * u + wave) * 256));
    }
    const uint32_t scl0 = (uint32_t)(uintptr_t)(lds_void *)&scl[0][0][0];
    auto request = [&](uint4v (&buf)[HB], int slot, int hs) __attribute__((always_inline)) {
        const int kt = hs >> 1, jh = hs & 1;
        const uint32_t base = (uint32_t)(uintptr_t)(lds_void *)buf, sbase = scl0 + (uint32_t)slot * (8 * 256);
#pragma unroll
        for (int u = 0; u < AU; u++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(asrc[u] + (size_t)kt * 256 + (2 * jh + j) * 64), "s"(base + aoff[u][j]) : "m0");
        if (f16_cols) {                                    // the same four copies: slice j of the F16 row block into W place w (j = 0) / 4 + w (j = 1)
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(fsrc + (size_t)kt * 256 + (2 * jh + j) * 64), "s"(base + qoff[j]) : "m0");
        } else {
#pragma unroll
            for (int u = 0; u < 2; u++) {
                asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(qsrc[u] + (size_t)kt * 128 + jh * 64), "s"(base + qoff[u]) : "m0");
                asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off" :: "v"(dsrc[u] + (size_t)kt * 32), "s"(sbase + doff[u]) : "m0");
            }
        }
    };
    half8 a0[MI], w0[4];                                   // fragments of slice 0 of the half step about to be multiplied
    // slice j (0 / 1) of the half step in `cur` / scale slot `slot`: A as it lies, W unpacked
    auto read = [&](half8 (&a)[MI], half8 (&w)[4], const uint4v (&cur)[HB], int slot, int jh, int j) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < MI; i++) a[i] = __builtin_bit_cast(half8, cur[((MI * wm + i) * 2 + j) * 64 + lane]);
        if (f16_cols) {                                    // (wave 0's copies; every fragment of the block is that one row block)
#pragma unroll
            for (int k = 0; k < 4; k++) w[k] = __builtin_bit_cast(half8, cur[2 * AB * 64 + (j ? 4 : 0) * 64 + lane]);
            return;
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int blk = 4 * wn + k;
            const uint2v q = reinterpret_cast<const uint2v *>(&cur[2 * AB * 64 + blk * 64 + lane])[j];
            half8 sc;
            if (WF == 1) sc = bcast8(scl[slot][blk][lane]);
            else sc = reinterpret_cast<const half8 *>(&scl[slot][blk][0])[h * 4 + 2 * jh + j];
            w[k] = q8_unpack8(q[0], q[1]) * sc;
        }
    };
    auto multiply = [&](const half8 (&a)[MI], const half8 (&w)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int k = 0; k < 4; k++) acc[i][k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], w[k], acc[i][k], 0, 0, 0);
    };
    // Half step hs is multiplied out of buffer hs % 6 (see gemm_big_f16_256): the barrier that ends half step hs - 1 has
    // found hs and hs + 1 in LDS, slice 0 of hs + 1 is read and unpacked while slice 1 of hs is multiplied, hs + 5 is
    // requested into the buffer hs - 1 left.  Eight copies per wave and half step.
    auto step = [&](int hs, const uint4v (&cur)[HB], int slot, const uint4v (&nxt)[HB], int nslot, uint4v (&free_buf)[HB], int fslot)
        __attribute__((always_inline)) {
        request(free_buf, fslot, min(hs + 5, last));
        half8 a1[MI], w1[4];
        read(a1, w1, cur, slot, hs & 1, 1);
        multiply(a0, w0);
        read(a0, w0, nxt, nslot, (hs + 1) & 1, 0);
        multiply(a1, w1);
        // in flight: this wave's copies of hs + 1 .. hs + 5, Q8_LOADS each; hs + 1 and hs + 2 must have landed
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(Q8_WAIT) : "memory");
    };
    if (nhalf > 0) {
        request(lb0, 0, 0); request(lb1, 1, min(1, last)); request(lb2, 2, min(2, last)); request(lb3, 3, min(3, last));
        request(lb4, 4, min(4, last));
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(Q8_WAIT) : "memory");   // five requests out: the first two have landed
        read(a0, w0, lb0, 0, 0, 0);
        const int full = nhalf / 6 * 6;
        for (int h0 = 0; h0 < full; h0 += 6) {
            step(h0, lb0, 0, lb1, 1, lb5, 5);
            step(h0 + 1, lb1, 1, lb2, 2, lb0, 0);
            step(h0 + 2, lb2, 2, lb3, 3, lb1, 1);
            step(h0 + 3, lb3, 3, lb4, 4, lb2, 2);
            step(h0 + 4, lb4, 4, lb5, 5, lb3, 3);
            step(h0 + 5, lb5, 5, lb0, 0, lb4, 4);
        }
        if (full < nhalf) step(full, lb0, 0, lb1, 1, lb5, 5);
        if (full + 1 < nhalf) step(full + 1, lb1, 1, lb2, 2, lb0, 0);
        if (full + 2 < nhalf) step(full + 2, lb2, 2, lb3, 3, lb1, 1);
        if (full + 3 < nhalf) step(full + 3, lb3, 3, lb4, 4, lb2, 2);
        if (full + 4 < nhalf) step(full + 4, lb4, 4, lb5, 5, lb3, 3);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    if (WF == 2) {
        // the F16 K steps at the end of this chunk (adapter rows): operands straight from memory
        for (int kt = max(kq_end, k_beg); kt < k_end; kt++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                half8 a[MI], w[4];
#pragma unroll
                for (int i = 0; i < MI; i++) a[i] = g.A[((size_t)min(mb0 + MI * wm + i, g.Mb - 1) * g.Kb + kt) * 256 + j * 64 + a_lane(lane)];
#pragma unroll
                for (int k = 0; k < 4; k++)
                    w[k] = reinterpret_cast<const half8 *>(g.W.w16)[((size_t)min(nb0 + 4 * wn + k, g.Nb - 1) * (g.Kb - g.W.kbq) + kt - g.W.kbq) * 256 + j * 64 + lane];
                multiply(a, w);
            }
        }
    }

    if (mb0 * 32 + BM <= g.M && (nb0 + 8) * 32 <= g.N) {   // a block inside the matrix: stores without tests, factors first
        float sc[MI][16];
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                sc[i][v] = g.a_inv_scale ? g.a_inv_scale[(mb0 + MI * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3)] : 1.0f;
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = (mb0 + MI * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                float *row = Cp + (size_t)m * g.ldp + (nb0 + 4 * wn) * 32 + r;
#pragma unroll
                for (int k = 0; k < 4; k++) row[k * 32] = acc[i][k][v] * sc[i][v];
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = (mb0 + MI * wm + i) * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
            if (m >= g.M) continue;
            const float sc = g.a_inv_scale ? g.a_inv_scale[m] : 1.0f;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int n = (nb0 + 4 * wn + k) * 32 + r;
                if (n < g.N) Cp[(size_t)m * g.ldp + n] = acc[i][k][v] * sc;
            }
        }
}

}  // namespace

// How many K chunks the large-M kernel should cut a product with F16 tiles into: three when its 128 x 256 output blocks
// would leave a third of the CUs or more without work and K is at least 4096, else one.  Measured on MI355X at 2048
// rows: the products with 2560 output columns (160 blocks for 256 CUs) go from 66 / 140 / 281 / 93 us to 54 / 103 /
// 199 / 73 us (K = 4096 / 9728 / 19456 / 6176) with three chunks dealt evenly to the XCDs; two chunks change nothing
// (320 blocks are two rounds again) and every product with K = 2560 loses (13 K steps per workgroup).
int big_gemm_chunks(int M, int N, int K, int fmt)
{
    if (fmt != 0 || g_big_split == 0) return 1;
    if (g_big_split > 1) return g_big_split;
    const long blocks = (long)((M + 127) / 128) * ((N + 128 * WPW - 1) / (128 * WPW));
    const int cus = num_cus() > 0 ? num_cus() : 256;
    // a handful of blocks over a very long K (the LM head's backward at a few hundred rows: 25 blocks, K = 262 144): as
    // many chunks as it takes to give every CU a block, each still thousands of columns long (640 rows: 930 us on the
    // streaming kernel, 3 680 / 1 340 / 840 / 640 us with 1 / 3 / 5 / 8-10 chunks)
    if (blocks * 8 <= cus && K >= 65536) return (int)std::min<long>(std::min<long>(cus / blocks, K / 8192), 16);
    return (blocks * 3 <= cus * 2 && K >= 4096) ? 3 : 1;
}

// Whether a Q8_0 operand can run on gemm_big_q8: the row blocks of a row-scaled operand all quantised, or one F16 row
// block (the adapter rows of the fused QKV weight) that begins a column block of its own; at most two F16 K steps at the
// end of a column-scaled one.
bool q8_wide_ok(const WeightOp &W, int N, int K)
{
    if (g_big_block == 1) return false;
    if (W.fmt == 1) return W.nbq >= tiled_rb(N) || (W.nbq % 8 == 0 && tiled_rb(N) - W.nbq == 1 && W.w16);
    if (W.fmt == 2) return W.kbq >= 1 && tiled_kb(K) - W.kbq <= 2;
    return false;
}

// K chunks for any operand: big_gemm_chunks for F16 tiles; for Q8_0 tiles on the 256 x 256 block, two or three chunks
// where they fill at least half as many CUs again as one does (each chunk 20 K steps or more), else one.
int big_gemm_chunks_for(int M, int N, int K, const WeightOp &W)
{
    if (W.fmt == 0) return big_gemm_chunks(M, N, K, 0);
    if (g_big_split == 0 || !q8_wide_ok(W, N, K)) return 1;
    if (g_big_split > 1) return g_big_split;
    const int cus = num_cus() > 0 ? num_cus() : 256;
    const long blocks = (long)((M + 255) / 256) * ((N + 255) / 256);
    auto share = [&](int c) { return (double)(blocks * c) / (double)((blocks * c + cus - 1) / cus * cus); };
    int best = 1;
    for (int c = 2; c <= 3; c++)
        if (tiled_kb(K) / c >= 20 && share(c) >= 1.5 * share(1) && share(c) > share(best)) best = c;
    return best;
}

int launch_gemm_big(const half_t *A, const float *a_inv_scale, const WeightOp &W, float *C, int ldc, int M, int N, int K,
                    int chunks, size_t plane_stride)
{
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const int Kb = tiled_kb(K), Nb = tiled_rb(N), Mb = tiled_rb(M);
    bool ok = ldc >= N && W.fmt >= 0 && W.fmt <= 2;
    if (W.fmt == 0) ok = ok && W.w16;
    if (W.fmt == 1) ok = ok && W.q && W.d && W.nbq >= 0 && W.nbq <= Nb && (W.nbq == Nb || W.w16);
    if (W.fmt == 2) ok = ok && W.q && W.d && W.kbq >= 0 && W.kbq <= Kb && (W.kbq == Kb || W.w16);
    if (!ok) { fprintf(stderr, "[fast_hip] gemm_big: bad launch M=%d N=%d K=%d ldc=%d fmt=%d\n", M, N, K, ldc, W.fmt); abort(); }
    GemmKArgs g{};
    g.A = reinterpret_cast<const half8 *>(A); g.a_inv_scale = a_inv_scale; g.W = W;
    const bool q8_wide = W.fmt != 0 && q8_wide_ok(W, N, K);
    if (chunks < 1 || (chunks > 1 && W.fmt != 0 && !q8_wide)) { fprintf(stderr, "[fast_hip] gemm_big: K chunks need F16 tiles or the 256 x 256 Q8_0 kernel\n"); abort(); }
    g.P = C; g.ldp = ldc; g.plane_stride = plane_stride;
    g.M = M; g.N = N; g.Mb = Mb; g.Nb = Nb; g.Kb = Kb;
    g.steps_per_chunk = (Kb + chunks - 1) / chunks;
    g.S = (Kb + g.steps_per_chunk - 1) / g.steps_per_chunk;
    const dim3 block(256);
    hipEvent_t ev_a = nullptr, ev_b = nullptr;
    const bool prof = gemm_prof_begin(weight_stream_bytes(W, N, K), 2.0 * M * N * K, &ev_a, &ev_b);
    // grid of either block shape: with K chunks one workgroup per (chunk, block); else whole patches of 8 x 32 ids (see
    // the kernels), the ids past the matrix returning at once
    auto grid_of = [&](const GemmKArgs &a, int bm, int bn) {
        const int mt = (a.M + bm - 1) / bm, nt = (a.N + bn - 1) / bn;
        return dim3(a.S > 1 ? mt * nt * a.S : 8 * 32 * ((mt + 7) / 8) * (((nt + 7) / 8 + 3) / 4));
    };
    if (W.fmt == 0 || q8_wide) {
        // 128 x 256 or 256 x 256 blocks, whichever keeps more of the GPU on useful work -- the share of the last round's
        // CUs that have a block times the share of the tiles' area that lies inside the matrix.  The wide block is faster
        // in its loop and wins from 0.9 of the other's share, given 20 K steps per block to win them in (below, its larger
        // prologue and epilogue take the gain back).  Measured at 2048 rows inside the step: 200 and 240 wide blocks win
        // against 400 and 480, 4752 against 9504; 608, 304 and 128 lose against 1216, 608 and 256.
        const int cus = num_cus() > 0 ? num_cus() : 256;
        auto share = [&](int bm, int bn) {
            const long tm = (M + bm - 1) / bm, tn = (N + bn - 1) / bn, blocks = tm * tn * g.S;
            return (double)M * N / ((double)tm * bm * tn * bn) * (double)blocks / (double)((blocks + cus - 1) / cus * cus);
        };
        const bool deep = g.steps_per_chunk >= 20;
        // (Q8_0 tiles: the wide block only, see gemm_big_q8)
        const bool wide = W.fmt != 0 || g_big_block == 2 || (g_big_block == 0 && deep && share(256, 256) >= 0.9 * share(128, 128 * WPW));
        // A product of at least one full round of wide blocks whose last round would be half empty or less: the columns
        // of the full rounds go to wide blocks, the rest to 128 x 256 blocks in a launch of their own
        const int MX = (M + 255) / 256, NX = (N + 255) / 256, full = MX * NX / cus, rest = MX * NX % cus;
        const int wide_cols = full * cus / MX * 256;
        auto launch = [&](const GemmKArgs &a, bool w, hipEvent_t e0, hipEvent_t e1) {
            const dim3 grid = w ? grid_of(a, 256, 256) : grid_of(a, 128, 128 * WPW);
#define BIG_LAUNCH(KERNEL) do { if (prof) hipExtLaunchKernelGGL((KERNEL), grid, block, 0, stream(), e0, e1, 0, a); \
                                else hipLaunchKernelGGL((KERNEL), grid, block, 0, stream(), a); } while (0)
            if (W.fmt == 0) { if (w) BIG_LAUNCH(gemm_big_f16_256); else BIG_LAUNCH(gemm_big_f16); }
            else if (W.fmt == 1) { if (a.W.nbq < a.Nb) BIG_LAUNCH((gemm_big_q8<1, 256, true>)); else BIG_LAUNCH((gemm_big_q8<1, 256>)); }
            else BIG_LAUNCH((gemm_big_q8<2, 256>));
#undef BIG_LAUNCH
        };
        if (g_big_block == 0 && !wide && deep && g.S == 1 && full >= 1 && rest > 0 && rest * 2 <= cus && wide_cols < N) {
            GemmKArgs g1 = g, g2 = g;
            const int rb = wide_cols / 32;                 // weight row blocks that go to the wide launch
            g1.N = wide_cols; g1.Nb = rb;
            g2.N = N - wide_cols; g2.Nb = tiled_rb(g2.N);
            g2.P = C + wide_cols;
            g2.W.w16 = W.w16 + (size_t)rb * Kb * 2048;    // (F16 tiles: Q8_0 products are all wide)
            launch(g1, true, ev_a, nullptr);
            launch(g2, false, nullptr, ev_b);
        } else launch(g, wide, ev_a, ev_b);
        HIP_CHECK(hipGetLastError());
        return g.S;
    }
    const dim3 grid = grid_of(g, 128, 128 * WPW);
    const size_t lds = (size_t)2 * (4 + 4 * WPW) * 256 * sizeof(half8);
    static bool attr_set = false;
    if (!attr_set) {
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_big<1>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_big<2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    if (prof) {
        if (W.fmt == 1) hipExtLaunchKernelGGL(gemm_big<1>, grid, block, lds, stream(), ev_a, ev_b, 0, g);
        else hipExtLaunchKernelGGL(gemm_big<2>, grid, block, lds, stream(), ev_a, ev_b, 0, g);
    } else {
        if (W.fmt == 1) hipLaunchKernelGGL(gemm_big<1>, grid, block, lds, stream(), g);
        else hipLaunchKernelGGL(gemm_big<2>, grid, block, lds, stream(), g);
    }
    HIP_CHECK(hipGetLastError());
    return 1;
}

void set_big_gemm_split(int mode) { g_big_split = mode; }
void set_big_gemm_block(int mode) { g_big_block = mode; }

}  // namespace lmhip
