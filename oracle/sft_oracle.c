/*
 * sft_oracle.c — CPU restatement of llm.metal's fused LoRA SFT step.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product path may link, load or
 * call this file: it exists so that tests, the smoke check and the benchmark's
 * CPU-baseline leg have something independent of the HIP code to compare with.
 *
 * Built twice from this one source: -DREAL=float (the arithmetic the reference
 * uses for activations, gradients and LoRA tensors) and -DREAL=double (used to
 * pin the float build and for finite-difference checks).  Frozen weights and
 * norm gammas are always passed as float arrays holding the values "as used"
 * (already rounded through F16 or quantised/dequantised through Q8_0).
 *
 * Every op states the reference location whose arithmetic it restates
 * (paths relative to the reference tree).  Single-threaded, naive loops.
 *
 * Pinning status of each function is recorded in tests/test_oracle_*.py; the
 * reference ships no golden vectors for this path, so the pins are closed
 * forms, library routines (numpy float16 casts, torch fp64 autograd / AdamW),
 * hand-derived known answers and finite differences.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef REAL
#define REAL float
#endif
typedef REAL real;

#define OR_API __attribute__((visibility("default")))

/* type-generic libm wrappers so the float build really computes in float */
#define R_EXP(x)  _Generic((x), float: expf,  double: exp)(x)
#define R_LOG(x)  _Generic((x), float: logf,  double: log)(x)
#define R_TANH(x) _Generic((x), float: tanhf, double: tanh)(x)
#define R_SQRT(x) _Generic((x), float: sqrtf, double: sqrt)(x)
#define R_POW(x,y) _Generic((x), float: powf, double: pow)(x, y)
#define R_COS(x)  _Generic((x), float: cosf,  double: cos)(x)
#define R_SIN(x)  _Generic((x), float: sinf,  double: sin)(x)

OR_API int or_real_bytes(void) { return (int)sizeof(real); }

/* ------------------------------------------------------------------ */
/* F16 conversion and Q8_0 — src/nn/wmat.c:19-75                       */
/* ------------------------------------------------------------------ */

/* fp32 -> fp16 bits, round to nearest even, the conversion `(__fp16)x`
 * performs in wmat_create_f16 (src/nn/wmat.c:63-75) and for the Q8_0 scale
 * (src/nn/wmat.c:31-32).  Written on the bit pattern so any C compiler
 * builds it. */
OR_API uint16_t or_f32_to_f16_bits(float f)
{
    uint32_t x; memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) {                 /* inf / nan */
        uint32_t mant = absx & 0x007fffffu;
        return (uint16_t)(sign | 0x7c00u | (mant ? (0x0200u | (mant >> 13)) : 0));
    }
    if (absx >= 0x477ff000u)                   /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (absx < 0x38800000u) {                  /* below the smallest normal half: subnormal or zero */
        if (absx < 0x33000000u) return (uint16_t)sign;      /* < 2^-25 -> 0 */
        int e = (int)(absx >> 23);                          /* biased exponent, 102..112 */
        uint32_t mant = (absx & 0x007fffffu) | 0x00800000u; /* 24-bit significand */
        int shift = 126 - e;                                /* 14..24: target unit is 2^-24 */
        uint32_t q = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t e = (absx >> 23) - 112u;          /* rebias 127 -> 15 */
    uint32_t mant = absx & 0x007fffffu;
    uint32_t h = (e << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;  /* carry may bump the exponent: correct */
    return (uint16_t)(sign | h);
}

OR_API float or_f16_bits_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu, x;
    if (e == 0) {
        if (m == 0) x = sign;
        else {                                   /* subnormal: normalise */
            int s = 0;
            while (!(m & 0x400u)) { m <<= 1; s++; }
            m &= 0x3ffu;
            x = sign | ((uint32_t)(113 - s) << 23) | (m << 13);
        }
    } else if (e == 31) x = sign | 0x7f800000u | (m << 13);
    else x = sign | ((e + 112u) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4);
    return f;
}

OR_API void or_f32_to_f16_array(const float *src, uint16_t *dst, size_t n)
{
    for (size_t i = 0; i < n; i++) dst[i] = or_f32_to_f16_bits(src[i]);
}

OR_API void or_f16_to_f32_array(const uint16_t *src, float *dst, size_t n)
{
    for (size_t i = 0; i < n; i++) dst[i] = or_f16_bits_to_f32(src[i]);
}

/* One Q8_0 block is 34 bytes: fp16 scale bits (little endian) then 32 int8.
 * quantize_row_q8, src/nn/wmat.c:19-44: amax over the block, scale = amax/127
 * in fp32, stored scale = fp16(scale); the quantiser divides by the UN-rounded
 * fp32 scale (inv = 1.0f/scale), q = clamp((int)roundf(x*inv), -128, 127);
 * an all-zero block stores zeros.  roundf rounds halves away from zero. */
OR_API void or_q8_quantize(const float *src, uint8_t *dst, int rows, int cols)
{
    int nb = cols / 32;                         /* truncating, as wmat_create_q8 does (src/nn/wmat.c:53) */
    for (int r = 0; r < rows; r++) {
        for (int b = 0; b < nb; b++) {
            const float *sp = src + (size_t)r * cols + (size_t)b * 32;
            uint8_t *blk = dst + ((size_t)r * nb + b) * 34;
            float amax = 0.0f;
            for (int j = 0; j < 32; j++) {
                float a = fabsf(sp[j]);
                if (a > amax) amax = a;
            }
            float scale = amax / 127.0f;
            uint16_t d = or_f32_to_f16_bits(scale);
            blk[0] = (uint8_t)(d & 0xff); blk[1] = (uint8_t)(d >> 8);
            if (scale != 0.0f) {
                float inv = 1.0f / scale;
                for (int j = 0; j < 32; j++) {
                    int v = (int)roundf(sp[j] * inv);
                    if (v < -128) v = -128;
                    if (v > 127) v = 127;
                    blk[2 + j] = (uint8_t)(int8_t)v;
                }
            } else {
                memset(blk + 2, 0, 32);
            }
        }
    }
}

/* Dequantise: value = float(fp16 scale) * q, computed in fp32
 * (src/data/gguf.c:225-253 and the q8_matvec kernel,
 * shaders/q8_kernels.metal:10-47, which multiplies float(d) by the int8). */
OR_API void or_q8_dequant(const uint8_t *src, float *dst, int rows, int cols)
{
    int nb = cols / 32;
    for (int r = 0; r < rows; r++)
        for (int b = 0; b < nb; b++) {
            const uint8_t *blk = src + ((size_t)r * nb + b) * 34;
            float d = or_f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
            for (int j = 0; j < 32; j++)
                dst[(size_t)r * cols + (size_t)b * 32 + j] = d * (float)(int8_t)blk[2 + j];
        }
}

/* ------------------------------------------------------------------ */
/* Matrix products                                                     */
/* ------------------------------------------------------------------ */

/* f16_matmul, shaders/q8_kernels.metal:383-407: C[M,N] = A[M,K] * W[N,K]^T,
 * W holds F16 values (here already widened to float), accumulation in `real`. */
OR_API void or_wmatmul(const real *A, const float *W, real *C, int M, int N, int K)
{
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            const real *a = A + (size_t)m * K;
            const float *w = W + (size_t)n * K;
            real s = 0;
            for (int k = 0; k < K; k++) s += a[k] * (real)w[k];
            C[(size_t)m * N + n] = s;
        }
}

/* f16_matmul_nt, shaders/q8_kernels.metal:411-435: C[M,K] = A[M,N] * W[N,K]. */
OR_API void or_wmatmul_nt(const real *A, const float *W, real *C, int M, int N, int K)
{
    for (int m = 0; m < M; m++) {
        real *c = C + (size_t)m * K;
        for (int k = 0; k < K; k++) c[k] = 0;
        for (int n = 0; n < N; n++) {
            real a = A[(size_t)m * N + n];
            const float *w = W + (size_t)n * K;
            for (int k = 0; k < K; k++) c[k] += a * (real)w[k];
        }
    }
}

/* float_matmul, shaders/q8_kernels.metal:1043-1067: C[M,N] = A[M,K] * W[N,K]^T. */
OR_API void or_matmul(const real *A, const real *W, real *C, int M, int N, int K)
{
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            real s = 0;
            for (int k = 0; k < K; k++) s += A[(size_t)m * K + k] * W[(size_t)n * K + k];
            C[(size_t)m * N + n] = s;
        }
}

/* float_matmul_tn, shaders/q8_kernels.metal:1070-1094: C[M,N] = A[K,M]^T * B[K,N]. */
OR_API void or_matmul_tn(const real *A, const real *B, real *C, int M, int N, int K)
{
    for (size_t i = 0; i < (size_t)M * N; i++) C[i] = 0;
    for (int k = 0; k < K; k++)
        for (int m = 0; m < M; m++) {
            real a = A[(size_t)k * M + m];
            for (int n = 0; n < N; n++) C[(size_t)m * N + n] += a * B[(size_t)k * N + n];
        }
}

/* float_matmul_nt, shaders/q8_kernels.metal:1128-1152: C[M,K] = A[M,N] * W[N,K]. */
OR_API void or_matmul_nt(const real *A, const real *W, real *C, int M, int N, int K)
{
    for (int m = 0; m < M; m++) {
        real *c = C + (size_t)m * K;
        for (int k = 0; k < K; k++) c[k] = 0;
        for (int n = 0; n < N; n++) {
            real a = A[(size_t)m * N + n];
            for (int k = 0; k < K; k++) c[k] += a * W[(size_t)n * K + k];
        }
    }
}

/* ------------------------------------------------------------------ */
/* Row ops                                                             */
/* ------------------------------------------------------------------ */

/* rms_norm, shaders/q8_kernels.metal:133-158: out = x * rsqrt(mean(x^2)+eps) * gamma.
 * In place (out == x) is relied upon by src/nn/fast_sft.c:668-669. */
OR_API void or_rms_norm(const real *x, const float *gamma, real *out, int dim, float eps, int B)
{
    for (int b = 0; b < B; b++) {
        const real *xr = x + (size_t)b * dim;
        real *o = out + (size_t)b * dim;
        real ss = 0;
        for (int i = 0; i < dim; i++) ss += xr[i] * xr[i];
        real inv = (real)1 / R_SQRT(ss / (real)dim + (real)eps);
        for (int i = 0; i < dim; i++) o[i] = xr[i] * inv * (real)gamma[i];
    }
}

/* rms_norm_train_backward, shaders/q8_kernels.metal:584-625:
 * r = rsqrt(mean(x^2)+eps); c = sum(dy*gamma*x) * r^2 / dim;
 * dx = (gamma*dy - c*x) * r.  No gamma gradient.  dx may alias dy
 * (src/nn/fast_sft.c:914-917). */
OR_API void or_rms_norm_backward(const real *x, const real *dy, const float *gamma, real *dx,
                                 int batch, int dim, float eps)
{
    for (int b = 0; b < batch; b++) {
        const real *xr = x + (size_t)b * dim, *dyr = dy + (size_t)b * dim;
        real *dxr = dx + (size_t)b * dim;
        real ss = 0, dot = 0;
        for (int i = 0; i < dim; i++) ss += xr[i] * xr[i];
        real inv = (real)1 / R_SQRT(ss / (real)dim + (real)eps);
        for (int i = 0; i < dim; i++) dot += dyr[i] * (real)gamma[i] * xr[i];
        real coeff = dot * inv * inv / (real)dim;
        for (int i = 0; i < dim; i++)
            dxr[i] = ((real)gamma[i] * dyr[i] - coeff * xr[i]) * inv;
    }
}

/* transpose_heads_fwd / _rev, shaders/q8_kernels.metal:438-474:
 * [N, H*D] <-> [H, N, D]. */
OR_API void or_transpose_heads_fwd(const real *src, real *dst, int N, int H, int D)
{
    for (int n = 0; n < N; n++)
        for (int h = 0; h < H; h++)
            memcpy(dst + ((size_t)h * N + n) * D, src + ((size_t)n * H + h) * D, sizeof(real) * D);
}

OR_API void or_transpose_heads_rev(const real *src, real *dst, int N, int H, int D)
{
    for (int n = 0; n < N; n++)
        for (int h = 0; h < H; h++)
            memcpy(dst + ((size_t)n * H + h) * D, src + ((size_t)h * N + n) * D, sizeof(real) * D);
}

/* repeat_kv, shaders/q8_kernels.metal:476-492: q-head hq reads kv-head hq / ratio. */
OR_API void or_repeat_kv(const real *src, real *dst, int n_kv, int N, int D, int ratio)
{
    size_t ND = (size_t)N * D;
    for (int hq = 0; hq < n_kv * ratio; hq++)
        memcpy(dst + hq * ND, src + (size_t)(hq / ratio) * ND, sizeof(real) * ND);
}

/* repeat_kv_bwd, shaders/q8_kernels.metal:973-992: sum the `ratio` copies. */
OR_API void or_repeat_kv_bwd(const real *dexp, real *dkv, int n_kv, int N, int D, int ratio)
{
    size_t ND = (size_t)N * D;
    for (int h = 0; h < n_kv; h++)
        for (size_t r = 0; r < ND; r++) {
            real s = 0;
            for (int g = 0; g < ratio; g++) s += dexp[((size_t)h * ratio + g) * ND + r];
            dkv[(size_t)h * ND + r] = s;
        }
}

/* rope_train / rope_train_bwd, shaders/q8_kernels.metal:495-538, 997-1038:
 * half-split pairs (d, d + hd/2), freq = 1 / theta^(2d/hd), angle = pos*freq;
 * forward rotates by +angle, backward by -angle.  Buffer is [H, N, hd], pos is
 * the index along N. */
static void rope_heads(real *buf, int H, int N, int hd, float theta, int inverse)
{
    int half = hd / 2;
    for (int h = 0; h < H; h++)
        for (int pos = 0; pos < N; pos++) {
            real *vec = buf + ((size_t)h * N + pos) * hd;
            for (int d = 0; d < half; d++) {
                real freq = (real)1 / R_POW((real)theta, (real)(2 * d) / (real)hd);
                real ang = (real)pos * freq;
                real c = R_COS(ang), s = R_SIN(ang);
                if (inverse) s = -s;
                real x0 = vec[d], x1 = vec[d + half];
                vec[d]        = x0 * c - x1 * s;
                vec[d + half] = x0 * s + x1 * c;
            }
        }
}

OR_API void or_rope_train(real *q, real *k, int Hq, int Hkv, int hd, int N, float theta)
{
    rope_heads(q, Hq, N, hd, theta, 0);
    rope_heads(k, Hkv, N, hd, theta, 0);
}

OR_API void or_rope_train_bwd(real *q, real *k, int Hq, int Hkv, int hd, int N, float theta)
{
    rope_heads(q, Hq, N, hd, theta, 1);
    rope_heads(k, Hkv, N, hd, theta, 1);
}

/* attn_train_fwd, shaders/q8_kernels.metal:769-851: per (head, query i):
 * s_j = q_i.k_j * scale for j <= i, softmax over j <= i, probs row saved
 * (zeros for j > i), out_i = sum_j p_j v_j.  The row reduction is the exact
 * sum (the reference's tree reduction leaves lanes out when the group size is
 * not a power of two; for power-of-two sizes both give the same sum up to
 * fp32 rounding order). */
OR_API void or_attn_train_fwd_window(const real *Q, const real *K, const real *V, real *out, real *probs,
                                     int H, int N, int D, float scale, int window);

OR_API void or_attn_train_fwd(const real *Q, const real *K, const real *V, real *out, real *probs,
                              int H, int N, int D, float scale)
{
    or_attn_train_fwd_window(Q, K, V, out, probs, H, N, D, scale, 0);
}

/* The same with a sliding window: query i sees keys max(0, i - window + 1) .. i; window <= 0: every key up to i, which
 * is all the reference's kernel does (it has no window argument; Gemma3's sliding_window is stored by
 * src/nn/gemma3.c:20,99 and never read).  The saved probabilities are zero outside the window, so the backward
 * kernels, which weigh every key by them, need no window of their own. */
OR_API void or_attn_train_fwd_window(const real *Q, const real *K, const real *V, real *out, real *probs,
                                     int H, int N, int D, float scale, int window)
{
    real *s = (real *)malloc(sizeof(real) * N);
    for (int h = 0; h < H; h++)
        for (int i = 0; i < N; i++) {
            const real *q = Q + ((size_t)h * N + i) * D;
            real mx = (real)-1e30;
            const int lo = (window > 0 && i >= window) ? i - window + 1 : 0;
            for (int j = lo; j <= i; j++) {
                const real *k = K + ((size_t)h * N + j) * D;
                real dot = 0;
                for (int d = 0; d < D; d++) dot += q[d] * k[d];
                s[j] = dot * (real)scale;
                if (s[j] > mx) mx = s[j];
            }
            real sum = 0;
            for (int j = lo; j <= i; j++) { s[j] = R_EXP(s[j] - mx); sum += s[j]; }
            real inv = (real)1 / sum;
            real *pr = probs + ((size_t)h * N + i) * N;
            for (int j = 0; j < N; j++) pr[j] = (j >= lo && j <= i) ? s[j] * inv : (real)0;
            real *o = out + ((size_t)h * N + i) * D;
            for (int d = 0; d < D; d++) o[d] = 0;
            for (int j = lo; j <= i; j++) {
                const real *v = V + ((size_t)h * N + j) * D;
                for (int d = 0; d < D; d++) o[d] += pr[j] * v[d];
            }
        }
    free(s);
}

/* attn_bwd_dq, shaders/q8_kernels.metal:857-925: d_raw_j = dO_i.v_j,
 * ds_j = p_j (d_raw_j - sum_k p_k d_raw_k) scale, dQ_i = sum_j ds_j k_j. */
OR_API void or_attn_bwd_dq(const real *dO, const real *probs, const real *V, const real *K,
                           real *dscore, real *dQ, int H, int N, int D, float scale)
{
    real *dr = (real *)malloc(sizeof(real) * N);
    for (int h = 0; h < H; h++)
        for (int i = 0; i < N; i++) {
            const real *dout = dO + ((size_t)h * N + i) * D;
            const real *pr = probs + ((size_t)h * N + i) * N;
            real dp = 0;
            for (int j = 0; j <= i; j++) {
                const real *v = V + ((size_t)h * N + j) * D;
                real dot = 0;
                for (int d = 0; d < D; d++) dot += dout[d] * v[d];
                dr[j] = dot;
                dp += pr[j] * dot;
            }
            real *ds = dscore + ((size_t)h * N + i) * N;
            for (int j = 0; j < N; j++)
                ds[j] = (j <= i) ? pr[j] * (dr[j] - dp) * (real)scale : (real)0;
            real *dq = dQ + ((size_t)h * N + i) * D;
            for (int d = 0; d < D; d++) dq[d] = 0;
            for (int j = 0; j <= i; j++) {
                const real *k = K + ((size_t)h * N + j) * D;
                for (int d = 0; d < D; d++) dq[d] += ds[j] * k[d];
            }
        }
    free(dr);
}

/* attn_bwd_dkv, shaders/q8_kernels.metal:931-968: dK_j = sum_{i>=j} ds_ij q_i,
 * dV_j = sum_{i>=j} p_ij dO_i. */
OR_API void or_attn_bwd_dkv(const real *dscore, const real *Q, const real *probs, const real *dO,
                            real *dK, real *dV, int H, int N, int D)
{
    for (int h = 0; h < H; h++)
        for (int j = 0; j < N; j++) {
            real *dk = dK + ((size_t)h * N + j) * D, *dv = dV + ((size_t)h * N + j) * D;
            for (int d = 0; d < D; d++) { dk[d] = 0; dv[d] = 0; }
            for (int i = j; i < N; i++) {
                real ds = dscore[((size_t)h * N + i) * N + j];
                real p = probs[((size_t)h * N + i) * N + j];
                const real *q = Q + ((size_t)h * N + i) * D;
                const real *dout = dO + ((size_t)h * N + i) * D;
                for (int d = 0; d < D; d++) { dk[d] += ds * q[d]; dv[d] += p * dout[d]; }
            }
        }
}

/* ------------------------------------------------------------------ */
/* Elementwise                                                         */
/* ------------------------------------------------------------------ */

static inline real gelu_inner(real g)
{
    real in = (real)0.7978845608 * (g + (real)0.044715 * g * g * g);
    if (in > 15) in = 15;
    if (in < -15) in = -15;
    return in;
}

/* silu_mul, shaders/q8_kernels.metal:337-344: gate = gate/(1+exp(-gate)) * up. */
OR_API void or_silu_mul(real *gate, const real *up, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        real g = gate[i];
        gate[i] = (g / ((real)1 + R_EXP(-g))) * up[i];
    }
}

/* gelu_mul, shaders/q8_kernels.metal:351-362: tanh-approximate GELU, tanh
 * argument clamped to +-15. */
OR_API void or_gelu_mul(real *gate, const real *up, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        real g = gate[i];
        gate[i] = (real)0.5 * g * ((real)1 + R_TANH(gelu_inner(g))) * up[i];
    }
}

/* silu_mul_backward, shaders/q8_kernels.metal:540-556.  dgate may alias dout
 * (src/nn/fast_sft.c:850-851): each index is read before it is written. */
OR_API void or_silu_mul_backward(const real *dout, const real *gate, const real *up,
                                 real *dgate, real *dup, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        real g = gate[i], u = up[i], dy = dout[i];
        real sig = (real)1 / ((real)1 + R_EXP(-g));
        dgate[i] = dy * u * (sig * ((real)1 + g * ((real)1 - sig)));
        dup[i] = dy * (g * sig);
    }
}

/* gelu_mul_backward, shaders/q8_kernels.metal:561-580. */
OR_API void or_gelu_mul_backward(const real *dout, const real *gate, const real *up,
                                 real *dgate, real *dup, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        real g = gate[i], u = up[i], dy = dout[i];
        real t = R_TANH(gelu_inner(g));
        real gelu = (real)0.5 * g * ((real)1 + t);
        real grad = (real)0.5 * ((real)1 + t)
                  + (real)0.5 * g * ((real)1 - t * t) * (real)0.7978845608
                    * ((real)1 + (real)3 * (real)0.044715 * g * g);
        dgate[i] = dy * u * grad;
        dup[i] = dy * gelu;
    }
}

/* residual_add / scale_tensor / add_scaled / clamp_tensor,
 * shaders/q8_kernels.metal:369-375, 627-643, 1155-1161. */
OR_API void or_residual_add(real *x, const real *y, size_t n) { for (size_t i = 0; i < n; i++) x[i] += y[i]; }
OR_API void or_scale(real *x, float a, size_t n) { for (size_t i = 0; i < n; i++) x[i] *= (real)a; }
OR_API void or_add_scaled(real *y, const real *x, float a, size_t n) { for (size_t i = 0; i < n; i++) y[i] += (real)a * x[i]; }
OR_API void or_clamp(real *x, float mx, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        if (x[i] > (real)mx) x[i] = (real)mx;
        if (x[i] < -(real)mx) x[i] = -(real)mx;
    }
}

/* softmax_ce_train, shaders/q8_kernels.metal:646-690: per row
 * loss = logsumexp - logit[target]; dlogits = softmax - onehot (unscaled). */
OR_API void or_softmax_ce(const real *logits, const uint32_t *targets, real *losses, real *dlogits,
                          int batch, int V)
{
    for (int b = 0; b < batch; b++) {
        const real *lg = logits + (size_t)b * V;
        real mx = (real)-1e30;
        for (int i = 0; i < V; i++) if (lg[i] > mx) mx = lg[i];
        real sum = 0;
        for (int i = 0; i < V; i++) sum += R_EXP(lg[i] - mx);
        real lse = R_LOG(sum) + mx;
        losses[b] = lse - lg[targets[b]];
        real *dl = dlogits + (size_t)b * V;
        for (int i = 0; i < V; i++)
            dl[i] = R_EXP(lg[i] - lse) - ((uint32_t)i == targets[b] ? (real)1 : (real)0);
    }
}

/* grpo_policy_grad, shaders/q8_kernels.metal:698-761: PPO-clip gate on the
 * probability ratio, dlogits = w * ratio * (softmax - onehot(action)). */
OR_API void or_grpo_policy_grad(const real *logits, const uint32_t *actions, const real *old_lp,
                                const real *advs, real *new_lp, real *dlogits,
                                int N, int V, float clip_eps)
{
    for (int p = 0; p < N; p++) {
        const real *lg = logits + (size_t)p * V;
        real mx = (real)-1e30;
        for (int i = 0; i < V; i++) if (lg[i] > mx) mx = lg[i];
        real sum = 0;
        for (int i = 0; i < V; i++) sum += R_EXP(lg[i] - mx);
        real lse = R_LOG(sum) + mx;
        real lp = lg[actions[p]] - lse;
        new_lp[p] = lp;
        real ratio = R_EXP(lp - old_lp[p]);
        real lo = (real)1 - (real)clip_eps, hi = (real)1 + (real)clip_eps;
        real clipped = ratio < lo ? lo : (ratio > hi ? hi : ratio);
        real adv = advs[p], w;
        if (adv >= 0) w = (ratio <= clipped) ? -adv : (real)0;
        else          w = (ratio >= clipped) ? -adv : (real)0;
        real *dl = dlogits + (size_t)p * V;
        for (int i = 0; i < V; i++)
            dl[i] = w * ratio * (R_EXP(lg[i] - lse) - ((uint32_t)i == actions[p] ? (real)1 : (real)0));
    }
}

/* f16_grad_accum, shaders/q8_kernels.metal:1164-1190:
 * G[M,N] (f16) = half(float(G) + sum_k dY[k,M]... ) with dY [K,M], X [K,N];
 * rounds to F16 once per call.  The sum is formed in `real`, the add in fp32. */
OR_API void or_f16_grad_accum(uint16_t *G, const real *dY, const real *X, int M, int K, int N)
{
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            real s = 0;
            for (int k = 0; k < K; k++) s += dY[(size_t)k * M + m] * X[(size_t)k * N + n];
            size_t idx = (size_t)m * N + n;
            G[idx] = or_f32_to_f16_bits(or_f16_bits_to_f32(G[idx]) + (float)s);
        }
}

/* f16_sgd_fused, shaders/q8_kernels.metal:1097-1125: W = half(float(W) - lr * dY^T X). */
OR_API void or_f16_sgd_fused(uint16_t *W, const real *dY, const real *X, int M, int K, int N, float lr)
{
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            real s = 0;
            for (int k = 0; k < K; k++) s += dY[(size_t)k * M + m] * X[(size_t)k * N + n];
            size_t idx = (size_t)m * N + n;
            W[idx] = or_f32_to_f16_bits(or_f16_bits_to_f32(W[idx]) - lr * (float)s);
        }
}

/* f16_sgd_apply, shaders/q8_kernels.metal:1195-1206: W = half(float(W) - lr*float(G)); G = 0. */
OR_API void or_f16_sgd_apply(uint16_t *W, uint16_t *G, size_t n, float lr)
{
    for (size_t i = 0; i < n; i++) {
        W[i] = or_f32_to_f16_bits(or_f16_bits_to_f32(W[i]) - lr * or_f16_bits_to_f32(G[i]));
        G[i] = 0;
    }
}

/* ------------------------------------------------------------------ */
/* Decode-step ops — shaders/q8_kernels.metal:10-331                   */
/* ------------------------------------------------------------------ */

/* q8_matvec, shaders/q8_kernels.metal:10-42: W is rows x nb blocks of
 * {fp16 d; int8 q[32]} (34 bytes, little endian); per block the 32 products
 * q * x are summed first and the block sum is scaled by d. */
OR_API void or_q8_matvec(const uint8_t *W, const real *x, real *y, int rows, int nb)
{
    for (int r = 0; r < rows; r++) {
        const uint8_t *rp = W + (size_t)r * nb * 34;
        real sum = 0;
        for (int b = 0; b < nb; b++) {
            const uint8_t *blk = rp + (size_t)b * 34;
            real scale = (real)or_f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
            real bs = 0;
            for (int j = 0; j < 32; j++) bs += (real)(int8_t)blk[2 + j] * x[b * 32 + j];
            sum += scale * bs;
        }
        y[r] = sum;
    }
}

/* f16_batch_matvec, shaders/q8_kernels.metal:49-91 (B = 1: f16_matvec, :97-127):
 * Y[b, row] = sum_c float(W[row, c]) * X[b, c], W given as fp16 bit patterns. */
OR_API void or_f16_batch_matvec(const uint16_t *W, const real *X, real *Y, int rows, int cols, int B)
{
    for (int b = 0; b < B; b++)
        for (int r = 0; r < rows; r++) {
            real s = 0;
            for (int c = 0; c < cols; c++)
                s += (real)or_f16_bits_to_f32(W[(size_t)r * cols + c]) * X[(size_t)b * cols + c];
            Y[(size_t)b * rows + r] = s;
        }
}

/* rope, shaders/q8_kernels.metal:195-231: the pairs (d, d + hd/2) of every q and
 * k head rotated by pos / theta^(2d/hd); q is [Hq, hd], k is [Hkv, hd]. */
OR_API void or_rope(real *q, real *k, int Hq, int Hkv, int hd, int pos, float theta)
{
    int half = hd / 2;
    for (int t = 0; t < Hq + Hkv; t++) {
        real *vec = t < Hq ? q + (size_t)t * hd : k + (size_t)(t - Hq) * hd;
        for (int d = 0; d < half; d++) {
            real freq = (real)1 / R_POW((real)theta, (real)(2 * d) / (real)hd);
            real ang = (real)pos * freq;
            real c = R_COS(ang), s = R_SIN(ang);
            real x0 = vec[d], x1 = vec[d + half];
            vec[d]        = x0 * c - x1 * s;
            vec[d + half] = x0 * s + x1 * c;
        }
    }
}

/* kv_cache_store, shaders/q8_kernels.metal:237-256: caches are [Hkv, max_seq, hd]. */
OR_API void or_kv_cache_store(const real *k, const real *v, real *kc, real *vc, int Hkv, int max_seq, int hd, int pos)
{
    for (int h = 0; h < Hkv; h++)
        for (int d = 0; d < hd; d++) {
            size_t ci = ((size_t)h * max_seq + pos) * hd + d;
            kc[ci] = k[h * hd + d];
            vc[ci] = v[h * hd + d];
        }
}

/* attention, shaders/q8_kernels.metal:262-331; scale 1/sqrt(hd) from the dispatch
 * (src/nn/fast_metal.m:414): per query head h (KV head h / group_ratio)
 * s_j = q.k_j * scale for j < n_attend, softmax with the maximum subtracted,
 * out = sum_j p_j v_j. */
OR_API void or_attention(const real *Q, const real *Kc, const real *Vc, real *out, int n_attend, int hd, int max_seq,
                         int Hq, int group_ratio)
{
    real *sc = (real *)malloc((size_t)n_attend * sizeof(real));
    real inv_sqrt = (real)(1.0f / sqrtf((float)hd));         /* a float in the dispatch */
    for (int h = 0; h < Hq; h++) {
        const real *qp = Q + (size_t)h * hd;
        const real *kp = Kc + (size_t)(h / group_ratio) * max_seq * hd;
        const real *vp = Vc + (size_t)(h / group_ratio) * max_seq * hd;
        real mx = (real)-1e30;
        for (int j = 0; j < n_attend; j++) {
            real dot = 0;
            for (int d = 0; d < hd; d++) dot += qp[d] * kp[(size_t)j * hd + d];
            sc[j] = dot * inv_sqrt;
            if (sc[j] > mx) mx = sc[j];
        }
        real sum = 0;
        for (int j = 0; j < n_attend; j++) { sc[j] = R_EXP(sc[j] - mx); sum += sc[j]; }
        real inv_sum = (real)1 / sum;
        for (int j = 0; j < n_attend; j++) sc[j] *= inv_sum;
        for (int d = 0; d < hd; d++) {
            real val = 0;
            for (int j = 0; j < n_attend; j++) val += sc[j] * vp[(size_t)j * hd + d];
            out[(size_t)h * hd + d] = val;
        }
    }
    free(sc);
}

/* ------------------------------------------------------------------ */
/* Optimiser — src/nn/fast_sft.c:1045-1107                             */
/* ------------------------------------------------------------------ */

/* adamw_update, src/nn/fast_sft.c:1045-1058 (bias corrections via powf on the
 * float step count; weight decay uses the parameter before the update). */
OR_API void or_adamw(real *p, const real *g, real *m, real *v, size_t n, float lr,
                     float b1, float b2, float eps, float wd, int step)
{
    real bc1 = (real)1 - R_POW((real)b1, (real)step);
    real bc2 = (real)1 - R_POW((real)b2, (real)step);
    for (size_t i = 0; i < n; i++) {
        real gi = g[i];
        m[i] = (real)b1 * m[i] + ((real)1 - (real)b1) * gi;
        v[i] = (real)b2 * v[i] + ((real)1 - (real)b2) * gi * gi;
        real mh = m[i] / bc1, vh = v[i] / bc2;
        p[i] -= (real)lr * (mh / (R_SQRT(vh) + (real)eps) + (real)wd * p[i]);
    }
}

/* clip_grad_norm, src/nn/fast_sft.c:1060-1088: global L2 norm over all LoRA
 * gradients with a double accumulator; if norm > max_norm scale every gradient
 * by max_norm / norm (no epsilon).  Returns the norm before clipping. */
OR_API double or_clip_grad_norm(real *g, size_t n, float max_norm)
{
    double sq = 0;
    for (size_t i = 0; i < n; i++) sq += (double)g[i] * (double)g[i];
    float norm = (float)sqrt(sq);
    if (norm > max_norm) {
        float sc = max_norm / norm;
        for (size_t i = 0; i < n; i++) g[i] *= (real)sc;
    }
    return sqrt(sq);
}

/* ------------------------------------------------------------------ */
/* The step — src/nn/fast_sft.c:616-982, 1113-1157                     */
/* ------------------------------------------------------------------ */

typedef struct {
    int model_type;          /* 0 = Qwen3 (SwiGLU, 2 norms), 1 = Gemma3 (GeGLU, 4 norms) */
    int NL, D, Hq, Hkv, hd, IS, V;
    int batch, seq;          /* rows BN = batch*seq; positions and attention restart per sequence */
    int R;                   /* LoRA rank */
    float lora_scaling;      /* alpha / R */
    float eps;               /* RMSNorm epsilon, 1e-6 (src/nn/fast_sft.c:190) */
    float emb_scale;         /* 1 for Qwen3, sqrtf(D) for Gemma3 (src/nn/fast_sft.c:302) */
    int window;              /* sliding-window attention on the local layers; 0 = none, the reference's behaviour */
} OrCfg;

typedef struct {
    const float *const *wq, *const *wk, *const *wv, *const *wo, *const *wg, *const *wu, *const *wd; /* [NL] */
    const float *const *g_in, *const *g_post_attn, *const *g_pre_ff, *const *g_post_ff;          /* [NL] */
    const float *const *g_q, *const *g_k;                                                      /* [NL], [hd] each */
    const float *g_final;    /* [D] */
    const float *lm_head;    /* [V, D] */
    const float *token_emb;  /* [V, D] fp32 table used for the lookup (src/nn/fast_sft.c:1119-1120) */
    const float *rope_theta; /* [NL] */
} OrWeights;

/* per-layer LoRA arena: A_q [R,D] | B_q [Hq*hd,R] | A_v [R,D] | B_v [Hkv*hd,R] */
OR_API size_t or_lora_layer_size(const OrCfg *c)
{
    return (size_t)2 * c->R * c->D + (size_t)c->Hq * c->hd * c->R + (size_t)c->Hkv * c->hd * c->R;
}

typedef struct {
    real *x_in, *ln1, *q_pre, *k_pre, *q_fin, *k_exp, *v_exp, *probs;
    real *x_mid, *ln2, *gate_pre, *up_val, *tq, *tv, *o_out, *ff_raw;
    real *act, *attn_flat;   /* save_gate_act, save_attn_flat: inputs of down_proj / o_proj (weight gradients) */
} OrSave;

typedef struct {
    OrCfg c;
    OrSave *sv;
    real *x_final, *ln_final, *logits, *dlogits, *losses;
} OrRun;

static real *ralloc(size_t n) { return (real *)calloc(n ? n : 1, sizeof(real)); }

static OrRun *run_alloc(const OrCfg *c)
{
    OrRun *r = (OrRun *)calloc(1, sizeof(OrRun));
    r->c = *c;
    size_t BN = (size_t)c->batch * c->seq, N = c->seq;
    size_t qd = (size_t)c->Hq * c->hd, kd = (size_t)c->Hkv * c->hd;
    r->sv = (OrSave *)calloc(c->NL, sizeof(OrSave));
    for (int L = 0; L < c->NL; L++) {
        OrSave *s = &r->sv[L];
        s->x_in = ralloc(BN * c->D);  s->ln1 = ralloc(BN * c->D);
        s->q_pre = ralloc(BN * qd);   s->k_pre = ralloc(BN * kd);
        s->q_fin = ralloc(BN * qd);   s->k_exp = ralloc(BN * qd);  s->v_exp = ralloc(BN * qd);
        s->probs = ralloc((size_t)c->batch * c->Hq * N * N);
        s->x_mid = ralloc(BN * c->D); s->ln2 = ralloc(BN * c->D);
        s->gate_pre = ralloc(BN * c->IS); s->up_val = ralloc(BN * c->IS);
        s->tq = ralloc(BN * (c->R ? c->R : 1)); s->tv = ralloc(BN * (c->R ? c->R : 1));
        s->o_out = ralloc(BN * c->D); s->ff_raw = ralloc(BN * c->D);
        s->act = ralloc(BN * c->IS);  s->attn_flat = ralloc(BN * qd);
    }
    r->x_final = ralloc(BN * c->D); r->ln_final = ralloc(BN * c->D);
    r->logits = ralloc(BN * c->V);  r->dlogits = ralloc(BN * c->V);
    r->losses = ralloc(BN);
    return r;
}

static void run_free(OrRun *r)
{
    for (int L = 0; L < r->c.NL; L++) {
        OrSave *s = &r->sv[L];
        free(s->x_in); free(s->ln1); free(s->q_pre); free(s->k_pre); free(s->q_fin);
        free(s->k_exp); free(s->v_exp); free(s->probs); free(s->x_mid); free(s->ln2);
        free(s->gate_pre); free(s->up_val); free(s->tq); free(s->tv); free(s->o_out); free(s->ff_raw);
        free(s->act); free(s->attn_flat);
    }
    free(r->sv); free(r->x_final); free(r->ln_final); free(r->logits); free(r->dlogits); free(r->losses);
    free(r);
}

/* forward_to_logits, src/nn/fast_sft.c:616-752.  `x` holds the embedded input
 * [BN, D] on entry and is consumed.  Sequences are independent in attention
 * and RoPE positions (batch is this build's extension; at batch 1 this is the
 * reference sequence of operations). */
static void forward(OrRun *r, const OrWeights *w, const real *lora, real *x)
{
    const OrCfg *c = &r->c;
    int BN = c->batch * c->seq, N = c->seq, D = c->D, Hq = c->Hq, Hkv = c->Hkv, hd = c->hd;
    int IS = c->IS, R = c->R, ratio = Hq / Hkv;
    int qd = Hq * hd, kd = Hkv * hd;
    size_t lsz = or_lora_layer_size(c);
    float attn_scale = 1.0f / sqrtf((float)hd);
    real *ln = ralloc((size_t)BN * D), *q = ralloc((size_t)BN * qd), *k = ralloc((size_t)BN * kd);
    real *v = ralloc((size_t)BN * kd), *lo = ralloc((size_t)BN * qd);
    real *qt = ralloc((size_t)N * qd), *kt = ralloc((size_t)N * kd), *vt = ralloc((size_t)N * kd);
    real *ao = ralloc((size_t)N * qd), *af = ralloc((size_t)BN * qd), *x2 = ralloc((size_t)BN * D);
    real *gate = ralloc((size_t)BN * IS), *up = ralloc((size_t)BN * IS), *ff = ralloc((size_t)BN * D);

    for (int L = 0; L < c->NL; L++) {
        OrSave *s = &r->sv[L];
        const real *Aq = lora + L * lsz, *Bq = Aq + (size_t)R * D;
        const real *Av = Bq + (size_t)qd * R, *Bv = Av + (size_t)R * D;

        memcpy(s->x_in, x, sizeof(real) * BN * D);
        or_rms_norm(x, w->g_in[L], ln, D, c->eps, BN);
        memcpy(s->ln1, ln, sizeof(real) * BN * D);

        or_wmatmul(ln, w->wq[L], q, BN, qd, D);
        or_wmatmul(ln, w->wk[L], k, BN, kd, D);
        or_wmatmul(ln, w->wv[L], v, BN, kd, D);
        if (R > 0) {                                   /* src/nn/fast_sft.c:639-644, 651-656 */
            or_matmul(ln, Aq, s->tq, BN, R, D);
            or_matmul(s->tq, Bq, lo, BN, qd, R);
            or_add_scaled(q, lo, c->lora_scaling, (size_t)BN * qd);
            or_matmul(ln, Av, s->tv, BN, R, D);
            or_matmul(s->tv, Bv, lo, BN, kd, R);
            or_add_scaled(v, lo, c->lora_scaling, (size_t)BN * kd);
        }

        for (int b = 0; b < c->batch; b++) {           /* attention core, one sequence at a time */
            size_t ro = (size_t)b * N;
            or_transpose_heads_fwd(q + ro * qd, qt, N, Hq, hd);
            or_transpose_heads_fwd(k + ro * kd, kt, N, Hkv, hd);
            or_transpose_heads_fwd(v + ro * kd, vt, N, Hkv, hd);
            memcpy(s->q_pre + ro * qd, qt, sizeof(real) * N * qd);
            memcpy(s->k_pre + ro * kd, kt, sizeof(real) * N * kd);
            or_rms_norm(qt, w->g_q[L], qt, hd, c->eps, Hq * N);
            or_rms_norm(kt, w->g_k[L], kt, hd, c->eps, Hkv * N);
            or_rope_train(qt, kt, Hq, Hkv, hd, N, w->rope_theta[L]);
            memcpy(s->q_fin + ro * qd, qt, sizeof(real) * N * qd);
            or_repeat_kv(kt, s->k_exp + ro * qd, Hkv, N, hd, ratio);
            or_repeat_kv(vt, s->v_exp + ro * qd, Hkv, N, hd, ratio);
            /* local layers: Gemma3's pattern (src/nn/gemma3.c:49-57), every layer of other models */
            const int local = c->window > 0 && (c->model_type == 1 ? (L % 6) != 0 : 1);
            or_attn_train_fwd_window(qt, s->k_exp + ro * qd, s->v_exp + ro * qd, ao,
                                     s->probs + (size_t)b * Hq * N * N, Hq, N, hd, attn_scale, local ? c->window : 0);
            or_transpose_heads_rev(ao, af + ro * qd, N, Hq, hd);
        }

        memcpy(s->attn_flat, af, sizeof(real) * BN * qd);
        or_wmatmul(af, w->wo[L], x2, BN, D, qd);
        if (c->model_type == 1) {                      /* src/nn/fast_sft.c:698-705 */
            memcpy(s->o_out, x2, sizeof(real) * BN * D);
            or_rms_norm(x2, w->g_post_attn[L], x2, D, c->eps, BN);
            or_residual_add(x, x2, (size_t)BN * D);
            memcpy(s->x_mid, x, sizeof(real) * BN * D);
            or_rms_norm(x, w->g_pre_ff[L], ln, D, c->eps, BN);
        } else {                                       /* src/nn/fast_sft.c:706-711 */
            or_residual_add(x, x2, (size_t)BN * D);
            memcpy(s->x_mid, x, sizeof(real) * BN * D);
            or_rms_norm(x, w->g_post_attn[L], ln, D, c->eps, BN);
        }
        memcpy(s->ln2, ln, sizeof(real) * BN * D);

        or_wmatmul(ln, w->wg[L], gate, BN, IS, D);
        or_wmatmul(ln, w->wu[L], up, BN, IS, D);
        memcpy(s->gate_pre, gate, sizeof(real) * BN * IS);
        memcpy(s->up_val, up, sizeof(real) * BN * IS);
        if (c->model_type == 1) or_gelu_mul(gate, up, (size_t)BN * IS);
        else                    or_silu_mul(gate, up, (size_t)BN * IS);
        memcpy(s->act, gate, sizeof(real) * BN * IS);
        or_wmatmul(gate, w->wd[L], ff, BN, D, IS);
        if (c->model_type == 1) {                      /* src/nn/fast_sft.c:732-736 */
            memcpy(s->ff_raw, ff, sizeof(real) * BN * D);
            or_rms_norm(ff, w->g_post_ff[L], ff, D, c->eps, BN);
        }
        or_residual_add(x, ff, (size_t)BN * D);
    }
    memcpy(r->x_final, x, sizeof(real) * BN * D);
    or_rms_norm(x, w->g_final, ln, D, c->eps, BN);
    memcpy(r->ln_final, ln, sizeof(real) * BN * D);
    or_wmatmul(ln, w->lm_head, r->logits, BN, c->V, D);

    free(ln); free(q); free(k); free(v); free(lo); free(qt); free(kt); free(vt);
    free(ao); free(af); free(x2); free(gate); free(up); free(ff);
}

/* Full-parameter mode of sft_backward_ex (src/nn/fast_sft.c:778-786, 804-811,
 * 817-833, 883-901, 922-946).  Every frozen matrix gets dW = dY^T X either added
 * into an F16 accumulator (accum = 1, f16_grad_accum) or applied at once as
 * W = half(W - lr dW) (accum = 0, f16_sgd_fused).  The matrices of OrWeights hold
 * F16 values widened to float; in SGD mode they are updated in place (the const
 * of OrWeights is cast away) and stay F16-representable. */
typedef struct {
    int accum;
    float lr;
    uint16_t *const *gq, *const *gk, *const *gv, *const *go, *const *gg, *const *gu, *const *gd;   /* [NL] F16 bits */
    uint16_t *glm;
} OrFull;

static void weight_grad(const OrFull *fp, const float *W_const, uint16_t *G,
                        const real *dY, const real *X, int M, int K, int N)
{
    if (fp->accum) { or_f16_grad_accum(G, dY, X, M, K, N); return; }
    float *W = (float *)W_const;
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {                   /* f16_sgd_fused on widened values */
            real s = 0;
            for (int k = 0; k < K; k++) s += dY[(size_t)k * M + m] * X[(size_t)k * N + n];
            size_t idx = (size_t)m * N + n;
            W[idx] = or_f16_bits_to_f32(or_f32_to_f16_bits(W[idx] - fp->lr * (float)s));
        }
}

/* sft_backward_ex, src/nn/fast_sft.c:766-982: the LoRA branch when fp is NULL,
 * the full-parameter branch (c->R must be 0) otherwise.  r->dlogits must
 * hold the loss gradient.  Writes the LoRA gradients (overwritten, never
 * accumulated) and, if dx_out is given, the gradient w.r.t. the embedded input. */
static void backward(OrRun *r, const OrWeights *w, const real *lora, real *grad, real *dx_out, const OrFull *fp)
{
    const OrCfg *c = &r->c;
    int BN = c->batch * c->seq, N = c->seq, D = c->D, Hq = c->Hq, Hkv = c->Hkv, hd = c->hd;
    int IS = c->IS, R = c->R, ratio = Hq / Hkv;
    int qd = Hq * hd, kd = Hkv * hd;
    size_t lsz = or_lora_layer_size(c);
    float attn_scale = 1.0f / sqrtf((float)hd), sc = c->lora_scaling;
    real *dx = ralloc((size_t)BN * D), *dx2 = ralloc((size_t)BN * D), *ln = ralloc((size_t)BN * D);
    real *x2 = ralloc((size_t)BN * D), *gate = ralloc((size_t)BN * IS), *up = ralloc((size_t)BN * IS);
    real *af = ralloc((size_t)BN * qd), *ao = ralloc((size_t)N * qd), *dsc = ralloc((size_t)Hq * N * N);
    real *qt = ralloc((size_t)N * qd), *ke = ralloc((size_t)N * qd), *ve = ralloc((size_t)N * qd);
    real *kt = ralloc((size_t)N * kd), *vt = ralloc((size_t)N * kd);
    real *dq = ralloc((size_t)BN * qd), *dk = ralloc((size_t)BN * kd), *dv = ralloc((size_t)BN * kd);
    real *dh = ralloc((size_t)BN * (R ? R : 1)), *lo = ralloc((size_t)BN * D);

    or_wmatmul_nt(r->dlogits, w->lm_head, dx, BN, c->V, D);
    if (fp) weight_grad(fp, w->lm_head, fp->glm, r->dlogits, r->ln_final, c->V, BN, D);
    or_rms_norm_backward(r->x_final, dx, w->g_final, dx2, BN, D, c->eps);
    memcpy(dx, dx2, sizeof(real) * BN * D);

    for (int L = c->NL - 1; L >= 0; L--) {
        OrSave *s = &r->sv[L];
        const real *Aq = lora + L * lsz, *Bq = Aq + (size_t)R * D;
        const real *Av = Bq + (size_t)qd * R, *Bv = Av + (size_t)R * D;
        real *dAq = grad + L * lsz, *dBq = dAq + (size_t)R * D;
        real *dAv = dBq + (size_t)qd * R, *dBv = dAv + (size_t)R * D;
        const real *d = dx;

        /* FFN, src/nn/fast_sft.c:798-874 */
        if (c->model_type == 1) {
            or_rms_norm_backward(s->ff_raw, dx, w->g_post_ff[L], dx2, BN, D, c->eps);
            d = dx2;
        }
        or_wmatmul_nt(d, w->wd[L], gate, BN, D, IS);
        if (fp) weight_grad(fp, w->wd[L], fp->accum ? fp->gd[L] : NULL, d, s->act, D, BN, IS);
        if (c->model_type == 1) or_gelu_mul_backward(gate, s->gate_pre, s->up_val, gate, up, (size_t)BN * IS);
        else                    or_silu_mul_backward(gate, s->gate_pre, s->up_val, gate, up, (size_t)BN * IS);
        or_wmatmul_nt(gate, w->wg[L], ln, BN, IS, D);
        if (fp) weight_grad(fp, w->wg[L], fp->accum ? fp->gg[L] : NULL, gate, s->ln2, IS, BN, D);
        or_wmatmul_nt(up, w->wu[L], x2, BN, IS, D);
        if (fp) weight_grad(fp, w->wu[L], fp->accum ? fp->gu[L] : NULL, up, s->ln2, IS, BN, D);
        or_residual_add(ln, x2, (size_t)BN * D);
        or_rms_norm_backward(s->x_mid, ln, c->model_type == 1 ? w->g_pre_ff[L] : w->g_post_attn[L],
                             dx2, BN, D, c->eps);
        or_residual_add(dx, dx2, (size_t)BN * D);

        /* attention output projection, src/nn/fast_sft.c:877-903 */
        d = dx;
        if (c->model_type == 1) {
            or_rms_norm_backward(s->o_out, dx, w->g_post_attn[L], dx2, BN, D, c->eps);
            d = dx2;
        }
        or_wmatmul_nt(d, w->wo[L], af, BN, D, qd);
        if (fp) weight_grad(fp, w->wo[L], fp->accum ? fp->go[L] : NULL, d, s->attn_flat, D, BN, qd);

        /* attention core, src/nn/fast_sft.c:905-920 */
        for (int b = 0; b < c->batch; b++) {
            size_t ro = (size_t)b * N;
            const real *pr = s->probs + (size_t)b * Hq * N * N;
            or_transpose_heads_fwd(af + ro * qd, ao, N, Hq, hd);
            or_attn_bwd_dq(ao, pr, s->v_exp + ro * qd, s->k_exp + ro * qd, dsc, qt, Hq, N, hd, attn_scale);
            or_attn_bwd_dkv(dsc, s->q_fin + ro * qd, pr, ao, ke, ve, Hq, N, hd);
            or_repeat_kv_bwd(ke, kt, Hkv, N, hd, ratio);
            or_repeat_kv_bwd(ve, vt, Hkv, N, hd, ratio);
            or_rope_train_bwd(qt, kt, Hq, Hkv, hd, N, w->rope_theta[L]);
            or_rms_norm_backward(s->q_pre + ro * qd, qt, w->g_q[L], qt, Hq * N, hd, c->eps);
            or_rms_norm_backward(s->k_pre + ro * kd, kt, w->g_k[L], kt, Hkv * N, hd, c->eps);
            or_transpose_heads_rev(qt, dq + ro * qd, N, Hq, hd);
            or_transpose_heads_rev(kt, dk + ro * kd, N, Hkv, hd);
            or_transpose_heads_rev(vt, dv + ro * kd, N, Hkv, hd);
        }

        /* full-parameter: the three weight updates come BEFORE the dX products, which therefore see
         * the new weights in SGD mode (src/nn/fast_sft.c:922-946) */
        if (fp) {
            weight_grad(fp, w->wq[L], fp->accum ? fp->gq[L] : NULL, dq, s->ln1, qd, BN, D);
            weight_grad(fp, w->wk[L], fp->accum ? fp->gk[L] : NULL, dk, s->ln1, kd, BN, D);
            weight_grad(fp, w->wv[L], fp->accum ? fp->gv[L] : NULL, dv, s->ln1, kd, BN, D);
        }

        /* LoRA Q, base Q/K, LoRA V, base V: src/nn/fast_sft.c:948-971 */
        or_wmatmul_nt(dq, w->wq[L], ln, BN, qd, D);
        if (R > 0) {
            or_matmul_tn(dq, s->tq, dBq, qd, R, BN);
            or_scale(dBq, sc, (size_t)qd * R);
            or_matmul_nt(dq, Bq, dh, BN, qd, R);
            or_scale(dh, sc, (size_t)BN * R);
            or_matmul_tn(dh, s->ln1, dAq, R, D, BN);
            or_matmul_nt(dh, Aq, lo, BN, R, D);
            or_residual_add(ln, lo, (size_t)BN * D);
        }
        or_wmatmul_nt(dk, w->wk[L], x2, BN, kd, D);
        or_residual_add(ln, x2, (size_t)BN * D);
        if (R > 0) {
            or_matmul_tn(dv, s->tv, dBv, kd, R, BN);
            or_scale(dBv, sc, (size_t)kd * R);
            or_matmul_nt(dv, Bv, dh, BN, kd, R);
            or_scale(dh, sc, (size_t)BN * R);
            or_matmul_tn(dh, s->ln1, dAv, R, D, BN);
            or_matmul_nt(dh, Av, lo, BN, R, D);
        }
        or_wmatmul_nt(dv, w->wv[L], x2, BN, kd, D);
        or_residual_add(ln, x2, (size_t)BN * D);
        if (R > 0) or_residual_add(ln, lo, (size_t)BN * D);

        /* input norm + residual + clamp, src/nn/fast_sft.c:975-980 */
        or_rms_norm_backward(s->x_in, ln, w->g_in[L], dx2, BN, D, c->eps);
        or_residual_add(dx, dx2, (size_t)BN * D);
        or_clamp(dx, 1e6f, (size_t)BN * D);
    }
    if (dx_out) memcpy(dx_out, dx, sizeof(real) * BN * D);

    free(dx); free(dx2); free(ln); free(x2); free(gate); free(up); free(af); free(ao); free(dsc);
    free(qt); free(ke); free(ve); free(kt); free(vt); free(dq); free(dk); free(dv); free(dh); free(lo);
}

/* Embedding gather of sft_train_step, src/nn/fast_sft.c:1119-1126. */
static real *embed(const OrCfg *c, const OrWeights *w, const uint32_t *tokens)
{
    int BN = c->batch * c->seq;
    real *x = ralloc((size_t)BN * c->D);
    for (int i = 0; i < BN; i++)
        for (int d = 0; d < c->D; d++) {
            float e = w->token_emb[(size_t)tokens[i] * c->D + d];
            x[(size_t)i * c->D + d] = (c->model_type == 1) ? (real)e * (real)c->emb_scale : (real)e;
        }
    return x;
}

/* Forward + mean cross-entropy only.  logits_out (optional) receives [BN, V]. */
OR_API double or_sft_loss(const OrCfg *c, const OrWeights *w, const real *lora,
                          const uint32_t *tokens, const uint32_t *targets, real *logits_out)
{
    OrRun *r = run_alloc(c);
    real *x = embed(c, w, tokens);
    forward(r, w, lora, x);
    int BN = c->batch * c->seq;
    or_softmax_ce(r->logits, targets, r->losses, r->dlogits, BN, c->V);
    real tot = 0;
    for (int i = 0; i < BN; i++) tot += r->losses[i];
    if (logits_out) memcpy(logits_out, r->logits, sizeof(real) * BN * c->V);
    double loss = (double)(tot / (real)BN);
    free(x); run_free(r);
    return loss;
}

/* sft_train_step, src/nn/fast_sft.c:1113-1157: embed, forward, CE with
 * dlogits /= BN (src/nn/fast_sft.c:754-760), backward, then — when do_update —
 * step_count++, clip_grad_norm(1.0), AdamW(b1 .9, b2 .999, eps 1e-8, wd .01)
 * (src/nn/fast_sft.c:1090-1107).  grad receives the gradients as they stand
 * after clipping when do_update, else raw.  Optional outputs may be NULL. */
OR_API double or_sft_train_step(const OrCfg *c, const OrWeights *w, real *lora, real *grad,
                                real *adam_m, real *adam_v, int *step_count,
                                const uint32_t *tokens, const uint32_t *targets, float lr,
                                int do_update, real *logits_out, real *dx_out, double *grad_norm_out)
{
    OrRun *r = run_alloc(c);
    int BN = c->batch * c->seq;
    real *x = embed(c, w, tokens);
    forward(r, w, lora, x);
    or_softmax_ce(r->logits, targets, r->losses, r->dlogits, BN, c->V);
    or_scale(r->dlogits, 1.0f / (float)BN, (size_t)BN * c->V);
    backward(r, w, lora, grad, dx_out, NULL);
    real tot = 0;
    for (int i = 0; i < BN; i++) tot += r->losses[i];
    double loss = (double)(tot / (real)BN);
    if (logits_out) memcpy(logits_out, r->logits, sizeof(real) * BN * c->V);
    size_t n = or_lora_layer_size(c) * c->NL;
    if (do_update) {
        (*step_count)++;
        double gn = or_clip_grad_norm(grad, n, 1.0f);
        if (grad_norm_out) *grad_norm_out = gn;
        or_adamw(lora, grad, adam_m, adam_v, n, lr, 0.9f, 0.999f, 1e-8f, 0.01f, *step_count);
    } else if (grad_norm_out) {
        double sq = 0;
        for (size_t i = 0; i < n; i++) sq += (double)grad[i] * (double)grad[i];
        *grad_norm_out = sqrt(sq);
    }
    free(x); run_free(r);
    return loss;
}

/* One forward + backward on one batch of rows, in full-parameter mode (full != NULL,
 * c->R == 0) or in LoRA mode (full == NULL: lora holds the adapters and grad receives
 * their gradients, overwritten).
 *   kind 0: cross-entropy against `targets`, dlogits / BN — sft_train_step with
 *           s->full_param (src/nn/fast_sft.c:1129-1139); returns the mean loss.
 *   kind 1: GRPO — grpo_policy_grad(actions = targets, old_lp, advs, clip_eps),
 *           dlogits * dl_scale (1/G), src/nn/fast_grpo.c:437-452; new_lp_out gets the
 *           log-probabilities; returns 0.
 * x_rows, when given, is the embedded input [BN, D] (GRPO zero-pads rows past the
 * sequence, src/nn/fast_grpo.c:420-422) and `tokens` is ignored.
 * full->accum selects sft_backward_accum or sft_backward_sgd(lr). */
OR_API double or_full_param_pass(const OrCfg *c, const OrWeights *w, const OrFull *full,
                                 const real *lora, real *grad,
                                 const uint32_t *tokens, const real *x_rows, int kind,
                                 const uint32_t *targets, const real *old_lp, const real *advs,
                                 float clip_eps, float dl_scale,
                                 real *logits_out, real *new_lp_out, real *dx_out)
{
    OrRun *r = run_alloc(c);
    int BN = c->batch * c->seq;
    real *x;
    if (x_rows) {
        x = ralloc((size_t)BN * c->D);
        memcpy(x, x_rows, sizeof(real) * BN * c->D);
    } else {
        x = embed(c, w, tokens);
    }
    forward(r, w, lora, x);
    if (logits_out) memcpy(logits_out, r->logits, sizeof(real) * BN * c->V);
    double ret = 0;
    if (kind == 0) {
        or_softmax_ce(r->logits, targets, r->losses, r->dlogits, BN, c->V);
        or_scale(r->dlogits, 1.0f / (float)BN, (size_t)BN * c->V);
        real tot = 0;
        for (int i = 0; i < BN; i++) tot += r->losses[i];
        ret = (double)(tot / (real)BN);
    } else {
        real *nl = ralloc(BN);
        or_grpo_policy_grad(r->logits, targets, old_lp, advs, nl, r->dlogits, BN, c->V, clip_eps);
        or_scale(r->dlogits, dl_scale, (size_t)BN * c->V);
        if (new_lp_out) memcpy(new_lp_out, nl, sizeof(real) * BN);
        free(nl);
    }
    backward(r, w, lora, grad, dx_out, full);
    free(x); run_free(r);
    return ret;
}

/* sft_apply_grad_sgd, src/nn/fast_sft.c:1021-1039, on widened weights:
 * W = half(W - lr * G), G = 0 for the seven matrices of every layer and lm_head. */
OR_API void or_apply_grad_sgd(const OrCfg *c, const OrWeights *w, const OrFull *full, float lr)
{
    size_t qd = (size_t)c->Hq * c->hd, kd = (size_t)c->Hkv * c->hd, D = c->D, IS = c->IS;
    for (int L = 0; L <= c->NL; L++) {
        const float *W[7]; uint16_t *G[7]; size_t n[7]; int cnt = 7;
        if (L < c->NL) {
            W[0] = w->wq[L]; G[0] = full->gq[L]; n[0] = qd * D;
            W[1] = w->wk[L]; G[1] = full->gk[L]; n[1] = kd * D;
            W[2] = w->wv[L]; G[2] = full->gv[L]; n[2] = kd * D;
            W[3] = w->wo[L]; G[3] = full->go[L]; n[3] = D * qd;
            W[4] = w->wg[L]; G[4] = full->gg[L]; n[4] = IS * D;
            W[5] = w->wu[L]; G[5] = full->gu[L]; n[5] = IS * D;
            W[6] = w->wd[L]; G[6] = full->gd[L]; n[6] = D * IS;
        } else {
            W[0] = w->lm_head; G[0] = full->glm; n[0] = (size_t)c->V * D; cnt = 1;
        }
        for (int j = 0; j < cnt; j++) {
            float *Wm = (float *)W[j];
            for (size_t i = 0; i < n[j]; i++) {
                Wm[i] = or_f16_bits_to_f32(or_f32_to_f16_bits(Wm[i] - lr * or_f16_bits_to_f32(G[j][i])));
                G[j][i] = 0;
            }
        }
    }
}
