/* Scalar C restatement of the INT8 quantized-linear arithmetic -- TEST
 * INFRASTRUCTURE ONLY (the checker of the checker).  Written independently of the
 * torch oracle, one element at a time, so that a vectorisation, broadcasting or
 * dtype-promotion mistake in either shows up as a bit difference between them.
 * Build with -ffp-contract=off: every product and sum below must round separately.
 *
 * Reference lines followed (paths relative to the reference checkout):
 *   block quantiser      triton/block_channel_fwd32.py:160-192 (clamped),
 *                        triton/block_channel_bwd33.py:87-120 (unclamped)
 *   per-token quantiser  triton/block_channel_fwd32.py:101-129
 *   two-pass row quant   triton/double-channle_fwd32.py:93-175
 *   block-channel GEMM   triton/block_channel_fwd32.py:51-66, block_channel_bwd33.py:42-56
 *   double-channel GEMM  triton/double-channle_fwd32.py:44-59
 *   fused quantiser      triton/fused_triton_fwd32.py:49-65
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even fp32 -> bf16 (finite inputs; NaN kept quiet) */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline int8_t round_q(float x, float scale, int clamp) {
    volatile float p = x * scale; /* volatile: forbid contraction even without the flag */
    volatile float a = p + 0.5f;
    float r = floorf(a);
    if (clamp) {
        if (r < -128.0f) r = -128.0f;
        if (r > 127.0f) r = 127.0f;
    }
    return (int8_t)(int32_t)r;
}

/* eps_mode 0: amax = amax > 1e-4 ? amax : 1e-4      (block / token kernels)
 * eps_mode 1: amax = amax + 1e-5                    (fused kernels)            */
static inline float apply_eps(float amax, int eps_mode) {
    if (eps_mode == 1) { volatile float t = amax + 1e-5f; return t; }
    return amax > 1e-4f ? amax : 1e-4f;
}

/* inv_mode 0: s = 1/(127/amax)   1: s = amax/127   2: s = amax*(1/127)
 * inv_mode 3: s = 127/amax (the multiplier itself, fused kernels)              */
static inline float stored_scale(float amax, float scale, int inv_mode) {
    switch (inv_mode) {
    case 0: return 1.0f / scale;
    case 1: return amax / 127.0f;
    case 2: { volatile float r = 1.0f / 127.0f; return amax * r; }
    default: return scale;
    }
}

/* x: [B, M, N] bf16 bits, dense.  Groups of bm x bn.  s: [B, M/bm, N/bn]. */
void ti8ref_group_quant(const uint16_t* x, int64_t B, int64_t M, int64_t N, int64_t bm, int64_t bn,
                        int clamp, int eps_mode, int inv_mode, int scale_bf16, int8_t* q, float* s) {
    for (int64_t b = 0; b < B; ++b)
        for (int64_t mb = 0; mb < M / bm; ++mb)
            for (int64_t nb = 0; nb < N / bn; ++nb) {
                float amax = 0.0f;
                for (int64_t i = 0; i < bm; ++i)
                    for (int64_t j = 0; j < bn; ++j) {
                        float v = fabsf(bf16_to_f32(x[(b * M + mb * bm + i) * N + nb * bn + j]));
                        if (v > amax) amax = v;
                    }
                amax = apply_eps(amax, eps_mode);
                float scale = 127.0f / amax;
                for (int64_t i = 0; i < bm; ++i)
                    for (int64_t j = 0; j < bn; ++j) {
                        int64_t o = (b * M + mb * bm + i) * N + nb * bn + j;
                        q[o] = round_q(bf16_to_f32(x[o]), scale, clamp);
                    }
                float st = stored_scale(amax, scale, inv_mode);
                if (scale_bf16) st = bf16_to_f32(f32_to_bf16(st));
                s[(b * (M / bm) + mb) * (N / bn) + nb] = st;
            }
}

/* Exact int32 C[M,N] = A[M,K] * B[N,K]^T. */
void ti8ref_gemm_i32(const int8_t* A, const int8_t* Bm, int64_t M, int64_t N, int64_t K, int32_t* C) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            int32_t acc = 0;
            for (int64_t k = 0; k < K; ++k) acc += (int32_t)A[m * K + k] * (int32_t)Bm[n * K + k];
            C[m * N + n] = acc;
        }
}

/* Scale descriptor: mode 0 = per row s[r]; mode 1 = per 128x128 block s[r/128][kb];
 * mode 2 = per (row, K block) s[r][kb]; mode 3 = per 128x256 block s[r/128][kb/2]. */
static inline float scale_at(const float* s, int mode, int64_t r, int64_t kb, int64_t nkb) {
    switch (mode) {
    case 0: return s[r];
    case 1: return s[(r / 128) * nkb + kb];
    case 2: return s[r * nkb + kb];
    default: return s[(r / 128) * (nkb / 2) + kb / 2];
    }
}

/* Block-channel promotion GEMM, one batch.
 * combine 0: acc = acc + (f32(dot)*sa)*sb      (Triton kernels)
 * combine 1: acc = acc + f32(dot)*(sa*sb)      (TileLang kernels)
 * combine 2: acc = acc + f32(dot)/(sa*sb)      (fused kernels; s holds multipliers)
 * out_scale multiplies the fp32 accumulator before the bf16 store (1.0f = none).
 * accf (optional) receives the fp32 accumulators. */
void ti8ref_gemm_promote(const int8_t* A, const int8_t* Bm, const float* sA, int modeA, const float* sB,
                         int modeB, int64_t M, int64_t N, int64_t K, int combine, float out_scale,
                         uint16_t* C, float* accf) {
    int64_t nkb = K / 128;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float acc = 0.0f;
            for (int64_t kb = 0; kb < nkb; ++kb) {
                int32_t d = 0;
                for (int64_t k = kb * 128; k < (kb + 1) * 128; ++k)
                    d += (int32_t)A[m * K + k] * (int32_t)Bm[n * K + k];
                float sa = scale_at(sA, modeA, m, kb, nkb), sb = scale_at(sB, modeB, n, kb, nkb);
                volatile float t;
                if (combine == 0) { volatile float u = (float)d * sa; t = u * sb; }
                else if (combine == 1) { volatile float u = sa * sb; t = (float)d * u; }
                else { volatile float u = sa * sb; t = (float)d / u; }
                volatile float nacc = acc + t;
                acc = nacc;
            }
            if (accf) accf[m * N + n] = acc;
            volatile float o = acc * out_scale;
            C[m * N + n] = f32_to_bf16(o);
        }
}

/* Double-channel epilogue: bf16((f32(acc)*sA[m])*sB[n]); if inv_k != 0 a second
 * rounding bf16(f32(c)*inv_k) follows (triton/double-channle_fwd32.py:59,284). */
void ti8ref_dequant_rows(const int32_t* acc, const float* sA, const float* sB, int64_t M, int64_t N,
                         float inv_k, uint16_t* C) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            volatile float t = (float)acc[m * N + n] * sA[m];
            volatile float u = t * sB[n];
            uint16_t c = f32_to_bf16(u);
            if (inv_k != 0.0f) { volatile float w = bf16_to_f32(c) * inv_k; c = f32_to_bf16(w); }
            C[m * N + n] = c;
        }
}

/* In-place un-normalised FWHT of rows of length n (power of two), fp32,
 * stage strides 1, 2, 4, ...; out-of-place bf16 rounding left to the caller. */
void ti8ref_fwht_f32(float* x, int64_t rows, int64_t n) {
    for (int64_t r = 0; r < rows; ++r) {
        float* v = x + r * n;
        for (int64_t h = 1; h < n; h <<= 1)
            for (int64_t i = 0; i < n; i += 2 * h)
                for (int64_t j = i; j < i + h; ++j) {
                    volatile float a = v[j] + v[j + h];
                    volatile float b = v[j] - v[j + h];
                    v[j] = a;
                    v[j + h] = b;
                }
    }
}

void ti8ref_f32_to_bf16(const float* x, int64_t n, uint16_t* y) {
    for (int64_t i = 0; i < n; ++i) y[i] = f32_to_bf16(x[i]);
}
