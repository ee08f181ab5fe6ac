/*
 * TEST INFRASTRUCTURE ONLY -- parity checker and CPU-baseline leg.  See pi_oracle.h.
 *
 * Plain-C restatement of the reference's CPU arithmetic for the sparse decode token loop.  The
 * x86 (AVX2/F16C) paths of the reference are what is restated, because those are the paths the
 * reference takes on the hosts this runs on; the lane-wise accumulation order of its SIMD dot
 * products is kept so that results can be compared against the compiled reference at fp32
 * round-off level.  Citations are file:line into the reference tree.
 *
 * How each function is pinned (tests/test_oracle_*.py): against golden vectors produced by the
 * compiled reference (oracle/_ref, tests/golden/), against numpy.float16 / closed forms, and
 * against dense fp64 matmul with an all-true mask.  pio_model_eval (the graph wiring of
 * llama.cpp:4949-5084, 5326-5468) is pinned by greedy tokens and logits that the reference's own
 * llama.cpp CPU path produced on synthetic PowerInfer GGUF files (tests/golden/ref_*.npz,
 * LLaMA F16, LLaMA Q4_0, Falcon F16 with grouped KV heads), to 1e-5 of the logit range.
 */
#include "pi_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__F16C__) || defined(__AVX2__)
#include <immintrin.h>
#endif

#define QK 32
typedef struct { uint16_t d; uint8_t qs[QK / 2]; } blk_q4_0;   /* ggml-quants.h:10-15, 18 bytes */
typedef struct { uint16_t d; int8_t  qs[QK];     } blk_q8_0;   /* ggml-quants.h:42-46, 34 bytes */
_Static_assert(sizeof(blk_q4_0) == 18, "q4_0 block");
_Static_assert(sizeof(blk_q8_0) == 34, "q8_0 block");

#define MAXI(a, b) ((a) > (b) ? (a) : (b))
#define MINI(a, b) ((a) < (b) ? (a) : (b))

static int clamp_threads(int n) {
#ifdef _OPENMP
    if (n <= 0) n = 1;
    return n;
#else
    (void)n; return 1;
#endif
}

/* ------------------------------------------------------------------------------------------
 * fp16 <-> fp32: IEEE-754 binary16, round-to-nearest-even (the reference uses F16C
 * _cvtss_sh(x, 0) / _cvtsh_ss on x86, ggml.c:289-308).
 * ---------------------------------------------------------------------------------------- */
static inline uint16_t f32_to_f16_sw(float f) {
    uint32_t x; memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7FFFFFFFu;
    if (x >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (x > 0x7F800000u ? 0x0200u | ((x >> 13) & 0x3FFu) : 0));
    if (x >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);               /* rounds to inf */
    if (x < 0x33000001u)  return (uint16_t)sign;                           /* rounds to zero */
    int e = (int)(x >> 23) - 127;
    uint32_t m = (x & 0x7FFFFFu) | 0x800000u;
    int shift; uint32_t base;
    if (e < -14) { shift = 13 + (-14 - e); base = 0; }                     /* subnormal half */
    else         { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7FFFFFu; }
    uint32_t q = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) q++;
    return (uint16_t)(sign | (base + q));
}
static inline float f16_to_f32_sw(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1F, m = h & 0x3FF, x;
    if (e == 0) {
        if (m == 0) x = sign;
        else { int s = 0; while (!(m & 0x400)) { m <<= 1; s++; } m &= 0x3FF; x = sign | ((uint32_t)(113 - s) << 23) | (m << 13); }
    } else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else x = sign | ((e + 112) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4); return f;
}
#if defined(__F16C__)
static inline uint16_t F2H(float f) { return (uint16_t)_cvtss_sh(f, 0); }
static inline float    H2F(uint16_t h) { return _cvtsh_ss(h); }
#else
#define F2H f32_to_f16_sw
#define H2F f16_to_f32_sw
#endif

uint16_t pio_f32_to_f16(float x) { return f32_to_f16_sw(x); }   /* exported as the software path so tests can pin it against F16C/numpy */
float    pio_f16_to_f32(uint16_t h) { return f16_to_f32_sw(h); }
void pio_f32_to_f16_row(const float * x, uint16_t * y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = F2H(x[i]); }
void pio_f16_to_f32_row(const uint16_t * x, float * y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = H2F(x[i]); }

size_t pio_row_bytes(int type, int64_t n) {
    switch (type) {
        case PIO_F32: case PIO_I32: return (size_t)n * 4;
        case PIO_F16:  return (size_t)n * 2;
        case PIO_Q4_0: return (size_t)(n / QK) * sizeof(blk_q4_0);
        default: return 0;
    }
}

/* ------------------------------------------------------------------------------------------
 * Q4_0 codec: ggml-quants.c:428-463 (quantize_row_q4_0_reference; the non-reference entry just
 * forwards to it) and :1074-1092 (dequantize_row_q4_0).  d = (signed value of largest magnitude)/-8,
 * q = min(15, trunc(x/d + 8.5)); element j in the low nibble of qs[j], element j+16 in the high.
 * ---------------------------------------------------------------------------------------- */
void pio_quantize_row_q4_0(const float * x, void * vy, int64_t n) {
    blk_q4_0 * y = (blk_q4_0 *)vy;
    for (int64_t b = 0; b < n / QK; ++b) {
        float amax = 0.0f, mx = 0.0f;
        for (int j = 0; j < QK; ++j) { float v = x[b * QK + j]; if (amax < fabsf(v)) { amax = fabsf(v); mx = v; } }
        const float d = mx / -8, id = d ? 1.0f / d : 0.0f;
        y[b].d = F2H(d);
        for (int j = 0; j < QK / 2; ++j) {
            const float x0 = x[b * QK + j] * id, x1 = x[b * QK + QK / 2 + j] * id;
            const uint8_t q0 = (uint8_t)MINI(15, (int8_t)(x0 + 8.5f)), q1 = (uint8_t)MINI(15, (int8_t)(x1 + 8.5f));
            y[b].qs[j] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}
void pio_dequantize_row_q4_0(const void * vx, float * y, int64_t n) {
    const blk_q4_0 * x = (const blk_q4_0 *)vx;
    for (int64_t b = 0; b < n / QK; ++b) {
        const float d = H2F(x[b].d);
        for (int j = 0; j < QK / 2; ++j) {
            y[b * QK + j]          = (float)((x[b].qs[j] & 0x0F) - 8) * d;
            y[b * QK + j + QK / 2] = (float)((x[b].qs[j] >> 4) - 8) * d;
        }
    }
}

/* Q8_0 activation quantiser, x86 path the executor uses for from_float: ggml-quants.c:702-760.
 * d = amax/127 stored as fp16; the multiplier is 127/amax (not 1/d) and rounding is to nearest even. */
void pio_quantize_row_q8_0(const float * x, void * vy, int64_t n) {
    blk_q8_0 * y = (blk_q8_0 *)vy;
    for (int64_t b = 0; b < n / QK; ++b) {
        float amax = 0.0f;
        for (int j = 0; j < QK; ++j) amax = fmaxf(amax, fabsf(x[b * QK + j]));
        const float d = amax / 127.f, id = (amax != 0.0f) ? 127.f / amax : 0.0f;
        y[b].d = F2H(d);
        for (int j = 0; j < QK; ++j) y[b].qs[j] = (int8_t)(int)rintf(x[b * QK + j] * id);
    }
}

/* ------------------------------------------------------------------------------------------
 * fp16 dot: ggml_vec_dot_f16, ggml.c:1188-1222 with the AVX2 macros (:745-800): steps of 32
 * elements into 4 accumulators of 8 fp32 lanes by FMA, the reduce of :760-778, leftovers in double.
 * ---------------------------------------------------------------------------------------- */
#if defined(__AVX2__) && defined(__F16C__) && defined(__FMA__)
#define PIO_SIMD 1
/* same arithmetic as the portable loops below, written with the x86 vector instructions so that the CPU
 * baseline runs at a realistic speed: 4 accumulators x 8 lanes, lane l of accumulator j holds the elements
 * 32k + 8j + l in increasing k */
static inline float dot_f16_simd(int64_t n, const uint16_t * x, const uint16_t * y, int64_t * done) {
    __m256 a0 = _mm256_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
    const int64_t np = n & ~(int64_t)31;
    for (int64_t i = 0; i < np; i += 32) {
        a0 = _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(x + i))),      _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(y + i))),      a0);
        a1 = _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(x + i + 8))),  _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(y + i + 8))),  a1);
        a2 = _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(x + i + 16))), _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(y + i + 16))), a2);
        a3 = _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(x + i + 24))), _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(y + i + 24))), a3);
    }
    a0 = _mm256_add_ps(_mm256_add_ps(a0, a2), _mm256_add_ps(a1, a3));
    const __m128 t0 = _mm_add_ps(_mm256_castps256_ps128(a0), _mm256_extractf128_ps(a0, 1));
    const __m128 t1 = _mm_hadd_ps(t0, t0);
    *done = np;
    return _mm_cvtss_f32(_mm_hadd_ps(t1, t1));
}
#endif

float pio_vec_dot_f16(int64_t n, const uint16_t * x, const uint16_t * y) {
#ifdef PIO_SIMD
    {
        int64_t np;
        double sumf = dot_f16_simd(n, x, y, &np);
        for (int64_t i = np; i < n; ++i) sumf += (double)(H2F(x[i]) * H2F(y[i]));
        return (float)sumf;
    }
#endif
    float acc[4][8];
    memset(acc, 0, sizeof acc);
    const int64_t np = n & ~(int64_t)31;
    for (int64_t i = 0; i < np; i += 32)
        for (int j = 0; j < 4; ++j)
            for (int l = 0; l < 8; ++l)
                acc[j][l] = fmaf(H2F(x[i + j * 8 + l]), H2F(y[i + j * 8 + l]), acc[j][l]);
    float t0[4];
    for (int l = 0; l < 8; ++l) { acc[0][l] += acc[2][l]; acc[1][l] += acc[3][l]; }
    for (int l = 0; l < 8; ++l) acc[0][l] += acc[1][l];
    for (int l = 0; l < 4; ++l) t0[l] = acc[0][l] + acc[0][l + 4];
    const float r = (t0[0] + t0[1]) + (t0[2] + t0[3]);
    double sumf = r;
    for (int64_t i = np; i < n; ++i) sumf += (double)(H2F(x[i]) * H2F(y[i]));
    return (float)sumf;
}

/* Q4_0 x Q8_0 dot: ggml_vec_dot_q4_0_q8_0 AVX2 path, ggml-quants.c:2585-2610.  Per block the 32
 * int8 products are summed exactly in groups of four adjacent bytes (nibble-unpacked order: the
 * sixteen low nibbles then the sixteen high nibbles), converted to fp32, and FMA'd with
 * d4*d8 into eight fp32 lanes; final horizontal sum as hsum_float_8 (ggml-quants.c:67-73). */
float pio_vec_dot_q4_0_q8_0(int64_t n, const void * vx, const void * vy) {
    const blk_q4_0 * x = (const blk_q4_0 *)vx;
    const blk_q8_0 * y = (const blk_q8_0 *)vy;
#ifdef PIO_SIMD
    {
        __m256 accv = _mm256_setzero_ps();
        const __m256i m4 = _mm256_set1_epi8(0x0F), off = _mm256_set1_epi8(8), ones = _mm256_set1_epi16(1);
        for (int64_t b = 0; b < n / QK; ++b) {
            const __m256 d = _mm256_set1_ps(H2F(x[b].d) * H2F(y[b].d));
            const __m128i raw = _mm_loadu_si128((const __m128i *)x[b].qs);
            __m256i q = _mm256_and_si256(_mm256_set_m128i(_mm_srli_epi16(raw, 4), raw), m4);   /* low nibbles | high nibbles */
            q = _mm256_sub_epi8(q, off);
            const __m256i yv = _mm256_loadu_si256((const __m256i *)y[b].qs);
            const __m256i p16 = _mm256_maddubs_epi16(_mm256_sign_epi8(q, q), _mm256_sign_epi8(yv, q));
            const __m256i p32 = _mm256_madd_epi16(ones, p16);                                  /* 8 sums of 4 adjacent products */
            accv = _mm256_fmadd_ps(d, _mm256_cvtepi32_ps(p32), accv);
        }
        __m128 r = _mm_add_ps(_mm256_extractf128_ps(accv, 1), _mm256_castps256_ps128(accv));
        r = _mm_add_ps(r, _mm_movehl_ps(r, r));
        r = _mm_add_ss(r, _mm_movehdup_ps(r));
        return _mm_cvtss_f32(r);
    }
#endif
    float acc[8] = {0};
    for (int64_t b = 0; b < n / QK; ++b) {
        const float d = H2F(x[b].d) * H2F(y[b].d);
        int8_t q[QK];
        for (int j = 0; j < QK / 2; ++j) { q[j] = (int8_t)((x[b].qs[j] & 0x0F) - 8); q[j + 16] = (int8_t)((x[b].qs[j] >> 4) - 8); }
        for (int l = 0; l < 8; ++l) {
            int s = 0;
            for (int k = 0; k < 4; ++k) s += (int)q[4 * l + k] * (int)y[b].qs[4 * l + k];
            acc[l] = fmaf(d, (float)s, acc[l]);
        }
    }
    float r[4];
    for (int l = 0; l < 4; ++l) r[l] = acc[l + 4] + acc[l];
    r[0] += r[2]; r[1] += r[3];
    return r[0] + r[1];
}

/* activation rows -> the weight type's dot type (type_traits[].vec_dot_type, ggml.c:429-455;
 * conversion done in the INIT phase, ggml.c:9703-9716 / 14151-14163) */
static size_t dot_row_bytes(int wtype, int64_t n) { return wtype == PIO_Q4_0 ? (size_t)(n / QK) * sizeof(blk_q8_0) : (size_t)n * 2; }
static void to_dot_type(int wtype, const float * x, void * y, int64_t n) {
    if (wtype == PIO_Q4_0) pio_quantize_row_q8_0(x, y, n); else pio_f32_to_f16_row(x, (uint16_t *)y, n);
}
static inline float vec_dot(int wtype, int64_t n, const void * w, const void * xq) {
    return wtype == PIO_Q4_0 ? pio_vec_dot_q4_0_q8_0(n, w, xq) : pio_vec_dot_f16(n, (const uint16_t *)w, (const uint16_t *)xq);
}

/* dense mul_mat: ggml_compute_forward_mul_mat, ggml.c:9598-9807 */
int pio_mul_mat(int wtype, const void * w, int64_t rows, int64_t cols, const float * x, int T, float * out, int n_threads) {
    if (wtype != PIO_F16 && wtype != PIO_Q4_0) return 1;
    const size_t wrb = pio_row_bytes(wtype, cols), xrb = dot_row_bytes(wtype, cols);
    char * xq = (char *)malloc(xrb * (size_t)T);
    if (!xq) return 2;
    for (int t = 0; t < T; ++t) to_dot_type(wtype, x + (size_t)t * cols, xq + xrb * t, cols);
    n_threads = clamp_threads(n_threads);
    #pragma omp parallel for num_threads(n_threads) schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int t = 0; t < T; ++t)
            out[(size_t)t * rows + r] = vec_dot(wtype, cols, (const char *)w + wrb * r, xq + xrb * t);
    free(xq);
    return 0;
}

/* sparse mul_mat: ggml_compute_forward_mul_mat_sparse, ggml.c:14030-14282 (test at :14256) */
int pio_mul_mat_sparse(int wtype, const void * w, int64_t rows, int64_t cols, const float * x, int T,
                       const float * idx, const int32_t * gpu_idx, float threshold, float * out, int n_threads) {
    if (wtype != PIO_F16 && wtype != PIO_Q4_0) return 1;
    /* The executor sends a MUL_MAT_SPARSE node here only when the predictor output is wider than 1000 (ggml.c:14904-14911); at or
     * below that it takes ..._sparse_head, a leftover of an attention-head experiment that reads one flag per 128 rows against a fixed
     * -7 and ignores the threshold.  No supported model has an FFN that narrow; that path is not restated, and asking for it is an error. */
    if (rows <= 1000) return 4;
    const size_t wrb = pio_row_bytes(wtype, cols), xrb = dot_row_bytes(wtype, cols);
    char * xq = (char *)malloc(xrb * (size_t)T);
    if (!xq) return 2;
    for (int t = 0; t < T; ++t) to_dot_type(wtype, x + (size_t)t * cols, xq + xrb * t, cols);
    n_threads = clamp_threads(n_threads);
    #pragma omp parallel for num_threads(n_threads) schedule(dynamic, 64)
    for (int64_t r = 0; r < rows; ++r)
        for (int t = 0; t < T; ++t) {
            float * o = out + (size_t)t * rows + r;
            if ((gpu_idx && gpu_idx[r] == 1) || idx[(size_t)t * rows + r] < threshold) { *o = 0.0f; continue; }
            *o = vec_dot(wtype, cols, (const char *)w + wrb * r, xq + xrb * t);
        }
    free(xq);
    return 0;
}

/* one axpy row, F16: ggml_axpy_avx_f16, ggml.c:14292-14312 (FMA of fp32(w) * fp32(fp16 alpha) into fp32) */
static void axpy_row_f16(int64_t n, const uint16_t * w, float * acc, uint16_t alpha) {
    const float a = H2F(alpha);
#ifdef PIO_SIMD
    if ((n & 7) == 0) {
        const __m256 av = _mm256_set1_ps(a);
        for (int64_t i = 0; i < n; i += 8)
            _mm256_storeu_ps(acc + i, _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(w + i))), av, _mm256_loadu_ps(acc + i)));
        return;
    }
#endif
    for (int64_t i = 0; i < n; ++i) acc[i] = fmaf(H2F(w[i]), a, acc[i]);
}
/* one axpy row, Q4_0: ggml_axpy_q4_0_q8_0, ggml-quants.c:2426-2509: int16 product (q-8)*alpha,
 * converted to fp32, multiplied by d_w*d_h, then a separate add (no FMA) */
static void axpy_row_q4_0(int64_t n, const blk_q4_0 * w, float * acc, int8_t alpha, uint16_t scale) {
    const float sc = H2F(scale);
#ifdef PIO_SIMD
    {
        const __m256i al = _mm256_set1_epi16((short)alpha), m4 = _mm256_set1_epi8(0x0F), off = _mm256_set1_epi8(8);
        for (int64_t b = 0; b < n / QK; ++b) {
            const __m256 d = _mm256_set1_ps(H2F(w[b].d) * sc);
            const __m128i raw = _mm_loadu_si128((const __m128i *)w[b].qs);
            __m256i q = _mm256_sub_epi8(_mm256_and_si256(_mm256_set_m128i(_mm_srli_epi16(raw, 4), raw), m4), off);
            float * o = acc + b * QK;
            for (int half = 0; half < 2; ++half) {
                const __m256i p16 = _mm256_mullo_epi16(_mm256_cvtepi8_epi16(half ? _mm256_extracti128_si256(q, 1) : _mm256_castsi256_si128(q)), al);
                const __m256 f0 = _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_cvtepi16_epi32(_mm256_castsi256_si128(p16))), d);
                const __m256 f1 = _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_cvtepi16_epi32(_mm256_extracti128_si256(p16, 1))), d);
                _mm256_storeu_ps(o + half * 16,     _mm256_add_ps(_mm256_loadu_ps(o + half * 16), f0));
                _mm256_storeu_ps(o + half * 16 + 8, _mm256_add_ps(_mm256_loadu_ps(o + half * 16 + 8), f1));
            }
        }
        return;
    }
#endif
    for (int64_t b = 0; b < n / QK; ++b) {
        const float d = H2F(w[b].d) * sc;
        float * o = acc + b * QK;
        for (int j = 0; j < QK / 2; ++j) {
            const int v0 = (w[b].qs[j] & 0x0F) - 8, v1 = (w[b].qs[j] >> 4) - 8;
            const float p0 = (float)(v0 * (int)alpha) * d, p1 = (float)(v1 * (int)alpha) * d;
            o[j] = o[j] + p0;
            o[j + QK / 2] = o[j + QK / 2] + p1;
        }
    }
}

/*
 * axpy: ggml_compute_forward_mul_mat_axpy (F16, ggml.c:14314-14463) and _axpy_q4_0 (:14465-14618).
 * Thread t owns rows [t*dr, (t+1)*dr), dr = ceil(rows/nth), accumulates into a private fp32 vector
 * and adds it into the zero-initialised output.  The reference performs that final add without a
 * lock; here the per-thread vectors are added in thread order, which is what the reference
 * computes whenever its threads do not collide, and exactly what it computes with one thread.
 */
int pio_axpy(int wtype, const void * wt, int64_t rows, int64_t cols, const float * h, int T,
             const float * idx, const int32_t * gpu_idx, float threshold, float * out, int n_threads) {
    if (wtype != PIO_F16 && wtype != PIO_Q4_0) return 1;
    if (!gpu_idx) return 3;   /* the reference F16 kernel skips every row when the aux tensor is NULL (ggml.c:14424) */
    const size_t wrb = pio_row_bytes(wtype, cols), hrb = dot_row_bytes(wtype, rows);
    n_threads = clamp_threads(n_threads);
    char  * hq  = (char *)malloc(hrb * (size_t)T);
    float * acc = (float *)malloc(sizeof(float) * (size_t)cols * n_threads);
    if (!hq || !acc) { free(hq); free(acc); return 2; }
    for (int t = 0; t < T; ++t) to_dot_type(wtype, h + (size_t)t * rows, hq + hrb * t, rows);
    memset(out, 0, sizeof(float) * (size_t)cols * T);
    const int64_t dr = (rows + n_threads - 1) / n_threads;
    for (int t = 0; t < T; ++t) {
        const float * id = idx + (size_t)t * rows;
        #pragma omp parallel num_threads(n_threads)
        {
#ifdef _OPENMP
            const int ith = omp_get_thread_num();
#else
            const int ith = 0;
#endif
            float * a = acc + (size_t)ith * cols;
            memset(a, 0, sizeof(float) * (size_t)cols);
            const int64_t r0 = dr * ith, r1 = MINI(r0 + dr, rows);
            if (wtype == PIO_F16) {
                const uint16_t * hh = (const uint16_t *)(hq + hrb * t);
                for (int64_t r = r0; r < r1; ++r) {
                    if (hh[r] == 0) continue;
                    if (gpu_idx[r] == 1) continue;
                    if (id[r] < threshold) continue;
                    axpy_row_f16(cols, (const uint16_t *)((const char *)wt + wrb * r), a, hh[r]);
                }
            } else {
                const blk_q8_0 * hb = (const blk_q8_0 *)(hq + hrb * t);
                for (int64_t r = r0; r < r1; ++r) {
                    if (gpu_idx[r] == 1) continue;
                    if (id[r] < threshold) continue;
                    const int8_t b = hb[r / QK].qs[r % QK];
                    if (b == 0) continue;
                    axpy_row_q4_0(cols, (const blk_q4_0 *)((const char *)wt + wrb * r), a, b, hb[r / QK].d);
                }
            }
        }
        float * o = out + (size_t)t * cols;
        for (int ith = 0; ith < n_threads; ++ith) {
            const float * a = acc + (size_t)ith * cols;
            for (int64_t c = 0; c < cols; ++c) o[c] += a[c];
        }
    }
    free(hq); free(acc);
    return 0;
}

/* RMSNorm: ggml_compute_forward_rms_norm_f32, ggml.c:9238-9284 (double sum of fp32 squares) */
void pio_rms_norm(const float * x, int64_t n, int T, float eps, float * out) {
    for (int t = 0; t < T; ++t) {
        const float * xr = x + (size_t)t * n; float * y = out + (size_t)t * n;
        double sum = 0.0;
        for (int64_t i = 0; i < n; ++i) sum += (double)(xr[i] * xr[i]);
        const float mean = (float)(sum / n);
        const float scale = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < n; ++i) y[i] = xr[i] * scale;
    }
}
/* LayerNorm without affine: ggml_compute_forward_norm_f32, ggml.c:9169-9236 */
void pio_norm(const float * x, int64_t n, int T, float eps, float * out) {
    for (int t = 0; t < T; ++t) {
        const float * xr = x + (size_t)t * n; float * y = out + (size_t)t * n;
        double sum = 0.0;
        for (int64_t i = 0; i < n; ++i) sum += (double)xr[i];
        const float mean = (float)(sum / n);
        double sum2 = 0.0;
        for (int64_t i = 0; i < n; ++i) { const float v = xr[i] - mean; y[i] = v; sum2 += (double)(v * v); }
        const float variance = (float)(sum2 / n);
        const float scale = 1.0f / sqrtf(variance + eps);
        for (int64_t i = 0; i < n; ++i) y[i] *= scale;
    }
}

/* RoPE forward, no YaRN (ext_factor 0, attn_factor 1): ggml_compute_forward_rope_f32,
 * ggml.c:11163-11325.  theta is advanced by repeated fp32 multiplication with
 * theta_scale = powf(base, -2/n_dims); NeoX mode multiplies theta_base by freq_scale once more
 * before the loop (:11294). */
void pio_rope(const float * x, int n_embd_head, int n_head, int T, const int32_t * pos, int n_dims, int mode,
              float freq_base, float freq_scale, float * out) {
    const float theta_scale = powf(freq_base, -2.0f / n_dims);
    const int is_neox = mode & 2;
    memcpy(out, x, sizeof(float) * (size_t)n_embd_head * n_head * T);
    for (int t = 0; t < T; ++t)
        for (int hd = 0; hd < n_head; ++hd) {
            const float * s = x + ((size_t)t * n_head + hd) * n_embd_head;
            float * o = out + ((size_t)t * n_head + hd) * n_embd_head;
            float theta_base = (float)pos[t];
            if (!is_neox) {
                for (int i0 = 0; i0 < n_embd_head; i0 += 2) {
                    const float th = freq_scale * theta_base;
                    const float c = cosf(th), sn = sinf(th);
                    theta_base *= theta_scale;
                    const float x0 = s[i0], x1 = s[i0 + 1];
                    o[i0]     = x0 * c - x1 * sn;
                    o[i0 + 1] = x0 * sn + x1 * c;
                }
            } else {
                theta_base *= freq_scale;
                for (int ib = 0; ib < n_embd_head / n_dims; ++ib)
                    for (int ic = 0; ic < n_dims; ic += 2) {
                        const float th = freq_scale * theta_base;
                        const float c = cosf(th), sn = sinf(th);
                        theta_base *= theta_scale;
                        const int i0 = ib * n_dims + ic / 2;
                        const float x0 = s[i0], x1 = s[i0 + n_dims / 2];
                        o[i0]              = x0 * c - x1 * sn;
                        o[i0 + n_dims / 2] = x0 * sn + x1 * c;
                    }
            }
        }
}

/* RoPE with the scaling operands (ggml_compute_forward_rope_f32 with rope_yarn, ggml.c:11124-11161, 11163-11325): the angle is
 * freq_scale * theta (linear scaling); with ext_factor != 0 it is mixed with the unscaled angle by a ramp over the pair index
 * between the two correction dimensions, and cos / sin are multiplied by attn_factor * (1 + 0.1 ln(1 / freq_scale)).  NeoX mode
 * hands the ramp the rotation fraction (ic / n_dims - ib) through an integer parameter, as the reference does: for ib == 0 that
 * is always 0. */
static float yarn_corr_dim(int n_dims, int n_orig_ctx, float n_rot, float base) {
    return n_dims * logf(n_orig_ctx / (n_rot * 2 * (float)M_PI)) / (2 * logf(base));
}
static void yarn_angle(float theta_extrap, float freq_scale, const float corr[2], int64_t i0, float ext_factor, float mscale, float * c, float * sn) {
    const float theta_interp = freq_scale * theta_extrap;
    float theta = theta_interp;
    if (ext_factor != 0.0f) {
        const float y = (i0 / 2 - corr[0]) / fmaxf(0.001f, corr[1] - corr[0]);
        const float ramp_mix = (1 - fminf(1, fmaxf(0, y))) * ext_factor;
        theta = theta_interp * (1 - ramp_mix) + theta_extrap * ramp_mix;
        mscale *= 1.0f + 0.1f * logf(1.0f / freq_scale);
    }
    *c = cosf(theta) * mscale;
    *sn = sinf(theta) * mscale;
}
void pio_rope_ext(const float * x, int n_embd_head, int n_head, int T, const int32_t * pos, int n_dims, int mode, int n_orig_ctx,
                  float freq_base, float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow, float * out) {
    const float theta_scale = powf(freq_base, -2.0f / n_dims);
    const float inv_ndims = -1.0f / n_dims;
    const int is_neox = mode & 2;
    float corr[2];
    corr[0] = fmaxf(0, floorf(yarn_corr_dim(n_dims, n_orig_ctx, beta_fast, freq_base)));
    corr[1] = fminf(n_dims - 1, ceilf(yarn_corr_dim(n_dims, n_orig_ctx, beta_slow, freq_base)));
    memcpy(out, x, sizeof(float) * (size_t)n_embd_head * n_head * T);
    for (int t = 0; t < T; ++t)
        for (int hd = 0; hd < n_head; ++hd) {
            const float * s = x + ((size_t)t * n_head + hd) * n_embd_head;
            float * o = out + ((size_t)t * n_head + hd) * n_embd_head;
            float theta_base = (float)pos[t];
            if (!is_neox) {
                for (int i0 = 0; i0 < n_embd_head; i0 += 2) {
                    float c, sn;
                    yarn_angle(theta_base, freq_scale, corr, i0, ext_factor, attn_factor, &c, &sn);
                    theta_base *= theta_scale;
                    const float x0 = s[i0], x1 = s[i0 + 1];
                    o[i0]     = x0 * c - x1 * sn;
                    o[i0 + 1] = x0 * sn + x1 * c;
                }
            } else {
                theta_base *= freq_scale;
                for (int ib = 0; ib < n_embd_head / n_dims; ++ib)
                    for (int ic = 0; ic < n_dims; ic += 2) {
                        const float cur_rot = inv_ndims * ic - ib;
                        float c, sn;
                        yarn_angle(theta_base, freq_scale, corr, (int64_t)cur_rot, ext_factor, attn_factor, &c, &sn);
                        theta_base *= theta_scale;
                        const int i0 = ib * n_dims + ic / 2;
                        const float x0 = s[i0], x1 = s[i0 + n_dims / 2];
                        o[i0]              = x0 * c - x1 * sn;
                        o[i0 + n_dims / 2] = x0 * sn + x1 * c;
                    }
            }
        }
}

/* softmax: ggml_compute_forward_soft_max_f32, ggml.c:10708-10775.  exp goes through a table indexed
 * by the fp16 bit pattern of (x - max) holding fp16(expf(fp32(that fp16))) (table built at
 * ggml.c:2188-2196); the sum is in double; the row is scaled by (float)(1/sum). */
static float * g_exp_f16;   /* 65536 entries, value already widened to fp32 */
static void exp_table_init(void) {
    if (g_exp_f16) return;
    float * tb = (float *)malloc(sizeof(float) * 65536);
    for (uint32_t i = 0; i < 65536; ++i) tb[i] = H2F(F2H(expf(H2F((uint16_t)i))));
    #pragma omp critical(pio_exp_tbl)
    { if (!g_exp_f16) g_exp_f16 = tb; else free(tb); }
}
void pio_soft_max(const float * x, int64_t n, int64_t rows, float * out) {
    exp_table_init();
    for (int64_t r = 0; r < rows; ++r) {
        const float * sp = x + r * n; float * dp = out + r * n;
        float mx = -INFINITY;
        for (int64_t i = 0; i < n; ++i) mx = fmaxf(mx, sp[i]);
        double sum = 0.0;
        for (int64_t i = 0; i < n; ++i) {
            if (sp[i] == -INFINITY) { dp[i] = 0.0f; continue; }
            const float v = g_exp_f16[F2H(sp[i] - mx)];
            sum += (double)v; dp[i] = v;
        }
        const float inv = (float)(1.0 / sum);
        for (int64_t i = 0; i < n; ++i) dp[i] *= inv;
    }
}

int pio_active_list(const float * idx, int64_t n, float threshold, int32_t * list) {
    int c = 0;
    for (int64_t i = 0; i < n; ++i) if (!(idx[i] < threshold)) list[c++] = (int32_t)i;
    return c;
}

/* the FFN block: llm_build_ffn_sparse, llama.cpp:4652-4757 (CPU-only build: the gpu_idx variants of
 * llm_build_sparse_mul_mat :4546 and llm_build_sparse_axpy :4599; no merge node) */
int pio_ffn_sparse(int d, int ff, int r, int T, int wtype, int has_gate,
                   const void * up_w, const void * gate_w, const void * down_t,
                   const uint16_t * fc1, const uint16_t * fc2,
                   const float * x_ffn, const float * x_pred, const int32_t * gpu_idx,
                   float threshold, int n_threads,
                   float * logits, float * up_out, float * gate_out, float * h_out, float * out) {
    int rc = 0;
    float * hid = (float *)malloc(sizeof(float) * (size_t)r * T);
    float * lg  = logits   ? logits   : (float *)malloc(sizeof(float) * (size_t)ff * T);
    float * up  = up_out   ? up_out   : (float *)malloc(sizeof(float) * (size_t)ff * T);
    float * gt  = gate_out ? gate_out : (float *)malloc(sizeof(float) * (size_t)ff * T);
    float * hh  = h_out    ? h_out    : (float *)malloc(sizeof(float) * (size_t)ff * T);
    rc |= pio_mul_mat(PIO_F16, fc1, r, d, x_pred, T, hid, n_threads);
    for (size_t i = 0; i < (size_t)r * T; ++i) hid[i] = hid[i] > 0.f ? hid[i] : 0.f;        /* ggml_vec_relu_f32, ggml.c:1403 */
    rc |= pio_mul_mat(PIO_F16, fc2, ff, r, hid, T, lg, n_threads);
    rc |= pio_mul_mat_sparse(wtype, up_w, ff, d, x_ffn, T, lg, gpu_idx, threshold, up, n_threads);
    if (has_gate) {
        rc |= pio_mul_mat_sparse(wtype, gate_w, ff, d, x_ffn, T, lg, gpu_idx, threshold, gt, n_threads);
        for (size_t i = 0; i < (size_t)ff * T; ++i) hh[i] = (gt[i] > 0.f ? gt[i] : 0.f) * up[i];
    } else {
        for (size_t i = 0; i < (size_t)ff * T; ++i) hh[i] = up[i] > 0.f ? up[i] : 0.f;
    }
    rc |= pio_axpy(wtype, down_t, ff, d, hh, T, lg, gpu_idx, threshold, out, n_threads);
    free(hid);
    if (!logits) free(lg);
    if (!up_out) free(up);
    if (!gate_out) free(gt);
    if (!h_out) free(hh);
    return rc;
}

/*
 * Attention for T new tokens: llm_build_kv_store (llama.cpp:4383-4418) then llm_build_kqv
 * (llama.cpp:4764-4850), each mul_mat being the fp16 dot above (K and V are F16 in the cache;
 * q and the softmax output are rounded to fp16 by the executor before the dot).
 * Layout of one layer's cache: K [n_ctx][n_embd_gqa] (cell-major), V [n_embd_gqa][n_ctx] (transposed).
 * kv_slot[t] = cell the new token t is written to; kq_mask [T][n_kv]; out [T][n_embd].
 */
int pio_attention(int n_embd_head, int n_head, int n_head_kv, int n_ctx, int n_kv, int T,
                  const int32_t * kv_slot, const float * kq_mask,
                  const float * q, const float * k_cur, const float * v_cur,
                  uint16_t * k_cache, uint16_t * v_cache, float * out) {
    const int n_embd_gqa = n_embd_head * n_head_kv, n_embd = n_embd_head * n_head, grp = n_head / n_head_kv;
    for (int t = 0; t < T; ++t) {
        const int cell = kv_slot[t];
        if (cell < 0 || cell >= n_ctx) return 1;
        for (int i = 0; i < n_embd_gqa; ++i) {
            k_cache[(size_t)cell * n_embd_gqa + i] = F2H(k_cur[(size_t)t * n_embd_gqa + i]);
            v_cache[(size_t)i * n_ctx + cell]      = F2H(v_cur[(size_t)t * n_embd_gqa + i]);
        }
    }
    const float scale = 1.0f / sqrtf((float)n_embd_head);
    uint16_t * qh = (uint16_t *)malloc(sizeof(uint16_t) * n_embd_head);
    float    * s  = (float *)malloc(sizeof(float) * n_kv * 2);
    uint16_t * ph = (uint16_t *)malloc(sizeof(uint16_t) * n_kv);
    float    * p  = s + n_kv;
    for (int t = 0; t < T; ++t)
        for (int h = 0; h < n_head; ++h) {
            const int hk = h / grp;     /* broadcast of K/V heads over query heads: ggml.c:9748-9760 (i02 = i12 / r2) */
            pio_f32_to_f16_row(q + ((size_t)t * n_head + h) * n_embd_head, qh, n_embd_head);
            for (int c = 0; c < n_kv; ++c) {
                float v = pio_vec_dot_f16(n_embd_head, k_cache + (size_t)c * n_embd_gqa + (size_t)hk * n_embd_head, qh);
                v = v * scale;
                s[c] = v + kq_mask[(size_t)t * n_kv + c];
            }
            pio_soft_max(s, n_kv, 1, p);
            pio_f32_to_f16_row(p, ph, n_kv);
            for (int e = 0; e < n_embd_head; ++e)
                out[(size_t)t * n_embd + (size_t)h * n_embd_head + e] =
                    pio_vec_dot_f16(n_kv, v_cache + ((size_t)hk * n_embd_head + e) * n_ctx, ph);
        }
    free(qh); free(s); free(ph);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * whole model
 * ---------------------------------------------------------------------------------------- */
typedef struct { int type; const void * data; int64_t ne0, ne1; } pio_tensor;

struct pio_model {
    pio_hparams hp;
    pio_tensor  glob[4];
    pio_tensor * layer;           /* [n_layer][PIO_T_COUNT] */
    uint16_t  * k_cache;          /* [n_layer][n_ctx][n_embd_gqa] */
    uint16_t  * v_cache;          /* [n_layer][n_embd_gqa][n_ctx] */
    int32_t   * zero_gpu_idx;     /* used when a layer has no GPU_IDX: everything is computed (llama.cpp:2984-2990) */
    float     * cap_ffn, * cap_logits, * cap_src;
};

pio_model * pio_model_new(const pio_hparams * hp) {
    pio_model * m = (pio_model *)calloc(1, sizeof *m);
    m->hp = *hp;
    m->layer = (pio_tensor *)calloc((size_t)hp->n_layer * PIO_T_COUNT, sizeof(pio_tensor));
    const size_t kv = (size_t)hp->n_layer * hp->n_ctx * (hp->n_embd / hp->n_head) * hp->n_head_kv;
    m->k_cache = (uint16_t *)calloc(kv, 2);
    m->v_cache = (uint16_t *)calloc(kv, 2);
    m->zero_gpu_idx = (int32_t *)calloc((size_t)hp->n_ff, 4);
    return m;
}
void pio_model_free(pio_model * m) {
    if (!m) return;
    free(m->layer); free(m->k_cache); free(m->v_cache); free(m->zero_gpu_idx); free(m);
}
int pio_model_set_tensor(pio_model * m, int layer, int kind, int type, const void * data, int64_t ne0, int64_t ne1) {
    if (kind < 0 || kind >= PIO_T_COUNT) return 1;
    pio_tensor * t;
    if (kind <= PIO_T_OUTPUT) t = &m->glob[kind];
    else { if (layer < 0 || layer >= m->hp.n_layer) return 1; t = &m->layer[(size_t)layer * PIO_T_COUNT + kind]; }
    t->type = type; t->data = data; t->ne0 = ne0; t->ne1 = ne1;
    return 0;
}
void pio_model_kv_clear(pio_model * m) {
    const size_t kv = (size_t)m->hp.n_layer * m->hp.n_ctx * (m->hp.n_embd / m->hp.n_head) * m->hp.n_head_kv;
    memset(m->k_cache, 0, kv * 2); memset(m->v_cache, 0, kv * 2);
}
void pio_model_set_capture(pio_model * m, float * ffn_out, float * pred_logits, float * ffn_src) { m->cap_ffn = ffn_out; m->cap_logits = pred_logits; m->cap_src = ffn_src; }

/* embedding gather: ggml_compute_forward_get_rows, ggml.c:10402 (dequantise the row to fp32) */
static int get_row(const pio_tensor * t, int64_t row, float * y) {
    const char * p = (const char *)t->data + pio_row_bytes(t->type, t->ne0) * (size_t)row;
    switch (t->type) {
        case PIO_F32:  memcpy(y, p, (size_t)t->ne0 * 4); return 0;
        case PIO_F16:  pio_f16_to_f32_row((const uint16_t *)p, y, t->ne0); return 0;
        case PIO_Q4_0: pio_dequantize_row_q4_0(p, y, t->ne0); return 0;
        default: return 1;
    }
}
/* llm_build_norm, llama.cpp:4420-4450: norm, then * weight (ggml_mul), then + bias (ggml_add) */
static void norm_affine(int rms, const float * x, int64_t n, int T, float eps, const pio_tensor * w, const pio_tensor * b, float * out) {
    if (rms) pio_rms_norm(x, n, T, eps, out); else pio_norm(x, n, T, eps, out);
    if (w && w->data) { const float * ww = (const float *)w->data; for (int t = 0; t < T; ++t) for (int64_t i = 0; i < n; ++i) out[(size_t)t * n + i] *= ww[i]; }
    if (b && b->data) { const float * bb = (const float *)b->data; for (int t = 0; t < T; ++t) for (int64_t i = 0; i < n; ++i) out[(size_t)t * n + i] += bb[i]; }
}
static int mm(const pio_tensor * w, const float * x, int T, float * out, int nt) {
    if (!w->data) return 1;
    return pio_mul_mat(w->type, w->data, w->ne1, w->ne0, x, T, out, nt);
}

/*
 * llama_decode for T tokens: build_llama_variants (llama.cpp:4949-5084) / build_falcon
 * (llama.cpp:5326-5468) with llm_build_ffn_sparse as the FFN.
 */
int pio_model_eval(pio_model * m, const int32_t * tokens, const int32_t * pos, const int32_t * kv_slot,
                   int T, int n_kv, const float * kq_mask, int all_logits, float * logits_out, int n_threads) {
    const pio_hparams * hp = &m->hp;
    const int d = hp->n_embd, ff = hp->n_ff, hd = d / hp->n_head, gqa = hd * hp->n_head_kv;
    const int falcon = hp->arch == PIO_ARCH_FALCON;
    const float fscale = hp->rope_freq_scale == 0.0f ? 1.0f : hp->rope_freq_scale;      /* cparams.rope_freq_scale, llama.cpp:9857 */
    int rc = 0;
    const size_t nd = (size_t)d * T;
    float * inpL = (float *)malloc(sizeof(float) * nd);
    float * cur  = (float *)malloc(sizeof(float) * nd);
    float * nrm  = (float *)malloc(sizeof(float) * nd);
    float * nrm2 = (float *)malloc(sizeof(float) * nd);
    float * qkv  = (float *)malloc(sizeof(float) * (size_t)(d + 2 * gqa) * T);
    float * q    = (float *)malloc(sizeof(float) * nd);
    float * k    = (float *)malloc(sizeof(float) * (size_t)gqa * T);
    float * v    = (float *)malloc(sizeof(float) * (size_t)gqa * T);
    float * qr   = (float *)malloc(sizeof(float) * nd);
    float * kr   = (float *)malloc(sizeof(float) * (size_t)gqa * T);
    float * att  = (float *)malloc(sizeof(float) * nd);
    float * ffi  = (float *)malloc(sizeof(float) * nd);
    float * ffo  = (float *)malloc(sizeof(float) * nd);
    float * lgt  = (float *)malloc(sizeof(float) * (size_t)ff * T);
    float * inpL_in = (float *)malloc(sizeof(float) * nd);

    for (int t = 0; t < T; ++t) {
        if (tokens[t] < 0 || tokens[t] >= hp->n_vocab) { rc = 1; goto done; }
        rc |= get_row(&m->glob[PIO_T_TOK_EMBD], tokens[t], inpL + (size_t)t * d);
    }
    for (int il = 0; il < hp->n_layer && !rc; ++il) {
        const pio_tensor * L = m->layer + (size_t)il * PIO_T_COUNT;
        uint16_t * kc = m->k_cache + (size_t)il * hp->n_ctx * gqa;
        uint16_t * vc = m->v_cache + (size_t)il * hp->n_ctx * gqa;
        const int32_t * gid = L[PIO_T_GPU_IDX].data ? (const int32_t *)L[PIO_T_GPU_IDX].data : m->zero_gpu_idx;
        const int r = (int)L[PIO_T_FC1].ne1;
        memcpy(inpL_in, inpL, sizeof(float) * nd);
        if (!falcon) {
            norm_affine(1, inpL, d, T, hp->norm_eps, &L[PIO_T_ATTN_NORM], NULL, nrm);
            rc |= mm(&L[PIO_T_WQ], nrm, T, q, n_threads);
            rc |= mm(&L[PIO_T_WK], nrm, T, k, n_threads);
            rc |= mm(&L[PIO_T_WV], nrm, T, v, n_threads);
            pio_rope(q, hd, hp->n_head,    T, pos, hd, 0, hp->rope_freq_base, fscale, qr);
            pio_rope(k, hd, hp->n_head_kv, T, pos, hd, 0, hp->rope_freq_base, fscale, kr);
            rc |= pio_attention(hd, hp->n_head, hp->n_head_kv, hp->n_ctx, n_kv, T, kv_slot, kq_mask, qr, kr, v, kc, vc, att);
            rc |= mm(&L[PIO_T_WO], att, T, cur, n_threads);
            for (size_t i = 0; i < nd; ++i) ffi[i] = cur[i] + inpL[i];                       /* ffn_inp */
            norm_affine(1, ffi, d, T, hp->norm_eps, &L[PIO_T_FFN_NORM], NULL, nrm);
            rc |= pio_ffn_sparse(d, ff, r, T, L[PIO_T_FFN_UP].type, 1,
                                 L[PIO_T_FFN_UP].data, L[PIO_T_FFN_GATE].data, L[PIO_T_FFN_DOWN_T].data,
                                 (const uint16_t *)L[PIO_T_FC1].data, (const uint16_t *)L[PIO_T_FC2].data,
                                 nrm, ffi, gid, hp->sparse_threshold, n_threads, lgt, NULL, NULL, NULL, ffo);
            for (size_t i = 0; i < nd; ++i) inpL[i] = ffo[i] + ffi[i];                       /* l_out */
        } else {
            norm_affine(0, inpL, d, T, hp->norm_eps, &L[PIO_T_ATTN_NORM], &L[PIO_T_ATTN_NORM_B], nrm);
            const float * attn_in = nrm;
            if (L[PIO_T_ATTN_NORM_2].data) {
                norm_affine(0, inpL, d, T, hp->norm_eps, &L[PIO_T_ATTN_NORM_2], &L[PIO_T_ATTN_NORM_2_B], nrm2);
                attn_in = nrm2;
            }
            rc |= mm(&L[PIO_T_WQKV], attn_in, T, qkv, n_threads);
            const int w = d + 2 * gqa;
            for (int t = 0; t < T; ++t) {
                memcpy(q + (size_t)t * d,   qkv + (size_t)t * w,           sizeof(float) * d);
                memcpy(k + (size_t)t * gqa, qkv + (size_t)t * w + d,       sizeof(float) * gqa);
                memcpy(v + (size_t)t * gqa, qkv + (size_t)t * w + d + gqa, sizeof(float) * gqa);
            }
            pio_rope(q, hd, hp->n_head,    T, pos, hd, 2, hp->rope_freq_base, fscale, qr);
            pio_rope(k, hd, hp->n_head_kv, T, pos, hd, 2, hp->rope_freq_base, fscale, kr);
            rc |= pio_attention(hd, hp->n_head, hp->n_head_kv, hp->n_ctx, n_kv, T, kv_slot, kq_mask, qr, kr, v, kc, vc, att);
            rc |= mm(&L[PIO_T_WO], att, T, cur, n_threads);                                   /* ffn_inp = attention output */
            rc |= pio_ffn_sparse(d, ff, r, T, L[PIO_T_FFN_UP].type, 0,
                                 L[PIO_T_FFN_UP].data, NULL, L[PIO_T_FFN_DOWN_T].data,
                                 (const uint16_t *)L[PIO_T_FC1].data, (const uint16_t *)L[PIO_T_FC2].data,
                                 nrm, inpL, gid, hp->sparse_threshold, n_threads, lgt, NULL, NULL, NULL, ffo);
            for (size_t i = 0; i < nd; ++i) { const float a = ffo[i] + cur[i]; inpL[i] = a + inpL[i]; }
        }
        if (m->cap_src)    memcpy(m->cap_src    + (size_t)il * nd, falcon ? inpL_in : ffi, sizeof(float) * nd);
        if (m->cap_ffn)    memcpy(m->cap_ffn    + (size_t)il * nd,              ffo, sizeof(float) * nd);
        if (m->cap_logits) memcpy(m->cap_logits + (size_t)il * (size_t)ff * T,  lgt, sizeof(float) * (size_t)ff * T);
    }
    if (!rc) {
        norm_affine(!falcon, inpL, d, T, hp->norm_eps, &m->glob[PIO_T_OUTPUT_NORM], falcon ? &m->glob[PIO_T_OUTPUT_NORM_B] : NULL, nrm);
        if (all_logits) rc |= mm(&m->glob[PIO_T_OUTPUT], nrm, T, logits_out, n_threads);
        else            rc |= mm(&m->glob[PIO_T_OUTPUT], nrm + (size_t)(T - 1) * d, 1, logits_out, n_threads);
    }
done:
    free(inpL); free(cur); free(nrm); free(nrm2); free(qkv); free(q); free(k); free(v); free(qr); free(kr);
    free(att); free(ffi); free(ffo); free(lgt); free(inpL_in);
    return rc;
}

/* K-shift (llm_build_k_shift, llama.cpp:4332-4381): every layer's K cache, viewed [n_rot = head size][n_head_kv][n_ctx], goes
 * through the in-place RoPE of fp16 data (ggml_compute_forward_rope_f16, ggml.c:11327-11478) with the cells' accumulated
 * position deltas as "positions" (delta[n_ctx], llama.cpp:6533-6547): fp16 -> fp32, rotate by delta * theta_i with theta
 * advanced by repeated fp32 multiplication, round back to fp16.  A cell with delta 0 is rotated by angle 0 and keeps its bits. */
int pio_model_k_shift(pio_model * m, const int32_t * delta) {
    const pio_hparams * hp = &m->hp;
    const int hd = hp->n_embd / hp->n_head, gqa = hd * hp->n_head_kv;
    const int is_neox = hp->arch == 1;
    const float theta_scale = powf(hp->rope_freq_base, -2.0f / hd);
    const float fscale = hp->rope_freq_scale == 0.0f ? 1.0f : hp->rope_freq_scale;
    for (int il = 0; il < hp->n_layer; ++il) {
        uint16_t * kc = m->k_cache + (size_t)il * hp->n_ctx * gqa;
        for (int c = 0; c < hp->n_ctx; ++c)
            for (int h = 0; h < hp->n_head_kv; ++h) {
                uint16_t * row = kc + (size_t)c * gqa + (size_t)h * hd;
                float theta_base = (float)delta[c];
                if (is_neox) theta_base *= fscale;                     /* ggml.c:11447 */
                for (int i = 0; i < hd / 2; ++i) {
                    const float th = fscale * theta_base;              /* rope_yarn with ext_factor 0, ggml.c:11124-11146 */
                    const float c_ = cosf(th), s_ = sinf(th);
                    theta_base *= theta_scale;
                    const int i0 = is_neox ? i : 2 * i, i1 = is_neox ? i + hd / 2 : 2 * i + 1;
                    const float x0 = H2F(row[i0]), x1 = H2F(row[i1]);
                    row[i0] = F2H(x0 * c_ - x1 * s_);
                    row[i1] = F2H(x0 * s_ + x1 * c_);
                }
            }
    }
    return 0;
}

/* single sequence: cell = position, n_kv = max(32, n_past + T) (llama.cpp:6842), mask as llama.cpp:6506-6531;
 * returns the greedy token of the last position (first maximum wins, llama.cpp:8617-8631) or -1 */
int pio_model_eval_simple(pio_model * m, const int32_t * tokens, int T, int n_past, float * logits_out, int n_threads) {
    const int n_kv = MINI(m->hp.n_ctx, MAXI(32, n_past + T));
    if (n_past + T > m->hp.n_ctx) return -1;
    int32_t * pos = (int32_t *)malloc(sizeof(int32_t) * T);
    float * mask = (float *)malloc(sizeof(float) * (size_t)T * n_kv);
    for (int t = 0; t < T; ++t) {
        pos[t] = n_past + t;
        for (int c = 0; c < n_kv; ++c) mask[(size_t)t * n_kv + c] = (c > n_past + t) ? -INFINITY : 0.0f;
    }
    float * lg = logits_out ? logits_out : (float *)malloc(sizeof(float) * m->hp.n_vocab);
    int rc = pio_model_eval(m, tokens, pos, pos, T, n_kv, mask, 0, lg, n_threads);
    int best = -1;
    if (!rc) { best = 0; for (int i = 1; i < m->hp.n_vocab; ++i) if (lg[i] > lg[best]) best = i; }
    if (!logits_out) free(lg);
    free(pos); free(mask);
    return best;
}
