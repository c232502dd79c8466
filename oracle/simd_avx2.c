/* CPU oracle, AVX2 + FMA + F16C row dots.  TEST INFRASTRUCTURE ONLY.
 *
 * These keep the lane structure of the reference's `simd` feature
 * (langtax/src/simd/x86.rs:207-775): eight f32 lanes, the dequantized weight
 * formed with separate multiply / add so it is bit-identical to the scalar
 * kernel, an FMA only into the accumulator, one horizontal sum per 256-element
 * super-block for Q4_K / Q6_K and one per row for the 32-element dtypes.  This
 * is the CPU path that is timed beside the GPU. */
#include "oracle.h"

#include <immintrin.h>
#include <string.h>

/* x86.rs:178-186: (lo128 + hi128), then halves, then the last pair */
static inline float hsum8(__m256 v) {
    __m128 q = _mm_add_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    __m128 p = _mm_add_ps(q, _mm_movehl_ps(q, q));
    __m128 o = _mm_add_ss(p, _mm_shuffle_ps(p, p, 0x55));
    return _mm_cvtss_f32(o);
}

static inline __m256 bcast_f16(const uint8_t *p) { /* x86.rs:507-512 */
    uint16_t h;
    memcpy(&h, p, 2);
    return _mm256_broadcastss_ps(_mm_cvtph_ps(_mm_cvtsi32_si128((int)h)));
}

static inline __m256i bytes8_to_i32(const uint8_t *p) {
    return _mm256_cvtepu8_epi32(_mm_loadl_epi64((const __m128i *)p));
}

/* x86.rs:207-232 */
static float dot_f32(size_t n, const uint8_t *row, const float *x) {
    __m256 a0 = _mm256_setzero_ps(), a1 = _mm256_setzero_ps();
    size_t full = n / 8, i = 0;
    for (; i + 1 < full; i += 2) {
        a0 = _mm256_fmadd_ps(_mm256_loadu_ps((const float *)(row + 32 * i)), _mm256_loadu_ps(x + 8 * i), a0);
        a1 = _mm256_fmadd_ps(_mm256_loadu_ps((const float *)(row + 32 * (i + 1))),
                             _mm256_loadu_ps(x + 8 * (i + 1)), a1);
    }
    if (i < full)
        a0 = _mm256_fmadd_ps(_mm256_loadu_ps((const float *)(row + 32 * i)), _mm256_loadu_ps(x + 8 * i), a0);
    float sum = hsum8(_mm256_add_ps(a0, a1));
    for (size_t c = full * 8; c < n; c++) {
        float w;
        memcpy(&w, row + 4 * c, 4);
        sum += w * x[c];
    }
    return sum;
}

/* x86.rs:237-265 */
static float dot_f16(size_t n, const uint8_t *row, const float *x) {
    __m256 a0 = _mm256_setzero_ps(), a1 = _mm256_setzero_ps();
    size_t full = n / 8, i = 0;
    for (; i + 1 < full; i += 2) {
        a0 = _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(row + 16 * i))),
                             _mm256_loadu_ps(x + 8 * i), a0);
        a1 = _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(row + 16 * (i + 1)))),
                             _mm256_loadu_ps(x + 8 * (i + 1)), a1);
    }
    if (i < full)
        a0 = _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(row + 16 * i))),
                             _mm256_loadu_ps(x + 8 * i), a0);
    float sum = hsum8(_mm256_add_ps(a0, a1));
    for (size_t c = full * 8; c < n; c++) {
        uint16_t h;
        memcpy(&h, row + 2 * c, 2);
        sum += lro_f16_to_f32(h) * x[c];
    }
    return sum;
}

/* x86.rs:270-336 */
static float dot_q4_k(size_t nb, const uint8_t *row, const float *x) {
    float sum = 0.0f;
    const __m256i nibmask = _mm256_set1_epi32(0x0f);
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *wb = row + 144 * b;
        const float *xb = x + 256 * b;
        uint16_t hd, hm;
        memcpy(&hd, wb, 2);
        memcpy(&hm, wb + 2, 2);
        float d = lro_f16_to_f32(hd), dmin = lro_f16_to_f32(hm);
        __m256 acc = _mm256_setzero_ps();
        for (int g = 0; g < 4; g++) {
            uint8_t sc0, m0, sc1, m1;
            lro_scale_min_k4(wb + 4, 2 * g, &sc0, &m0);
            lro_scale_min_k4(wb + 4, 2 * g + 1, &sc1, &m1);
            __m256 a0 = _mm256_set1_ps(d * (float)sc0), b0 = _mm256_set1_ps(dmin * (float)m0);
            __m256 a1 = _mm256_set1_ps(d * (float)sc1), b1 = _mm256_set1_ps(dmin * (float)m1);
            const uint8_t *qs = wb + 16 + 32 * g;
            for (int c = 0; c < 4; c++) {
                __m256i by = bytes8_to_i32(qs + 8 * c);
                __m256 lo = _mm256_cvtepi32_ps(_mm256_and_si256(by, nibmask));
                __m256 hi = _mm256_cvtepi32_ps(_mm256_srli_epi32(by, 4));
                __m256 wlo = _mm256_sub_ps(_mm256_mul_ps(a0, lo), b0);
                __m256 whi = _mm256_sub_ps(_mm256_mul_ps(a1, hi), b1);
                acc = _mm256_fmadd_ps(wlo, _mm256_loadu_ps(xb + 64 * g + 8 * c), acc);
                acc = _mm256_fmadd_ps(whi, _mm256_loadu_ps(xb + 64 * g + 32 + 8 * c), acc);
            }
        }
        sum += hsum8(acc);
    }
    return sum;
}

/* x86.rs:341-417 */
static float dot_q6_k(size_t nb, const uint8_t *row, const float *x) {
    float sum = 0.0f;
    const __m256i nibmask = _mm256_set1_epi32(0x0f), two = _mm256_set1_epi32(3),
                  bias = _mm256_set1_epi32(32);
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *wb = row + 210 * b;
        const float *xb = x + 256 * b;
        uint16_t hd;
        memcpy(&hd, wb + 208, 2);
        float d = lro_f16_to_f32(hd);
        __m256 acc = _mm256_setzero_ps();
        for (int n = 0; n < 2; n++) {
            for (int step = 0; step < 4; step++) {
                int l = 8 * step, is = l / 16;
                const int8_t *sc = (const int8_t *)(wb + 192 + 8 * n + is);
                __m256i lo = bytes8_to_i32(wb + 64 * n + l);
                __m256i hi = bytes8_to_i32(wb + 64 * n + 32 + l);
                __m256i h = bytes8_to_i32(wb + 128 + 32 * n + l);
                __m256i q[4];
                q[0] = _mm256_and_si256(lo, nibmask);
                q[1] = _mm256_and_si256(hi, nibmask);
                q[2] = _mm256_srli_epi32(lo, 4);
                q[3] = _mm256_srli_epi32(hi, 4);
                __m256i hs[4] = {h, _mm256_srli_epi32(h, 2), _mm256_srli_epi32(h, 4),
                                 _mm256_srli_epi32(h, 6)};
                for (int k = 0; k < 4; k++) {
                    __m256i code = _mm256_or_si256(q[k], _mm256_slli_epi32(_mm256_and_si256(hs[k], two), 4));
                    __m256 qf = _mm256_cvtepi32_ps(_mm256_sub_epi32(code, bias));
                    __m256 ds = _mm256_set1_ps(d * (float)sc[2 * k]);
                    acc = _mm256_fmadd_ps(_mm256_mul_ps(ds, qf), _mm256_loadu_ps(xb + 128 * n + 32 * k + l), acc);
                }
            }
        }
        sum += hsum8(acc);
    }
    return sum;
}

/* x86.rs:585-627 */
static float dot_q4_0(size_t nb, const uint8_t *row, const float *x) {
    __m256 acc = _mm256_setzero_ps();
    const __m256i nibmask = _mm256_set1_epi32(0x0f), eight = _mm256_set1_epi32(8);
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *wb = row + 18 * b;
        const float *xb = x + 32 * b;
        __m256 dv = bcast_f16(wb);
        for (int c = 0; c < 2; c++) {
            __m256i by = bytes8_to_i32(wb + 2 + 8 * c);
            __m256i lo = _mm256_sub_epi32(_mm256_and_si256(by, nibmask), eight);
            __m256i hi = _mm256_sub_epi32(_mm256_srli_epi32(by, 4), eight);
            __m256 wlo = _mm256_mul_ps(_mm256_cvtepi32_ps(lo), dv);
            __m256 whi = _mm256_mul_ps(_mm256_cvtepi32_ps(hi), dv);
            acc = _mm256_fmadd_ps(wlo, _mm256_loadu_ps(xb + 8 * c), acc);
            acc = _mm256_fmadd_ps(whi, _mm256_loadu_ps(xb + 16 + 8 * c), acc);
        }
    }
    return hsum8(acc);
}

/* fifth bit of elements base..base+7 moved to bit 4 of each lane (x86.rs:548-555) */
static inline __m256i fifth_bits(__m256i qh, int base) {
    const __m256i lanes = _mm256_setr_epi32(0, 1, 2, 3, 4, 5, 6, 7);
    __m256i sh = _mm256_srlv_epi32(qh, _mm256_add_epi32(_mm256_set1_epi32(base), lanes));
    return _mm256_slli_epi32(_mm256_and_si256(sh, _mm256_set1_epi32(1)), 4);
}

/* x86.rs:643-700 */
static float dot_q5_0(size_t nb, const uint8_t *row, const float *x) {
    __m256 acc = _mm256_setzero_ps();
    const __m256i nibmask = _mm256_set1_epi32(0x0f), sixteen = _mm256_set1_epi32(16);
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *wb = row + 22 * b;
        const float *xb = x + 32 * b;
        __m256 dv = bcast_f16(wb);
        uint32_t qhu;
        memcpy(&qhu, wb + 2, 4);
        __m256i qh = _mm256_set1_epi32((int)qhu);
        for (int c = 0; c < 2; c++) {
            __m256i by = bytes8_to_i32(wb + 6 + 8 * c);
            __m256i lo = _mm256_or_si256(_mm256_and_si256(by, nibmask), fifth_bits(qh, 8 * c));
            __m256i hi = _mm256_or_si256(_mm256_srli_epi32(by, 4), fifth_bits(qh, 8 * c + 16));
            __m256 wlo = _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_sub_epi32(lo, sixteen)), dv);
            __m256 whi = _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_sub_epi32(hi, sixteen)), dv);
            acc = _mm256_fmadd_ps(wlo, _mm256_loadu_ps(xb + 8 * c), acc);
            acc = _mm256_fmadd_ps(whi, _mm256_loadu_ps(xb + 16 + 8 * c), acc);
        }
    }
    return hsum8(acc);
}

/* x86.rs:707-757 */
static float dot_q5_1(size_t nb, const uint8_t *row, const float *x) {
    __m256 acc = _mm256_setzero_ps();
    const __m256i nibmask = _mm256_set1_epi32(0x0f);
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *wb = row + 24 * b;
        const float *xb = x + 32 * b;
        __m256 dv = bcast_f16(wb), mv = bcast_f16(wb + 2);
        uint32_t qhu;
        memcpy(&qhu, wb + 4, 4);
        __m256i qh = _mm256_set1_epi32((int)qhu);
        for (int c = 0; c < 2; c++) {
            __m256i by = bytes8_to_i32(wb + 8 + 8 * c);
            __m256i lo = _mm256_or_si256(_mm256_and_si256(by, nibmask), fifth_bits(qh, 8 * c));
            __m256i hi = _mm256_or_si256(_mm256_srli_epi32(by, 4), fifth_bits(qh, 8 * c + 16));
            __m256 wlo = _mm256_add_ps(_mm256_mul_ps(_mm256_cvtepi32_ps(lo), dv), mv);
            __m256 whi = _mm256_add_ps(_mm256_mul_ps(_mm256_cvtepi32_ps(hi), dv), mv);
            acc = _mm256_fmadd_ps(wlo, _mm256_loadu_ps(xb + 8 * c), acc);
            acc = _mm256_fmadd_ps(whi, _mm256_loadu_ps(xb + 16 + 8 * c), acc);
        }
    }
    return hsum8(acc);
}

/* x86.rs:764-775 */
static float dot_q8_0(size_t nb, const uint8_t *row, const float *x) {
    __m256 acc = _mm256_setzero_ps();
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *wb = row + 34 * b;
        const float *xb = x + 32 * b;
        __m256 dv = bcast_f16(wb);
        for (int c = 0; c < 4; c++) {
            __m256i qi = _mm256_cvtepi8_epi32(_mm_loadl_epi64((const __m128i *)(wb + 2 + 8 * c)));
            __m256 w = _mm256_mul_ps(_mm256_cvtepi32_ps(qi), dv);
            acc = _mm256_fmadd_ps(w, _mm256_loadu_ps(xb + 8 * c), acc);
        }
    }
    return hsum8(acc);
}

float lro_simd_dot_row(int type, size_t n_cols, const uint8_t *row, const float *x) {
    switch (type) {
    case LRO_F32: return dot_f32(n_cols, row, x);
    case LRO_F16: return dot_f16(n_cols, row, x);
    case LRO_Q4_0: return dot_q4_0(n_cols / 32, row, x);
    case LRO_Q5_0: return dot_q5_0(n_cols / 32, row, x);
    case LRO_Q5_1: return dot_q5_1(n_cols / 32, row, x);
    case LRO_Q8_0: return dot_q8_0(n_cols / 32, row, x);
    case LRO_Q4_K: return dot_q4_k(n_cols / 256, row, x);
    case LRO_Q6_K: return dot_q6_k(n_cols / 256, row, x);
    default: return 0.0f;
    }
}
