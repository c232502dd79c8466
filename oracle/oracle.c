/* CPU oracle: scalar restatement of the reference's kernels.  TEST INFRASTRUCTURE ONLY.
 * Build with -ffp-contract=off: every product and sum below must round
 * separately, as Rust's f32 arithmetic does. */
#include "oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

/* ---------------------------------------------------------------- binary16 */

/* langtax/src/fp16.rs:4-33.  Written from the format definition: a finite
 * binary16 is man * 2^-24 (exp field 0) or (1024 + man) * 2^(exp-25). */
float lro_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    uint32_t bits;
    if (e == 31u) {
        bits = sign | 0x7f800000u | (m << 13);
    } else if (e != 0u) {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0u) {
        bits = sign;
    } else {
        /* normalise the subnormal: find the leading one of the 10-bit field */
        int lead = 9;
        while (((m >> lead) & 1u) == 0u) lead--;
        uint32_t frac = (m << (10 - lead)) & 0x3ffu;
        /* value = 2^(lead-24) * (1 + frac/1024) */
        bits = sign | ((uint32_t)(lead - 24 + 127) << 23) | (frac << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* langtax/src/fp16.rs:36-62: truncating (round-toward-zero) encoder that
 * keeps binary16 subnormals and saturates to infinity. */
uint16_t lro_f32_to_f16(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
    int32_t biased = (int32_t)((b >> 23) & 0xffu);
    int32_t e = biased - 112; /* -127 + 15 */
    uint32_t man = (b >> 13) & 0x3ffu;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e > 0) return (uint16_t)(sign | ((uint32_t)e << 10) | man);
    if (biased == 0) return sign; /* f32 zero / subnormal */
    int32_t shift = 1 - e;
    if (shift > 11) return sign;
    uint32_t full = 0x400u | man;
    return (uint16_t)(sign | ((full >> shift) & 0x3ffu));
}

static inline float rd_f16(const uint8_t *p) {
    return lro_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}
static inline uint32_t rd_u32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}
static inline float rd_f32(const uint8_t *p) {
    uint32_t b = rd_u32(p);
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static inline void wr_f16(uint8_t *p, float v) {
    uint16_t h = lro_f32_to_f16(v);
    p[0] = (uint8_t)(h & 0xff);
    p[1] = (uint8_t)(h >> 8);
}

/* ---------------------------------------------------------------- shapes */

size_t lro_block_elems(int type) {
    switch (type) {
    case LRO_F32:
    case LRO_F16: return 1;
    case LRO_Q4_0:
    case LRO_Q5_0:
    case LRO_Q5_1:
    case LRO_Q8_0: return 32;
    case LRO_Q4_K:
    case LRO_Q6_K: return 256;
    default: return 0;
    }
}

size_t lro_block_bytes(int type) {
    switch (type) {
    case LRO_F32: return 4;
    case LRO_F16: return 2;
    case LRO_Q4_0: return 18;
    case LRO_Q5_0: return 22;
    case LRO_Q5_1: return 24;
    case LRO_Q8_0: return 34;
    case LRO_Q4_K: return 144;
    case LRO_Q6_K: return 210;
    default: return 0;
    }
}

size_t lro_row_bytes(int type, size_t n_cols) {
    size_t qk = lro_block_elems(type), bb = lro_block_bytes(type);
    if (qk == 0 || n_cols % qk != 0) return 0;
    size_t nb = n_cols / qk;
    if (nb != 0 && bb > (size_t)-1 / nb) return 0;
    return nb * bb;
}

/* langtax/src/quant.rs:8901-8912 */
void lro_scale_min_k4(const uint8_t s[12], int j, uint8_t *sc, uint8_t *mn) {
    if (j < 4) {
        *sc = s[j] & 63;
        *mn = s[j + 4] & 63;
    } else {
        *sc = (uint8_t)((s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4));
        *mn = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

/* 5-bit code of element e (0..31) of a Q5 block: nibble from qs, fifth bit
 * from bit e of qh.  langtax/src/quant.rs:7751-7756 */
static inline uint32_t q5_code(const uint8_t *qs, uint32_t qh, int e) {
    uint32_t nib = (e < 16) ? (qs[e] & 0x0fu) : (uint32_t)(qs[e - 16] >> 4);
    return nib | (((qh >> e) & 1u) << 4);
}

/* 6-bit code, already recentred, of element e (0..255) of a Q6_K block.
 * langtax/src/quant.rs:8806-8821, 5751-5753 */
static inline int q6_code(const uint8_t *ql, const uint8_t *qh, int e) {
    int n = e >> 7, r = e & 127, quarter = r >> 5, l = r & 31;
    uint8_t lo = ql[64 * n + l + ((quarter & 1) ? 32 : 0)];
    uint32_t nib = (quarter >= 2) ? (uint32_t)(lo >> 4) : (lo & 0x0fu);
    uint32_t two = (qh[32 * n + l] >> (2 * quarter)) & 3u;
    return (int)(nib | (two << 4)) - 32;
}

/* ---------------------------------------------------------------- dequant */

int lro_dequant_row(int type, size_t n_cols, const uint8_t *row, float *y) {
    size_t qk = lro_block_elems(type);
    if (qk == 0 || n_cols % qk != 0) return -1;
    size_t nb = n_cols / qk;
    switch (type) {
    case LRO_F32:
        for (size_t c = 0; c < n_cols; c++) y[c] = rd_f32(row + 4 * c);
        return 0;
    case LRO_F16:
        for (size_t c = 0; c < n_cols; c++) y[c] = rd_f16(row + 2 * c);
        return 0;
    case LRO_Q8_0: /* quant.rs:7884-7910: f32(q) * d */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 34 * b;
            float d = rd_f16(wb);
            for (int j = 0; j < 32; j++) y[32 * b + j] = (float)(int8_t)wb[2 + j] * d;
        }
        return 0;
    case LRO_Q4_0: /* quant.rs:7918-7950: f32(nibble - 8) * d */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 18 * b;
            float d = rd_f16(wb);
            for (int j = 0; j < 16; j++) {
                y[32 * b + j] = (float)((int)(wb[2 + j] & 0x0f) - 8) * d;
                y[32 * b + 16 + j] = (float)((int)(wb[2 + j] >> 4) - 8) * d;
            }
        }
        return 0;
    case LRO_Q5_0: /* quant.rs:7734-7765: f32(code - 16) * d */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 22 * b;
            float d = rd_f16(wb);
            uint32_t qh = rd_u32(wb + 2);
            for (int e = 0; e < 32; e++)
                y[32 * b + e] = (float)((int)q5_code(wb + 6, qh, e) - 16) * d;
        }
        return 0;
    case LRO_Q5_1: /* quant.rs:8046-8080: (f32(code) * d) + m, two roundings */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 24 * b;
            float d = rd_f16(wb), m = rd_f16(wb + 2);
            uint32_t qh = rd_u32(wb + 4);
            for (int e = 0; e < 32; e++) {
                float p = (float)q5_code(wb + 8, qh, e) * d;
                y[32 * b + e] = p + m;
            }
        }
        return 0;
    case LRO_Q4_K: /* quant.rs:8083-8130: (a * f32(q)) - b with a = d*sc, b = dmin*m */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 144 * b;
            float d = rd_f16(wb), dmin = rd_f16(wb + 2);
            for (int sub = 0; sub < 8; sub++) {
                uint8_t sc, mn;
                lro_scale_min_k4(wb + 4, sub, &sc, &mn);
                float a = d * (float)sc, bb = dmin * (float)mn;
                const uint8_t *qs = wb + 16 + 32 * (sub >> 1);
                for (int l = 0; l < 32; l++) {
                    uint32_t q = (sub & 1) ? (uint32_t)(qs[l] >> 4) : (qs[l] & 0x0fu);
                    float p = a * (float)q;
                    y[256 * b + 32 * sub + l] = p - bb;
                }
            }
        }
        return 0;
    case LRO_Q6_K: /* quant.rs:8783-8853: (d * f32(sc)) * f32(q) */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 210 * b;
            float d = rd_f16(wb + 208);
            for (int e = 0; e < 256; e++) {
                int n = e >> 7, r = e & 127;
                int sidx = 8 * n + 2 * (r >> 5) + ((r & 31) >> 4);
                float ds = d * (float)(int8_t)wb[192 + sidx];
                y[256 * b + e] = ds * (float)q6_code(wb, wb + 128, e);
            }
        }
        return 0;
    default:
        return -1;
    }
}

/* ---------------------------------------------------------------- scalar dots */

float lro_vec_dot_row(int type, size_t n_cols, const uint8_t *row, const float *x) {
    size_t qk = lro_block_elems(type);
    if (qk == 0) return 0.0f;
    size_t nb = n_cols / qk;
    float sum = 0.0f;
    switch (type) {
    case LRO_F32: /* quant.rs:8979-8985 */
        for (size_t c = 0; c < n_cols; c++) sum += rd_f32(row + 4 * c) * x[c];
        break;
    case LRO_F16: /* quant.rs:8963-8969 */
        for (size_t c = 0; c < n_cols; c++) sum += rd_f16(row + 2 * c) * x[c];
        break;
    case LRO_Q8_0: /* quant.rs:9326-9341: (f32(q) * d) * x, elements in order */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 34 * b;
            float d = rd_f16(wb);
            const float *xb = x + 32 * b;
            for (int j = 0; j < 32; j++) {
                float w = (float)(int8_t)wb[2 + j] * d;
                sum += w * xb[j];
            }
        }
        break;
    case LRO_Q4_0: /* quant.rs:9301-9324: element j then element j+16 */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 18 * b;
            float d = rd_f16(wb);
            const float *xb = x + 32 * b;
            for (int j = 0; j < 16; j++) {
                float w0 = (float)((int)(wb[2 + j] & 0x0f) - 8) * d;
                float w1 = (float)((int)(wb[2 + j] >> 4) - 8) * d;
                sum += w0 * xb[j];
                sum += w1 * xb[j + 16];
            }
        }
        break;
    case LRO_Q5_0: /* quant.rs:9150-9176 */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 22 * b;
            float d = rd_f16(wb);
            uint32_t qh = rd_u32(wb + 2);
            const float *xb = x + 32 * b;
            for (int j = 0; j < 16; j++) {
                float w0 = (float)((int)q5_code(wb + 6, qh, j) - 16) * d;
                float w1 = (float)((int)q5_code(wb + 6, qh, j + 16) - 16) * d;
                sum += w0 * xb[j];
                sum += w1 * xb[j + 16];
            }
        }
        break;
    case LRO_Q5_1: /* quant.rs:9178-9207 */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 24 * b;
            float d = rd_f16(wb), m = rd_f16(wb + 2);
            uint32_t qh = rd_u32(wb + 4);
            const float *xb = x + 32 * b;
            for (int j = 0; j < 16; j++) {
                float p0 = (float)q5_code(wb + 8, qh, j) * d;
                float p1 = (float)q5_code(wb + 8, qh, j + 16) * d;
                float w0 = p0 + m, w1 = p1 + m;
                sum += w0 * xb[j];
                sum += w1 * xb[j + 16];
            }
        }
        break;
    case LRO_Q4_K: /* quant.rs:9414-9467: per pair of sub-blocks, 32 low then 32 high */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 144 * b;
            float d = rd_f16(wb), dmin = rd_f16(wb + 2);
            const float *xb = x + 256 * b;
            for (int sub = 0; sub < 8; sub++) {
                uint8_t sc, mn;
                lro_scale_min_k4(wb + 4, sub, &sc, &mn);
                float a = d * (float)sc, bb = dmin * (float)mn;
                const uint8_t *qs = wb + 16 + 32 * (sub >> 1);
                for (int l = 0; l < 32; l++) {
                    uint32_t q = (sub & 1) ? (uint32_t)(qs[l] >> 4) : (qs[l] & 0x0fu);
                    float p = a * (float)q;
                    float w = p - bb;
                    sum += w * xb[32 * sub + l];
                }
            }
        }
        break;
    case LRO_Q6_K: /* quant.rs:10095-10163: for each l the four quarters l, l+32, l+64, l+96 */
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *wb = row + 210 * b;
            float d = rd_f16(wb + 208);
            const float *xb = x + 256 * b;
            for (int n = 0; n < 2; n++) {
                for (int l = 0; l < 32; l++) {
                    for (int quarter = 0; quarter < 4; quarter++) {
                        int e = 128 * n + 32 * quarter + l;
                        int sidx = 8 * n + 2 * quarter + (l >> 4);
                        float ds = d * (float)(int8_t)wb[192 + sidx];
                        float w = ds * (float)q6_code(wb, wb + 128, e);
                        sum += w * xb[e];
                    }
                }
            }
        }
        break;
    default:
        break;
    }
    return sum;
}

/* ---------------------------------------------------------------- f64 oracle */

double lro_row_dot_f64(int type, size_t n_cols, const uint8_t *row, const float *x) {
    float *w = (float *)malloc((n_cols ? n_cols : 1) * sizeof(float));
    if (!w || lro_dequant_row(type, n_cols, row, w) != 0) {
        free(w);
        return NAN;
    }
    double s = 0.0;
    for (size_t c = 0; c < n_cols; c++) s += (double)w[c] * (double)x[c];
    free(w);
    return s;
}

double lro_row_abs_dot_f64(int type, size_t n_cols, const uint8_t *row, const float *x) {
    float *w = (float *)malloc((n_cols ? n_cols : 1) * sizeof(float));
    if (!w || lro_dequant_row(type, n_cols, row, w) != 0) {
        free(w);
        return NAN;
    }
    double s = 0.0;
    for (size_t c = 0; c < n_cols; c++) s += fabs((double)w[c] * (double)x[c]);
    free(w);
    return s;
}

int lro_gemm_f64(int type, size_t n_cols, size_t n_tokens, size_t n_rows, const uint8_t *w,
                 const float *x, double *y) {
    size_t rb = lro_row_bytes(type, n_cols);
    if (rb == 0 && n_cols != 0) return -1;
    float *wr = (float *)malloc((n_cols ? n_cols : 1) * sizeof(float));
    if (!wr) return -2;
    for (size_t r = 0; r < n_rows; r++) {
        if (lro_dequant_row(type, n_cols, w + r * rb, wr) != 0) {
            free(wr);
            return -1;
        }
        for (size_t t = 0; t < n_tokens; t++) {
            const float *xt = x + t * n_cols;
            double s = 0.0;
            for (size_t c = 0; c < n_cols; c++) s += (double)wr[c] * (double)xt[c];
            y[t * n_rows + r] = s;
        }
    }
    free(wr);
    return 0;
}

/* f64 product and the magnitude sum |w||x| of every output in one pass. */
int lro_gemm_f64_mag(int type, size_t n_cols, size_t n_tokens, size_t n_rows, const uint8_t *w,
                     const float *x, double *y, double *mag) {
    size_t rb = lro_row_bytes(type, n_cols);
    if (rb == 0 && n_cols != 0) return -1;
    float *wr = (float *)malloc((n_cols ? n_cols : 1) * sizeof(float));
    if (!wr) return -2;
    for (size_t r = 0; r < n_rows; r++) {
        if (lro_dequant_row(type, n_cols, w + r * rb, wr) != 0) {
            free(wr);
            return -1;
        }
        for (size_t t = 0; t < n_tokens; t++) {
            const float *xt = x + t * n_cols;
            double s = 0.0, a = 0.0;
            for (size_t c = 0; c < n_cols; c++) {
                double p = (double)wr[c] * (double)xt[c];
                s += p;
                a += fabs(p);
            }
            y[t * n_rows + r] = s;
            mag[t * n_rows + r] = a;
        }
    }
    free(wr);
    return 0;
}

/* ---------------------------------------------------------------- threaded GEMM */

/* langtax/src/pool.rs:43, 70-79 */
int lro_worker_count(size_t n_rows) {
    if (n_rows <= 1) return 1;
    long hw = sysconf(_SC_NPROCESSORS_ONLN);
    size_t n = hw > 0 ? (size_t)hw : 1;
    if (n > n_rows) n = n_rows;
    if (n > 10) n = 10;
    return (int)n;
}

typedef struct {
    int type, kind;
    size_t n_cols, n_tokens, n_rows, rb, r0, r1;
    const uint8_t *w;
    const float *x;
    float *scratch; /* row-major [n_rows][n_tokens] */
} gemm_job;

static void *gemm_worker(void *arg) {
    gemm_job *j = (gemm_job *)arg;
    for (size_t r = j->r0; r < j->r1; r++) {
        const uint8_t *row = j->w + r * j->rb;
        for (size_t t = 0; t < j->n_tokens; t++) {
            const float *xt = j->x + t * j->n_cols;
            j->scratch[r * j->n_tokens + t] =
                j->kind ? lro_simd_dot_row(j->type, j->n_cols, row, xt)
                        : lro_vec_dot_row(j->type, j->n_cols, row, xt);
        }
    }
    return NULL;
}

/* langtax/src/quant.rs:6760-6888: validate, compute every token against each
 * weight row into row-major scratch over contiguous row chunks (pool.rs:113-148),
 * then copy transposed into the token-major output. */
int lro_gemm(int type, int kind, int threads, size_t n_cols, size_t n_tokens, size_t n_rows,
             const uint8_t *w, size_t w_len, const float *x, size_t x_len, float *y,
             size_t y_len) {
    if (n_tokens == 0) return -1;
    if (n_cols != 0 && n_tokens > (size_t)-1 / n_cols) return -2;
    if (x_len != n_tokens * n_cols) return -3;
    if (y_len % n_tokens != 0 || y_len / n_tokens != n_rows) return -4;
    size_t qk = lro_block_elems(type);
    if (qk == 0) return -5;
    if (n_cols % qk != 0) return -6; /* UnalignedCols */
    size_t rb = lro_row_bytes(type, n_cols);
    if (n_rows != 0 && rb > (size_t)-1 / n_rows) return -7;
    if (w_len != rb * n_rows) return -8;
    if (n_rows == 0) return 0;
    float *scratch = (float *)malloc(y_len * sizeof(float));
    if (!scratch) return -9;
    int workers = threads > 0 ? threads : lro_worker_count(n_rows);
    if ((size_t)workers > n_rows) workers = (int)n_rows;
    size_t chunk = (n_rows + (size_t)workers - 1) / (size_t)workers;
    gemm_job jobs[64];
    pthread_t tid[64];
    if (workers > 64) workers = 64;
    int n_jobs = 0;
    for (size_t r0 = 0; r0 < n_rows; r0 += chunk) {
        gemm_job *j = &jobs[n_jobs++];
        j->type = type;
        j->kind = kind;
        j->n_cols = n_cols;
        j->n_tokens = n_tokens;
        j->n_rows = n_rows;
        j->rb = rb;
        j->r0 = r0;
        j->r1 = r0 + chunk < n_rows ? r0 + chunk : n_rows;
        j->w = w;
        j->x = x;
        j->scratch = scratch;
    }
    if (n_jobs == 1) {
        gemm_worker(&jobs[0]);
    } else {
        for (int i = 0; i < n_jobs; i++) pthread_create(&tid[i], NULL, gemm_worker, &jobs[i]);
        for (int i = 0; i < n_jobs; i++) pthread_join(tid[i], NULL);
    }
    for (size_t t = 0; t < n_tokens; t++)
        for (size_t r = 0; r < n_rows; r++) y[t * n_rows + r] = scratch[r * n_tokens + t];
    free(scratch);
    return 0;
}

/* ---------------------------------------------------------------- packers */

/* quant.rs:4342-4351 */
void lro_pack_q8_0_block(float d, const int8_t qs[32], uint8_t out[34]) {
    wr_f16(out, d);
    for (int j = 0; j < 32; j++) out[2 + j] = (uint8_t)qs[j];
}

/* quant.rs:4581-4605: v[j] in -8..7 -> low nibble of qs[j], v[j+16] -> high nibble */
void lro_pack_q4_0_block(float d, const int8_t v[32], uint8_t out[18]) {
    wr_f16(out, d);
    for (int j = 0; j < 16; j++) {
        uint8_t lo = (uint8_t)(v[j] + 8) & 0x0f, hi = (uint8_t)(v[j + 16] + 8) & 0x0f;
        out[2 + j] = (uint8_t)(lo | (hi << 4));
    }
}

static uint32_t pack_q5_codes(const uint8_t q5[32], uint8_t *qs) {
    uint32_t qh = 0;
    for (int j = 0; j < 16; j++) {
        qs[j] = (uint8_t)((q5[j] & 0x0f) | ((q5[j + 16] & 0x0f) << 4));
        if (q5[j] & 0x10) qh |= 1u << j;
        if (q5[j + 16] & 0x10) qh |= 1u << (j + 16);
    }
    return qh;
}
static void wr_u32(uint8_t *p, uint32_t v) {
    for (int i = 0; i < 4; i++) p[i] = (uint8_t)(v >> (8 * i));
}

/* quant.rs:4639-4672 */
void lro_pack_q5_0_block(float d, const uint8_t q5[32], uint8_t out[22]) {
    wr_f16(out, d);
    wr_u32(out + 2, pack_q5_codes(q5, out + 6));
}

/* quant.rs:4680-4721 */
void lro_pack_q5_1_block(float d, float m, const uint8_t q5[32], uint8_t out[24]) {
    wr_f16(out, d);
    wr_f16(out + 2, m);
    wr_u32(out + 4, pack_q5_codes(q5, out + 8));
}

/* quant.rs:4852-4878, 4977-5012 */
void lro_pack_q4_k_block(float d, float dmin, const uint8_t sc[8], const uint8_t mn[8],
                         const uint8_t q4[256], uint8_t out[144]) {
    wr_f16(out, d);
    wr_f16(out + 2, dmin);
    uint8_t *s = out + 4;
    memset(s, 0, 12);
    for (int j = 0; j < 4; j++) {
        s[j] = sc[j] & 63;
        s[j + 4] = mn[j] & 63;
    }
    for (int j = 4; j < 8; j++) {
        uint8_t a = sc[j] & 63, b = mn[j] & 63;
        s[j + 4] = (uint8_t)((a & 0x0f) | ((b & 0x0f) << 4));
        s[j - 4] |= (uint8_t)((a >> 4) << 6);
        s[j] |= (uint8_t)((b >> 4) << 6);
    }
    for (int g = 0; g < 4; g++)
        for (int l = 0; l < 32; l++)
            out[16 + 32 * g + l] =
                (uint8_t)((q4[64 * g + l] & 0x0f) | ((q4[64 * g + 32 + l] & 0x0f) << 4));
}

/* quant.rs:5712-5753 */
void lro_pack_q6_k_block(float d, const int8_t sc[16], const int8_t q6[256], uint8_t out[210]) {
    memset(out, 0, 210);
    for (int n = 0; n < 2; n++) {
        for (int l = 0; l < 32; l++) {
            uint8_t c[4];
            for (int k = 0; k < 4; k++) c[k] = (uint8_t)(q6[128 * n + 32 * k + l] + 32) & 63;
            out[64 * n + l] = (uint8_t)((c[0] & 0x0f) | ((c[2] & 0x0f) << 4));
            out[64 * n + 32 + l] = (uint8_t)((c[1] & 0x0f) | ((c[3] & 0x0f) << 4));
            out[128 + 32 * n + l] =
                (uint8_t)((c[0] >> 4) | ((c[1] >> 4) << 2) | ((c[2] >> 4) << 4) | ((c[3] >> 4) << 6));
        }
    }
    for (int i = 0; i < 16; i++) out[192 + i] = (uint8_t)sc[i];
    wr_f16(out + 208, d);
}

/* quant.rs:5694-5701 */
void lro_pack_f16(const float *v, size_t n, uint8_t *out) {
    for (size_t i = 0; i < n; i++) wr_f16(out + 2 * i, v[i]);
}

/* ---------------------------------------------------------------- RNG + demo */

/* langtax/src/sample.rs:306-312 */
uint64_t lro_splitmix64(uint64_t *state) {
    *state += 0x9E3779B97F4A7C15ull;
    uint64_t z = *state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* langtax/src/main.rs:40-48 */
static uint32_t demo_rnd(uint64_t *seed) {
    *seed = *seed * 6364136223846793005ull + 1ull;
    return (uint32_t)(*seed >> 33);
}
static int8_t demo_i8(uint32_t u) { return (int8_t)((int32_t)(u % 255u) - 128); }

/* Q8_0 x Q8_0 integer block dot, langtax/src/quant.rs:8860-8876: per block an
 * exact i32 dot, then sum = sum + f32(acc) * (dw * dx) with every step rounded. */
static float q8q8_row(const uint8_t *row, const uint8_t *x, size_t nb) {
    volatile float sum = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *wb = row + 34 * b, *xb = x + 34 * b;
        float dw = rd_f16(wb), dx = rd_f16(xb);
        int32_t acc = 0;
        for (int j = 0; j < 32; j++) acc += (int32_t)(int8_t)wb[2 + j] * (int32_t)(int8_t)xb[2 + j];
        float scale = dw * dx;
        float term = (float)acc * scale;
        sum = sum + term;
    }
    return sum;
}

/* langtax/src/main.rs:31-38 (checksum), :63-102 (data), :168-196 (run) */
uint64_t lro_demo_q8_gemv(size_t n_cols, size_t n_rows, float *y) {
    size_t nb = n_cols / 32;
    uint8_t *w = (uint8_t *)malloc(n_rows * nb * 34 + 1);
    uint8_t *x = (uint8_t *)malloc(nb * 34 + 1);
    if (!w || !x) {
        free(w);
        free(x);
        return 0;
    }
    uint64_t seed = 1;
    int8_t qs[32];
    for (size_t r = 0; r < n_rows; r++) {
        for (size_t b = 0; b < nb; b++) {
            for (int j = 0; j < 32; j++) qs[j] = demo_i8(demo_rnd(&seed));
            uint32_t extra = demo_rnd(&seed) % 80u;
            float amax = 20.0f / 1000.0f + (float)extra / 1000.0f;
            lro_pack_q8_0_block(amax, qs, w + (r * nb + b) * 34);
        }
    }
    for (size_t b = 0; b < nb; b++) {
        for (int j = 0; j < 32; j++) qs[j] = demo_i8(demo_rnd(&seed));
        lro_pack_q8_0_block(1.0f / 127.0f, qs, x + b * 34);
    }
    uint64_t h = 0xcbf29ce484222325ull;
    for (size_t r = 0; r < n_rows; r++) {
        y[r] = q8q8_row(w + r * nb * 34, x, nb);
        uint32_t bits;
        memcpy(&bits, &y[r], 4);
        h ^= (uint64_t)bits;
        h *= 0x100000001b3ull;
    }
    free(w);
    free(x);
    return h;
}

/* native-cuda/src/lib.rs:37-53 */
long lro_validate(const float *actual, const double *expected, size_t n) {
    for (size_t i = 0; i < n; i++) {
        double a = (double)actual[i], e = expected[i];
        double tol = 1e-4 + 1e-4 * fabs(e);
        if (!isfinite(a) || !isfinite(e) || fabs(a - e) > tol) return (long)i;
    }
    return -1;
}
