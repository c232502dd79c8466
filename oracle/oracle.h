/* CPU oracle for the GGUF block-quantized matrix products (TEST INFRASTRUCTURE).
 *
 * This library restates, in plain C, the arithmetic of the reference's CPU
 * kernels for the eight in-scope GGUF dtypes.  It exists to CHECK the HIP
 * executor; nothing in the product path may call, link or load it.  Only the
 * test-suite, the smoke check and the benchmark's cpu-baseline leg use it.
 *
 * Every function names the reference source it follows (paths relative to the
 * reference checkout).  The scalar kernels keep the reference's operation
 * order exactly (one f32 accumulator, no contraction), so that on any input a
 * bit-for-bit agreement with the reference's `--no-default-features` build is
 * expected; the AVX2 kernels (simd_avx2.c) keep the lane structure of the
 * reference's `simd` feature and are the timed CPU baseline.
 *
 * Pinning status (what each part is checked against, see tests/):
 *   f16 decode/encode ....... arithmetic definition over all 65 536 patterns,
 *                             numpy float16, the reference's published
 *                             Q8_0 GEMV checksum
 *   Q8_0 layout + LCG ....... published y_checksum=80e188057fa1eef0, y0=78.165176
 *   SplitMix64 .............. published first outputs (seed 0 and 1)
 *   packers ................. byte-level known answers from the reference's tests
 *   dequant / scalar dots ... hand-computable cases, closed-form dyadic fixtures
 *                             with exact f64 sums, independent numpy dequantizers,
 *                             fused-dot == dequant-then-dot (bitwise for Q4_K)
 *   AVX2 dots ............... the reference's proven bound against the scalar
 *                             kernels and an f64 dot
 * No function here is "parity unpinned".
 */
#ifndef LLAMA_RUST_ORACLE_H
#define LLAMA_RUST_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids (langtax/src/gguf.rs:245-258). */
enum {
    LRO_F32 = 0,
    LRO_F16 = 1,
    LRO_Q4_0 = 2,
    LRO_Q5_0 = 6,
    LRO_Q5_1 = 7,
    LRO_Q8_0 = 8,
    LRO_Q4_K = 12,
    LRO_Q6_K = 14
};

/* langtax/src/fp16.rs:4-33 and :36-62 */
float lro_f16_to_f32(uint16_t h);
uint16_t lro_f32_to_f16(float f);

/* Elements per block / bytes per block; 0 for an unknown type.
 * langtax/src/quant.rs:87-163 */
size_t lro_block_elems(int type);
size_t lro_block_bytes(int type);
/* Packed bytes of one row, or 0 when n_cols is not a whole number of blocks
 * (the reference's UnalignedCols) or the product overflows.
 * langtax/src/quant.rs:4210-4218, 4254-4284, 5647-5682 */
size_t lro_row_bytes(int type, size_t n_cols);

/* One packed row -> n_cols f32.  Returns 0, or -1 on a bad type/shape.
 * langtax/src/quant.rs:7511-7541, 7734-7765, 7884-7950, 8046-8130, 8783-8853 */
int lro_dequant_row(int type, size_t n_cols, const uint8_t *row, float *y);

/* Scalar fused dequant-dot of one row, reference operation order.
 * langtax/src/quant.rs:8963-8985, 9150-9207, 9301-9341, 9414-9467, 10095-10163 */
float lro_vec_dot_row(int type, size_t n_cols, const uint8_t *row, const float *x);

/* AVX2+FMA+F16C row dot with the lane structure of the reference's `simd`
 * feature.  langtax/src/simd/x86.rs:207-775 */
float lro_simd_dot_row(int type, size_t n_cols, const uint8_t *row, const float *x);

/* f64 dot of the dequantized row with x: the parity oracle the reference's
 * integration test uses.  langtax/tests/native_cuda_parity.rs:124-148 */
double lro_row_dot_f64(int type, size_t n_cols, const uint8_t *row, const float *x);
/* sum |w_i * x_i| in f64 (the error-bound scale, langtax/src/simd/tests.rs:18-91) */
double lro_row_abs_dot_f64(int type, size_t n_cols, const uint8_t *row, const float *x);

/* Token-major products  y[t*n_rows + r] = W[r,:] . x[t*n_cols ...].
 * kind: 0 = scalar kernels, 1 = AVX2 kernels.  threads <= 0 means the
 * reference's rule min(hardware threads, n_rows, 10) over contiguous row
 * chunks (langtax/src/pool.rs:43, 70-148); layout and validation follow
 * langtax/src/quant.rs:6760-6888.  Returns 0 or a negative error. */
int lro_gemm(int type, int kind, int threads, size_t n_cols, size_t n_tokens,
             size_t n_rows, const uint8_t *w, size_t w_len, const float *x,
             size_t x_len, float *y, size_t y_len);
/* Same product as exact-as-possible f64 sums over the dequantized weights. */
int lro_gemm_f64(int type, size_t n_cols, size_t n_tokens, size_t n_rows,
                 const uint8_t *w, const float *x, double *y);
/* The f64 product together with sum_c |W[r,c] x[t,c]| per output (the scale of
 * the reference's error bound, langtax/src/simd/tests.rs:93-105). */
int lro_gemm_f64_mag(int type, size_t n_cols, size_t n_tokens, size_t n_rows, const uint8_t *w,
                     const float *x, double *y, double *mag);
/* Worker count the reference would use for n_rows rows (pool.rs:70-79). */
int lro_worker_count(size_t n_rows);

/* Block packers.  langtax/src/quant.rs:4342-4351, 4581-4605, 4639-4721,
 * 4852-4878, 4977-5012, 5712-5753 */
void lro_pack_q8_0_block(float d, const int8_t qs[32], uint8_t out[34]);
void lro_pack_q4_0_block(float d, const int8_t v[32], uint8_t out[18]);
void lro_pack_q5_0_block(float d, const uint8_t q5[32], uint8_t out[22]);
void lro_pack_q5_1_block(float d, float m, const uint8_t q5[32], uint8_t out[24]);
void lro_pack_q4_k_block(float d, float dmin, const uint8_t sc[8], const uint8_t mn[8],
                         const uint8_t q4[256], uint8_t out[144]);
void lro_pack_q6_k_block(float d, const int8_t sc[16], const int8_t q6[256], uint8_t out[210]);
void lro_pack_f16(const float *v, size_t n, uint8_t *out);

/* Unpack the j-th 6-bit (scale, min) pair of a Q4_K block.
 * langtax/src/quant.rs:8901-8912 */
void lro_scale_min_k4(const uint8_t scales[12], int j, uint8_t *sc, uint8_t *mn);

/* SplitMix64 (langtax/src/sample.rs:306-312). */
uint64_t lro_splitmix64(uint64_t *state);

/* The `gguf_gemv write|gemv` demo: LCG-generated Q8_0 weights and Q8_0
 * activations, integer block dot, FNV-style checksum over the f32 outputs.
 * langtax/src/main.rs:31-102, langtax/src/quant.rs:8860-8876.
 * Fills y[n_rows] and returns the checksum. */
uint64_t lro_demo_q8_gemv(size_t n_cols, size_t n_rows, float *y);

/* The reference's acceptance test for one output: both finite and
 * |a - e| <= 1e-4 + 1e-4 |e|.  native-cuda/src/lib.rs:37-53.
 * Returns -1 when all pass, else the first failing index. */
long lro_validate(const float *actual, const double *expected, size_t n);

#ifdef __cplusplus
}
#endif
#endif
