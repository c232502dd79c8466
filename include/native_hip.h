/* native-hip: C ABI of the MI355X (gfx950) matrix executor for llama-rust's
 * GGUF block-quantized matrix products.
 *
 * This is the boundary a Rust `native-hip` crate binds (one `extern "C"` block,
 * no other FFI), and the only way host code reaches the HIP kernels.  Every
 * entry point names the reference interface it stands in for; paths are
 * relative to the reference checkout.
 *
 * Conventions
 *   - Plain pointers and sizes only.  `*_len` arguments are ELEMENT counts of
 *     the buffer they follow (f32 elements, or bytes for packed weights).
 *   - Return value: LNH_OK (0) or an lnh_status error code.  The message of the
 *     most recent failure on an executor is lnh_last_error(exec); for calls
 *     without an executor (lnh_create, lnq_*) it is lnh_thread_error() /
 *     lnq_last_error(), both thread-local.  Strings stay valid until the next
 *     call on the same executor / thread.
 *   - Validation happens before any device work and never touches `y`.
 *     After any error the executor remains usable.
 *   - There is no CPU fallback: a missing device or a failed launch is an error.
 *   - An executor and its matrices are confined to one host thread at a time
 *     (the reference takes `&mut self` on every operation).
 *   - Products are token-major: x[t*cols + c], y[t*rows + r],
 *     y[t, r] = sum_c W[r, c] * x[t, c], f32 activations, f32 accumulation.
 */
#ifndef NATIVE_HIP_H
#define NATIVE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct lnh_exec lnh_exec;     /* stands in for CudaGemv   (native-cuda/src/gpu.rs:132-141) */
typedef struct lnh_matrix lnh_matrix; /* stands in for CudaMatrix (native-cuda/src/gpu.rs:125-130) */

typedef enum lnh_status {
    LNH_OK = 0,
    LNH_ERR_INVALID = 1,     /* shape / length / argument validation failed; nothing was launched */
    LNH_ERR_DEVICE = 2,      /* a HIP runtime call or kernel failed */
    LNH_ERR_OOM = 3,         /* device allocation failed (after the scratch pool was released and retried) */
    LNH_ERR_FOREIGN = 4,     /* matrix belongs to a different executor */
    LNH_ERR_UNSUPPORTED = 5  /* dtype outside F32, F16, Q4_0, Q4_K, Q5_0, Q5_1, Q6_K, Q8_0 */
} lnh_status;

/* ggml type ids (langtax/src/gguf.rs:245-258); the Rust shim maps GemmKind to these. */
enum {
    LNH_TYPE_F32 = 0,
    LNH_TYPE_F16 = 1,
    LNH_TYPE_Q4_0 = 2,
    LNH_TYPE_Q5_0 = 6,
    LNH_TYPE_Q5_1 = 7,
    LNH_TYPE_Q8_0 = 8,
    LNH_TYPE_Q4_K = 12,
    LNH_TYPE_Q6_K = 14
};

/* ------------------------------------------------------------------ executor */

/* CudaGemv::new(device_ordinal)            native-cuda/src/gpu.rs:148-161 */
int lnh_create(int device_ordinal, lnh_exec **out);
void lnh_destroy(lnh_exec *exec);
/* CudaGemv::memory_info -> (free, total)   native-cuda/src/gpu.rs:164-175 */
int lnh_memory_info(lnh_exec *exec, size_t *free_bytes, size_t *total_bytes);
/* Err(String) of the last failed call on this executor ("" if none). */
const char *lnh_last_error(const lnh_exec *exec);
/* Message of the last failed lnh_create / host-only helper on this thread. */
const char *lnh_thread_error(void);

/* ------------------------------------------------------------------ resident matrices */

/* CudaGemv::upload(rows, cols, &[f32])     native-cuda/src/gpu.rs:264-277
 * Same checks and messages as Shape::checked (native-cuda/src/lib.rs:19-34). */
int lnh_upload_f32(lnh_exec *exec, size_t rows, size_t cols, const float *weights, size_t weights_len,
                   lnh_matrix **out);
/* Packed residency: takes the GGUF bytes of a rows x cols tensor as they lie in
 * the file and keeps them packed in HBM.  Replaces the host-side expansion to
 * F32 at langtax/src/quant.rs:6746-6755 followed by upload (native_gpu.rs:190-194).
 * `nbytes` must equal rows * row_bytes(type, cols); cols must be a whole number
 * of blocks (32 for Q4_0/Q5_0/Q5_1/Q8_0, 256 for Q4_K/Q6_K).
 * A quantized matrix has two layouts in HBM: the one the single-token kernels
 * stream is made here; the one the multi-token (matrix-core) kernels stream is
 * made from it by the first product of three or more tokens (or by
 * lnh_matrix_prepare), so a matrix that only ever meets one token at a time
 * (an output head, an embedding table) takes its GGUF size once, the others
 * about twice (lnh_matrix_info reports the figure as it stands). */
int lnh_upload_packed(lnh_exec *exec, uint32_t ggml_type, size_t rows, size_t cols, const uint8_t *bytes,
                      size_t nbytes, lnh_matrix **out);
/* Same, from bytes that already sit in device memory of this executor's GPU. */
int lnh_upload_packed_device(lnh_exec *exec, uint32_t ggml_type, size_t rows, size_t cols,
                             const void *device_bytes, size_t nbytes, lnh_matrix **out);
/* Drop of a CudaMatrix.  Safe after its executor was destroyed. */
void lnh_matrix_free(lnh_matrix *matrix);
/* device_bytes: what the matrix holds in HBM now (it grows once, when the multi-token layout is made). */
int lnh_matrix_info(const lnh_matrix *matrix, uint32_t *ggml_type, size_t *rows, size_t *cols,
                    size_t *device_bytes);
/* Makes now whatever products of up to max_tokens tokens by this matrix will need beyond the upload (the
 * multi-token layout when max_tokens >= 3 and the dtype is quantized): allocates, runs on the executor's own
 * stream and returns when the copy is complete.  For callers that will run such products where allocating is
 * not possible: inside a stream capture (a product that finds the layout missing there fails with
 * LNH_ERR_INVALID before anything is launched) or through lnh_gemm_device_noalloc.  No counterpart in the
 * reference, whose resident form is one F32 array. */
int lnh_matrix_prepare(lnh_exec *exec, const lnh_matrix *matrix, size_t max_tokens);

/* ------------------------------------------------------------------ products (host buffers) */

/* CudaGemv::gemv_resident(matrix, input, output)          native-cuda/src/gpu.rs:280-335 */
int lnh_gemv(lnh_exec *exec, const lnh_matrix *matrix, const float *x, size_t x_len, float *y, size_t y_len);
/* CudaGemv::gemm_resident(matrix, tokens, input, output)  native-cuda/src/gpu.rs:351-417
 * (tokens == 1 runs the GEMV kernel; native_gpu::matmul always calls this one). */
int lnh_gemm(lnh_exec *exec, const lnh_matrix *matrix, size_t tokens, const float *x, size_t x_len, float *y,
             size_t y_len);
/* CudaGemv::gemv(weights, input, output): upload + product native-cuda/src/gpu.rs:339-347 */
int lnh_gemv_once(lnh_exec *exec, const float *weights, size_t weights_len, const float *x, size_t x_len,
                  float *y, size_t y_len);
/* Expert-grouped GEMM: group g multiplies tokens[g] packed rows of x by mats[g].
 * Stands in for the per-expert loop of three gemm calls at
 * langtax/src/decode.rs:10035-10058 / 10148-10261 (one call per projection).
 * x holds the groups' token rows back to back (sum_g tokens[g]*cols[g] floats),
 * y likewise (sum_g tokens[g]*rows[g]).  Groups with tokens[g] == 0 are skipped. */
int lnh_gemm_grouped(lnh_exec *exec, size_t n_groups, const lnh_matrix *const *mats, const size_t *tokens,
                     const float *x, size_t x_len, float *y, size_t y_len);

/* Several matrices times one shared input in a single call: stands in for the back-to-back
 * gemm calls on the same activations at langtax/src/decode.rs:2754-2790 (q, k, v) and
 * 2968-2979 (gate, up).  x holds tokens * cols floats (all matrices have the same column
 * count); y receives the products back to back, matrix after matrix (tokens * rows[i] each).
 * One input copy, one launch for single-token calls, one output copy. */
int lnh_gemm_shared(lnh_exec *exec, size_t n_mats, const lnh_matrix *const *mats, size_t tokens, const float *x,
                    size_t x_len, float *y, size_t y_len);

/* ------------------------------------------------------------------ products (device buffers) */

/* The same products with x and y already in this GPU's memory, enqueued on
 * `stream` (a hipStream_t; NULL = the executor's own stream) without any host
 * synchronisation.  No counterpart in the reference, whose every call copies
 * through the host (native-cuda/src/gpu.rs:301-303, 332-334).
 * Products of three or more tokens by a quantized matrix use a workspace that
 * belongs to the executor and grows on demand (growing allocates, so it cannot
 * happen while `stream` is being captured into a graph: such a call fails with
 * LNH_ERR_INVALID before anything is launched - run the largest shape once
 * before capturing; a workspace that captured launches point at stays
 * allocated until the executor is destroyed, also after a later call has
 * made the executor move to a larger one).  Calls of one executor must therefore be enqueued on
 * one stream at a time; calls that overlap on different streams race on it.
 * Every device buffer a call reads (device_x, device_x2, device_residual, device_norm_w; in this and the following
 * sections) must be 16-byte aligned, as anything hipMalloc returns is: LNH_ERR_INVALID otherwise. */
int lnh_gemm_device(lnh_exec *exec, const lnh_matrix *matrix, size_t tokens, const float *device_x,
                    float *device_y, void *stream);
int lnh_gemm_grouped_device(lnh_exec *exec, size_t n_groups, const lnh_matrix *const *mats,
                            const size_t *tokens, const float *device_x, float *device_y, void *stream);
/* lnh_gemm_device for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid it).  No counterpart in the reference.  Same product, same
 * kernels, same results as lnh_gemm_device, but the workspace of the multi-token kernels is a fixed
 * array inside the library's device code (LNH_NOALLOC_WORKSPACE_BYTES per GPU, held from lnh_create on
 * that GPU until the process ends) instead of the executor's grow-on-demand allocation: the call
 * never allocates or frees.  A product that needs more fails with LNH_ERR_INVALID
 * (the message states the need) before anything is launched; so does a product of three or more tokens by a
 * quantized matrix whose multi-token layout has not been made yet (lnh_matrix_prepare, or any earlier such product
 * through an allocating entry point, makes it).  Every call on one GPU, from any executor, uses the
 * same array and nothing in it outlives a call: calls that may overlap on one GPU (different streams,
 * different threads) race on it and must be ordered by the caller. */
#define LNH_NOALLOC_WORKSPACE_BYTES ((size_t)64 << 20)
int lnh_gemm_device_noalloc(lnh_exec *exec, const lnh_matrix *matrix, size_t tokens, const float *device_x,
                            float *device_y, void *stream);

/* n independent products enqueued back to back in one call: product i multiplies
 * tokens[i] rows at device_x[i] by mats[i] into device_y[i].  This is how a decode
 * step's products (langtax/src/decode.rs:2755-2996: q, k, v, o, gate, up, down per
 * layer) are issued without a host round trip each. */
int lnh_gemm_batch_device(lnh_exec *exec, size_t n, const lnh_matrix *const *mats, const size_t *tokens,
                          const float *const *device_x, float *const *device_y, void *stream);
/* Up to eight single-token products that read the same device_x (equal dtype and column count), one
 * launch: device_ys[i] = mats[i] * x, or, with accumulate != 0, device_ys[i] += mats[i] * x.  The
 * second form is the product followed by the residual addition of langtax/src/decode.rs:2957 and
 * 3043 (x = attn_proj + residual, x = ffn_out + residual) done in the product's epilogue; a
 * y must then not alias x.  LNH_ERR_UNSUPPORTED when a row is too long for the single-token kernels. */
int lnh_gemv_shared_device(lnh_exec *exec, size_t n_mats, const lnh_matrix *const *mats, const float *device_x,
                           float *const *device_ys, int accumulate, void *stream);
/* The same launch with the operation that precedes the product in the decode graph applied to x as the
 * kernel stages it (x itself is left as it is):
 *   LNH_PROLOGUE_RMSNORM  x := x * inv_rms(x, eps) * x2, x2 = norm weights   (langtax/src/decode.rs:11498-11513,
 *                         called at 2745 and 2960 before the q/k/v and gate/up products)
 *   LNH_PROLOGUE_SWIGLU   x := SiLU(x) * x2, x = gate, x2 = up               (decode.rs:11826-11830, 2981-2984)
 * LNH_ERR_UNSUPPORTED (nothing launched) unless the matrices are Q4_K with rows of at most 16384 columns:
 * the caller then runs the operation as a kernel of its own and calls lnh_gemv_shared_device. */
enum { LNH_PROLOGUE_NONE = 0, LNH_PROLOGUE_RMSNORM = 1, LNH_PROLOGUE_SWIGLU = 2 };
int lnh_gemv_fused_device(lnh_exec *exec, size_t n_mats, const lnh_matrix *const *mats, const float *device_x,
                          float *const *device_ys, int accumulate, int prologue, const float *device_x2, float eps,
                          void *stream);
/* device_h = SiLU(gate x') * (up x'), x' = device_x or, with LNH_PROLOGUE_RMSNORM, its RMSNorm times
 * device_x2: the gate and up products of one launch (langtax/src/decode.rs:2968-2979) and the element-wise
 * step that follows them (decode.rs:2981-2984, 11826-11830) in the launch's epilogue, so that neither gate
 * nor up is written out.  LNH_ERR_UNSUPPORTED (nothing launched) unless both are Q4_K of one shape with
 * rows of 2048 to 16384 columns and the launch gives every 256-column unit its own wavefront (up to about
 * 67 M weights per matrix on this part): the caller then uses lnh_gemv_fused_device. */
int lnh_gemv_swiglu_device(lnh_exec *exec, const lnh_matrix *gate, const lnh_matrix *up, const float *device_x,
                           float *device_h, int prologue, const float *device_x2, float eps, void *stream);
/* Activations kept in the form the multi-token kernels read, for steps that stay on the device.  No counterpart in
 * the reference, whose every product takes and returns plain f32 rows on the host (langtax/src/native_gpu.rs:124-213).
 * A multi-token product is up to three launches: the activations are cut into three bf16 parts in the matrix's column
 * order (a launch of its own for more than 32 tokens; the matrix-core launch does it for fewer), the matrix-core launch
 * writes one partial result per share of the columns, a last launch sums the shares.
 * Between two products of a decode step lies only element-wise work; lnh_gemm_act_device does that work in the
 * launch that sums the shares and leaves its result already cut for the next matrix, so a chain of products costs
 * two launches each instead of three plus the element-wise kernels.
 *   lnh_act_create        a buffer for up to max_tokens tokens of `cols` columns under matrices of `ggml_type`
 *                         (LNH_ERR_UNSUPPORTED for F32 / F16, whose products take plain rows)
 *   lnh_act_split_device  fills it from `tokens` plain f32 rows on the device
 *   lnh_gemm_act_device   multiplies it by up to 8 resident matrices of that dtype and column count (tokens >= 3;
 *                         LNH_ERR_UNSUPPORTED below: single-token launches take plain rows), then
 *     LNH_EPILOGUE_NONE         device_ys[i] = mats[i] x                        (any number of matrices)
 *     LNH_EPILOGUE_ADD_RMSNORM  device_residual += mats[0] x, then RMSNorm of the new residual times device_norm_w
 *                               (langtax/src/decode.rs:2957 / 3043 and 11498-11513) into device_xn (plain rows, may
 *                               be NULL) and into `next` (may be NULL), whose columns are the matrix's rows;
 *                               LNH_ERR_UNSUPPORTED for matrices of more than 12288 rows
 *     LNH_EPILOGUE_SWIGLU       SiLU(mats[0] x) * (mats[1] x) (decode.rs:11826-11830, 2981-2984) into `next`
 *     LNH_EPILOGUE_ADD_RMSNORM_DEFERRED  as ADD_RMSNORM into `next` (required; device_xn must be NULL), for at most
 *                               32 tokens (LNH_ERR_UNSUPPORTED beyond): only the addition and the rows' sums of squares
 *                               are formed now, by many small workgroups instead of one per token, and the product
 *                               that reads `next` scales the rows as it loads them.  device_residual and
 *                               device_norm_w must stay as they are until that product has run, and it must be
 *                               called with the same token count.  Same bits as ADD_RMSNORM.
 *   lnh_gemm_plain_act_device  the same product and epilogues with the product's own activations as `tokens` plain
 *                         f32 rows at device_x (the first product of a chain, or one whose input another kernel of
 *                         the caller wrote: the attention output): up to 32 tokens no launch is spent on cutting them
 *   Sums run in share order and the row operations in the order of a one-workgroup-per-row kernel, so results
 *   equal those of the three-launch product followed by separate element-wise kernels bit for bit.
 * Like lnh_gemm_device it may grow the executor's workspace and make a matrix's multi-token layout on first use;
 * neither is possible while the stream is being captured (run the step once before capturing it). */
typedef struct lnh_act lnh_act;
enum { LNH_EPILOGUE_NONE = 0, LNH_EPILOGUE_ADD_RMSNORM = 1, LNH_EPILOGUE_SWIGLU = 2, LNH_EPILOGUE_ADD_RMSNORM_DEFERRED = 3 };
int lnh_act_create(lnh_exec *exec, uint32_t ggml_type, size_t cols, size_t max_tokens, lnh_act **out);
void lnh_act_free(lnh_act *act);
int lnh_act_split_device(lnh_exec *exec, lnh_act *act, size_t tokens, const float *device_x, void *stream);
int lnh_gemm_act_device(lnh_exec *exec, size_t n_mats, const lnh_matrix *const *mats, const lnh_act *x, size_t tokens,
                        float *const *device_ys, int epilogue, float *device_residual, const float *device_norm_w, float eps,
                        float *device_xn, lnh_act *next, void *stream);
int lnh_gemm_plain_act_device(lnh_exec *exec, size_t n_mats, const lnh_matrix *const *mats, const float *device_x,
                              size_t tokens, float *const *device_ys, int epilogue, float *device_residual,
                              const float *device_norm_w, float eps, float *device_xn, lnh_act *next, void *stream);
/* Measurement aid, no counterpart in the reference: a plain device-to-device copy kernel
 * (nbytes a multiple of 16) whose known traffic calibrates HBM byte counters. */
int lnh_calibration_copy(lnh_exec *exec, void *device_dst, const void *device_src, size_t nbytes, void *stream);
/* Measurement aid, no counterpart in the reference: a kernel that reads nbytes (a multiple of 16, at least 32)
 * of device memory once, requested the way the single-token kernels request their weights, and does nothing
 * with them.  Its duration at the sizes of a decode step's launches is the ceiling those launches are held
 * against beside the 8 TB/s figure. */
int lnh_calibration_read(lnh_exec *exec, const void *device_src, size_t nbytes, void *stream);
/* Block the host until everything enqueued on the executor's own stream is done. */
int lnh_synchronize(lnh_exec *exec);

/* ------------------------------------------------------------------ host-only helpers */

/* Shape::checked(rows, cols, weights, input)   native-cuda/src/lib.rs:19-34 */
int lnh_shape_checked(size_t rows, size_t cols, size_t weights_len, size_t input_len, uint32_t *rows_out,
                      uint32_t *cols_out);
/* validate(actual, expected)                   native-cuda/src/lib.rs:37-53
 * Returns LNH_OK when every |a-e| <= 1e-4 + 1e-4|e| with both finite. */
int lnh_validate(const float *actual, size_t actual_len, const double *expected, size_t expected_len);
/* Packed bytes of one row, 0 if cols is not a whole number of blocks or the type is unknown
 * (langtax/src/quant.rs:4210-4218, 4254-4284, 5647-5682). */
size_t lnh_row_bytes(uint32_t ggml_type, size_t cols);
/* Device bytes a packed rows x cols matrix holds once it has met products of up to `tokens` tokens: the
 * single-token layout, plus the multi-token layout when such a product reads it (tokens >= 3, quantized
 * dtypes).  What a residency cache charges before the upload, where the reference charges rows * cols * 4
 * (langtax/src/native_gpu.rs:178-182); after the product lnh_matrix_info gives the figure as it stands.
 * 0 for an unknown dtype, columns that are not whole blocks, or a size beyond size_t. */
size_t lnh_resident_bytes(uint32_t ggml_type, size_t rows, size_t cols, size_t tokens);

/* ------------------------------------------------------------------ dispatch + residency
 * The layer above the executor: the twin of langtax/src/native_gpu.rs plus the
 * validation of quant::native_matmul (langtax/src/quant.rs:6683-6758), i.e. what
 * gemv_<t>_f32 / gemm_<t>_f32 (quant.rs:6144-6293, 6366-6478, 6891-7199) run
 * when the GPU backend is compiled in.  One executor and one residency cache
 * per host thread; identity of a weight is its dtype, shape and ALL its bytes. */

/* gemv_<t>_f32(n_cols, w, x, y):  n_rows = y_len */
int lnq_gemv(uint32_t ggml_type, size_t n_cols, const uint8_t *w, size_t w_len, const float *x, size_t x_len,
             float *y, size_t y_len);
/* gemm_<t>_f32(n_cols, n_tokens, w, x, y):  n_rows = y_len / n_tokens */
int lnq_gemm(uint32_t ggml_type, size_t n_cols, size_t n_tokens, const uint8_t *w, size_t w_len,
             const float *x, size_t x_len, float *y, size_t y_len);
/* The per-expert products of one MoE projection in one call; part g is the
 * byte slice of expert g (langtax/src/decode.rs:9853-9913).  All parts share
 * dtype, n_cols and n_rows. */
int lnq_gemm_grouped(uint32_t ggml_type, size_t n_cols, size_t n_rows, size_t n_groups,
                     const uint8_t *const *parts, size_t part_len, const size_t *tokens, const float *x,
                     size_t x_len, float *y, size_t y_len);
const char *lnq_last_error(void);
/* Residency policy, exposed for host tests (native_gpu.rs:20-43, 217-360). */
int lnq_parse_cache_bytes(const char *value_or_null, int *is_auto, size_t *bytes);
size_t lnq_automatic_cache_bytes(size_t free_bytes, size_t total_bytes);
int lnq_admission_requires_eviction(size_t used, size_t incoming, size_t limit);
/* Counters of this thread's cache; any pointer may be NULL. */
void lnq_cache_stats(size_t *entries, size_t *bytes, size_t *limit, size_t *hits, size_t *misses);
/* Drop this thread's executor and cache (the next call re-reads LLAMA_HIP_CACHE_BYTES). */
void lnq_reset(void);

#ifdef __cplusplus
}
#endif
#endif
