/*
 * native-hip, host side of a Llama decode (dense or routed feed-forward): the caller of the matrix products.
 *
 * The matrix executor (native_hip.h) replaces one seam of the reference; this header is
 * the code either side of that seam, restated in C++ so that an end-to-end greedy decode
 * of a GGUF model can run and be checked without the reference's Rust toolchain:
 *
 *   GGUF v3 reader / writer             langtax/src/gguf.rs:64-68, 626-702, 728-828, 922-947
 *   model load (llama architecture)     langtax/src/decode.rs:1910-1958, 2050-2090, 7461-7475
 *   forward pass of n tokens            langtax/src/decode.rs:2710-3099 (llama branch; routed experts 9938-10292)
 *     RMSNorm 11498-11513, RoPE (adjacent pairs) 11578-11602, attention 11126-11197,
 *     softmax 12021-12033, SiLU 11826-11830, argmax 12104-12114, embedding 10761-10800
 *   paged K/V addressing                langtax/src/kv_page.rs:410-438, decode.rs:12059-12100
 *
 * All host arithmetic is f32 in the reference's operation order.  Every weight product
 * goes through one of three routes, chosen per model:
 *   LNM_PRODUCTS_RESIDENT  matrices uploaded once (lnh_upload_packed), products by lnh_gemm
 *   LNM_PRODUCTS_DISPATCH  lnq_gemv / lnq_gemm, i.e. the reference's call shape with the
 *                          content-identified residency cache behind it
 *   LNM_PRODUCTS_CALLBACK  a function of the caller (tests plug their CPU checker in here;
 *                          the library itself contains no CPU implementation of a product)
 *
 * Errors: every call returns 0 on success; otherwise a non-zero code with the text in
 * lnm_last_error() (thread-local, valid until the next lnm call on the thread).
 */
#ifndef NATIVE_HIP_LLAMA_H
#define NATIVE_HIP_LLAMA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct lnm_model lnm_model;
typedef struct lnm_session lnm_session;

typedef struct lnm_hparams {
    uint32_t n_layer, n_embd, n_head, n_head_kv, n_ff, n_vocab, head_dim, n_rot;
    float rope_base, rms_eps;
    uint32_t block_type, embd_type, output_type; /* ggml type ids of blk.0.attn_q, token_embd, output */
    uint32_t n_expert, n_expert_used;            /* llama.expert_count / expert_used_count; 0, 0: dense feed-forward */
} lnm_hparams;

enum { LNM_PRODUCTS_RESIDENT = 0, LNM_PRODUCTS_DISPATCH = 1, LNM_PRODUCTS_CALLBACK = 2 };

/* y[t * n_rows + r] = sum_c W[r, c] * x[t * n_cols + c]; returns 0 on success. */
typedef int (*lnm_matmul_fn)(void *user, uint32_t ggml_type, size_t n_rows, size_t n_cols, size_t n_tokens,
                             const uint8_t *w, size_t w_len, const float *x, float *y);

const char *lnm_last_error(void);

/* Maps the file and validates the llama hyper-parameters and tensor shapes. */
int lnm_load(const char *gguf_path, lnm_model **out);
/* Same from memory; the bytes are copied. */
int lnm_load_bytes(const uint8_t *bytes, size_t len, lnm_model **out);
void lnm_free(lnm_model *model);
int lnm_info(const lnm_model *model, lnm_hparams *out);
/* Route of the products; `fn` and `user` are used by LNM_PRODUCTS_CALLBACK only.  Default: RESIDENT. */
int lnm_set_products(lnm_model *model, int route, lnm_matmul_fn fn, void *user);

/* One sequence with a paged K/V cache of `kv_block` positions per block.  `block_ids` (may be
 * NULL) gives the physical block of each logical block, any permutation of 0 .. n_block_ids-1;
 * NULL allocates blocks in order as the sequence grows. */
int lnm_session_new(lnm_model *model, size_t kv_block, const uint32_t *block_ids, size_t n_block_ids,
                    lnm_session **out);
/* A session whose whole decode step stays on the GPU (needs the RESIDENT route): embedding row, RMSNorm,
 * RoPE, attention over the paged K/V cache (device memory, same addressing), SiLU(gate)*up and the greedy
 * pick are small kernels between the single-token products, the residual additions are done in the
 * epilogue of the o and down products, and one step is one HIP graph whose replays pass the picked token
 * on in device memory.  No counterpart in the reference, whose every product returns to the host
 * (langtax/src/native_gpu.rs:124-213); the arithmetic of the small kernels is the host code's, element for
 * element, except for the order of the sums inside RMSNorm and the softmax denominator.
 * `max_positions` sizes the cache (rounded up to whole blocks).  A batch of n >= 3 tokens runs its first n - 1
 * tokens through the multi-token products in chunks of up to 128 (only their K and V are kept) and the last one
 * as a step; the environment variable LLAMA_HIP_DECODE_STEP_PREFILL makes every token a step. */
int lnm_session_new_device(lnm_model *model, size_t kv_block, const uint32_t *block_ids, size_t n_block_ids,
                           size_t max_positions, lnm_session **out);
/* A device session for `n_sequences` (at most 128) independent sequences of up to `max_positions` each, decoded
 * together: every step processes one token of every sequence, the weight products as one multi-token product
 * each (the continuous-batching shape of langtax/src/engine.rs:1423-1510, where M = the number of running
 * sequences), attention per sequence over its own blocks of the paged cache.  Like the device session above it
 * has no counterpart in the reference, whose batches return to the host after every product.  Freed with
 * lnm_session_free; lnm_forward and lnm_generate_greedy refuse it. */
int lnm_session_new_device_batch(lnm_model *model, size_t kv_block, size_t n_sequences, size_t max_positions,
                                 lnm_session **out);
/* Greedy decode of all sequences from scratch: `prompts` holds the prompts one after the other, prompt_lens[b]
 * tokens for sequence b (at least 1); out[b * n_new + i] is token i of sequence b.  Prompts run one sequence
 * after the other (all tokens but the last in chunks of up to 128, K and V only), then n_new steps of all
 * sequences together, step 0 taking every prompt's last token. */
int lnm_batch_generate_greedy(lnm_session *session, const uint32_t *prompts, const size_t *prompt_lens, size_t n_new,
                              uint32_t *out, double *prefill_seconds, double *decode_seconds);
void lnm_session_free(lnm_session *session);
/* Runs the n tokens as one batch at positions past .. past+n-1 (products with n_tokens = n) and
 * writes the logits of the last one (n_vocab floats). */
int lnm_forward(lnm_session *session, const uint32_t *tokens, size_t n, float *logits);
/* A whole prompt for a session that may already hold part of it (the reference's prompt_logits with prefix
 * reuse, langtax/src/decode.rs:1106-1196, 3931-3962; its test scenario langtax/tests/native_cuda_parity.rs:236-249):
 * the session remembers the tokens it has forwarded; positions 0 .. lcp-1 of the cache are kept, where lcp is
 * the longest common prefix of those tokens and `tokens`, the rest is forwarded as one batch at positions
 * lcp .. n-1 and replaces what the cache held there.  A full hit (lcp == n) recomputes the last token, so the
 * logits are always those of tokens[n-1].  `prefix_hit` (may be NULL) receives lcp.  A session whose remembered
 * tokens do not cover its cache (after a failed call) starts over from position 0. */
int lnm_prompt(lnm_session *session, const uint32_t *tokens, size_t n, float *logits, size_t *prefix_hit);
/* Greedy decode: the prompt as one batch, then one token at a time; out[0] comes from the prompt's
 * logits, out[i] from decode step i, n_new tokens and n_new - 1 decode steps in all.  The two
 * wall times (seconds) may be NULL. */
int lnm_generate_greedy(lnm_session *session, const uint32_t *prompt, size_t n_prompt, size_t n_new,
                        uint32_t *out, double *prefill_seconds, double *decode_seconds);

/* Where a session's wall time went so far: inside weight products (host round trips included),
 * inside RoPE + attention, and how many products it ran.  Any pointer may be NULL. */
int lnm_session_timing(const lnm_session *session, double *products_seconds, double *attention_seconds,
                       uint64_t *n_products);

/* Building blocks, exported so that each can be checked on its own. */
int lnm_dequant_row(uint32_t ggml_type, size_t n_cols, const uint8_t *row, size_t row_len, float *y);
int lnm_rmsnorm(float *x, const float *w, size_t n, float eps);
int lnm_rope(float *head, size_t head_len, size_t pos, size_t n_rot, float base);
void lnm_softmax(float *x, size_t n);
uint32_t lnm_argmax(const float *x, size_t n);
/* Routed feed-forward (langtax/src/decode.rs:9938-10116, 10148-10292, 10366-10409).
 * lnm_topk: indices of the k largest of n values, descending, ties to the lower index (decode.rs:11363-11379).
 * lnm_router_weights: weights[j] = probs[order[j]], divided by max(their sum, 2^-14) when norm_w (decode.rs:11391-11409).
 * lnm_moe_ffn: the whole routed feed-forward of `layer` on n_tokens rows x (n_embd each, already normed) by the
 * model's product route: router product, softmax, top-k, renormalised weights, tokens bucketed per expert in
 * ascending expert order, gate / up products, SiLU(gate) * up, down product, ffn_out[t] += y * w. */
int lnm_topk(const float *values, size_t n, size_t k, uint32_t *order);
int lnm_router_weights(const float *probs, const uint32_t *order, size_t k, int norm_w, float *weights);
int lnm_moe_ffn(lnm_model *model, size_t layer, size_t n_tokens, const float *x, float *ffn_out);

/* A random dense llama model written as GGUF v3: packed blocks are drawn directly (codes uniform,
 * block scales sized so that the dequantized weights have mean 0 and standard deviation
 * `weight_std`), norm weights are 1 + N(0, 0.05).  Deterministic in `seed`. */
typedef struct lnm_synth_spec {
    uint32_t n_layer, n_embd, n_head, n_head_kv, n_ff, n_vocab;
    uint32_t block_type, embd_type, output_type; /* ggml type ids */
    float rope_base, rms_eps, weight_std;
    uint64_t seed;
    uint32_t n_expert, n_expert_used; /* > 0: routed feed-forward (ffn_gate_inp F32 + 3-D ffn_{gate,up,down}_exps of block_type) */
} lnm_synth_spec;
int lnm_write_synthetic_llama(const char *gguf_path, const lnm_synth_spec *spec);

/* GGUF container checks without a model: number of tensors and keys, or an error. */
int lnm_gguf_inspect(const uint8_t *bytes, size_t len, size_t *n_tensors, size_t *n_kv, size_t *alignment);
/* Tensor i of a GGUF blob: name (copied, NUL-terminated, truncated to name_cap), type, dims, byte range. */
int lnm_gguf_tensor(const uint8_t *bytes, size_t len, size_t index, char *name, size_t name_cap, uint32_t *ggml_type,
                    uint64_t shape[4], uint32_t *n_dims, size_t *start, size_t *end);

#ifdef __cplusplus
}
#endif
#endif
