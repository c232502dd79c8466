// Host-callable launchers of the gfx950 kernels (kernels.hip).
#pragma once
#include <hip/hip_runtime.h>

#include "matview.h"

namespace nh {

// CU count and the largest dynamic LDS a workgroup may ask for on this device.  Held once per process: the
// first call sets them, a later call returns false when its values differ (the caller refuses the executor).
bool set_device_limits(int cu_count, size_t lds_per_block);

// What the device's converts give for nibble bytes: the value of byte 0x01 under the fp8 (E4M3) unpack when bytes
// 0..15 decode linearly (n * unit, a power of two), else 0 (nibble kernels then take the byte-convert path);
// whether the packed fp8 -> bf16 convert with scale 512 gives the integers 0..15; whether the signed 4-bit
// convert with a byte select gives (n - 8) / 16.  Probed by a 16-thread kernel, held once per process like the limits.
hipError_t probe_nibble_converts(hipStream_t stream, float *unit_out, bool *bf16_out, bool *i4_out);
bool set_nibble_converts(float unit, bool bf16_exact, bool i4_exact);

// Scatter the GGUF bytes at src_device (device memory) into the planes of m.
hipError_t launch_repack(hipStream_t stream, const MatView &m, const void *src_device);
// The tiled copy (matview.h) from the planes of the same matrix, both on the device; tiled.s0..s3 hold the units
// per row of each plane.
hipError_t launch_retile(hipStream_t stream, const MatView &tiled, const MatView &planes);

// y[t, r] = sum_c W[r, c] x[t, c]; x and y are device pointers, token-major.
// Products of three or more tokens by a quantized matrix run on the matrix cores (two tokens: two
// single-token launches),
// read the tiled copy of the matrix and need device workspace: ws must hold gemm_workspace_bytes() for the same
// arguments (hipErrorInvalidValue otherwise).  The workspace is only used by
// work queued on `stream`, so calls on one stream may share it.
size_t gemm_workspace_bytes(const MatView *mats, const uint32_t *tokens, uint32_t n);
hipError_t launch_gemm(hipStream_t stream, const MatView &m, const MatView &tiled, uint32_t tokens, const float *x,
                       float *y, void *ws, size_t ws_bytes);
// n independent products (the experts of one MoE projection, say): consecutive
// groups of equal dtype and column count share launches, up to 8 per launch.
hipError_t launch_gemm_groups(hipStream_t stream, const MatView *mats, const MatView *tiled, const uint32_t *tokens,
                              const float *const *xs, float *const *ys, uint32_t n, void *ws, size_t ws_bytes);

// Activations that stay in the form the matrix-core kernels read (three bf16 parts per group of 16 columns, in the
// column order of the dtype that will multiply them) between products, for callers whose steps stay on the device:
// act_bytes sizes a buffer for up to max_tokens tokens of `cols` columns under a matrix of dtype `type` (0: not a
// dtype / shape of the matrix-core path); launch_act_split fills it from plain f32 rows; launch_gemm_act multiplies
// it by n matrices of that dtype and column count (tiled copies, tokens >= 3) and either writes ys (epilogue NONE:
// main launch + share sum, as launch_gemm_groups without its split launch) or applies, in the launch that sums the
// shares, the step that follows the product and leaves the result split in next_act for the next product:
//   ADD_RMSNORM (n = 1)   residual[t] += W x[t]; xn = RMSNorm(residual[t]) * norm_w -> xn_out (may be null), next_act
//                         (may be null; next_cols = rows of W)
//   SWIGLU (n = 2)        SiLU(W0 x[t]) * (W1 x[t]) -> next_act (next_cols = rows of W0 = rows of W1)
//   ADD_DEFER (n = 1)     residual[t] += W x[t], and the sixteen partial sums of squares of the new row into
//                         `partial` (16 floats per token): the normalisation itself is left to the product that
//                         reads the residual rows next (ActNorm below), so that many small workgroups take the place
//                         of one per token.  tokens <= ACT_DEFER_MAX_TOKENS.
// ws must hold gemm_act_workspace_bytes() for the same arguments.  hipErrorInvalidValue = not this path's case,
// nothing launched.
enum { ACT_EPILOGUE_NONE = 0, ACT_EPILOGUE_ADD_RMSNORM = 1, ACT_EPILOGUE_SWIGLU = 2, ACT_EPILOGUE_ADD_DEFER = 3 };
constexpr size_t ACT_NORM_MAX_ROW_BYTES = 48 * 1024;  // ADD_RMSNORM: rows of at most 12288 floats
constexpr uint32_t ACT_DEFER_MAX_TOKENS = 32;         // the products whose main launch cuts plain rows itself
constexpr size_t ACT_DEFER_PARTIAL_BYTES = ACT_DEFER_MAX_TOKENS * 16 * sizeof(float);
struct ActEpilogue {
    int kind = ACT_EPILOGUE_NONE;
    float *residual = nullptr;
    const float *norm_w = nullptr;
    float eps = 0.f;
    float *xn_out = nullptr;
    float *partial = nullptr;  // ADD_DEFER
    void *next_act = nullptr;
    uint32_t next_type = 0, next_cols = 0, next_max_tokens = 0;
};
size_t act_bytes(uint32_t type, uint32_t cols, uint32_t max_tokens);
hipError_t launch_act_split(hipStream_t stream, void *act, uint32_t type, uint32_t cols, uint32_t max_tokens, uint32_t tokens,
                            const float *x);
// x_plain (with act == nullptr): the product's own activations are `tokens` plain f32 rows; up to 32 tokens the
// main launch cuts them itself, more are cut into the workspace by a launch of their own first.
// norm (with x_plain, tokens <= ACT_DEFER_MAX_TOKENS): the plain rows are a residual stream an ADD_DEFER epilogue
// left; the product reads RMSNorm(row) * w, bit for bit what ADD_RMSNORM would have left split.
struct ActNorm {
    const float *w = nullptr, *partial = nullptr;
    float eps = 0.f;
};
size_t gemm_act_workspace_bytes(const MatView *mats, uint32_t n, uint32_t tokens, bool with_epilogue, bool plain_x = false);
hipError_t launch_gemm_act(hipStream_t stream, const MatView *tiled, uint32_t n, uint32_t tokens, void *act, uint32_t act_max_tokens,
                           const float *x_plain, const ActNorm *norm, float *const *ys, const ActEpilogue &ep, void *ws,
                           size_t ws_bytes);

// One launch for up to 8 single-token products that read the same x and share dtype
// and column count (q/k/v, gate/up).  hipErrorInvalidValue = not fusable this way;
// the caller then launches them one by one.  accumulate: y += W x instead of y = W x.
hipError_t launch_gemv_multi(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n, const float *x,
                             bool accumulate = false);

// The same launch with a prologue applied to x on its way into LDS (Q4_K matrices whose rows fit one
// launch; hipErrorInvalidValue otherwise, nothing launched):
//   prologue 1: x := x * inv_rms(x, eps) * x2   (RMSNorm, x2 = norm weights)
//   prologue 2: x := SiLU(x) * x2               (x = gate, x2 = up)
hipError_t launch_gemv_multi_prologue(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n, const float *x,
                                      bool accumulate, int prologue, const float *x2, float eps);

// h = SiLU(gate x') * (up x'), x' = x or, with prologue 1, RMSNorm(x) * x2: the two products of one launch
// combined in its epilogue (Q4_K matrices of equal shape whose launch gives every unit its own wavefront;
// hipErrorInvalidValue otherwise, nothing launched).
hipError_t launch_gemv_swiglu_pair(hipStream_t stream, const MatView &gate, const MatView &up, const float *x, float *h,
                                   int prologue, const float *x2, float eps);

// Device memory that belongs to the code object instead of an allocation: STATIC_SCRATCH_BYTES per GPU,
// usable as the workspace of launch_gemm_groups by callers that may not allocate.
// static_scratch_init(device) looks the address up (the device must be current; once per device,
// repeated calls are free); static_scratch(device) returns it, null before that.  Everything that
// uses it on one GPU shares it: such launches must not overlap.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)64 << 20;
hipError_t static_scratch_init(int device);
void *static_scratch(int device);

// dst[0, nbytes) = src[0, nbytes) (nbytes a multiple of 16): reference traffic for counter calibration.
hipError_t launch_copy(hipStream_t stream, void *dst, const void *src, size_t nbytes);
// Reads src[0, nbytes) once and writes nothing (sink: any 4 writable device bytes, never written in practice):
// the streaming-read yardstick the single-token kernels are measured against.
hipError_t launch_read(hipStream_t stream, const void *src, size_t nbytes, void *sink);
// The same copy with a grid sized by nbytes: activations between pinned host staging memory (which the
// device reads and writes directly) and device scratch, a few KB at a time.
hipError_t launch_copy_small(hipStream_t stream, void *dst, const void *src, size_t nbytes);

}  // namespace nh
