// C ABI of the executor (include/native_hip.h): device context, resident
// matrices, scratch reuse and the validation rules of the reference's
// CudaGemv / CudaMatrix / Shape / validate
// (native-cuda/src/gpu.rs:125-418, native-cuda/src/lib.rs:8-53).
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/native_hip.h"
#include "kernels.h"

static_assert(LNH_NOALLOC_WORKSPACE_BYTES == nh::STATIC_SCRATCH_BYTES, "header and device array disagree");

namespace {

struct Ctx {
    int device;
    uint64_t id;
};

std::atomic<uint64_t> g_next_ctx{1};
thread_local std::string t_error;

}  // namespace

struct lnh_matrix {
    std::shared_ptr<Ctx> ctx;
    void *dev = nullptr;
    size_t dev_bytes = 0;
    nh::MatView view{};   // planes the single-token kernels read
    // Row-interleaved copy the multi-token kernels read (quantized dtypes).  Made from the planes by the first
    // product that needs it (or lnh_matrix_prepare), so that a matrix only ever used with one token (an output
    // head, an embedding table) is resident once.  p0 is null until then.
    mutable std::mutex lazy;
    mutable void *dev_tiled = nullptr;
    mutable size_t tiled_bytes = 0;
    mutable nh::MatView tiled{};
};

struct lnh_act {
    std::shared_ptr<Ctx> ctx;
    void *dev = nullptr;
    size_t bytes = 0;  // of the split form; the partial sums of a deferred norm follow it in the allocation
    uint32_t type = 0, cols = 0, max_tokens = 0;
    // Set by LNH_EPILOGUE_ADD_RMSNORM_DEFERRED, cleared by everything else that fills the activations: the
    // content is RMSNorm(deferred_x rows) * deferred_w, formed by the product that reads it.  Host state, in the
    // order of the calls that enqueue the work, like the device content it describes.
    const float *deferred_x = nullptr, *deferred_w = nullptr;
    float deferred_eps = 0.f;
    uint32_t deferred_tokens = 0;
    float *partial() const { return reinterpret_cast<float *>(static_cast<uint8_t *>(dev) + bytes); }
};

struct lnh_exec {
    std::shared_ptr<Ctx> ctx;
    hipStream_t stream = nullptr;
    float *d_in = nullptr, *d_out = nullptr;  // device scratch, grow-only
    size_t in_cap = 0, out_cap = 0;           // capacities in floats
    float *h_in = nullptr, *h_out = nullptr;  // pinned host staging for small calls, grow-only
    size_t hin_cap = 0, hout_cap = 0;
    void *d_ws = nullptr;                     // kernel workspace (multi-token products), grow-only
    std::vector<void *> ws_retired;           // earlier, smaller workspaces: captured graphs may still point at them
    size_t ws_cap = 0;
    std::string err;
};

namespace {

int fail(lnh_exec *e, int code, const std::string &msg) {
    if (e) e->err = msg;
    t_error = msg;
    return code;
}

// The kernels read activations, norm weights and residual rows in 16-byte pieces.
bool misaligned(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }

int hip_fail(lnh_exec *e, hipError_t h, const char *what) {
    (void)hipGetLastError();  // clear the sticky error so the executor stays usable
    int code = h == hipErrorOutOfMemory ? LNH_ERR_OOM : LNH_ERR_DEVICE;
    return fail(e, code, std::string(what) + ": " + hipGetErrorString(h));
}

bool mul_overflows(size_t a, size_t b, size_t *out) {
    if (a != 0 && b > SIZE_MAX / a) return true;
    *out = a * b;
    return false;
}

// native-cuda/src/lib.rs:19-34, message for message.
const char *shape_checked(size_t rows, size_t cols, size_t weights, size_t input, uint32_t *r32, uint32_t *c32) {
    if (rows == 0 || cols == 0) return "GEMV dimensions must be positive";
    size_t elements;
    if (mul_overflows(rows, cols, &elements)) return "GEMV shape overflow";
    if (elements > UINT32_MAX) return "GEMV matrix exceeds u32 indexing";
    if (weights != elements || input != cols) return "GEMV buffer lengths do not match shape";
    if (rows > UINT32_MAX) return "GEMV rows exceed u32";
    if (cols > UINT32_MAX) return "GEMV columns exceed u32";
    if (r32) *r32 = (uint32_t)rows;
    if (c32) *c32 = (uint32_t)cols;
    return nullptr;
}

// Device scratch that recurring shapes reuse across layers and tokens
// (native-cuda/src/gpu.rs:143-262).  Grow-only; an out-of-memory on growth
// releases both buffers and retries once (gpu.rs:198-210).
int ensure_scratch(lnh_exec *e, size_t in_floats, size_t out_floats) {
    auto grow = [&](float *&buf, size_t &cap, size_t want) -> hipError_t {
        if (want <= cap) return hipSuccess;
        if (buf) {
            (void)hipFree(buf);
            buf = nullptr;
            cap = 0;
        }
        size_t n = want < 4096 ? 4096 : (want + 3) & ~(size_t)3;  // whole 16-byte vectors (launch_copy_small)
        hipError_t h = hipMalloc(reinterpret_cast<void **>(&buf), n * sizeof(float));
        if (h == hipSuccess) cap = n;
        return h;
    };
    for (int attempt = 0; attempt < 2; attempt++) {
        hipError_t h = grow(e->d_in, e->in_cap, in_floats);
        if (h == hipSuccess) h = grow(e->d_out, e->out_cap, out_floats);
        if (h == hipSuccess) return LNH_OK;
        (void)hipGetLastError();
        if (h != hipErrorOutOfMemory || attempt == 1) return hip_fail(e, h, "HIP scratch allocation");
        if (e->d_in) (void)hipFree(e->d_in);
        if (e->d_out) (void)hipFree(e->d_out);
        e->d_in = e->d_out = nullptr;
        e->in_cap = e->out_cap = 0;
    }
    return LNH_ERR_OOM;
}

// Pinned host staging for calls whose activations are small (a decode step's vectors, a few tokens).
// A copy from or to pageable memory makes the runtime stage and synchronise on its own, tens of
// microseconds per call; from pinned memory a small kernel moves the data at PCIe latency.  False = no
// pinned memory to be had: the caller takes the plain copies.
constexpr size_t PINNED_MAX_FLOATS = (size_t)1 << 20;  // 4 MB each way
bool ensure_pinned(lnh_exec *e, size_t in_floats, size_t out_floats) {
    auto grow = [&](float *&buf, size_t &cap, size_t want) {
        if (want <= cap) return true;
        if (buf) (void)hipHostFree(buf);
        buf = nullptr;
        cap = 0;
        size_t n = want < 16384 ? 16384 : (want + 3) & ~(size_t)3;
        if (hipHostMalloc(reinterpret_cast<void **>(&buf), n * sizeof(float), hipHostMallocDefault) != hipSuccess) {
            (void)hipGetLastError();
            buf = nullptr;
            return false;
        }
        cap = n;
        return true;
    };
    return grow(e->h_in, e->hin_cap, in_floats) && grow(e->h_out, e->hout_cap, out_floats);
}

// Workspace of the multi-token kernels.  A workspace that has become too small is kept until the executor
// goes: a caller may have captured launches that point at it into a HIP graph (a decode step that is replayed
// while another call, a longer prompt say, makes the workspace grow), and work already queued may still use
// it.  Growth is by at least half, so everything retired together is smaller than twice the live buffer.
int ensure_workspace(lnh_exec *e, hipStream_t s, size_t bytes) {
    if (bytes <= e->ws_cap) return LNH_OK;
    // Growing allocates, which a stream under capture cannot record: refuse before anything is launched
    // instead of leaving the caller with a broken capture.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (s && hipStreamIsCapturing(s, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone)
        return fail(e, LNH_ERR_INVALID,
                    "the multi-token workspace must grow to " + std::to_string(bytes) +
                        " bytes while the stream is being captured: run the largest product once before capturing, "
                        "or use lnh_gemm_device_noalloc");
    (void)hipGetLastError();
    size_t want = bytes > e->ws_cap + e->ws_cap / 2 ? bytes : e->ws_cap + e->ws_cap / 2;
    want += want / 4;
    void *fresh = nullptr;
    hipError_t h = hipMalloc(&fresh, want);
    if (h != hipSuccess) {
        (void)hipGetLastError();
        want = bytes;
        h = hipMalloc(&fresh, want);
    }
    if (h != hipSuccess) return hip_fail(e, h, "HIP workspace allocation");
    if (e->d_ws) e->ws_retired.push_back(e->d_ws);
    e->d_ws = fresh;
    e->ws_cap = want;
    return LNH_OK;
}

// The tiled copy of m, made now if no product has needed it yet.  Making it allocates, which a stream under capture
// cannot record, and the copy must be complete before any stream reads it: the one-time build is followed by a
// synchronisation of the building stream.
// `view` (may be null) receives the copy's addresses, read under the matrix's lock.
int ensure_tiled(lnh_exec *e, hipStream_t s, const lnh_matrix *m, nh::MatView *view = nullptr) {
    std::lock_guard<std::mutex> lock(m->lazy);
    if (view) *view = m->tiled;
    if (m->tiled.p0) return LNH_OK;
    const nh::TiledSpec ts = nh::tiled_spec(m->view.type, m->view.rows, m->view.cols);
    if (ts.total == 0) return LNH_OK;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (s && hipStreamIsCapturing(s, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone)
        return fail(e, LNH_ERR_INVALID,
                    "the matrix has no multi-token copy yet and the stream is being captured: call lnh_matrix_prepare (or run one "
                    "multi-token product) before capturing");
    (void)hipGetLastError();
    hipError_t h = hipSetDevice(m->ctx->device);
    if (h != hipSuccess) return hip_fail(e, h, "hipSetDevice");
    void *dev = nullptr;
    h = hipMalloc(&dev, ts.total);
    if (h != hipSuccess) return hip_fail(e, h, "HIP matrix allocation (multi-token copy)");
    uint8_t *tb = static_cast<uint8_t *>(dev);
    nh::MatView t = m->view;
    t.p0 = tb + ts.offset[0];
    t.p1 = tb + ts.offset[1];
    t.p2 = tb + ts.offset[2];
    t.p3 = tb + ts.offset[3];
    t.s0 = (uint32_t)ts.per_row[0];
    t.s1 = (uint32_t)ts.per_row[1];
    t.s2 = (uint32_t)ts.per_row[2];
    t.s3 = (uint32_t)ts.per_row[3];
    hipStream_t bs = s ? s : e->stream;
    // rows that pad the last tile are decoded like any other and then dropped: give them defined bytes
    h = hipMemsetAsync(tb, 0, ts.total, bs);
    if (h == hipSuccess) h = nh::launch_retile(bs, t, m->view);
    const hipError_t hs = hipStreamSynchronize(bs);
    if (h == hipSuccess) h = hs;
    if (h != hipSuccess) {
        (void)hipFree(dev);
        return hip_fail(e, h, "HIP matrix re-layout (multi-token copy)");
    }
    m->dev_tiled = dev;
    m->tiled_bytes = ts.total;
    m->tiled = t;
    if (view) *view = t;
    return LNH_OK;
}

// Launch n products; xs/ys are device pointers.
int launch_products(lnh_exec *e, hipStream_t s, size_t n, const lnh_matrix *const *mats, const size_t *tokens,
                    const float *const *xs, float *const *ys) {
    std::vector<nh::MatView> views(n), tiled(n);
    std::vector<uint32_t> toks(n);
    for (size_t g = 0; g < n; g++) {
        views[g] = mats[g]->view;
        toks[g] = (uint32_t)tokens[g];
        tiled[g] = nh::MatView{};  // single-token products never look at it
        if (nh::product_reads_tiled(views[g].type, toks[g]) && views[g].rows != 0) {
            const int rt = ensure_tiled(e, s, mats[g], &tiled[g]);
            if (rt != LNH_OK) return rt;
        }
    }
    int rc = ensure_workspace(e, s, nh::gemm_workspace_bytes(views.data(), toks.data(), (uint32_t)n));
    if (rc != LNH_OK) return rc;
    hipError_t h = nh::launch_gemm_groups(s, views.data(), tiled.data(), toks.data(), xs, ys, (uint32_t)n, e->d_ws, e->ws_cap);
    if (h != hipSuccess) return hip_fail(e, h, "HIP kernel launch");
    return LNH_OK;
}

int make_matrix(lnh_exec *e, uint32_t type, size_t rows, size_t cols, const void *src, bool src_on_device,
                size_t nbytes, lnh_matrix **out) {
    nh::PlaneSpec ps = nh::plane_spec(type, rows, cols);
    hipError_t h = hipSetDevice(e->ctx->device);
    if (h != hipSuccess) return hip_fail(e, h, "hipSetDevice");
    void *dev = nullptr;
    h = hipMalloc(&dev, ps.total);
    if (h != hipSuccess) return hip_fail(e, h, "HIP matrix allocation");
    void *staging = nullptr;
    const void *src_dev = src;
    if (!src_on_device) {
        h = hipMalloc(&staging, nbytes ? nbytes : 1);
        if (h != hipSuccess) {
            (void)hipFree(dev);
            return hip_fail(e, h, "HIP upload staging allocation");
        }
        h = hipMemcpyAsync(staging, src, nbytes, hipMemcpyHostToDevice, e->stream);
        src_dev = staging;
    }
    auto m = std::make_unique<lnh_matrix>();
    m->ctx = e->ctx;
    m->dev = dev;
    m->dev_bytes = ps.total;
    uint8_t *base = static_cast<uint8_t *>(dev);
    m->view.p0 = base + ps.offset[0];
    m->view.p1 = base + ps.offset[1];
    m->view.p2 = base + ps.offset[2];
    m->view.p3 = base + ps.offset[3];
    m->view.s0 = (uint32_t)ps.stride[0];
    m->view.s1 = (uint32_t)ps.stride[1];
    m->view.s2 = (uint32_t)ps.stride[2];
    m->view.s3 = (uint32_t)ps.stride[3];
    m->view.type = type;
    m->view.rows = (uint32_t)rows;
    m->view.cols = (uint32_t)cols;
    m->view.nb = (uint32_t)(cols / nh::block_elems(type));
    if (h == hipSuccess) h = nh::launch_repack(e->stream, m->view, src_dev);
    hipError_t hs = hipStreamSynchronize(e->stream);
    if (h == hipSuccess) h = hs;
    if (staging) (void)hipFree(staging);
    if (h != hipSuccess) {
        (void)hipFree(dev);
        return hip_fail(e, h, "HIP matrix upload");
    }
    *out = m.release();
    return LNH_OK;
}

int check_packed_shape(lnh_exec *e, uint32_t type, size_t rows, size_t cols, size_t nbytes) {
    if (!nh::type_supported(type)) return fail(e, LNH_ERR_UNSUPPORTED, "unsupported GGUF dtype " + std::to_string(type));
    if (rows == 0 || cols == 0) return fail(e, LNH_ERR_INVALID, "GEMV dimensions must be positive");
    size_t qk = nh::block_elems(type);
    if (cols % qk != 0)
        return fail(e, LNH_ERR_INVALID, "n_cols " + std::to_string(cols) + " is not a multiple of " + std::to_string(qk));
    if (rows > UINT32_MAX) return fail(e, LNH_ERR_INVALID, "GEMV rows exceed u32");
    if (cols > UINT32_MAX) return fail(e, LNH_ERR_INVALID, "GEMV columns exceed u32");
    size_t rb = nh::gguf_row_bytes(type, cols), total;
    if (rb == 0 || mul_overflows(rb, rows, &total)) return fail(e, LNH_ERR_INVALID, "GEMV shape overflow");
    // plane strides are kept in 32 bits
    if (nh::plane_spec(type, 1, cols).stride[0] > UINT32_MAX) return fail(e, LNH_ERR_INVALID, "GEMV columns exceed u32");
    // the Q4_K single-token kernel forms byte offsets inside a plane in 32 bits
    if (type == nh::T_Q4_K && rows * nh::plane_spec(type, 1, cols).stride[0] > UINT32_MAX)
        return fail(e, LNH_ERR_INVALID, "Q4_K matrix exceeds 4 GiB of codes: split it by rows");
    if (nbytes != total) return fail(e, LNH_ERR_INVALID, "GEMV buffer lengths do not match shape");
    return LNH_OK;
}

// Shared checks of gemm_resident (native-cuda/src/gpu.rs:358-371).
int check_gemm(lnh_exec *e, const lnh_matrix *m, size_t tokens, bool have_lens, size_t x_len, size_t y_len,
               size_t *inputs, size_t *outputs) {
    if (!e) return LNH_ERR_INVALID;
    if (!m) return fail(e, LNH_ERR_INVALID, "HIP matrix is null");
    if (m->ctx.get() != e->ctx.get()) return fail(e, LNH_ERR_FOREIGN, "HIP matrix belongs to a different executor");
    if (mul_overflows(tokens, m->view.cols, inputs)) return fail(e, LNH_ERR_INVALID, "HIP GEMM input shape overflow");
    if (mul_overflows(tokens, m->view.rows, outputs)) return fail(e, LNH_ERR_INVALID, "HIP GEMM output shape overflow");
    if (tokens == 0 || (have_lens && (x_len != *inputs || y_len != *outputs)))
        return fail(e, LNH_ERR_INVALID, "HIP GEMM buffer lengths do not match shape");
    if (*outputs > UINT32_MAX) return fail(e, LNH_ERR_INVALID, "HIP GEMM launch exceeds u32");
    if (*inputs > UINT32_MAX) return fail(e, LNH_ERR_INVALID, "HIP GEMM input exceeds u32");
    return LNH_OK;
}

// H2D x, kernel(s), blocking D2H y (native-cuda/src/gpu.rs:301-303, 332-334).
// shared_x: every group reads the same x (tokens[0] rows of it), copied to the device once.
int run_host(lnh_exec *e, size_t n_groups, const lnh_matrix *const *mats, const size_t *tokens, const float *x,
             size_t x_total, float *y, size_t y_total, bool shared_x = false) {
    hipError_t h = hipSetDevice(e->ctx->device);
    if (h != hipSuccess) return hip_fail(e, h, "hipSetDevice");
    int rc = ensure_scratch(e, x_total, y_total);
    if (rc != LNH_OK) return rc;
    const bool pinned = x_total <= PINNED_MAX_FLOATS && y_total <= PINNED_MAX_FLOATS && ensure_pinned(e, x_total, y_total);
    if (pinned) {
        std::memcpy(e->h_in, x, x_total * sizeof(float));
        h = nh::launch_copy_small(e->stream, e->d_in, e->h_in, ((x_total + 3) & ~(size_t)3) * sizeof(float));
    } else {
        h = hipMemcpyAsync(e->d_in, x, x_total * sizeof(float), hipMemcpyHostToDevice, e->stream);
    }
    if (h != hipSuccess) return hip_fail(e, h, "HIP input copy");
    std::vector<const float *> xs(n_groups);
    std::vector<float *> ys(n_groups);
    size_t xo = 0, yo = 0;
    for (size_t g = 0; g < n_groups; g++) {
        xs[g] = e->d_in + xo;
        ys[g] = e->d_out + yo;
        if (!shared_x) xo += tokens[g] * mats[g]->view.cols;
        yo += tokens[g] * mats[g]->view.rows;
    }
    rc = launch_products(e, e->stream, n_groups, mats, tokens, xs.data(), ys.data());
    if (rc != LNH_OK) {
        (void)hipStreamSynchronize(e->stream);
        return rc;
    }
    if (pinned)
        h = nh::launch_copy_small(e->stream, e->h_out, e->d_out, ((y_total + 3) & ~(size_t)3) * sizeof(float));
    else
        h = hipMemcpyAsync(y, e->d_out, y_total * sizeof(float), hipMemcpyDeviceToHost, e->stream);
    hipError_t hs = hipStreamSynchronize(e->stream);
    if (h == hipSuccess) h = hs;
    if (h != hipSuccess) return hip_fail(e, h, "HIP output copy");
    if (pinned) std::memcpy(y, e->h_out, y_total * sizeof(float));  // y is written only after everything succeeded
    return LNH_OK;
}

}  // namespace

extern "C" {

int lnh_create(int device_ordinal, lnh_exec **out) {
    if (!out) return fail(nullptr, LNH_ERR_INVALID, "lnh_create: out is null");
    *out = nullptr;
    int count = 0;
    hipError_t h = hipGetDeviceCount(&count);
    if (h != hipSuccess) return hip_fail(nullptr, h, "hipGetDeviceCount");
    if (device_ordinal < 0 || device_ordinal >= count)
        return fail(nullptr, LNH_ERR_DEVICE,
                    "HIP device " + std::to_string(device_ordinal) + " not present (" + std::to_string(count) +
                        " visible); no CPU fallback");
    h = hipSetDevice(device_ordinal);
    if (h != hipSuccess) return hip_fail(nullptr, h, "hipSetDevice");
    hipDeviceProp_t prop;
    h = hipGetDeviceProperties(&prop, device_ordinal);
    if (h != hipSuccess) return hip_fail(nullptr, h, "hipGetDeviceProperties");
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(nullptr, LNH_ERR_DEVICE, std::string("kernels are built for gfx950 only, device is ") + prop.gcnArchName);
    size_t lds = prop.sharedMemPerBlockOptin ? prop.sharedMemPerBlockOptin : prop.sharedMemPerBlock;
    if (lds > 80 * 1024) lds = 80 * 1024;  // two workgroups per CU must fit in the 160 KB LDS
    if (!nh::set_device_limits(prop.multiProcessorCount, lds))
        return fail(nullptr, LNH_ERR_DEVICE,
                    "HIP device " + std::to_string(device_ordinal) + " differs from the GPU this process already runs on (compute units or LDS per "
                    "workgroup): one kind of GPU per process");
    auto e = std::make_unique<lnh_exec>();
    e->ctx = std::make_shared<Ctx>();
    e->ctx->device = device_ordinal;
    e->ctx->id = g_next_ctx.fetch_add(1);
    h = hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking);
    if (h != hipSuccess) return hip_fail(nullptr, h, "hipStreamCreate");
    float unit = 0.f;
    bool bf16_exact = false, i4_exact = false;
    h = nh::probe_nibble_converts(e->stream, &unit, &bf16_exact, &i4_exact);
    if (h != hipSuccess) {
        (void)hipStreamDestroy(e->stream);
        return hip_fail(nullptr, h, "nibble convert probe");
    }
    if (!nh::set_nibble_converts(unit, bf16_exact, i4_exact)) {
        (void)hipStreamDestroy(e->stream);
        return fail(nullptr, LNH_ERR_DEVICE,
                    "HIP device " + std::to_string(device_ordinal) + " converts nibble bytes differently from the GPU this process already runs on: "
                    "one kind of GPU per process");
    }
    // address of this device's copy of the static workspace (lnh_gemm_device_noalloc), looked up while
    // the device is current
    h = nh::static_scratch_init(device_ordinal);
    if (h != hipSuccess) {
        (void)hipStreamDestroy(e->stream);
        return hip_fail(nullptr, h, "hipGetSymbolAddress(static workspace)");
    }
    *out = e.release();
    return LNH_OK;
}

void lnh_destroy(lnh_exec *e) {
    if (!e) return;
    (void)hipSetDevice(e->ctx->device);
    if (e->stream) {
        (void)hipStreamSynchronize(e->stream);
        (void)hipStreamDestroy(e->stream);
    }
    if (e->d_ws) (void)hipFree(e->d_ws);
    for (void *p : e->ws_retired) (void)hipFree(p);
    if (e->d_in) (void)hipFree(e->d_in);
    if (e->d_out) (void)hipFree(e->d_out);
    if (e->h_in) (void)hipHostFree(e->h_in);
    if (e->h_out) (void)hipHostFree(e->h_out);
    delete e;
}

int lnh_memory_info(lnh_exec *e, size_t *free_bytes, size_t *total_bytes) {
    if (!e) return LNH_ERR_INVALID;
    hipError_t h = hipSetDevice(e->ctx->device);
    size_t f = 0, t = 0;
    if (h == hipSuccess) h = hipMemGetInfo(&f, &t);
    if (h != hipSuccess) return hip_fail(e, h, "hipMemGetInfo");
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return LNH_OK;
}

const char *lnh_last_error(const lnh_exec *e) { return e ? e->err.c_str() : ""; }
const char *lnh_thread_error(void) { return t_error.c_str(); }

int lnh_upload_f32(lnh_exec *e, size_t rows, size_t cols, const float *weights, size_t weights_len, lnh_matrix **out) {
    if (!e || !out) return LNH_ERR_INVALID;
    *out = nullptr;
    if (const char *msg = shape_checked(rows, cols, weights_len, cols, nullptr, nullptr))
        return fail(e, LNH_ERR_INVALID, msg);
    if (!weights) return fail(e, LNH_ERR_INVALID, "weights pointer is null");
    return make_matrix(e, nh::T_F32, rows, cols, weights, false, weights_len * sizeof(float), out);
}

int lnh_upload_packed(lnh_exec *e, uint32_t type, size_t rows, size_t cols, const uint8_t *bytes, size_t nbytes,
                      lnh_matrix **out) {
    if (!e || !out) return LNH_ERR_INVALID;
    *out = nullptr;
    int rc = check_packed_shape(e, type, rows, cols, nbytes);
    if (rc != LNH_OK) return rc;
    if (!bytes) return fail(e, LNH_ERR_INVALID, "weights pointer is null");
    return make_matrix(e, type, rows, cols, bytes, false, nbytes, out);
}

int lnh_upload_packed_device(lnh_exec *e, uint32_t type, size_t rows, size_t cols, const void *device_bytes,
                             size_t nbytes, lnh_matrix **out) {
    if (!e || !out) return LNH_ERR_INVALID;
    *out = nullptr;
    int rc = check_packed_shape(e, type, rows, cols, nbytes);
    if (rc != LNH_OK) return rc;
    if (!device_bytes) return fail(e, LNH_ERR_INVALID, "weights pointer is null");
    return make_matrix(e, type, rows, cols, device_bytes, true, nbytes, out);
}

void lnh_matrix_free(lnh_matrix *m) {
    if (!m) return;
    (void)hipSetDevice(m->ctx->device);
    if (m->dev) (void)hipFree(m->dev);
    if (m->dev_tiled) (void)hipFree(m->dev_tiled);
    delete m;
}

int lnh_matrix_prepare(lnh_exec *e, const lnh_matrix *m, size_t max_tokens) {
    if (!e) return LNH_ERR_INVALID;
    if (!m) return fail(e, LNH_ERR_INVALID, "HIP matrix is null");
    if (m->ctx.get() != e->ctx.get()) return fail(e, LNH_ERR_FOREIGN, "HIP matrix belongs to a different executor");
    if (max_tokens > UINT32_MAX) return fail(e, LNH_ERR_INVALID, "GEMM tokens exceed u32");
    if (!nh::product_reads_tiled(m->view.type, (uint32_t)max_tokens)) return LNH_OK;
    return ensure_tiled(e, e->stream, m);
}

int lnh_matrix_info(const lnh_matrix *m, uint32_t *type, size_t *rows, size_t *cols, size_t *device_bytes) {
    if (!m) return LNH_ERR_INVALID;
    if (type) *type = m->view.type;
    if (rows) *rows = m->view.rows;
    if (cols) *cols = m->view.cols;
    if (device_bytes) {
        std::lock_guard<std::mutex> lock(m->lazy);
        *device_bytes = m->dev_bytes + m->tiled_bytes;  // the multi-token copy counts once it exists
    }
    return LNH_OK;
}

int lnh_gemv(lnh_exec *e, const lnh_matrix *m, const float *x, size_t x_len, float *y, size_t y_len) {
    if (!e) return LNH_ERR_INVALID;
    if (!m) return fail(e, LNH_ERR_INVALID, "HIP matrix is null");
    if (m->ctx.get() != e->ctx.get()) return fail(e, LNH_ERR_FOREIGN, "HIP matrix belongs to a different executor");
    if (x_len != m->view.cols || y_len != m->view.rows)
        return fail(e, LNH_ERR_INVALID, "HIP GEMV vector lengths do not match resident matrix");
    if (!x || !y) return fail(e, LNH_ERR_INVALID, "vector pointer is null");
    size_t one = 1;
    return run_host(e, 1, &m, &one, x, x_len, y, y_len);
}

int lnh_gemm(lnh_exec *e, const lnh_matrix *m, size_t tokens, const float *x, size_t x_len, float *y, size_t y_len) {
    size_t inputs, outputs;
    int rc = check_gemm(e, m, tokens, true, x_len, y_len, &inputs, &outputs);
    if (rc != LNH_OK) return rc;
    if (!x || !y) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    return run_host(e, 1, &m, &tokens, x, inputs, y, outputs);
}

int lnh_gemv_once(lnh_exec *e, const float *weights, size_t weights_len, const float *x, size_t x_len, float *y,
                  size_t y_len) {
    if (!e) return LNH_ERR_INVALID;
    lnh_matrix *m = nullptr;
    // upload(output.len(), input.len(), weights)
    if (const char *msg = shape_checked(y_len, x_len, weights_len, x_len, nullptr, nullptr))
        return fail(e, LNH_ERR_INVALID, msg);
    int rc = lnh_upload_f32(e, y_len, x_len, weights, weights_len, &m);
    if (rc != LNH_OK) return rc;
    rc = lnh_gemv(e, m, x, x_len, y, y_len);
    lnh_matrix_free(m);
    return rc;
}

static int check_groups(lnh_exec *e, size_t n_groups, const lnh_matrix *const *mats, const size_t *tokens,
                        size_t *x_total, size_t *y_total) {
    if (!e) return LNH_ERR_INVALID;
    if (n_groups != 0 && (!mats || !tokens)) return fail(e, LNH_ERR_INVALID, "group arrays are null");
    size_t xt = 0, yt = 0;
    for (size_t g = 0; g < n_groups; g++) {
        if (!mats[g]) return fail(e, LNH_ERR_INVALID, "HIP matrix is null");
        if (mats[g]->ctx.get() != e->ctx.get())
            return fail(e, LNH_ERR_FOREIGN, "HIP matrix belongs to a different executor");
        size_t in, outn;
        if (mul_overflows(tokens[g], mats[g]->view.cols, &in) || mul_overflows(tokens[g], mats[g]->view.rows, &outn) ||
            xt + in < xt || yt + outn < yt)
            return fail(e, LNH_ERR_INVALID, "HIP GEMM input shape overflow");
        if (in > UINT32_MAX || outn > UINT32_MAX) return fail(e, LNH_ERR_INVALID, "HIP GEMM launch exceeds u32");
        xt += in;
        yt += outn;
    }
    *x_total = xt;
    *y_total = yt;
    return LNH_OK;
}

int lnh_gemm_shared(lnh_exec *e, size_t n_mats, const lnh_matrix *const *mats, size_t tokens, const float *x,
                    size_t x_len, float *y, size_t y_len) {
    if (!e) return LNH_ERR_INVALID;
    if (n_mats == 0 || !mats) return fail(e, LNH_ERR_INVALID, "matrix array is empty");
    if (tokens == 0) return fail(e, LNH_ERR_INVALID, "HIP GEMM requires at least one token");
    std::vector<size_t> toks(n_mats, tokens);
    size_t xt, yt;
    int rc = check_groups(e, n_mats, mats, toks.data(), &xt, &yt);
    if (rc != LNH_OK) return rc;
    for (size_t g = 1; g < n_mats; g++)
        if (mats[g]->view.cols != mats[0]->view.cols)
            return fail(e, LNH_ERR_INVALID, "matrices that share an input must have the same column count");
    const size_t inputs = tokens * mats[0]->view.cols;
    if (x_len != inputs || y_len != yt) return fail(e, LNH_ERR_INVALID, "HIP GEMM buffer lengths do not match shape");
    if (!x || !y) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    return run_host(e, n_mats, mats, toks.data(), x, inputs, y, yt, true);
}

int lnh_gemm_grouped(lnh_exec *e, size_t n_groups, const lnh_matrix *const *mats, const size_t *tokens, const float *x,
                     size_t x_len, float *y, size_t y_len) {
    size_t xt, yt;
    int rc = check_groups(e, n_groups, mats, tokens, &xt, &yt);
    if (rc != LNH_OK) return rc;
    if (x_len != xt || y_len != yt) return fail(e, LNH_ERR_INVALID, "HIP GEMM buffer lengths do not match shape");
    if (yt == 0) return LNH_OK;
    if (!x || !y) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    return run_host(e, n_groups, mats, tokens, x, xt, y, yt);
}

int lnh_gemm_device(lnh_exec *e, const lnh_matrix *m, size_t tokens, const float *dx, float *dy, void *stream) {
    size_t inputs, outputs;
    int rc = check_gemm(e, m, tokens, false, 0, 0, &inputs, &outputs);
    if (rc != LNH_OK) return rc;
    if (!dx || !dy) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    if (misaligned(dx)) return fail(e, LNH_ERR_INVALID, "device input buffers must be 16-byte aligned");
    hipStream_t s = stream ? static_cast<hipStream_t>(stream) : e->stream;
    return launch_products(e, s, 1, &m, &tokens, &dx, &dy);
}

int lnh_gemm_device_noalloc(lnh_exec *e, const lnh_matrix *m, size_t tokens, const float *dx, float *dy, void *stream) {
    size_t inputs, outputs;
    int rc = check_gemm(e, m, tokens, false, 0, 0, &inputs, &outputs);
    if (rc != LNH_OK) return rc;
    if (!dx || !dy) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    if (misaligned(dx)) return fail(e, LNH_ERR_INVALID, "device input buffers must be 16-byte aligned");
    void *ws = nh::static_scratch(e->ctx->device);
    if (!ws) return fail(e, LNH_ERR_DEVICE, "static workspace of this device was not initialised");
    const uint32_t tok32 = (uint32_t)tokens;
    const size_t need = nh::gemm_workspace_bytes(&m->view, &tok32, 1);
    if (need > nh::STATIC_SCRATCH_BYTES)
        return fail(e, LNH_ERR_INVALID,
                    "product needs " + std::to_string(need) + " bytes of workspace, the allocation-free entry point holds " +
                        std::to_string(nh::STATIC_SCRATCH_BYTES) + ": use lnh_gemm_device or fewer tokens per call");
    hipStream_t s = stream ? static_cast<hipStream_t>(stream) : e->stream;
    nh::MatView tiled{};
    if (nh::product_reads_tiled(m->view.type, tok32)) {
        std::lock_guard<std::mutex> lock(m->lazy);
        if (!m->tiled.p0)
            return fail(e, LNH_ERR_INVALID,
                        "the matrix has no multi-token copy yet and this entry point does not allocate: call lnh_matrix_prepare first");
        tiled = m->tiled;
    }
    const hipError_t h = nh::launch_gemm_groups(s, &m->view, &tiled, &tok32, &dx, &dy, 1, ws, nh::STATIC_SCRATCH_BYTES);
    if (h != hipSuccess) return hip_fail(e, h, "HIP kernel launch");
    return LNH_OK;
}

int lnh_act_create(lnh_exec *e, uint32_t type, size_t cols, size_t max_tokens, lnh_act **out) {
    if (!e) return LNH_ERR_INVALID;
    if (!out) return fail(e, LNH_ERR_INVALID, "output pointer is null");
    *out = nullptr;
    if (cols > UINT32_MAX || max_tokens > UINT32_MAX) return fail(e, LNH_ERR_INVALID, "activation shape exceeds u32");
    const size_t bytes = nh::act_bytes(type, (uint32_t)cols, (uint32_t)max_tokens);
    if (bytes == 0)
        return fail(e, LNH_ERR_UNSUPPORTED, "split activations exist for the block-quantized dtypes, columns in multiples of 32 and at least one token");
    hipError_t h = hipSetDevice(e->ctx->device);
    if (h != hipSuccess) return hip_fail(e, h, "hipSetDevice");
    void *dev = nullptr;
    h = hipMalloc(&dev, bytes + nh::ACT_DEFER_PARTIAL_BYTES);
    if (h != hipSuccess) return hip_fail(e, h, "HIP activation allocation");
    // slots past the tokens of a call are multiplied like any other and dropped: keep them finite from the start
    h = hipMemsetAsync(dev, 0, bytes + nh::ACT_DEFER_PARTIAL_BYTES, e->stream);
    const hipError_t hs = hipStreamSynchronize(e->stream);
    if (h == hipSuccess) h = hs;
    if (h != hipSuccess) {
        (void)hipFree(dev);
        return hip_fail(e, h, "HIP activation allocation");
    }
    auto a = std::make_unique<lnh_act>();
    a->ctx = e->ctx;
    a->dev = dev;
    a->bytes = bytes;
    a->type = type;
    a->cols = (uint32_t)cols;
    a->max_tokens = (uint32_t)max_tokens;
    *out = a.release();
    return LNH_OK;
}

void lnh_act_free(lnh_act *a) {
    if (!a) return;
    if (a->dev) {
        (void)hipSetDevice(a->ctx->device);
        (void)hipFree(a->dev);
    }
    delete a;
}

int lnh_act_split_device(lnh_exec *e, lnh_act *a, size_t tokens, const float *dx, void *stream) {
    if (!e) return LNH_ERR_INVALID;
    if (!a || !dx) return fail(e, LNH_ERR_INVALID, "activation or buffer pointer is null");
    if (misaligned(dx)) return fail(e, LNH_ERR_INVALID, "device input buffers must be 16-byte aligned");
    if (a->ctx.get() != e->ctx.get()) return fail(e, LNH_ERR_FOREIGN, "activations belong to a different executor");
    if (tokens == 0 || tokens > a->max_tokens) return fail(e, LNH_ERR_INVALID, "token count outside the activations' capacity");
    hipStream_t s = stream ? static_cast<hipStream_t>(stream) : e->stream;
    const hipError_t h = nh::launch_act_split(s, a->dev, a->type, a->cols, a->max_tokens, (uint32_t)tokens, dx);
    if (h != hipSuccess) return hip_fail(e, h, "HIP kernel launch");
    a->deferred_x = nullptr;
    return LNH_OK;
}

}  // extern "C"

namespace {
// lnh_gemm_act_device (x) and lnh_gemm_plain_act_device (dx): the product's activations split or plain.
int gemm_act(lnh_exec *e, size_t n_mats, const lnh_matrix *const *mats, const lnh_act *x, const float *dx, size_t tokens,
             float *const *dys, int epilogue, float *d_residual, const float *d_norm_w, float eps, float *d_xn, lnh_act *next,
             void *stream) {
    if (!e) return LNH_ERR_INVALID;
    if (!mats || (!x && !dx) || n_mats == 0) return fail(e, LNH_ERR_INVALID, "matrix list or activations are null");
    if (misaligned(dx) || misaligned(d_residual) || misaligned(d_norm_w)) return fail(e, LNH_ERR_INVALID, "device input buffers must be 16-byte aligned");
    if (n_mats > 8) return fail(e, LNH_ERR_INVALID, "at most 8 matrices per call");
    if ((x && x->ctx.get() != e->ctx.get()) || (next && next->ctx.get() != e->ctx.get()))
        return fail(e, LNH_ERR_FOREIGN, "activations belong to a different executor");
    if (tokens == 0 || tokens > UINT32_MAX || (x && tokens > x->max_tokens) || (next && tokens > next->max_tokens))
        return fail(e, LNH_ERR_INVALID, "token count outside the activations' capacity");
    if (tokens < nh::MM_MIN_TOKENS)
        return fail(e, LNH_ERR_UNSUPPORTED, "split activations serve products of three or more tokens");
    nh::ActNorm norm;
    if (x && x->deferred_x) {  // the rows are a residual stream whose norm this product applies as it reads them
        if (tokens != x->deferred_tokens)
            return fail(e, LNH_ERR_INVALID, "the activations hold a deferred norm of another token count");
        norm.w = x->deferred_w;
        norm.partial = x->partial();
        norm.eps = x->deferred_eps;
        dx = x->deferred_x;
    }
    const bool plain = dx != nullptr;
    nh::MatView views[8], tiled[8];
    for (size_t i = 0; i < n_mats; i++) {
        const lnh_matrix *m = mats[i];
        if (!m) return fail(e, LNH_ERR_INVALID, "HIP matrix is null");
        if (m->ctx.get() != e->ctx.get()) return fail(e, LNH_ERR_FOREIGN, "HIP matrix belongs to a different executor");
        if (x ? (m->view.type != x->type || m->view.cols != x->cols)
              : (m->view.type != mats[0]->view.type || m->view.cols != mats[0]->view.cols))
            return fail(e, LNH_ERR_INVALID, x ? "the activations were split for another dtype or column count than the matrix has"
                                              : "matrices that share an input must have one dtype and column count");
        if (m->view.rows == 0) return fail(e, LNH_ERR_INVALID, "HIP matrix has no rows");
        views[i] = m->view;
    }
    nh::ActEpilogue ep;
    switch (epilogue) {
    case LNH_EPILOGUE_NONE:
        if (!dys) return fail(e, LNH_ERR_INVALID, "output list is null");
        for (size_t i = 0; i < n_mats; i++)
            if (!dys[i]) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
        break;
    case LNH_EPILOGUE_ADD_RMSNORM:
        if (n_mats != 1) return fail(e, LNH_ERR_INVALID, "the residual epilogue takes one matrix");
        if (!d_residual || !d_norm_w) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
        if (next && next->cols != views[0].rows) return fail(e, LNH_ERR_INVALID, "next activations do not have the product's width");
        ep.kind = nh::ACT_EPILOGUE_ADD_RMSNORM;
        break;
    case LNH_EPILOGUE_ADD_RMSNORM_DEFERRED:
        if (n_mats != 1) return fail(e, LNH_ERR_INVALID, "the residual epilogue takes one matrix");
        if (!d_residual || !d_norm_w || !next) return fail(e, LNH_ERR_INVALID, "buffer pointer or next activations are null");
        if (next->cols != views[0].rows) return fail(e, LNH_ERR_INVALID, "next activations do not have the product's width");
        if (d_xn) return fail(e, LNH_ERR_UNSUPPORTED, "a deferred norm leaves no plain normalised rows");
        if (tokens > nh::ACT_DEFER_MAX_TOKENS)
            return fail(e, LNH_ERR_UNSUPPORTED, "the norm is deferred for products of at most 32 tokens");
        if (next == x) return fail(e, LNH_ERR_INVALID, "a deferred norm cannot go into the activations the product reads");
        ep.kind = nh::ACT_EPILOGUE_ADD_DEFER;
        ep.partial = next->partial();
        break;
    case LNH_EPILOGUE_SWIGLU:
        if (n_mats != 2 || views[0].rows != views[1].rows) return fail(e, LNH_ERR_INVALID, "SiLU(gate) * up takes two matrices of one shape");
        if (!next) return fail(e, LNH_ERR_INVALID, "SiLU(gate) * up needs activations to leave its result in");
        if (next->cols != views[0].rows) return fail(e, LNH_ERR_INVALID, "next activations do not have the product's width");
        ep.kind = nh::ACT_EPILOGUE_SWIGLU;
        break;
    default: return fail(e, LNH_ERR_INVALID, "unknown epilogue");
    }
    ep.residual = d_residual;
    ep.norm_w = d_norm_w;
    ep.eps = eps;
    ep.xn_out = d_xn;
    if (next && ep.kind != nh::ACT_EPILOGUE_ADD_DEFER) {
        ep.next_act = next->dev;
        ep.next_type = next->type;
        ep.next_cols = next->cols;
        ep.next_max_tokens = next->max_tokens;
    }
    hipStream_t s = stream ? static_cast<hipStream_t>(stream) : e->stream;
    for (size_t i = 0; i < n_mats; i++) {
        const int rt = ensure_tiled(e, s, mats[i], &tiled[i]);
        if (rt != LNH_OK) return rt;
    }
    int rc = ensure_workspace(e, s, nh::gemm_act_workspace_bytes(tiled, (uint32_t)n_mats, (uint32_t)tokens,
                                                                 ep.kind != nh::ACT_EPILOGUE_NONE, plain));
    if (rc != LNH_OK) return rc;
    const hipError_t h = nh::launch_gemm_act(s, tiled, (uint32_t)n_mats, (uint32_t)tokens, plain ? nullptr : x->dev,
                                             plain ? 0 : x->max_tokens, dx, norm.w ? &norm : nullptr, dys, ep, e->d_ws, e->ws_cap);
    if (h == hipErrorInvalidValue) {
        (void)hipGetLastError();
        return fail(e, LNH_ERR_UNSUPPORTED, "this product is not one the split-activation path launches");
    }
    if (h != hipSuccess) return hip_fail(e, h, "HIP kernel launch");
    if (next) {  // what `next` holds from here on
        const bool deferred = ep.kind == nh::ACT_EPILOGUE_ADD_DEFER;
        next->deferred_x = deferred ? d_residual : nullptr;
        next->deferred_w = d_norm_w;
        next->deferred_eps = eps;
        next->deferred_tokens = (uint32_t)tokens;
    }
    return LNH_OK;
}
}  // namespace

extern "C" {

int lnh_gemm_act_device(lnh_exec *e, size_t n_mats, const lnh_matrix *const *mats, const lnh_act *x, size_t tokens,
                        float *const *dys, int epilogue, float *d_residual, const float *d_norm_w, float eps, float *d_xn,
                        lnh_act *next, void *stream) {
    if (e && !x) return fail(e, LNH_ERR_INVALID, "matrix list or activations are null");
    return gemm_act(e, n_mats, mats, x, nullptr, tokens, dys, epilogue, d_residual, d_norm_w, eps, d_xn, next, stream);
}

int lnh_gemm_plain_act_device(lnh_exec *e, size_t n_mats, const lnh_matrix *const *mats, const float *dx, size_t tokens,
                              float *const *dys, int epilogue, float *d_residual, const float *d_norm_w, float eps,
                              float *d_xn, lnh_act *next, void *stream) {
    if (e && !dx) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    return gemm_act(e, n_mats, mats, nullptr, dx, tokens, dys, epilogue, d_residual, d_norm_w, eps, d_xn, next, stream);
}

int lnh_gemm_grouped_device(lnh_exec *e, size_t n_groups, const lnh_matrix *const *mats, const size_t *tokens,
                            const float *dx, float *dy, void *stream) {
    size_t xt, yt;
    int rc = check_groups(e, n_groups, mats, tokens, &xt, &yt);
    if (rc != LNH_OK) return rc;
    if (yt == 0) return LNH_OK;
    if (!dx || !dy) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    if (misaligned(dx)) return fail(e, LNH_ERR_INVALID, "device input buffers must be 16-byte aligned");
    hipStream_t s = stream ? static_cast<hipStream_t>(stream) : e->stream;
    std::vector<const float *> xs(n_groups);
    std::vector<float *> ys(n_groups);
    size_t xo = 0, yo = 0;
    for (size_t g = 0; g < n_groups; g++) {
        xs[g] = dx + xo;
        ys[g] = dy + yo;
        xo += tokens[g] * mats[g]->view.cols;
        yo += tokens[g] * mats[g]->view.rows;
    }
    return launch_products(e, s, n_groups, mats, tokens, xs.data(), ys.data());
}

int lnh_gemm_batch_device(lnh_exec *e, size_t n, const lnh_matrix *const *mats, const size_t *tokens,
                          const float *const *dx, float *const *dy, void *stream) {
    if (!e) return LNH_ERR_INVALID;
    if (n != 0 && (!mats || !tokens || !dx || !dy)) return fail(e, LNH_ERR_INVALID, "batch arrays are null");
    for (size_t i = 0; i < n; i++) {  // validate everything before the first launch
        size_t inputs, outputs;
        int rc = check_gemm(e, mats[i], tokens[i], false, 0, 0, &inputs, &outputs);
        if (rc != LNH_OK) return rc;
        if (!dx[i] || !dy[i]) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
        if (misaligned(dx[i])) return fail(e, LNH_ERR_INVALID, "device input buffers must be 16-byte aligned");
    }
    hipStream_t s = stream ? static_cast<hipStream_t>(stream) : e->stream;
    for (size_t i = 0; i < n;) {
        // Single-token products that read the same x (q/k/v, gate/up) go out as one launch.
        size_t run = 1;
        while (tokens[i] == 1 && i + run < n && run < 8 && tokens[i + run] == 1 && dx[i + run] == dx[i] &&
               mats[i + run]->view.type == mats[i]->view.type && mats[i + run]->view.cols == mats[i]->view.cols)
            run++;
        hipError_t h = hipErrorInvalidValue;
        if (run > 1) {
            nh::MatView views[8];
            float *ys[8];
            for (size_t k = 0; k < run; k++) {
                views[k] = mats[i + k]->view;
                ys[k] = dy[i + k];
            }
            h = nh::launch_gemv_multi(s, views, ys, (uint32_t)run, dx[i]);
            if (h == hipErrorInvalidValue) (void)hipGetLastError();
        }
        if (h == hipErrorInvalidValue) {
            // consecutive multi-token products go out together: those of equal dtype and column count share launches
            run = 1;
            while (tokens[i] > 1 && i + run < n && tokens[i + run] > 1) run++;
            int rc = launch_products(e, s, run, &mats[i], &tokens[i], &dx[i], &dy[i]);
            if (rc != LNH_OK) return rc;
            h = hipSuccess;
        }
        if (h != hipSuccess) return hip_fail(e, h, "HIP kernel launch");
        i += run;
    }
    return LNH_OK;
}

// Shared checks and launch of the single-token device products.
static int gemv_shared_device(lnh_exec *e, size_t n_mats, const lnh_matrix *const *mats, const float *dx, float *const *dys,
                              int accumulate, int prologue, const float *dx2, float eps, void *stream) {
    if (!e) return LNH_ERR_INVALID;
    if (n_mats == 0 || n_mats > 8) return fail(e, LNH_ERR_INVALID, "between one and eight matrices share an input");
    if (!mats || !dx || !dys) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    if (prologue != LNH_PROLOGUE_NONE && prologue != LNH_PROLOGUE_RMSNORM && prologue != LNH_PROLOGUE_SWIGLU)
        return fail(e, LNH_ERR_INVALID, "unknown prologue");
    if (prologue != LNH_PROLOGUE_NONE && !dx2) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    if (misaligned(dx) || misaligned(dx2)) return fail(e, LNH_ERR_INVALID, "device input buffers must be 16-byte aligned");
    nh::MatView views[8];
    float *ys[8];
    for (size_t i = 0; i < n_mats; i++) {
        size_t inputs, outputs;
        int rc = check_gemm(e, mats[i], 1, false, 0, 0, &inputs, &outputs);
        if (rc != LNH_OK) return rc;
        if (!dys[i]) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
        if (mats[i]->view.type != mats[0]->view.type || mats[i]->view.cols != mats[0]->view.cols)
            return fail(e, LNH_ERR_INVALID, "matrices that share an input must share dtype and column count");
        views[i] = mats[i]->view;
        ys[i] = dys[i];
    }
    hipStream_t s = stream ? static_cast<hipStream_t>(stream) : e->stream;
    const hipError_t h = prologue == LNH_PROLOGUE_NONE
                             ? nh::launch_gemv_multi(s, views, ys, (uint32_t)n_mats, dx, accumulate != 0)
                             : nh::launch_gemv_multi_prologue(s, views, ys, (uint32_t)n_mats, dx, accumulate != 0, prologue, dx2, eps);
    if (h == hipErrorInvalidValue) {
        (void)hipGetLastError();
        return fail(e, LNH_ERR_UNSUPPORTED, prologue == LNH_PROLOGUE_NONE ? "rows too long for the single-token kernels"
                                                                         : "no fused prologue for this dtype or row length");
    }
    if (h != hipSuccess) return hip_fail(e, h, "HIP kernel launch");
    return LNH_OK;
}

int lnh_gemv_shared_device(lnh_exec *e, size_t n_mats, const lnh_matrix *const *mats, const float *dx,
                           float *const *dys, int accumulate, void *stream) {
    return gemv_shared_device(e, n_mats, mats, dx, dys, accumulate, LNH_PROLOGUE_NONE, nullptr, 0.f, stream);
}

int lnh_gemv_fused_device(lnh_exec *e, size_t n_mats, const lnh_matrix *const *mats, const float *dx, float *const *dys,
                          int accumulate, int prologue, const float *dx2, float eps, void *stream) {
    return gemv_shared_device(e, n_mats, mats, dx, dys, accumulate, prologue, dx2, eps, stream);
}

int lnh_gemv_swiglu_device(lnh_exec *e, const lnh_matrix *gate, const lnh_matrix *up, const float *dx, float *dh,
                           int prologue, const float *dx2, float eps, void *stream) {
    if (!e) return LNH_ERR_INVALID;
    if (!dx || !dh) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    if (prologue != LNH_PROLOGUE_NONE && prologue != LNH_PROLOGUE_RMSNORM) return fail(e, LNH_ERR_INVALID, "unknown prologue");
    if (prologue != LNH_PROLOGUE_NONE && !dx2) return fail(e, LNH_ERR_INVALID, "buffer pointer is null");
    if (misaligned(dx) || misaligned(dx2)) return fail(e, LNH_ERR_INVALID, "device input buffers must be 16-byte aligned");
    size_t inputs, outputs;
    int rc = check_gemm(e, gate, 1, false, 0, 0, &inputs, &outputs);
    if (rc == LNH_OK) rc = check_gemm(e, up, 1, false, 0, 0, &inputs, &outputs);
    if (rc != LNH_OK) return rc;
    if (gate->view.type != up->view.type || gate->view.cols != up->view.cols || gate->view.rows != up->view.rows)
        return fail(e, LNH_ERR_INVALID, "gate and up must share dtype and shape");
    hipStream_t s = stream ? static_cast<hipStream_t>(stream) : e->stream;
    const hipError_t h = nh::launch_gemv_swiglu_pair(s, gate->view, up->view, dx, dh, prologue, dx2, eps);
    if (h == hipErrorInvalidValue) {
        (void)hipGetLastError();
        return fail(e, LNH_ERR_UNSUPPORTED, "no paired SiLU*up epilogue for this dtype or shape");
    }
    if (h != hipSuccess) return hip_fail(e, h, "HIP kernel launch");
    return LNH_OK;
}

int lnh_calibration_copy(lnh_exec *e, void *device_dst, const void *device_src, size_t nbytes, void *stream) {
    if (!e) return LNH_ERR_INVALID;
    if (!device_dst || !device_src || nbytes % 16 != 0) return fail(e, LNH_ERR_INVALID, "copy needs device pointers and a multiple of 16 bytes");
    hipError_t h = nh::launch_copy(stream ? static_cast<hipStream_t>(stream) : e->stream, device_dst, device_src, nbytes);
    if (h != hipSuccess) return hip_fail(e, h, "HIP kernel launch");
    return LNH_OK;
}

int lnh_calibration_read(lnh_exec *e, const void *device_src, size_t nbytes, void *stream) {
    if (!e) return LNH_ERR_INVALID;
    if (!device_src || nbytes % 16 != 0 || nbytes == 16) return fail(e, LNH_ERR_INVALID, "read needs a device pointer and a multiple of 16 bytes, at least 32");
    hipError_t h = hipSetDevice(e->ctx->device);
    if (h != hipSuccess) return hip_fail(e, h, "hipSetDevice");
    const int rc = ensure_scratch(e, 0, 1);  // the kernel's never-written sink
    if (rc != LNH_OK) return rc;
    h = nh::launch_read(stream ? static_cast<hipStream_t>(stream) : e->stream, device_src, nbytes, e->d_out);
    if (h != hipSuccess) return hip_fail(e, h, "HIP kernel launch");
    return LNH_OK;
}

int lnh_synchronize(lnh_exec *e) {
    if (!e) return LNH_ERR_INVALID;
    hipError_t h = hipStreamSynchronize(e->stream);
    if (h != hipSuccess) return hip_fail(e, h, "hipStreamSynchronize");
    return LNH_OK;
}

int lnh_shape_checked(size_t rows, size_t cols, size_t weights_len, size_t input_len, uint32_t *rows_out,
                      uint32_t *cols_out) {
    if (const char *msg = shape_checked(rows, cols, weights_len, input_len, rows_out, cols_out))
        return fail(nullptr, LNH_ERR_INVALID, msg);
    return LNH_OK;
}

int lnh_validate(const float *actual, size_t actual_len, const double *expected, size_t expected_len) {
    if (actual_len != expected_len) return fail(nullptr, LNH_ERR_INVALID, "GEMV output length mismatch");
    for (size_t i = 0; i < actual_len; i++) {
        double a = (double)actual[i], ex = expected[i];
        double tol = 1e-4 + 1e-4 * std::fabs(ex);
        if (!std::isfinite(a) || !std::isfinite(ex) || std::fabs(a - ex) > tol) {
            char buf[160];
            std::snprintf(buf, sizeof buf, "GEMV mismatch at row %zu: expected %.17g, got %.9g", i, ex, a);
            return fail(nullptr, LNH_ERR_INVALID, buf);
        }
    }
    return LNH_OK;
}

size_t lnh_row_bytes(uint32_t type, size_t cols) { return nh::gguf_row_bytes(type, cols); }

size_t lnh_resident_bytes(uint32_t type, size_t rows, size_t cols, size_t tokens) {
    const size_t rb = nh::gguf_row_bytes(type, cols);
    if (rb == 0 || rows == 0 || rows > UINT32_MAX || cols > UINT32_MAX || rb > SIZE_MAX / 4 / rows) return 0;
    size_t bytes = nh::plane_spec(type, rows, cols).total;
    if (nh::product_reads_tiled(type, tokens > UINT32_MAX ? UINT32_MAX : (uint32_t)tokens))
        bytes += nh::tiled_spec(type, rows, cols).total;
    return bytes;
}

}  // extern "C"
