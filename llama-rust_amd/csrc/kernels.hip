// HIP kernels for gfx950 (MI355X) and their launchers: re-layout at upload, single-token GEMV,
// multi-token GEMM.  One translation unit; the kernels live in the .inc files below.
//
// All products are y[t, r] = sum_c W[r, c] * x[t, c] with f32 activations and
// f32 accumulation; W stays packed in HBM (see matview.h) and is decoded in
// registers.  Block scales are factored out of the inner sums
// (sum_j (d*q_j) x_j = d * sum_j q_j x_j; codes are brought to their signed value first),
// which changes only the order of f32 roundings, never the value being
// approximated: the exact product of the dequantized weights
// (langtax/src/quant.rs:7511-7541, 7734-7765, 7884-7950, 8046-8130, 8783-8853).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "kernels.h"

namespace nh {

#include "device_helpers.inc"
#include "repack.inc"
#include "gemv_kernels.inc"
#include "gemm_kernels.inc"

// ------------------------------------------------------------------ launchers

static bool g_nibble_bf16 = false;  // the packed fp8 -> bf16 convert turns nibble bytes into the integers 0..15
static bool g_nibble_i4 = false;    // the signed 4-bit convert with a byte select gives (n - 8) / 16 for nibble n ^ 8
static int g_cu_count = 256;
static size_t g_lds_limit = 64 * 1024;

// The launchers' view of the device is held once per process.  Every executor reports what it found on its
// device; the first report sets it, a later one that differs is refused by the caller (one kind of GPU per
// process: a second kind would need these per device).
static bool g_limits_set = false;
bool set_device_limits(int cu_count, size_t lds_per_block) {
    if (cu_count <= 0 || lds_per_block == 0) return false;
    if (g_limits_set) return cu_count == g_cu_count && lds_per_block == g_lds_limit;
    g_cu_count = cu_count;
    g_lds_limit = lds_per_block;
    g_limits_set = true;
    return true;
}

// Jobs must share x, dtype and column count.  hipErrorInvalidValue = "does not fit this
// kernel" (x too long for LDS); the caller then uses the tiled kernel.
template <uint32_t T, int R>
static hipError_t launch_gemv_t(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n_jobs,
                                const float *x, bool accumulate) {
    constexpr int E = Geo<T>::E;
    GemvBatch b;
    const uint32_t cols = mats[0].cols;
    b.n_chunks = (cols + E - 1) / E;
    b.x_pad = b.n_chunks * E;
    b.x = x;
    b.n_jobs = n_jobs;
    uint32_t rgs = 0;
    for (uint32_t j = 0; j < n_jobs; j++) {
        b.job[j].m = mats[j];
        b.job[j].y = ys[j];
        b.job[j].rg_begin = rgs;
        b.job[j].pad = 0;
        rgs += (mats[j].rows + R - 1) / R;
    }
    for (uint32_t j = n_jobs; j < GEMV_MAX_JOBS; j++) b.job[j] = b.job[0];
    b.total_rgs = rgs;
    b.unit0 = b.units = b.pad = 0;  // column windows are a lane-per-unit matter
    b.accumulate = accumulate;
    b.x2 = nullptr;
    b.eps = 0.f;
    b.pair = 0;
    const size_t lds = ((size_t)b.x_pad + (T == T_F32 || T == T_F16 ? 0 : 2 * (size_t)b.n_chunks)) * sizeof(float);
    if (lds > g_lds_limit) return hipErrorInvalidValue;
    auto kern = gemv_kernel<T, R>;
    static size_t configured = 0;  // per instantiation
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)g_lds_limit);
        if (e != hipSuccess) return e;
        configured = g_lds_limit;
    }
    size_t per_cu = g_lds_limit * 2 / (lds ? lds : 1);  // 160 KB of LDS per CU
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 2) per_cu = 2;                          // 16 wavefronts per CU
    uint32_t grid = (uint32_t)((size_t)g_cu_count * per_cu);
    const uint32_t needed = (rgs + GEMV_WAVES - 1) / GEMV_WAVES;
    if (grid > needed) grid = needed;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GEMV_WAVES * 64), lds, stream, b);
    return hipGetLastError();
}

// Decode the sixteen bytes 0x00..0x0f with the fp8 unpack on the device.
__global__ void fp8_nibble_probe(float *out) {
    const uint32_t n = threadIdx.x & 15u;
    auto v = __builtin_amdgcn_cvt_pk_f32_fp8((int)(n | (n << 8) | (n << 16) | (n << 24)), false);
    auto w = __builtin_amdgcn_cvt_pk_f32_fp8((int)(n | (n << 8) | (n << 16) | (n << 24)), true);
    out[4 * threadIdx.x] = v[0];
    out[4 * threadIdx.x + 1] = v[1];
    out[4 * threadIdx.x + 2] = w[0];
    out[4 * threadIdx.x + 3] = w[1];
    // the same bytes straight to bf16 with the scale 2^9 that makes nibble n the number n
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    const int packed = (int)(n | (n << 8) | (n << 16) | (n << 24));
    const bf16x2 lo = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(packed, 512.0f, false);
    const bf16x2 hi = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(packed, 512.0f, true);
    out[64 + 4 * threadIdx.x] = (float)lo[0];
    out[64 + 4 * threadIdx.x + 1] = (float)lo[1];
    out[64 + 4 * threadIdx.x + 2] = (float)hi[0];
    out[64 + 4 * threadIdx.x + 3] = (float)hi[1];
    // signed 4-bit convert of the low nibble of every byte, and of the high nibbles after a shift
    const uint32_t lo_n = (n | (n << 8) | (n << 16) | (n << 24)) ^ 0x88888888u, hi_n = ((n << 4) * 0x01010101u) ^ 0x88888888u;
    out[128 + 8 * threadIdx.x] = i4_of_byte<0>(lo_n);
    out[128 + 8 * threadIdx.x + 1] = i4_of_byte<1>(lo_n);
    out[128 + 8 * threadIdx.x + 2] = i4_of_byte<2>(lo_n);
    out[128 + 8 * threadIdx.x + 3] = i4_of_byte<3>(lo_n);
    out[128 + 8 * threadIdx.x + 4] = i4_of_byte<0>(hi_n >> 4);
    out[128 + 8 * threadIdx.x + 5] = i4_of_byte<1>(hi_n >> 4);
    out[128 + 8 * threadIdx.x + 6] = i4_of_byte<2>(hi_n >> 4);
    out[128 + 8 * threadIdx.x + 7] = i4_of_byte<3>(hi_n >> 4);
}

hipError_t probe_nibble_converts(hipStream_t stream, float *unit_out, bool *bf16_out, bool *i4_out) {
    *unit_out = 0.f;
    float *d = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&d), 256 * sizeof(float));
    if (e != hipSuccess) return e;
    float h[256];
    hipLaunchKernelGGL(fp8_nibble_probe, dim3(1), dim3(16), 0, stream, d);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpyAsync(h, d, sizeof h, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    (void)hipFree(d);
    if (e != hipSuccess) return e;
    const float unit = h[4];  // byte 0x01
    bool linear = unit > 0.f;
    for (int n = 0; n < 16 && linear; n++)
        for (int k = 0; k < 4; k++) linear = linear && h[4 * n + k] == (float)n * unit;
    // the unit must be a power of two so that folding it into a block scale is exact
    int ex;
    if (linear && std::frexp(unit, &ex) != 0.5f) linear = false;
    *unit_out = linear ? unit : 0.f;
    bool exact = true;  // fp8 -> bf16 with scale 512 must give the integers 0..15
    for (int n = 0; n < 16; n++)
        for (int k = 0; k < 4; k++) exact = exact && h[64 + 4 * n + k] == (float)n;
    const bool bf16_exact = exact;
    exact = true;
    for (int n = 0; n < 16; n++)
        for (int k = 0; k < 8; k++) exact = exact && h[128 + 8 * n + k] == (float)(n - 8) / 16.0f;
    if (bf16_out) *bf16_out = bf16_exact;
    if (i4_out) *i4_out = exact;
    return hipSuccess;
}

static float g_nib_mul = 0.f;  // 1 / (value of fp8 byte 0x01); 0 = fp8 unpack not usable
static bool g_converts_set = false;
bool set_nibble_converts(float unit, bool bf16_exact, bool i4_exact) {
    const float mul = unit > 0.f ? 1.0f / unit : 0.f;
    if (g_converts_set) return mul == g_nib_mul && bf16_exact == g_nibble_bf16 && i4_exact == g_nibble_i4;
    g_nib_mul = mul;
    g_nibble_bf16 = bf16_exact;
    g_nibble_i4 = i4_exact;
    g_converts_set = true;
    return true;
}

template <int LB, int NW, int PL, int PRO>
static hipError_t launch_q4k_lb(hipStream_t stream, const GemvBatch &b, uint32_t units, size_t lds) {
    const bool fp8 = g_nib_mul != 0.f;
    if (PRO != PRO_NONE && !fp8) return hipErrorInvalidValue;  // prologues are built for the fp8 unpack only
    size_t per_cu = g_lds_limit * 2 / (lds ? lds : 1);  // 160 KB of LDS per CU
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 32 / NW) per_cu = 32 / NW;             // 32 wavefronts per CU (measured +2.5 % on the decode step over 16)
    uint32_t grid = (uint32_t)((size_t)g_cu_count * per_cu);
    const uint32_t needed = (units + NW - 1) / NW;
    if (grid > needed) grid = needed;
    const bool one = grid == needed;  // a wavefront for every unit
    void (*kern)(GemvBatch, float) = nullptr;
    if (b.pair) {
        // the pair epilogue exists where a wavefront holds at most four rows, for one unit per wavefront
        if constexpr (LB >= 16 && PRO != PRO_SWIGLU) {
            if (one && fp8) kern = gemv_q4k_kernel<LB, NW, true, PL, true, PRO, true>;
        }
        if (!kern) return hipErrorInvalidValue;
    } else if constexpr (PRO == PRO_NONE) {
        kern = fp8 ? (one ? gemv_q4k_kernel<LB, NW, true, PL, true> : gemv_q4k_kernel<LB, NW, true, PL, false>)
                   : (one ? gemv_q4k_kernel<LB, NW, false, PL, true> : gemv_q4k_kernel<LB, NW, false, PL, false>);
    } else {
        kern = one ? gemv_q4k_kernel<LB, NW, true, PL, true, PRO> : gemv_q4k_kernel<LB, NW, true, PL, false, PRO>;
    }
    static size_t configured[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t &conf = configured[4 * (b.pair != 0) + 2 * fp8 + one];
    if (lds > 48 * 1024 && lds > conf) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)g_lds_limit);
        if (e != hipSuccess) return e;
        conf = g_lds_limit;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, stream, b, fp8 ? g_nib_mul : 1.0f);
    return hipGetLastError();
}

// Jobs of a lane-per-unit launch: lb lanes per row, 64 / lb rows per wavefront step.
static uint32_t fill_unit_jobs(GemvBatch &b, const MatView *mats, float *const *ys, uint32_t n_jobs, const float *x,
                               uint32_t lb) {
    const uint32_t rg_rows = 64 / lb;
    b.x = x;
    b.x2 = nullptr;
    b.eps = 0.f;
    b.pair = 0;
    b.n_jobs = n_jobs;
    b.n_chunks = 0;
    b.x_pad = mats[0].cols;
    b.pad = 0;
    uint32_t rgs = 0;
    for (uint32_t j = 0; j < n_jobs; j++) {
        b.job[j].m = mats[j];
        b.job[j].y = ys[j];
        b.job[j].rg_begin = rgs;
        b.job[j].pad = 0;
        rgs += (mats[j].rows + rg_rows - 1) / rg_rows;
    }
    for (uint32_t j = n_jobs; j < GEMV_MAX_JOBS; j++) b.job[j] = b.job[0];
    b.total_rgs = rgs;
    return rgs;
}

// Rows of nu units are cut into the fewest equal windows of at most max_units; window w
// covers units [first, first + count).
struct UnitWindows {
    uint32_t n, per;
    UnitWindows(uint32_t nu, uint32_t max_units) : n((nu + max_units - 1) / max_units), per((nu + n - 1) / n) {}
    uint32_t first(uint32_t w) const { return w * per; }
    uint32_t count(uint32_t w, uint32_t nu) const { return first(w) + per <= nu ? per : nu - first(w); }
};

struct GemvPrologue {
    int kind = PRO_NONE;        // PRO_RMSNORM: x2 = norm weights; PRO_SWIGLU: x2 = the up vector (x is gate)
    const float *x2 = nullptr;
    float eps = 0.f;
    bool pair = false;          // two jobs (gate, up): y of the first receives SiLU(gate) * up
};

template <int PRO>
static hipError_t launch_gemv_q4k_pro(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n_jobs,
                                      const float *x, bool accumulate, const GemvPrologue &pro) {
    const uint32_t nb = mats[0].nb;
    // one lane per super-block, at most 64 per row and launch: longer rows take several launches
    const UnitWindows win(nb, 64);
    if (PRO != PRO_NONE && win.n != 1) return hipErrorInvalidValue;  // a prologue needs all of x in one workgroup
    if (pro.pair && (win.n != 1 || n_jobs != 2 || mats[0].rows != mats[1].rows)) return hipErrorInvalidValue;
    for (uint32_t w = 0; w < win.n; w++) {
        const uint32_t units = win.count(w, nb);
        uint32_t lbb = 1;  // super-blocks per row, rounded up to a power of two
        while (lbb < 64 && lbb < units) lbb <<= 1;
        // Two lanes per super-block for matrices that would otherwise give the chip fewer than about ten
        // wavefront steps per CU (measured crossover: 8192 x 4096 gains 11 %, 12288 x 4096 loses 6 %).
        size_t full_steps = 0;
        for (uint32_t j = 0; j < n_jobs; j++) full_steps += (mats[j].rows + 64 / lbb - 1) / (64 / lbb);
        const bool halves = lbb <= 16 && full_steps <= (size_t)10 * g_cu_count;
        const uint32_t lb = halves ? 2 * lbb : lbb;
        GemvBatch b;
        const uint32_t rgs = fill_unit_jobs(b, mats, ys, n_jobs, x, lb);
        b.unit0 = win.first(w);
        b.units = units;
        b.accumulate = accumulate || w > 0;
        b.x2 = pro.x2;
        b.eps = pro.eps;
        b.pair = pro.pair ? 1u : 0u;
        // x slots, the sub-block sums of x, and room for one partial sum per wavefront (RMSNorm prologue)
        const size_t lds = (size_t)(64 * (lbb * 4 + 4) + lbb * 8 + 16) * sizeof(float);
        if (lds > g_lds_limit) return hipErrorInvalidValue;
        hipError_t e;
        if (halves) {
            switch (lb) {
            case 2: e = launch_q4k_lb<2, 4, 4, PRO>(stream, b, rgs, lds); break;
            case 4: e = launch_q4k_lb<4, 4, 4, PRO>(stream, b, rgs, lds); break;
            case 8: e = launch_q4k_lb<8, 4, 4, PRO>(stream, b, rgs, lds); break;
            case 16: e = launch_q4k_lb<16, 4, 4, PRO>(stream, b, rgs, lds); break;
            default: e = launch_q4k_lb<32, 4, 4, PRO>(stream, b, rgs, lds); break;
            }
        } else {
            switch (lb) {
            // Short rows: small workgroups, so that even a 1024-row matrix spreads over every CU.
            case 1: e = launch_q4k_lb<1, 4, 8, PRO>(stream, b, rgs, lds); break;
            case 2: e = launch_q4k_lb<2, 4, 8, PRO>(stream, b, rgs, lds); break;
            case 4: e = launch_q4k_lb<4, 4, 8, PRO>(stream, b, rgs, lds); break;
            case 8: e = launch_q4k_lb<8, 4, 8, PRO>(stream, b, rgs, lds); break;
            case 16: e = launch_q4k_lb<16, 4, 8, PRO>(stream, b, rgs, lds); break;
            case 32: e = launch_q4k_lb<32, 8, 8, PRO>(stream, b, rgs, lds); break;
            default: e = launch_q4k_lb<64, 8, 8, PRO>(stream, b, rgs, lds); break;
            }
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

static hipError_t launch_gemv_q4k(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n_jobs,
                                  const float *x, bool accumulate, const GemvPrologue &pro = GemvPrologue()) {
    switch (pro.kind) {
    case PRO_NONE: return launch_gemv_q4k_pro<PRO_NONE>(stream, mats, ys, n_jobs, x, accumulate, pro);
    case PRO_RMSNORM: return launch_gemv_q4k_pro<PRO_RMSNORM>(stream, mats, ys, n_jobs, x, accumulate, pro);
    case PRO_SWIGLU: return launch_gemv_q4k_pro<PRO_SWIGLU>(stream, mats, ys, n_jobs, x, accumulate, pro);
    default: return hipErrorInvalidValue;
    }
}

template <int LB, int NW>
static hipError_t launch_q6k_lb(hipStream_t stream, const GemvBatch &b, uint32_t units, size_t lds) {
    auto kern = gemv_q6k_kernel<LB, NW>;
    static size_t configured = 0;
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)g_lds_limit);
        if (e != hipSuccess) return e;
        configured = g_lds_limit;
    }
    size_t per_cu = g_lds_limit * 2 / (lds ? lds : 1);
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 16 / NW) per_cu = 16 / NW;             // 16 wavefronts per CU (32 measured 5 % slower on the 431 MB head)
    uint32_t grid = (uint32_t)((size_t)g_cu_count * per_cu);
    const uint32_t needed = (units + NW - 1) / NW;
    if (grid > needed) grid = needed;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, stream, b);
    return hipGetLastError();
}

static hipError_t launch_gemv_q6k(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n_jobs,
                                  const float *x, bool accumulate) {
    const uint32_t nb = mats[0].nb;
    const UnitWindows win(nb, 64);
    for (uint32_t w = 0; w < win.n; w++) {
        const uint32_t units = win.count(w, nb);
        uint32_t lb = 1;
        while (lb < 64 && lb < units) lb <<= 1;
        GemvBatch b;
        const uint32_t rgs = fill_unit_jobs(b, mats, ys, n_jobs, x, lb);
        b.unit0 = win.first(w);
        b.units = units;
        b.accumulate = accumulate || w > 0;
        const size_t lds = (size_t)(64 * (lb * 4 + 4)) * sizeof(float);
        if (lds > g_lds_limit) return hipErrorInvalidValue;
        hipError_t e;
        switch (lb) {
        case 1: e = launch_q6k_lb<1, 4>(stream, b, rgs, lds); break;
        case 2: e = launch_q6k_lb<2, 4>(stream, b, rgs, lds); break;
        case 4: e = launch_q6k_lb<4, 4>(stream, b, rgs, lds); break;
        case 8: e = launch_q6k_lb<8, 4>(stream, b, rgs, lds); break;
        case 16: e = launch_q6k_lb<16, 4>(stream, b, rgs, lds); break;
        case 32: e = launch_q6k_lb<32, 8>(stream, b, rgs, lds); break;
        default: e = launch_q6k_lb<64, 16>(stream, b, rgs, lds); break;  // measured 7 % faster than 8 wavefronts
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <uint32_t T, int LB, int NW>
static hipError_t launch_b32_lb(hipStream_t stream, const GemvBatch &b, uint32_t units, size_t lds) {
    const bool fp8 = T == T_Q4_0 && g_nibble_i4;  // which of the two instantiations
    const void *kern = fp8 ? reinterpret_cast<const void *>(gemv_b32_kernel<T, LB, NW, true>)
                           : reinterpret_cast<const void *>(gemv_b32_kernel<T, LB, NW, false>);
    static size_t configured[2] = {0, 0};
    if (lds > 48 * 1024 && lds > configured[fp8]) {
        hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)g_lds_limit);
        if (e != hipSuccess) return e;
        configured[fp8] = g_lds_limit;
    }
    size_t per_cu = g_lds_limit * 2 / (lds ? lds : 1);  // 160 KB of LDS per CU
    if (per_cu < 1) per_cu = 1;
    constexpr size_t wpc = T == T_Q8_0 ? 32 : 16;       // wavefronts per CU (measured: Q8_0 +5 % at 32, Q4_0 -4 %)
    if (per_cu > wpc / NW) per_cu = wpc / NW;
    uint32_t grid = (uint32_t)((size_t)g_cu_count * per_cu);
    const uint32_t needed = (units + NW - 1) / NW;
    if (grid > needed) grid = needed;
    if (fp8)
        hipLaunchKernelGGL((gemv_b32_kernel<T, LB, NW, true>), dim3(grid), dim3(NW * 64), lds, stream, b);
    else
        hipLaunchKernelGGL((gemv_b32_kernel<T, LB, NW, false>), dim3(grid), dim3(NW * 64), lds, stream, b);
    return hipGetLastError();
}

// hipErrorInvalidValue: rows are not whole units (block-order layout).
template <uint32_t T>
static hipError_t launch_gemv_b32(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n_jobs,
                                  const float *x, bool accumulate) {
    using G = B32Geo<T>;
    const uint32_t cols = mats[0].cols;
    if (!piece_major(T, cols)) return hipErrorInvalidValue;
    const uint32_t nu = cols / G::UC;
    // up to 64 lanes per row, and as many unit columns per lane as keep x within LDS
    const size_t iter_lds = (size_t)((G::UC / 4) * (64 * 4 + 4) + G::NBLK * 64) * sizeof(float);
    const uint32_t max_iter = (uint32_t)(g_lds_limit / iter_lds) ? (uint32_t)(g_lds_limit / iter_lds) : 1;
    const UnitWindows win(nu, 64 * max_iter);
    for (uint32_t w = 0; w < win.n; w++) {
        const uint32_t units = win.count(w, nu);
        uint32_t lb = 1;
        while (lb < 64 && lb < units) lb <<= 1;
        const uint32_t n_iter = (units + lb - 1) / lb;
        GemvBatch b;
        const uint32_t rgs = fill_unit_jobs(b, mats, ys, n_jobs, x, lb);
        b.unit0 = win.first(w);
        b.units = units;
        b.accumulate = accumulate || w > 0;
        const size_t lds = (size_t)n_iter * ((G::UC / 4) * (lb * 4 + 4) + G::NBLK * lb) * sizeof(float);
        if (lds > g_lds_limit) return hipErrorInvalidValue;
        hipError_t e;
        switch (lb) {
        case 1: e = launch_b32_lb<T, 1, 4>(stream, b, rgs, lds); break;
        case 2: e = launch_b32_lb<T, 2, 4>(stream, b, rgs, lds); break;
        case 4: e = launch_b32_lb<T, 4, 4>(stream, b, rgs, lds); break;
        case 8: e = launch_b32_lb<T, 8, 4>(stream, b, rgs, lds); break;
        case 16: e = launch_b32_lb<T, 16, 4>(stream, b, rgs, lds); break;
        case 32: e = launch_b32_lb<T, 32, 8>(stream, b, rgs, lds); break;
        default:  // 16 wavefronts per workgroup measured 3 % faster for Q8_0, 12 % slower for the nibble dtypes
            e = T == T_Q8_0 ? launch_b32_lb<T, 64, 16>(stream, b, rgs, lds) : launch_b32_lb<T, 64, 8>(stream, b, rgs, lds);
            break;
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <uint32_t T>
static hipError_t launch_tiled_t(hipStream_t stream, const MatView &m, uint32_t tokens, const float *x, float *y) {
    dim3 grid((m.rows + GT_ROWS - 1) / GT_ROWS, (tokens + GT_TOK - 1) / GT_TOK);
    hipLaunchKernelGGL(gemm_tiled_kernel<T>, grid, dim3(256), 0, stream, m, x, y, tokens);
    return hipGetLastError();
}

template <uint32_t T>
static hipError_t launch_multi_t(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n, const float *x,
                                 bool accumulate) {
    if constexpr (T == T_Q4_K) return launch_gemv_q4k(stream, mats, ys, n, x, accumulate);
    if constexpr (T == T_Q6_K) return launch_gemv_q6k(stream, mats, ys, n, x, accumulate);
    if constexpr (T == T_Q8_0 || T == T_Q4_0 || T == T_Q5_0 || T == T_Q5_1) {
        hipError_t e = launch_gemv_b32<T>(stream, mats, ys, n, x, accumulate);
        if (e != hipErrorInvalidValue) return e;
        (void)hipGetLastError();
    }
    // Rows per lane: four share the lane's activations, but a wavefront owns whole row groups, so
    // matrices with few rows take fewer rows per group to give every wavefront of the chip one.
    size_t rows = 0;
    for (uint32_t j = 0; j < n; j++) rows += mats[j].rows;
    const size_t wavefronts = (size_t)g_cu_count * 16;
    if (rows >= 4 * wavefronts) return launch_gemv_t<T, 4>(stream, mats, ys, n, x, accumulate);
    if (rows >= 2 * wavefronts) return launch_gemv_t<T, 2>(stream, mats, ys, n, x, accumulate);
    return launch_gemv_t<T, 1>(stream, mats, ys, n, x, accumulate);
}

// ---- MFMA GEMM: planning and launch

static bool mm_type(uint32_t type) { return type != T_F32 && type != T_F16 && type_supported(type); }

struct MmPlan {
    MmBatch b;
    int tt;             // token tiles of 32 per workgroup (1 or 2)
    bool tile16;        // 16-token tiles (gemm_mfma16_kernel) instead
    bool tile16x2;      // Q4_K, 17 to 32 tokens: gemm_mfma16_kernel with two 16-token tiles per workgroup (planned as a 32-token tile)
    uint32_t max_tok;   // most tokens of any job
    uint32_t n_groups;  // groups of 16 columns
    size_t xb_bytes, sx_bytes, part_bytes;
};

static size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }

// Jobs share dtype and column count; every job has at least MM_MIN_TOKENS tokens.
static void mm_plan(const MatView *mats, const uint32_t *tokens, const float *const *xs, float *const *ys, uint32_t n,
                    MmPlan &p) {
    MmBatch &b = p.b;
    uint32_t max_tok = 0, total_tok = 0;
    for (uint32_t j = 0; j < n; j++) max_tok = tokens[j] > max_tok ? tokens[j] : max_tok;
    p.tt = max_tok > 32 ? 2 : 1;
    p.max_tok = max_tok;
    p.tile16 = max_tok <= 16 && mats[0].type != T_Q6_K;
    // measured on 4096x14336 / 14336x4096 at 17, 24 and 32 tokens: Q4_K 26.4 / 27.7 / 30.4 -> 25.9 / 27.4 / 28.5 us, a
    // routed layer 394 -> 380 us, 32 sequences decoded together +3 %; Q4_0, Q5_0, Q5_1 and Q8_0 lose 1-2.5 us to the
    // 32-token tile, which skips the matrix-core work of empty token quarters
    p.tile16x2 = !p.tile16 && max_tok <= 32 && mats[0].type == T_Q4_K;
    const uint32_t tile_tok = p.tile16 ? 16u : 32u * (uint32_t)p.tt;
    uint32_t wgs = 0;
    bool any_split = false;
    const uint32_t n_steps = mats[0].cols / 32;
    // Columns are shared between workgroups as far as that shortens the launch: every share costs a partial
    // result written and read back.  A CU holds two workgroups of these kernels, and one alone already gets 0.63-0.7
    // of what the two get together (measured on the 16-token kernel: a step of 0.48 us alone, 0.76 us each
    // together), so what counts is how evenly the steps fall on the CUs.  The launch is priced in steps of a
    // workgroup that shares its CU: whole rounds of 2 x CUs workgroups, then the rest (alone on their CUs if they
    // are at most one per CU), two more steps per workgroup for its start and end; the shares at what the launch
    // that sums them costs (their bytes at 3 TB/s + 3.5 us).  The constants are fitted to 4096x14336 / 14336x4096
    // products of 8 to 512 tokens and to the grouped products of a routed layer (8 experts, 9 to 21 tokens each).
    uint32_t launch_tiles = 0;
    size_t share_bytes = 0;  // one share of every job
    for (uint32_t j = 0; j < n; j++) {
        launch_tiles += ((tokens[j] + tile_tok - 1) / tile_tok) * ((mats[j].rows + MM_ROWS - 1) / MM_ROWS);
        share_bytes += (size_t)tokens[j] * mats[j].rows * sizeof(float);
    }
    // a share is at least 256 columns: finer ones (32 shares of a 4096-column matrix) cost the launch that sums them
    // more than they gain (8 sequences decoded together: 2110 -> 2055 tok/s)
    uint32_t ks_max = n_steps / 8;
    if (ks_max > 32) ks_max = 32;
    if (ks_max < 1) ks_max = 1;
    const uint32_t slots = (uint32_t)(2 * g_cu_count), alone = (uint32_t)g_cu_count;
    const double step_us = p.tt == 2 ? 1.5 : 0.7;
    uint32_t ks_launch = 1;
    double best = 0.0;
    for (uint32_t ks = 1; ks <= ks_max; ks++) {
        const uint64_t wg = (uint64_t)(launch_tiles ? launch_tiles : 1) * ks;
        const double len = (double)((n_steps + ks - 1) / ks) + 2.0;
        const uint64_t rounds = wg / slots, rest = wg % slots;
        double cost = (double)rounds * len + (rest == 0 ? 0.0 : rest <= alone ? 0.7 * len : len);
        if (ks > 1) cost += ((double)ks * (double)share_bytes / 3.0e6 + 3.5) / step_us;
        if (ks == 1 || cost < best) {
            best = cost;
            ks_launch = ks;
        }
    }
    for (uint32_t j = 0; j < n; j++) {
        MmJob &job = b.job[j];
        job.m = mats[j];
        job.x = xs ? xs[j] : nullptr;
        job.y = ys ? ys[j] : nullptr;
        job.part = nullptr;
        job.tokens = tokens[j];
        // products of the same activations (q, k, v of one input) read one set of split slots
        const bool same_x = j > 0 && xs && xs[j] == xs[j - 1] && tokens[j] == tokens[j - 1];
        if (same_x) total_tok -= tokens[j];
        job.tok_off = total_tok;
        job.wg_begin = wgs;
        job.tok_tiles = (tokens[j] + tile_tok - 1) / tile_tok;
        const uint32_t tiles = job.tok_tiles * ((mats[j].rows + MM_ROWS - 1) / MM_ROWS);
        uint32_t ks = ks_launch;
        job.ksplit = ks;
        job.pad = 0;
        wgs += tiles * ks;
        any_split = any_split || ks > 1;
        total_tok += tokens[j];
    }
    for (uint32_t j = n; j < MM_MAX_JOBS; j++) b.job[j] = b.job[0];
    b.n_jobs = n;
    b.mpad = total_tok + (p.tile16 ? 16 : 64);  // a tile may read up to 15 resp. 63 slots past its job's last token
    b.total_wgs = wgs;
    b.any_split = any_split ? 1u : 0u;
    b.nibble_bf16 = g_nibble_bf16 ? 1u : 0u;
    b.pad0 = b.pad1 = b.pad2 = 0;
    p.n_groups = mats[0].cols / 16;
    p.xb_bytes = up256((size_t)p.n_groups * 6 * b.mpad * sizeof(uint4));
    p.sx_bytes = up256((size_t)p.n_groups * b.mpad * sizeof(float));
    size_t part = 0;
    for (uint32_t j = 0; j < n; j++)
        if (b.job[j].ksplit > 1) part += up256((size_t)b.job[j].ksplit * tokens[j] * mats[j].rows * sizeof(float));
    p.part_bytes = part;
}

// INLINE (TT = 1): the jobs' x are plain f32 rows and the kernel cuts them itself.
template <uint32_t T, int TT, int VQ, bool INLINE = false, bool FB = false, bool NORM = false>
static hipError_t launch_mm_main(hipStream_t stream, const MmBatch &b) {
    // FB: the device's shortcut from nibbles to bf16 codes is usable (probed at start-up): the packed
    // fp8 convert for Q4_K, the signed 4-bit convert for Q4_0
    if constexpr (T == T_Q4_K && !FB) {
        if (b.nibble_bf16) return launch_mm_main<T, TT, VQ, INLINE, true, NORM>(stream, b);
    }
    if constexpr (T == T_Q4_0 && !FB) {
        if (g_nibble_i4) return launch_mm_main<T, TT, VQ, INLINE, true, NORM>(stream, b);
    }
    constexpr size_t lds = 2 * MmStage<T, TT>::BYTES;  // two pipeline stages
    auto kern = gemm_mfma_kernel<T, TT, VQ, FB, INLINE, NORM>;
    static bool configured = false;
    if (lds > 48 * 1024 && !configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)lds);
        if (e != hipSuccess) return e;
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(b.total_wgs), dim3(256), lds, stream, b);
    return hipGetLastError();
}

// INLINE: the jobs' x are plain f32 rows and the kernel cuts them itself (no mm_xsplit launch before it).
// NT: 16-token tiles per workgroup (2: the plan's 32-token tiles).
template <uint32_t T, bool INLINE = false, bool FB = false, bool NORM = false, int NT = 1>
static hipError_t launch_mm16_main(hipStream_t stream, const MmBatch &b) {
    if constexpr (T == T_Q4_K && !FB) {
        if (b.nibble_bf16) return launch_mm16_main<T, INLINE, true, NORM, NT>(stream, b);
    }
    if constexpr (T == T_Q4_0 && !FB) {
        if (g_nibble_i4) return launch_mm16_main<T, INLINE, true, NORM, NT>(stream, b);
    }
    constexpr size_t lds = Mm16Traits<T, NT>::LDS_BYTES;  // two pipeline stages, the scale exchange
    static_assert(lds <= 48 * 1024, "within the default dynamic LDS limit");
    hipLaunchKernelGGL((gemm_mfma16_kernel<T, FB, INLINE, NORM, NT>), dim3(b.total_wgs), dim3(256), lds, stream, b);
    return hipGetLastError();
}

// Workgroups per job of the share reduction: one float4 per thread (one float for small jobs, as the kernel
// chooses) where that fills fewer than 512.
static uint32_t mm_reduce_blocks(const MmBatch &b) {
    size_t most = 1;
    for (uint32_t j = 0; j < b.n_jobs; j++) {
        const size_t total = (size_t)b.job[j].tokens * b.job[j].m.rows;
        const size_t per_thread = total >= MM_REDUCE_WIDE_MIN ? 4 : 1, blocks = ((total + per_thread - 1) / per_thread + 255) / 256;
        if (b.job[j].ksplit > 1 && blocks > most) most = blocks;
    }
    return (uint32_t)(most < 512 ? most : 512);
}

template <uint32_t T>
static hipError_t launch_mm_t(hipStream_t stream, MmPlan &p, void *ws, size_t ws_bytes) {
    if (p.xb_bytes + p.sx_bytes + p.part_bytes > ws_bytes) return hipErrorInvalidValue;
    MmBatch &b = p.b;
    uint8_t *base = static_cast<uint8_t *>(ws);
    b.xb = reinterpret_cast<uint4 *>(base);
    b.sx = reinterpret_cast<float *>(base + p.xb_bytes);
    uint8_t *part = base + p.xb_bytes + p.sx_bytes;
    for (uint32_t j = 0; j < b.n_jobs; j++)
        if (b.job[j].ksplit > 1) {
            b.job[j].part = reinterpret_cast<float *>(part);
            part += up256((size_t)b.job[j].ksplit * b.job[j].tokens * b.job[j].m.rows * sizeof(float));
        }
    hipError_t e;
    if constexpr (T != T_Q6_K) {
        if (p.tile16) {  // the 16-token kernel cuts the activations itself
            e = launch_mm16_main<T, true>(stream, b);
            if (e != hipSuccess) return e;
            if (b.any_split) hipLaunchKernelGGL(mm_reduce_kernel, dim3(mm_reduce_blocks(b), b.n_jobs), dim3(256), 0, stream, b);
            return hipGetLastError();
        }
    }
    if constexpr (T == T_Q4_K) {
        if (p.tile16x2) {
            e = launch_mm16_main<T, true, false, false, 2>(stream, b);
            if (e != hipSuccess) return e;
            if (b.any_split) hipLaunchKernelGGL(mm_reduce_kernel, dim3(mm_reduce_blocks(b), b.n_jobs), dim3(256), 0, stream, b);
            return hipGetLastError();
        }
    }
    if (p.tt == 2) {  // 64-token tiles: the activations are cut once, by a launch of their own
        hipLaunchKernelGGL(mm_xsplit_kernel<T>, dim3((b.mpad + XS_TOK - 1) / XS_TOK, (p.n_groups + XS_GRP - 1) / XS_GRP),
                           dim3(256), 0, stream, b, p.n_groups);
        e = launch_mm_main<T, 2, 4>(stream, b);
    } else if (p.max_tok <= 8) e = launch_mm_main<T, 1, 1, true>(stream, b);
    else if (p.max_tok <= 16) e = launch_mm_main<T, 1, 2, true>(stream, b);
    else if (p.max_tok <= 24) e = launch_mm_main<T, 1, 3, true>(stream, b);
    else e = launch_mm_main<T, 1, 4, true>(stream, b);
    if (e != hipSuccess) return e;
    if (b.any_split) hipLaunchKernelGGL(mm_reduce_kernel, dim3(mm_reduce_blocks(b), b.n_jobs), dim3(256), 0, stream, b);
    return hipGetLastError();
}

static hipError_t launch_mm(hipStream_t stream, MmPlan &p, void *ws, size_t ws_bytes) {
    switch (p.b.job[0].m.type) {
    case T_Q4_0: return launch_mm_t<T_Q4_0>(stream, p, ws, ws_bytes);
    case T_Q5_0: return launch_mm_t<T_Q5_0>(stream, p, ws, ws_bytes);
    case T_Q5_1: return launch_mm_t<T_Q5_1>(stream, p, ws, ws_bytes);
    case T_Q8_0: return launch_mm_t<T_Q8_0>(stream, p, ws, ws_bytes);
    case T_Q4_K: return launch_mm_t<T_Q4_K>(stream, p, ws, ws_bytes);
    case T_Q6_K: return launch_mm_t<T_Q6_K>(stream, p, ws, ws_bytes);
    default: return hipErrorInvalidValue;
    }
}

// F32 / F16 weights, two or more tokens: gemm_fmfma_kernel (+ fg_reduce_kernel when columns are shared).
struct FgPlan {
    FgJob job;
    int tt;
    uint32_t wgs;
    size_t part_bytes;
};
static void fg_plan(const MatView &m, uint32_t tokens, FgPlan &p) {
    p.tt = tokens > 32 ? 2 : tokens > 16 ? 1 : 0;   // 0: a 16-token tile
    const uint32_t tile_tok = p.tt == 0 ? 16u : 32u * (uint32_t)p.tt;
    const uint32_t tok_tiles = (tokens + tile_tok - 1) / tile_tok, row_tiles = (m.rows + FG_ROWS - 1) / FG_ROWS;
    const uint32_t tiles = tok_tiles * row_tiles, n_steps = (m.cols + FG_K - 1) / FG_K;
    // about two workgroups per CU (16-token tiles measured at 1 / 2 / 3 / 4 per CU: F16 4096x14336, 8 tokens, 51 / 40 / 40 / 44 us)
    uint32_t ks = (uint32_t)(2 * g_cu_count) / (tiles ? tiles : 1);
    if (ks > n_steps / 8) ks = n_steps / 8;                           // a share is at least 256 columns
    if (ks > 32) ks = 32;
    if (ks < 1) ks = 1;
    p.job.m = m;
    p.job.x = nullptr;
    p.job.y = nullptr;
    p.job.part = nullptr;
    p.job.tokens = tokens;
    p.job.tok_tiles = tok_tiles;
    p.job.ksplit = ks;
    p.job.pad = 0;
    p.wgs = tiles * ks;
    p.part_bytes = ks > 1 ? up256((size_t)ks * tokens * m.rows * sizeof(float)) : 0;
}

template <uint32_t T, int TT>
static hipError_t launch_fg_main(hipStream_t stream, const FgPlan &p) {
    constexpr size_t lds = (size_t)2 * (FG_ROWS + (TT == 0 ? 16 : 32 * TT)) * FG_LD * sizeof(float);
    auto kern = gemm_fmfma_kernel<T, TT>;
    static bool configured = false;
    if (lds > 48 * 1024 && !configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(p.wgs), dim3(256), lds, stream, p.job);
    return hipGetLastError();
}

static hipError_t launch_fg(hipStream_t stream, const MatView &m, uint32_t tokens, const float *x, float *y, void *ws,
                            size_t ws_bytes) {
    FgPlan p;
    fg_plan(m, tokens, p);
    if (p.part_bytes > ws_bytes) return hipErrorInvalidValue;
    p.job.x = x;
    p.job.y = y;
    p.job.part = static_cast<float *>(ws);
    hipError_t e;
    if (m.type == T_F16)
        e = p.tt == 2 ? launch_fg_main<T_F16, 2>(stream, p) : p.tt == 1 ? launch_fg_main<T_F16, 1>(stream, p) : launch_fg_main<T_F16, 0>(stream, p);
    else
        e = p.tt == 2 ? launch_fg_main<T_F32, 2>(stream, p) : p.tt == 1 ? launch_fg_main<T_F32, 1>(stream, p) : launch_fg_main<T_F32, 0>(stream, p);
    if (e != hipSuccess || p.job.ksplit < 2) return e;
    const size_t total = (size_t)tokens * m.rows, vec = (total + 3) / 4, blocks = (vec + 255) / 256;
    hipLaunchKernelGGL(fg_reduce_kernel, dim3((unsigned)(blocks < 512 ? blocks : 512)), dim3(256), 0, stream, p.job.part, y, total,
                       p.job.ksplit);
    return hipGetLastError();
}

// Single-token products, and whatever the other paths do not take.
static hipError_t launch_plain(hipStream_t stream, const MatView &m, uint32_t tokens, const float *x, float *y) {
    auto run = [&](auto tag) -> hipError_t {
        constexpr uint32_t T = decltype(tag)::value;
        if (tokens == 1) {
            hipError_t e = launch_multi_t<T>(stream, &m, &y, 1, x, false);
            if (e != hipErrorInvalidValue) return e;
            (void)hipGetLastError();
        }
        return launch_tiled_t<T>(stream, m, tokens, x, y);
    };
    switch (m.type) {
    case T_F32: return run(std::integral_constant<uint32_t, T_F32>{});
    case T_F16: return run(std::integral_constant<uint32_t, T_F16>{});
    case T_Q4_0: return run(std::integral_constant<uint32_t, T_Q4_0>{});
    case T_Q5_0: return run(std::integral_constant<uint32_t, T_Q5_0>{});
    case T_Q5_1: return run(std::integral_constant<uint32_t, T_Q5_1>{});
    case T_Q8_0: return run(std::integral_constant<uint32_t, T_Q8_0>{});
    case T_Q4_K: return run(std::integral_constant<uint32_t, T_Q4_K>{});
    case T_Q6_K: return run(std::integral_constant<uint32_t, T_Q6_K>{});
    default: return hipErrorInvalidValue;
    }
}

// Length of the run of groups starting at g that one MFMA launch can take.
// (Two tokens are two single-token launches: 2 x 9-15 us on the 33-44 MB matrices against 24-29 us for the
// three launches of the MFMA path, and row t of the result is then bit for bit the GEMV of token t.)
static uint32_t mm_run(const MatView *mats, const uint32_t *tokens, uint32_t n, uint32_t g) {
    if (!mm_type(mats[g].type) || tokens[g] < MM_MIN_TOKENS) return 0;
    uint32_t run = 1;
    while (g + run < n && run < (uint32_t)MM_MAX_JOBS && tokens[g + run] >= MM_MIN_TOKENS && mats[g + run].type == mats[g].type &&
           mats[g + run].cols == mats[g].cols)
        run++;
    return run;
}

// A run is launched as up to two batches: the products of at most 16 tokens (16-token tiles) and the
// others (32- or 64-token tiles); a product of 9 tokens beside one of 21 would otherwise pay for 32.
struct MmClass {
    MatView mats[MM_MAX_JOBS];
    uint32_t tokens[MM_MAX_JOBS];
    const float *xs[MM_MAX_JOBS];
    float *ys[MM_MAX_JOBS];
    uint32_t n;
};
static void mm_classes(const MatView *mats, const uint32_t *tokens, const float *const *xs, float *const *ys, uint32_t run,
                       MmClass (&cls)[2]) {
    cls[0].n = cls[1].n = 0;
    for (uint32_t j = 0; j < run; j++) {
        MmClass &c = cls[tokens[j] <= 16 && mats[j].type != T_Q6_K ? 0 : 1];
        c.mats[c.n] = mats[j];
        c.tokens[c.n] = tokens[j];
        c.xs[c.n] = xs ? xs[j] : nullptr;
        c.ys[c.n] = ys ? ys[j] : nullptr;
        c.n++;
    }
}

size_t gemm_workspace_bytes(const MatView *mats, const uint32_t *tokens, uint32_t n) {
    size_t need = 0;
    for (uint32_t g = 0; g < n;) {
        if (tokens[g] == 0 || mats[g].rows == 0) { g++; continue; }
        const uint32_t run = mm_run(mats, tokens, n, g);
        if (run == 0) {
            if ((mats[g].type == T_F32 || mats[g].type == T_F16) && tokens[g] > 1) {
                FgPlan p;
                fg_plan(mats[g], tokens[g], p);
                need = p.part_bytes > need ? p.part_bytes : need;
            }
            g++;
            continue;
        }
        MmClass cls[2];
        mm_classes(mats + g, tokens + g, nullptr, nullptr, run, cls);
        for (const MmClass &c : cls) {
            if (c.n == 0) continue;
            MmPlan p;
            mm_plan(c.mats, c.tokens, nullptr, nullptr, c.n, p);
            const size_t bytes = p.xb_bytes + p.sx_bytes + p.part_bytes;
            need = bytes > need ? bytes : need;
        }
        g += run;
    }
    return need;
}

hipError_t launch_gemm_groups(hipStream_t stream, const MatView *mats, const MatView *tiled, const uint32_t *tokens,
                              const float *const *xs, float *const *ys, uint32_t n, void *ws, size_t ws_bytes) {
    for (uint32_t g = 0; g < n;) {
        if (tokens[g] == 0 || mats[g].rows == 0) { g++; continue; }
        const uint32_t run = mm_run(mats, tokens, n, g);
        hipError_t e = hipSuccess;
        if (run == 0) {
            if (mm_type(mats[g].type) && tokens[g] > 1) {
                for (uint32_t t = 0; t < tokens[g] && e == hipSuccess; t++)
                    e = launch_plain(stream, mats[g], 1, xs[g] + (size_t)t * mats[g].cols, ys[g] + (size_t)t * mats[g].rows);
            } else if ((mats[g].type == T_F32 || mats[g].type == T_F16) && tokens[g] > 1) {
                e = launch_fg(stream, mats[g], tokens[g], xs[g], ys[g], ws, ws_bytes);
            } else {
                e = launch_plain(stream, mats[g], tokens[g], xs[g], ys[g]);
            }
            g++;
        } else {
            MmClass cls[2];
            mm_classes(tiled + g, tokens + g, xs + g, ys + g, run, cls);
            for (const MmClass &c : cls) {  // the batches follow each other on the stream and share the workspace
                if (c.n == 0 || e != hipSuccess) continue;
                MmPlan p;
                mm_plan(c.mats, c.tokens, c.xs, c.ys, c.n, p);
                e = launch_mm(stream, p, ws, ws_bytes);
            }
            g += run;
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// ---- activations that stay in the split form between products

static uint32_t act_mpad(uint32_t type, uint32_t tokens) { return tokens + (tokens <= 16 && type != T_Q6_K ? 16u : 64u); }

size_t act_bytes(uint32_t type, uint32_t cols, uint32_t max_tokens) {
    if (!mm_type(type) || cols % 32 != 0 || max_tokens == 0) return 0;
    const size_t n_groups = cols / 16, mpad = (size_t)max_tokens + 64;
    return up256(n_groups * 6 * mpad * sizeof(uint4)) + up256(n_groups * mpad * sizeof(float));
}

// Where `tokens` tokens lie in an activation buffer made for up to max_tokens (the slot stride follows the token
// count, as in a product's own workspace; the sums start where the planes of max_tokens would end).
static ActView act_view(void *act, uint32_t type, uint32_t cols, uint32_t max_tokens, uint32_t tokens) {
    ActView v;
    const size_t n_groups = cols / 16;
    v.xb = static_cast<uint4 *>(act);
    v.sx = reinterpret_cast<float *>(static_cast<uint8_t *>(act) + up256(n_groups * 6 * ((size_t)max_tokens + 64) * sizeof(uint4)));
    v.mpad = act_mpad(type, tokens);
    v.n_groups = (uint32_t)n_groups;
    return v;
}

template <typename F> static hipError_t mm_by_type(uint32_t type, F &&run) {
    switch (type) {
    case T_Q4_0: return run(std::integral_constant<uint32_t, T_Q4_0>{});
    case T_Q5_0: return run(std::integral_constant<uint32_t, T_Q5_0>{});
    case T_Q5_1: return run(std::integral_constant<uint32_t, T_Q5_1>{});
    case T_Q8_0: return run(std::integral_constant<uint32_t, T_Q8_0>{});
    case T_Q4_K: return run(std::integral_constant<uint32_t, T_Q4_K>{});
    case T_Q6_K: return run(std::integral_constant<uint32_t, T_Q6_K>{});
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_act_split(hipStream_t stream, void *act, uint32_t type, uint32_t cols, uint32_t max_tokens, uint32_t tokens,
                            const float *x) {
    if (!act || !x || act_bytes(type, cols, max_tokens) == 0 || tokens == 0 || tokens > max_tokens) return hipErrorInvalidValue;
    const ActView v = act_view(act, type, cols, max_tokens, tokens);
    MmBatch b{};
    b.job[0].m.type = type;
    b.job[0].m.cols = cols;
    b.job[0].x = x;
    b.job[0].tokens = tokens;
    b.job[0].tok_off = 0;
    for (uint32_t j = 1; j < MM_MAX_JOBS; j++) b.job[j] = b.job[0];
    b.n_jobs = 1;
    b.xb = v.xb;
    b.sx = v.sx;
    b.mpad = v.mpad;
    return mm_by_type(type, [&](auto t) {
        constexpr uint32_t T = decltype(t)::value;
        hipLaunchKernelGGL(mm_xsplit_kernel<T>, dim3((b.mpad + XS_TOK - 1) / XS_TOK, (v.n_groups + XS_GRP - 1) / XS_GRP), dim3(256),
                           0, stream, b, v.n_groups);
        return hipGetLastError();
    });
}

// The plan of n products (one dtype, one column count) of the same split activations, `tokens` tokens each.
// forced_shares: every job writes shares (one when its columns are not shared) into the workspace, for an
// epilogue launch to sum; otherwise jobs without shared columns write ys directly.
static bool act_plan(const MatView *tiled, uint32_t n, uint32_t tokens, float *const *ys, bool forced_shares, MmPlan &p) {
    if (n == 0 || n > (uint32_t)MM_MAX_JOBS || tokens < MM_MIN_TOKENS || !mm_type(tiled[0].type)) return false;
    for (uint32_t j = 1; j < n; j++)
        if (tiled[j].type != tiled[0].type || tiled[j].cols != tiled[0].cols) return false;
    uint32_t toks[MM_MAX_JOBS];
    const float *xs[MM_MAX_JOBS];
    static const float same_x = 0.f;  // any one address: the jobs then share their split slots
    for (uint32_t j = 0; j < n; j++) {
        toks[j] = tokens;
        xs[j] = &same_x;
    }
    mm_plan(tiled, toks, xs, ys, n, p);
    if (forced_shares) {
        size_t part = 0;
        for (uint32_t j = 0; j < n; j++) {
            const uint32_t ks = p.b.job[j].ksplit > 1 ? p.b.job[j].ksplit : 1;
            part += up256((size_t)ks * tokens * tiled[j].rows * sizeof(float));
        }
        p.part_bytes = part;
    }
    return true;
}

size_t gemm_act_workspace_bytes(const MatView *mats, uint32_t n, uint32_t tokens, bool with_epilogue, bool plain_x) {
    MmPlan p;
    if (!act_plan(mats, n, tokens, nullptr, with_epilogue, p)) return 0;
    // plain activations of more than 32 tokens are cut into the workspace first
    return p.part_bytes + (plain_x && p.tt == 2 ? p.xb_bytes + p.sx_bytes : 0);
}

hipError_t launch_gemm_act(hipStream_t stream, const MatView *tiled, uint32_t n, uint32_t tokens, void *act, uint32_t act_max_tokens,
                           const float *x_plain, const ActNorm *norm, float *const *ys, const ActEpilogue &ep, void *ws,
                           size_t ws_bytes) {
    // everything is checked before the first launch: a refusal leaves the stream as it was
    if (x_plain ? act != nullptr : (!act || tokens > act_max_tokens)) return hipErrorInvalidValue;
    if (norm && (!x_plain || tokens > ACT_DEFER_MAX_TOKENS || !norm->w || !norm->partial)) return hipErrorInvalidValue;
    const bool fused = ep.kind != ACT_EPILOGUE_NONE;
    if (fused && (ep.kind == ACT_EPILOGUE_SWIGLU ? n != 2 : n != 1)) return hipErrorInvalidValue;
    if (!fused && !ys) return hipErrorInvalidValue;
    MmPlan p;
    if (!act_plan(tiled, n, tokens, fused ? nullptr : ys, fused, p)) return hipErrorInvalidValue;
    const bool cut_first = x_plain && p.tt == 2;  // plain activations of more than 32 tokens: mm_xsplit into the workspace
    const size_t split_bytes = cut_first ? p.xb_bytes + p.sx_bytes : 0;
    if (p.part_bytes + split_bytes > ws_bytes) return hipErrorInvalidValue;
    MmBatch &b = p.b;
    ActView in{};
    if (!x_plain) {
        in = act_view(act, tiled[0].type, tiled[0].cols, act_max_tokens, tokens);
        if (in.mpad != b.mpad) return hipErrorInvalidValue;  // the plan's slots and the buffer's must be the same thing
    } else {
        for (uint32_t j = 0; j < b.n_jobs; j++) b.job[j].x = x_plain;
        for (uint32_t j = b.n_jobs; j < (uint32_t)MM_MAX_JOBS; j++) b.job[j].x = x_plain;
        if (cut_first) {
            in.xb = static_cast<uint4 *>(ws);
            in.sx = reinterpret_cast<float *>(static_cast<uint8_t *>(ws) + p.xb_bytes);
        }
    }
    const uint32_t rows = tiled[0].rows;
    ActView next{};
    if (ep.next_act) {
        if (!fused || act_bytes(ep.next_type, ep.next_cols, ep.next_max_tokens) == 0 || tokens > ep.next_max_tokens ||
            ep.next_cols != rows)
            return hipErrorInvalidValue;
        next = act_view(ep.next_act, ep.next_type, ep.next_cols, ep.next_max_tokens, tokens);
    }
    if (ep.kind == ACT_EPILOGUE_ADD_RMSNORM) {
        if (!ep.residual || !ep.norm_w) return hipErrorInvalidValue;
        // the row passes through LDS; rows beyond the default dynamic limit would need an attribute set outside captures
        if ((size_t)rows * sizeof(float) > ACT_NORM_MAX_ROW_BYTES) return hipErrorInvalidValue;
    }
    if (ep.kind == ACT_EPILOGUE_ADD_DEFER && (!ep.residual || !ep.partial || tokens > ACT_DEFER_MAX_TOKENS || ep.next_act || ep.xn_out))
        return hipErrorInvalidValue;
    if (ep.kind == ACT_EPILOGUE_SWIGLU && (!ep.next_act || tiled[1].rows != rows)) return hipErrorInvalidValue;
    if (norm && p.tt == 2) return hipErrorInvalidValue;  // cannot happen up to ACT_DEFER_MAX_TOKENS tokens

    b.xb = in.xb;
    b.sx = in.sx;
    if (norm) {  // what the cutting kernels read in place of split activations (gemm_mfma16_kernel's NORM)
        b.xb = reinterpret_cast<uint4 *>(const_cast<float *>(norm->w));  // read only
        b.sx = const_cast<float *>(norm->partial);
        std::memcpy(&b.pad0, &norm->eps, sizeof(float));
    }
    uint8_t *part = static_cast<uint8_t *>(ws) + split_bytes;
    for (uint32_t j = 0; j < b.n_jobs; j++) {
        MmJob &job = b.job[j];
        if (job.ksplit > 1 || fused) {
            job.part = reinterpret_cast<float *>(part);
            if (job.ksplit < 2) job.y = job.part;  // its one share
            part += up256((size_t)(job.ksplit > 1 ? job.ksplit : 1) * tokens * job.m.rows * sizeof(float));
        }
    }
    hipError_t e = mm_by_type(tiled[0].type, [&](auto t) {
        constexpr uint32_t T = decltype(t)::value;
        if constexpr (T != T_Q6_K) {
            if (p.tile16 && norm) return launch_mm16_main<T, true, false, true>(stream, b);
            if (p.tile16) return x_plain ? launch_mm16_main<T, true>(stream, b) : launch_mm16_main<T>(stream, b);
        }
        if constexpr (T == T_Q4_K) {
            if (p.tile16x2 && norm) return launch_mm16_main<T, true, false, true, 2>(stream, b);
            if (p.tile16x2)
                return x_plain ? launch_mm16_main<T, true, false, false, 2>(stream, b) : launch_mm16_main<T, false, false, false, 2>(stream, b);
        }
        if (norm) {
            if constexpr (T == T_Q6_K) {  // the other dtypes take 16-token tiles up to 16 tokens
                if (p.max_tok <= 8) return launch_mm_main<T, 1, 1, true, false, true>(stream, b);
                if (p.max_tok <= 16) return launch_mm_main<T, 1, 2, true, false, true>(stream, b);
            }
            if (p.max_tok <= 24) return launch_mm_main<T, 1, 3, true, false, true>(stream, b);
            return launch_mm_main<T, 1, 4, true, false, true>(stream, b);
        }
        if (cut_first)
            hipLaunchKernelGGL(mm_xsplit_kernel<T>, dim3((b.mpad + XS_TOK - 1) / XS_TOK, (p.n_groups + XS_GRP - 1) / XS_GRP),
                               dim3(256), 0, stream, b, p.n_groups);
        if (p.tt == 2) return launch_mm_main<T, 2, 4>(stream, b);
        if (x_plain) {  // 32-token tiles cut plain activations themselves
            if (p.max_tok <= 8) return launch_mm_main<T, 1, 1, true>(stream, b);
            if (p.max_tok <= 16) return launch_mm_main<T, 1, 2, true>(stream, b);
            if (p.max_tok <= 24) return launch_mm_main<T, 1, 3, true>(stream, b);
            return launch_mm_main<T, 1, 4, true>(stream, b);
        }
        if (p.max_tok <= 8) return launch_mm_main<T, 1, 1>(stream, b);
        if (p.max_tok <= 16) return launch_mm_main<T, 1, 2>(stream, b);
        if (p.max_tok <= 24) return launch_mm_main<T, 1, 3>(stream, b);
        return launch_mm_main<T, 1, 4>(stream, b);
    });
    if (e != hipSuccess) return e;
    if (!fused) {
        if (b.any_split) hipLaunchKernelGGL(mm_reduce_kernel, dim3(mm_reduce_blocks(b), b.n_jobs), dim3(256), 0, stream, b);
        return hipGetLastError();
    }
    const size_t total = (size_t)tokens * rows;
    auto shares = [&](uint32_t j) { return b.job[j].ksplit > 1 ? b.job[j].part : b.job[j].y; };
    auto count = [&](uint32_t j) { return b.job[j].ksplit > 1 ? b.job[j].ksplit : 1u; };
    const uint32_t nt = ep.next_act ? ep.next_type : (uint32_t)T_Q8_0;  // without next activations the column order is never used
    if (ep.kind == ACT_EPILOGUE_ADD_DEFER) {
        hipLaunchKernelGGL(mm_epi_add_partial_kernel, dim3(tokens, 4), dim3(256), 0, stream, shares(0), count(0), total, rows,
                           ep.residual, ep.partial);
        return hipGetLastError();
    }
    if (ep.kind == ACT_EPILOGUE_ADD_RMSNORM)
        return mm_by_type(nt, [&](auto t) {
            constexpr uint32_t TN = decltype(t)::value;
            hipLaunchKernelGGL(mm_epi_add_norm_kernel<TN>, dim3(tokens), dim3(1024), (size_t)rows * sizeof(float), stream, shares(0),
                               count(0), total, rows, ep.residual, ep.norm_w, ep.eps, ep.xn_out, next);
            return hipGetLastError();
        });
    return mm_by_type(nt, [&](auto t) {  // SiLU(gate) * up
        constexpr uint32_t TN = decltype(t)::value;
        constexpr int GRP = 8;  // 128 columns per workgroup: 16 measured 2-3 % slower on the batch steps, 4 (not Q6_K's order) the same
        hipLaunchKernelGGL((mm_epi_swiglu_kernel<TN, GRP>), dim3((next.mpad + XS_TOK - 1) / XS_TOK, (next.n_groups + GRP - 1) / GRP),
                           dim3(256), 0, stream, shares(0), count(0), shares(1), count(1), total, rows, tokens, next);
        return hipGetLastError();
    });
}

// Plain 16-byte-per-lane copy, used only to calibrate HBM traffic counters.
__global__ __launch_bounds__(256) void copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

hipError_t launch_copy(hipStream_t stream, void *dst, const void *src, size_t nbytes) {
    hipLaunchKernelGGL(copy_kernel, dim3(g_cu_count * 8), dim3(256), 0, stream, static_cast<uint4 *>(dst),
                       static_cast<const uint4 *>(src), nbytes / 16);
    return hipGetLastError();
}

// Plain streaming read: every thread requests eight consecutive-by-256 16-byte pieces at once and the
// grid covers the whole range in one go, like the single-token kernels' weight loads; nothing is written
// (the store is behind a condition that never holds).  What this takes is what the memory system gives
// a reader that does no arithmetic at all.
__global__ __launch_bounds__(256) void read_kernel(const uint4 *__restrict__ p, size_t n16, uint32_t *sink) {
    uint4 v[8];
    const size_t base = (size_t)blockIdx.x * 8 * 256 + threadIdx.x;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const size_t i = base + (size_t)k * 256;
        v[k] = stream_load16(reinterpret_cast<const uint8_t *>(p + (i < n16 ? i : 0)));  // read once: the products' own kind of load
    }
    uint32_t a = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) a ^= v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
    if (a == 0x9e3779b9u && n16 == 1) *sink = a;
}

hipError_t launch_read(hipStream_t stream, const void *src, size_t nbytes, void *sink) {
    const size_t n16 = nbytes / 16;
    if (n16 == 0) return hipSuccess;
    hipLaunchKernelGGL(read_kernel, dim3((unsigned)((n16 + 2047) / 2048)), dim3(256), 0, stream,
                       static_cast<const uint4 *>(src), n16, static_cast<uint32_t *>(sink));
    return hipGetLastError();
}

hipError_t launch_copy_small(hipStream_t stream, void *dst, const void *src, size_t nbytes) {
    const size_t n16 = nbytes / 16, want = (n16 + 255) / 256, most = (size_t)g_cu_count * 8;
    if (n16 == 0) return hipSuccess;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)(want < most ? want : most)), dim3(256), 0, stream,
                       static_cast<uint4 *>(dst), static_cast<const uint4 *>(src), n16);
    return hipGetLastError();
}

// ---- device memory that no call allocates
//
// Workspace of the multi-token kernels (split activations, their group sums, partial results of
// column shares) for callers that may not allocate: a file-scope device array, one copy per GPU that
// loads this code object, held until the process ends.  In host code the array's name only stands for
// the symbol; its device address comes from hipGetSymbolAddress, once per device, and only that
// address is ever handed to kernels.
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int SCRATCH_MAX_DEVICES = 64;
static void *g_scratch_ptr[SCRATCH_MAX_DEVICES];  // per device ordinal, null until static_scratch_init

hipError_t static_scratch_init(int device) {
    if (device < 0 || device >= SCRATCH_MAX_DEVICES) return hipErrorInvalidDevice;
    if (g_scratch_ptr[device]) return hipSuccess;
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));  // of the current device
    if (e != hipSuccess) return e;
    if (!ptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[device] = ptr;
    return hipSuccess;
}

void *static_scratch(int device) {
    return device >= 0 && device < SCRATCH_MAX_DEVICES ? g_scratch_ptr[device] : nullptr;
}

hipError_t launch_gemv_multi(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n, const float *x,
                             bool accumulate) {
    if (n == 0) return hipSuccess;
    if (n > GEMV_MAX_JOBS) return hipErrorInvalidValue;
    for (uint32_t j = 0; j < n; j++)
        if (mats[j].type != mats[0].type || mats[j].cols != mats[0].cols || mats[j].rows == 0) return hipErrorInvalidValue;
    switch (mats[0].type) {
    case T_F32: return launch_multi_t<T_F32>(stream, mats, ys, n, x, accumulate);
    case T_F16: return launch_multi_t<T_F16>(stream, mats, ys, n, x, accumulate);
    case T_Q4_0: return launch_multi_t<T_Q4_0>(stream, mats, ys, n, x, accumulate);
    case T_Q5_0: return launch_multi_t<T_Q5_0>(stream, mats, ys, n, x, accumulate);
    case T_Q5_1: return launch_multi_t<T_Q5_1>(stream, mats, ys, n, x, accumulate);
    case T_Q8_0: return launch_multi_t<T_Q8_0>(stream, mats, ys, n, x, accumulate);
    case T_Q4_K: return launch_multi_t<T_Q4_K>(stream, mats, ys, n, x, accumulate);
    case T_Q6_K: return launch_multi_t<T_Q6_K>(stream, mats, ys, n, x, accumulate);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gemv_multi_prologue(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n, const float *x,
                                      bool accumulate, int prologue, const float *x2, float eps) {
    if (n == 0 || n > GEMV_MAX_JOBS || !x2) return hipErrorInvalidValue;
    if (prologue != PRO_RMSNORM && prologue != PRO_SWIGLU) return hipErrorInvalidValue;
    for (uint32_t j = 0; j < n; j++)
        if (mats[j].type != T_Q4_K || mats[j].cols != mats[0].cols || mats[j].rows == 0) return hipErrorInvalidValue;
    GemvPrologue pro;
    pro.kind = prologue;
    pro.x2 = x2;
    pro.eps = eps;
    return launch_gemv_q4k(stream, mats, ys, n, x, accumulate, pro);
}

hipError_t launch_gemv_swiglu_pair(hipStream_t stream, const MatView &gate, const MatView &up, const float *x, float *h,
                                   int prologue, const float *x2, float eps) {
    if (gate.type != T_Q4_K || up.type != T_Q4_K || gate.cols != up.cols || gate.rows != up.rows || gate.rows == 0)
        return hipErrorInvalidValue;
    if (prologue != PRO_NONE && (prologue != PRO_RMSNORM || !x2)) return hipErrorInvalidValue;
    const MatView mats[2] = {gate, up};
    float *const ys[2] = {h, h};
    GemvPrologue pro;
    pro.kind = prologue;
    pro.x2 = x2;
    pro.eps = eps;
    pro.pair = true;
    return launch_gemv_q4k(stream, mats, ys, 2, x, false, pro);
}

hipError_t launch_gemm(hipStream_t stream, const MatView &m, const MatView &tiled, uint32_t tokens, const float *x,
                       float *y, void *ws, size_t ws_bytes) {
    return launch_gemm_groups(stream, &m, &tiled, &tokens, &x, &y, 1, ws, ws_bytes);
}

}  // namespace nh
