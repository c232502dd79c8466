// HIP kernels for gfx950 (MI355X): re-layout at upload, decode GEMV, tiled GEMM.
//
// All products are y[t, r] = sum_c W[r, c] * x[t, c] with f32 activations and
// f32 accumulation; W stays packed in HBM (see matview.h) and is decoded in
// registers.  Block scales are factored out of the inner sums
// (sum_j (d*q_j) x_j = d * sum_j q_j x_j, code biases via the per-lane sum of x),
// which changes only the order of f32 roundings, never the value being
// approximated: the exact product of the dequantized weights
// (langtax/src/quant.rs:7511-7541, 7734-7765, 7884-7950, 8046-8130, 8783-8853).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>
#include <type_traits>

#include "kernels.h"

namespace nh {

// ------------------------------------------------------------------ small device helpers

__device__ __forceinline__ float h2f(uint16_t bits) {
    // Hardware binary16 -> f32 is exact for every finite input, subnormals
    // included (same argument as langtax/src/simd/x86.rs:244-248).
    return __half2float(__ushort_as_half(bits));
}
__device__ __forceinline__ float ub0(uint32_t v) { return (float)(v & 0xffu); }
__device__ __forceinline__ float ub1(uint32_t v) { return (float)((v >> 8) & 0xffu); }
__device__ __forceinline__ float ub2(uint32_t v) { return (float)((v >> 16) & 0xffu); }
__device__ __forceinline__ float ub3(uint32_t v) { return (float)(v >> 24); }
__device__ __forceinline__ float sb(uint32_t v, int k) { return (float)(int)(int8_t)(v >> (8 * k)); }

// sum of 4 code bytes (0..255) times 4 activations
__device__ __forceinline__ float dot4_ub(uint32_t q, const float *x, float acc) {
    acc = fmaf(ub0(q), x[0], acc);
    acc = fmaf(ub1(q), x[1], acc);
    acc = fmaf(ub2(q), x[2], acc);
    acc = fmaf(ub3(q), x[3], acc);
    return acc;
}

// Same with a code bias taken off every code before the multiply.  (Factoring the bias out
// through the sum of x, sum q x - bias sum x, is cheaper but lets one large activation
// under a zero weight swamp the small terms of the row: the two big numbers only
// cancel at the end, after the accumulator has lost the small ones.)
__device__ __forceinline__ float dot4_ub_biased(uint32_t q, float bias, const float *x, float acc) {
    acc = fmaf(ub0(q) - bias, x[0], acc);
    acc = fmaf(ub1(q) - bias, x[1], acc);
    acc = fmaf(ub2(q) - bias, x[2], acc);
    acc = fmaf(ub3(q) - bias, x[3], acc);
    return acc;
}
// four signed bytes times four activations
__device__ __forceinline__ float dot4_sb(uint32_t q, const float *x, float acc) {
    acc = fmaf(sb(q, 0), x[0], acc);
    acc = fmaf(sb(q, 1), x[1], acc);
    acc = fmaf(sb(q, 2), x[2], acc);
    acc = fmaf(sb(q, 3), x[3], acc);
    return acc;
}
// Low nibble of byte K of w, read as a signed 4-bit integer, divided by 16 (v_cvt_off_f32_i4 with a
// byte select, so that no shift is spent on picking the byte).  With w = codes ^ 0x88888888 that
// is (n - 8) / 16 for the nibble n.
template <int K> __device__ __forceinline__ float i4_of_byte(uint32_t w) {
    float r;
    if constexpr (K == 0) asm("v_cvt_off_f32_i4_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(r) : "v"(w));
    if constexpr (K == 1) asm("v_cvt_off_f32_i4_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(r) : "v"(w));
    if constexpr (K == 2) asm("v_cvt_off_f32_i4_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(r) : "v"(w));
    if constexpr (K == 3) asm("v_cvt_off_f32_i4_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(r) : "v"(w));
    return r;
}
// sum over the low nibbles of the four bytes of w (signed, / 16) times four activations
__device__ __forceinline__ float dot4_i4(uint32_t w, const float *x, float acc) {
    acc = fmaf(i4_of_byte<0>(w), x[0], acc);
    acc = fmaf(i4_of_byte<1>(w), x[1], acc);
    acc = fmaf(i4_of_byte<2>(w), x[2], acc);
    acc = fmaf(i4_of_byte<3>(w), x[3], acc);
    return acc;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Q4_K: 6-bit (scale, min) pair j of the 12 packed bytes held in header dwords h1..h3
// (langtax/src/quant.rs:8901-8912).
__device__ __forceinline__ void q4k_scale_min(uint32_t h1, uint32_t h2, uint32_t h3, int j, float &sc, float &mn) {
    int sh = 8 * (j & 3);
    uint32_t a = (h1 >> sh) & 0xffu, b = (h2 >> sh) & 0xffu, c = (h3 >> sh) & 0xffu;
    uint32_t s, m;
    if (j < 4) {
        s = a & 63u;
        m = b & 63u;
    } else {
        s = (c & 15u) | ((a >> 6) << 4);
        m = (c >> 4) | ((b >> 6) << 4);
    }
    sc = (float)s;
    mn = (float)m;
}

// ------------------------------------------------------------------ re-layout at upload

struct MutView {
    uint8_t *p0, *p1, *p2, *p3;
    uint32_t s0, s1, s2, s3;
    uint32_t type, rows, cols, nb;
};

// One thread per GGUF block: copy its fields into the planes.  Byte-wise on
// purpose (GGUF blocks are only 2-byte aligned); this runs once per matrix.
__global__ void repack_blocks(MutView v, const uint8_t *__restrict__ src, size_t src_row_bytes) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t total = (size_t)v.rows * v.nb;
    if (idx >= total) return;
    size_t r = idx / v.nb, b = idx % v.nb;
    // code pieces of the 32-column dtypes: piece-major when the row is whole units (matview.h)
    const bool major = piece_major(v.type, v.cols);
    const size_t units = v.cols / unit_cols(v.type);
    switch (v.type) {
    case T_Q8_0: {
        const uint8_t *s = src + r * src_row_bytes + b * 34;
        uint8_t *d = v.p1 + r * v.s1 + b * 2;
        d[0] = s[0];
        d[1] = s[1];
        for (int h = 0; h < 2; h++) {
            uint8_t *q = v.p0 + r * v.s0 + piece_offset(major, units, 2 * b + h);
            for (int i = 0; i < 16; i++) q[i] = s[2 + 16 * h + i];
        }
        break;
    }
    case T_Q4_0: {
        const uint8_t *s = src + r * src_row_bytes + b * 18;
        uint8_t *d = v.p1 + r * v.s1 + b * 2;
        d[0] = s[0];
        d[1] = s[1];
        uint8_t *q = v.p0 + r * v.s0 + piece_offset(major, units, b);
        for (int i = 0; i < 16; i++) q[i] = s[2 + i];
        break;
    }
    case T_Q5_0: {
        const uint8_t *s = src + r * src_row_bytes + b * 22;
        uint8_t *d = v.p2 + r * v.s2 + b * 2;
        d[0] = s[0];
        d[1] = s[1];
        uint8_t *h = v.p1 + r * v.s1 + b * 4;
        for (int i = 0; i < 4; i++) h[i] = s[2 + i];
        uint8_t *q = v.p0 + r * v.s0 + piece_offset(major, units, b);
        for (int i = 0; i < 16; i++) q[i] = s[6 + i];
        break;
    }
    case T_Q5_1: {
        const uint8_t *s = src + r * src_row_bytes + b * 24;
        uint8_t *d = v.p2 + r * v.s2 + b * 4;
        for (int i = 0; i < 4; i++) d[i] = s[i];
        uint8_t *h = v.p1 + r * v.s1 + b * 4;
        for (int i = 0; i < 4; i++) h[i] = s[4 + i];
        uint8_t *q = v.p0 + r * v.s0 + piece_offset(major, units, b);
        for (int i = 0; i < 16; i++) q[i] = s[8 + i];
        break;
    }
    case T_Q4_K: {
        const uint8_t *s = src + r * src_row_bytes + b * 144;
        uint8_t *h = v.p1 + r * v.s1 + b * 16;
        for (int i = 0; i < 16; i++) h[i] = s[i];
        // 16-byte piece cc of block b goes to slot cc * nb + b of the row (matview.h)
        for (int cc = 0; cc < 8; cc++) {
            uint8_t *q = v.p0 + r * v.s0 + ((size_t)cc * v.nb + b) * 16;
            for (int i = 0; i < 16; i++) q[i] = s[16 + cc * 16 + i];
        }
        break;
    }
    case T_Q6_K: {
        const uint8_t *s = src + r * src_row_bytes + b * 210;
        for (int cc = 0; cc < 8; cc++) {  // ql: 16-byte piece cc of block b at slot cc * nb + b
            uint8_t *q = v.p0 + r * v.s0 + ((size_t)cc * v.nb + b) * 16;
            for (int i = 0; i < 16; i++) q[i] = s[cc * 16 + i];
        }
        for (int hc = 0; hc < 4; hc++) {  // qh: 16-byte piece hc of block b at slot hc * nb + b
            uint8_t *q = v.p1 + r * v.s1 + ((size_t)hc * v.nb + b) * 16;
            for (int i = 0; i < 16; i++) q[i] = s[128 + hc * 16 + i];
        }
        uint8_t *sc = v.p2 + r * v.s2 + b * 16;
        for (int i = 0; i < 16; i++) sc[i] = s[192 + i];
        uint8_t *d = v.p3 + r * v.s3 + b * 2;
        d[0] = s[208];
        d[1] = s[209];
        break;
    }
    default: break;
    }
}

// F32 / F16 rows: copy `elem` bytes per element into a row whose stride is padded.
__global__ void repack_plain(uint8_t *dst, size_t dst_stride, const uint8_t *__restrict__ src, size_t rows,
                             size_t row_bytes) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * dst_stride) return;
    size_t r = idx / dst_stride, c = idx % dst_stride;
    dst[idx] = c < row_bytes ? src[r * row_bytes + c] : (uint8_t)0;
}

// Tiled copy (matview.h): one thread per GGUF block.  In the MutView of a tiled
// copy s0..s3 hold the units per row of each plane.
__global__ void repack_blocks_tiled(MutView v, const uint8_t *__restrict__ src, size_t src_row_bytes) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t total = (size_t)v.rows * v.nb;
    if (idx >= total) return;
    const size_t r = idx / v.nb, b = idx % v.nb, tile = r / TILE_ROWS, rr = r % TILE_ROWS;
    auto unit = [&](uint8_t *p, uint32_t per_row, size_t i, size_t bytes) {
        return p + ((tile * per_row + i) * TILE_ROWS + rr) * bytes;
    };
    auto copy = [](uint8_t *d, const uint8_t *s, int n) {
        for (int i = 0; i < n; i++) d[i] = s[i];
    };
    switch (v.type) {
    case T_Q8_0: {
        const uint8_t *s = src + r * src_row_bytes + b * 34;
        copy(unit(v.p1, v.s1, b, 2), s, 2);
        copy(unit(v.p0, v.s0, 2 * b, 16), s + 2, 16);
        copy(unit(v.p0, v.s0, 2 * b + 1, 16), s + 18, 16);
        break;
    }
    case T_Q4_0: {
        const uint8_t *s = src + r * src_row_bytes + b * 18;
        copy(unit(v.p1, v.s1, b, 2), s, 2);
        copy(unit(v.p0, v.s0, b, 16), s + 2, 16);
        break;
    }
    case T_Q5_0: {
        const uint8_t *s = src + r * src_row_bytes + b * 22;
        copy(unit(v.p2, v.s2, b, 2), s, 2);
        copy(unit(v.p1, v.s1, b, 4), s + 2, 4);
        copy(unit(v.p0, v.s0, b, 16), s + 6, 16);
        break;
    }
    case T_Q5_1: {
        const uint8_t *s = src + r * src_row_bytes + b * 24;
        copy(unit(v.p2, v.s2, b, 4), s, 4);
        copy(unit(v.p1, v.s1, b, 4), s + 4, 4);
        copy(unit(v.p0, v.s0, b, 16), s + 8, 16);
        break;
    }
    case T_Q4_K: {
        const uint8_t *s = src + r * src_row_bytes + b * 144;
        copy(unit(v.p1, v.s1, b, 16), s, 16);
        for (int cc = 0; cc < 8; cc++) copy(unit(v.p0, v.s0, 8 * b + cc, 16), s + 16 + 16 * cc, 16);
        break;
    }
    case T_Q6_K: {
        const uint8_t *s = src + r * src_row_bytes + b * 210;
        for (int cc = 0; cc < 8; cc++) copy(unit(v.p0, v.s0, 8 * b + cc, 16), s + 16 * cc, 16);
        for (int hc = 0; hc < 4; hc++) copy(unit(v.p1, v.s1, 4 * b + hc, 16), s + 128 + 16 * hc, 16);
        for (int n = 0; n < 2; n++) copy(unit(v.p2, v.s2, 2 * b + n, 8), s + 192 + 8 * n, 8);
        copy(unit(v.p3, v.s3, b, 2), s + 208, 2);
        break;
    }
    default: break;
    }
}

static MutView mut_view(const MatView &m) {
    MutView v;
    v.p0 = const_cast<uint8_t *>(m.p0);
    v.p1 = const_cast<uint8_t *>(m.p1);
    v.p2 = const_cast<uint8_t *>(m.p2);
    v.p3 = const_cast<uint8_t *>(m.p3);
    v.s0 = m.s0; v.s1 = m.s1; v.s2 = m.s2; v.s3 = m.s3;
    v.type = m.type; v.rows = m.rows; v.cols = m.cols; v.nb = m.nb;
    return v;
}

hipError_t launch_repack_tiled(hipStream_t stream, const MatView &tiled, const void *src_device) {
    if (tiled.rows == 0 || tiled.p0 == nullptr) return hipSuccess;
    size_t total = (size_t)tiled.rows * tiled.nb;
    hipLaunchKernelGGL(repack_blocks_tiled, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, mut_view(tiled),
                       static_cast<const uint8_t *>(src_device), gguf_row_bytes(tiled.type, tiled.cols));
    return hipGetLastError();
}

hipError_t launch_repack(hipStream_t stream, const MatView &m, const void *src_device) {
    if (m.rows == 0) return hipSuccess;
    const uint8_t *src = static_cast<const uint8_t *>(src_device);
    if (m.type == T_F32 || m.type == T_F16) {
        size_t row_bytes = (size_t)m.cols * (m.type == T_F32 ? 4 : 2);
        size_t total = (size_t)m.rows * m.s0;
        size_t blocks = (total + 255) / 256;
        hipLaunchKernelGGL(repack_plain, dim3((unsigned)blocks), dim3(256), 0, stream, const_cast<uint8_t *>(m.p0),
                           (size_t)m.s0, src, (size_t)m.rows, row_bytes);
    } else {
        size_t total = (size_t)m.rows * m.nb;
        size_t blocks = (total + 255) / 256;
        hipLaunchKernelGGL(repack_blocks, dim3((unsigned)blocks), dim3(256), 0, stream, mut_view(m), src,
                           gguf_row_bytes(m.type, m.cols));
    }
    return hipGetLastError();
}

// ------------------------------------------------------------------ per-dtype lane steps (GEMV)
//
// A "chunk" is the slice of one row that one lane consumes per step: 16 bytes of
// the code plane (or of the row itself for F16/F32), i.e. E consecutive-ish
// columns.  Steps<T>::E is that column count; xs points at the E activations of
// the chunk in LDS, laid out in the order the lane consumes them.

template <uint32_t T> struct Geo;
template <> struct Geo<T_F32> { static constexpr int E = 4; };
template <> struct Geo<T_F16> { static constexpr int E = 8; };
template <> struct Geo<T_Q8_0> { static constexpr int E = 16; };
template <> struct Geo<T_Q4_0> { static constexpr int E = 32; };
template <> struct Geo<T_Q5_0> { static constexpr int E = 32; };
template <> struct Geo<T_Q5_1> { static constexpr int E = 32; };
template <> struct Geo<T_Q4_K> { static constexpr int E = 32; };
template <> struct Geo<T_Q6_K> { static constexpr int E = 32; };

// Activations of one chunk in registers plus the partial sums the dtype's bias
// terms need.  x[i] pairs with the i-th code the lane decodes.
template <int E> struct XChunk {
    float x[E];
    float s_lo, s_hi;  // sum of x[0..E/2), sum of x[E/2..E)
};

// Where the E activations of chunk c live in the row (column index of x[i]).
template <uint32_t T> __device__ __forceinline__ uint32_t chunk_col(uint32_t c, int i) {
    constexpr int E = Geo<T>::E;
    if constexpr (T == T_Q4_K) {
        // chunk = 16 bytes of a 64-column group: low nibbles are columns
        // [16h, 16h+16) of the group, high nibbles the same range 32 further on.
        uint32_t blk = c >> 3, cc = c & 7, g = cc >> 1, h = cc & 1;
        return blk * 256 + g * 64 + h * 16 + (i < 16 ? i : 16 + i);
    } else if constexpr (T == T_Q6_K) {
        // chunk = 16 bytes of ql: low nibbles are 16 columns of quarter h (of
        // half n), high nibbles the same 16 columns of quarter h+2.
        uint32_t blk = c >> 3, cc = c & 7, n = cc >> 2, h = (cc >> 1) & 1, k = cc & 1;
        return blk * 256 + n * 128 + h * 32 + k * 16 + (i < 16 ? i : 48 + i);
    } else {
        return c * E + i;  // Q4_0/Q5_x: x[0..16) low nibbles, x[16..32) high nibbles = natural order
    }
}

template <uint32_t T> __device__ __forceinline__ void load_x(const float *xs, uint32_t c, XChunk<Geo<T>::E> &o) {
    constexpr int E = Geo<T>::E;
    if constexpr (T == T_Q4_K || T == T_Q6_K) {
        const float4 *lo = reinterpret_cast<const float4 *>(xs + chunk_col<T>(c, 0));
        const float4 *hi = reinterpret_cast<const float4 *>(xs + chunk_col<T>(c, 16));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float4 a = lo[i], b = hi[i];
            o.x[4 * i] = a.x; o.x[4 * i + 1] = a.y; o.x[4 * i + 2] = a.z; o.x[4 * i + 3] = a.w;
            o.x[16 + 4 * i] = b.x; o.x[16 + 4 * i + 1] = b.y; o.x[16 + 4 * i + 2] = b.z; o.x[16 + 4 * i + 3] = b.w;
        }
    } else {
        const float4 *p = reinterpret_cast<const float4 *>(xs + (size_t)c * E);
#pragma unroll
        for (int i = 0; i < E / 4; i++) {
            float4 a = p[i];
            o.x[4 * i] = a.x; o.x[4 * i + 1] = a.y; o.x[4 * i + 2] = a.z; o.x[4 * i + 3] = a.w;
        }
    }
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int i = 0; i < E / 2; i++) {
        lo += o.x[i];
        hi += o.x[E / 2 + i];
    }
    o.s_lo = lo;
    o.s_hi = hi;
}

// Raw bytes of one chunk of one row.
template <uint32_t T> struct Raw;
template <> struct Raw<T_F32> { uint4 q; };
template <> struct Raw<T_F16> { uint4 q; };
template <> struct Raw<T_Q8_0> { uint4 q; uint16_t d; };
template <> struct Raw<T_Q4_0> { uint4 q; uint16_t d; };
template <> struct Raw<T_Q5_0> { uint4 q; uint32_t qh; uint16_t d; };
template <> struct Raw<T_Q5_1> { uint4 q; uint32_t qh; uint32_t dm; };
template <> struct Raw<T_Q4_K> { uint4 q; uint4 hdr; };
template <> struct Raw<T_Q6_K> { uint4 ql; uint4 qh; uint2 sc; uint16_t d; };

template <uint32_t T> __device__ __forceinline__ void load_raw(const MatView &m, uint32_t row, uint32_t c, Raw<T> &r) {
    const size_t ro = (size_t)row;
    if constexpr (T == T_F32 || T == T_F16) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + (size_t)c * 16);
    } else if constexpr (T == T_Q8_0) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + piece_offset(piece_major(T, m.cols), m.cols / unit_cols(T), c));
        r.d = *reinterpret_cast<const uint16_t *>(m.p1 + ro * m.s1 + (size_t)(c >> 1) * 2);
    } else if constexpr (T == T_Q4_0) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + piece_offset(piece_major(T, m.cols), m.cols / unit_cols(T), c));
        r.d = *reinterpret_cast<const uint16_t *>(m.p1 + ro * m.s1 + (size_t)c * 2);
    } else if constexpr (T == T_Q5_0) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + piece_offset(piece_major(T, m.cols), m.cols / unit_cols(T), c));
        r.qh = *reinterpret_cast<const uint32_t *>(m.p1 + ro * m.s1 + (size_t)c * 4);
        r.d = *reinterpret_cast<const uint16_t *>(m.p2 + ro * m.s2 + (size_t)c * 2);
    } else if constexpr (T == T_Q5_1) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + piece_offset(piece_major(T, m.cols), m.cols / unit_cols(T), c));
        r.qh = *reinterpret_cast<const uint32_t *>(m.p1 + ro * m.s1 + (size_t)c * 4);
        r.dm = *reinterpret_cast<const uint32_t *>(m.p2 + ro * m.s2 + (size_t)c * 4);
    } else if constexpr (T == T_Q4_K) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + ((size_t)(c & 7) * m.nb + (c >> 3)) * 16);
        r.hdr = *reinterpret_cast<const uint4 *>(m.p1 + ro * m.s1 + (size_t)(c >> 3) * 16);
    } else if constexpr (T == T_Q6_K) {
        uint32_t blk = c >> 3, cc = c & 7, n = cc >> 2, k = cc & 1;
        r.ql = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + ((size_t)cc * m.nb + blk) * 16);
        r.qh = *reinterpret_cast<const uint4 *>(m.p1 + ro * m.s1 + ((size_t)(2 * n + k) * m.nb + blk) * 16);
        r.sc = *reinterpret_cast<const uint2 *>(m.p2 + ro * m.s2 + (size_t)blk * 16 + n * 8);
        r.d = *reinterpret_cast<const uint16_t *>(m.p3 + ro * m.s3 + (size_t)blk * 2);
    }
}

// 5-bit codes of four consecutive elements as four bytes: nibbles in `nib`
// (one per byte), fifth bits = bits [e0, e0+4) of qh.
__device__ __forceinline__ uint32_t q5_bytes(uint32_t nib, uint32_t qh, int e0) {
    uint32_t h4 = (qh >> e0) & 0xfu;
    // spread bit k of h4 to bit 8k: 0x00204081 has bits 0, 7, 14, 21 set
    uint32_t spread = (h4 * 0x00204081u) & 0x01010101u;
    return nib | (spread << 4);
}

// Same for Q5_0 as signed bytes 8 (c - 16): nib8 holds the nibbles in bits 3..6 of every byte, the
// fifth bit goes to bit 7 and is flipped (c ^ 16 is c - 16 in 5-bit two's complement).
__device__ __forceinline__ uint32_t q5_signed_bytes(uint32_t nib8, uint32_t qh, int e0) {
    uint32_t h4 = (qh >> e0) & 0xfu;
    uint32_t spread = (h4 * 0x00204081u) & 0x01010101u;
    return (nib8 | (spread << 7)) ^ 0x80808080u;
}

// Contribution of one chunk of one row to that row's dot product.
template <uint32_t T>
__device__ __forceinline__ float chunk_dot(const Raw<T> &r, const XChunk<Geo<T>::E> &xc, uint32_t c, float acc) {
    const float *x = xc.x;
    if constexpr (T == T_F32) {
        acc = fmaf(__uint_as_float(r.q.x), x[0], acc);
        acc = fmaf(__uint_as_float(r.q.y), x[1], acc);
        acc = fmaf(__uint_as_float(r.q.z), x[2], acc);
        acc = fmaf(__uint_as_float(r.q.w), x[3], acc);
        return acc;
    } else if constexpr (T == T_F16) {
        const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            acc = fmaf(h2f((uint16_t)(w[i] & 0xffffu)), x[2 * i], acc);
            acc = fmaf(h2f((uint16_t)(w[i] >> 16)), x[2 * i + 1], acc);
        }
        return acc;
    } else if constexpr (T == T_Q8_0) {
        const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int k = 0; k < 4; k++) t = fmaf(sb(w[i], k), x[4 * i + k], t);
        }
        return fmaf(h2f(r.d), t, acc);
    } else if constexpr (T == T_Q4_0) {
        const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            t = dot4_ub_biased(w[i] & 0x0f0f0f0fu, 8.f, x + 4 * i, t);
            t = dot4_ub_biased((w[i] >> 4) & 0x0f0f0f0fu, 8.f, x + 16 + 4 * i, t);
        }
        return fmaf(h2f(r.d), t, acc);
    } else if constexpr (T == T_Q5_0 || T == T_Q5_1) {
        const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        float t = 0.f;
        constexpr float bias = T == T_Q5_0 ? 16.f : 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            t = dot4_ub_biased(q5_bytes(w[i] & 0x0f0f0f0fu, r.qh, 4 * i), bias, x + 4 * i, t);
            t = dot4_ub_biased(q5_bytes((w[i] >> 4) & 0x0f0f0f0fu, r.qh, 16 + 4 * i), bias, x + 16 + 4 * i, t);
        }
        if constexpr (T == T_Q5_0) {
            return fmaf(h2f(r.d), t, acc);
        } else {
            float d = h2f((uint16_t)(r.dm & 0xffffu)), mm = h2f((uint16_t)(r.dm >> 16));
            acc = fmaf(d, t, acc);
            return fmaf(mm, xc.s_lo + xc.s_hi, acc);
        }
    } else if constexpr (T == T_Q4_K) {
        const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        float tl = 0.f, th = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            tl = dot4_ub(w[i] & 0x0f0f0f0fu, x + 4 * i, tl);
            th = dot4_ub((w[i] >> 4) & 0x0f0f0f0fu, x + 16 + 4 * i, th);
        }
        int g = (c & 7) >> 1;
        float d = h2f((uint16_t)(r.hdr.x & 0xffffu)), dmin = h2f((uint16_t)(r.hdr.x >> 16));
        float sc0, m0, sc1, m1;
        q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * g, sc0, m0);
        q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * g + 1, sc1, m1);
        // sum (a q - b) x = a sum q x - b sum x, per 32-column sub-block
        acc = fmaf(d * sc0, tl, acc);
        acc = fmaf(-(dmin * m0), xc.s_lo, acc);
        acc = fmaf(d * sc1, th, acc);
        acc = fmaf(-(dmin * m1), xc.s_hi, acc);
        return acc;
    } else if constexpr (T == T_Q6_K) {
        const uint32_t lo[4] = {r.ql.x, r.ql.y, r.ql.z, r.ql.w};
        const uint32_t hb[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        uint32_t cc = c & 7, h = (cc >> 1) & 1, k = cc & 1;
        float tl = 0.f, th = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t two_lo = (hb[i] >> (2 * h)) & 0x03030303u;        // quarter h
            uint32_t two_hi = (hb[i] >> (2 * h + 4)) & 0x03030303u;    // quarter h + 2
            tl = dot4_ub_biased((lo[i] & 0x0f0f0f0fu) | (two_lo << 4), 32.f, x + 4 * i, tl);
            th = dot4_ub_biased(((lo[i] >> 4) & 0x0f0f0f0fu) | (two_hi << 4), 32.f, x + 16 + 4 * i, th);
        }
        int sh = 8 * (2 * h + k);
        float s_lo = (float)(int)(int8_t)(r.sc.x >> sh);  // scale 8n + 2h + k
        float s_hi = (float)(int)(int8_t)(r.sc.y >> sh);  // scale 8n + 2(h+2) + k
        float d = h2f(r.d);
        acc = fmaf(d * s_lo, tl, acc);
        acc = fmaf(d * s_hi, th, acc);
        return acc;
    }
    return acc;
}

// ------------------------------------------------------------------ GEMV (one token)
//
// Free-running wavefronts.  A workgroup (8 wavefronts) stages x and the
// per-chunk sums of x in LDS once; after that single barrier every wavefront
// streams on its own: it owns whole row groups (R consecutive rows, all of
// their columns), walks them in steps of 64 chunks, and always has the next
// step's weight bytes in flight while it does the arithmetic of the current one
// (two register buffers, used alternately).  One DPP reduction per row group,
// no barrier and no LDS traffic between wavefronts, so the sum of a row is
// formed in a fixed order that does not depend on scheduling.  One launch can
// serve several matrices that share the same x (q/k/v, gate/up): row groups of
// all jobs are numbered consecutively and dealt round-robin to the wavefronts.

constexpr int GEMV_WAVES = 8;
constexpr int GEMV_MAX_JOBS = 8;

struct GemvJob {
    MatView m;
    float *y;
    uint32_t rg_begin;  // first row group of this job in the launch-wide numbering
    uint32_t pad;
};
struct GemvBatch {
    GemvJob job[GEMV_MAX_JOBS];
    const float *x;
    uint32_t n_jobs, total_rgs, n_chunks, x_pad;
    // Column window of the lane-per-unit kernels: units [unit0, unit0 + units) of every row.
    // Rows too long for LDS are done in several launches, the later ones adding to y.
    uint32_t unit0, units, accumulate, pad;
};

template <uint32_t T> __device__ __forceinline__ void load_x_lds(const float *xs, const float *sums, uint32_t c,
                                                                  XChunk<Geo<T>::E> &o) {
    constexpr int E = Geo<T>::E;
    if constexpr (T == T_Q4_K || T == T_Q6_K) {
        const float4 *lo = reinterpret_cast<const float4 *>(xs + chunk_col<T>(c, 0));
        const float4 *hi = reinterpret_cast<const float4 *>(xs + chunk_col<T>(c, 16));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float4 a = lo[i], b = hi[i];
            o.x[4 * i] = a.x; o.x[4 * i + 1] = a.y; o.x[4 * i + 2] = a.z; o.x[4 * i + 3] = a.w;
            o.x[16 + 4 * i] = b.x; o.x[16 + 4 * i + 1] = b.y; o.x[16 + 4 * i + 2] = b.z; o.x[16 + 4 * i + 3] = b.w;
        }
    } else {
        const float4 *p = reinterpret_cast<const float4 *>(xs + (size_t)c * E);
#pragma unroll
        for (int i = 0; i < E / 4; i++) {
            float4 a = p[i];
            o.x[4 * i] = a.x; o.x[4 * i + 1] = a.y; o.x[4 * i + 2] = a.z; o.x[4 * i + 3] = a.w;
        }
    }
    if constexpr (T == T_F32 || T == T_F16) {  // no code bias, no sums kept
        o.s_lo = o.s_hi = 0.f;
    } else {
        float2 sm = *reinterpret_cast<const float2 *>(sums + 2 * c);
        o.s_lo = sm.x;
        o.s_hi = sm.y;
    }
}

// Sum over the 64 lanes, valid in lane 63.  Four DPP steps inside each row of 16
// lanes, then the two row broadcasts.
__device__ __forceinline__ float wave_sum_dpp(float v) {
#define NH_DPP_ADD(ctrl, rmask)                                                                              \
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, rmask, 0xf, false))
    NH_DPP_ADD(0xb1, 0xf);   // quad_perm [1,0,3,2]
    NH_DPP_ADD(0x4e, 0xf);   // quad_perm [2,3,0,1]
    NH_DPP_ADD(0x141, 0xf);  // row_half_mirror
    NH_DPP_ADD(0x140, 0xf);  // row_mirror
    NH_DPP_ADD(0x142, 0xa);  // row_bcast15 into rows 1 and 3
    NH_DPP_ADD(0x143, 0xc);  // row_bcast31 into rows 2 and 3
#undef NH_DPP_ADD
    return v;
}

template <uint32_t T, int R> struct GemvUnit {
    Raw<T> raw[R];
};

template <uint32_t T, int R>
__global__ __launch_bounds__(GEMV_WAVES * 64, 4) void gemv_kernel(const GemvBatch b) {
    constexpr int E = Geo<T>::E;
    extern __shared__ __align__(16) float lds[];
    float *xs = lds;               // x_pad activations, zero padded
    float *sums = lds + b.x_pad;   // per chunk: sum of its first half, sum of its second half

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n_steps = (b.n_chunks + 63u) / 64u;
    const uint32_t total_waves = gridDim.x * GEMV_WAVES;
    const uint32_t cols = b.job[0].m.cols;

    // Unit = (row group g, step s).  State of the unit being fetched:
    uint32_t g = blockIdx.x * GEMV_WAVES + wave, s = 0;

    auto fetch = [&](uint32_t gg, uint32_t ss, GemvUnit<T, R> &u) {
        uint32_t j = 0;
        while (j + 1 < b.n_jobs && gg >= b.job[j + 1].rg_begin) j++;
        const MatView &m = b.job[j].m;
        const uint32_t row0 = (gg - b.job[j].rg_begin) * R;
        uint32_t c = ss * 64u + lane;
        c = c < b.n_chunks ? c : b.n_chunks - 1;
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint32_t row = row0 + r < m.rows ? row0 + r : m.rows - 1;
            load_raw<T>(m, row, c, u.raw[r]);
        }
    };

    GemvUnit<T, R> ua, ub;
    bool have_a = g < b.total_rgs;
    if (have_a) fetch(g, s, ua);  // in flight while x is staged

    for (uint32_t i = tid; i < b.x_pad; i += GEMV_WAVES * 64) xs[i] = i < cols ? b.x[i] : 0.f;
    __syncthreads();
    for (uint32_t c = tid; c < (T == T_F32 || T == T_F16 ? 0u : b.n_chunks); c += GEMV_WAVES * 64) {
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int i = 0; i < E / 2; i++) {
            lo += xs[chunk_col<T>(c, i)];
            hi += xs[chunk_col<T>(c, E / 2 + i)];
        }
        sums[2 * c] = lo;
        sums[2 * c + 1] = hi;
    }
    __syncthreads();

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;

    auto consume = [&](uint32_t gg, uint32_t ss, const GemvUnit<T, R> &u) {
        uint32_t c = ss * 64u + lane;
        const bool active = c < b.n_chunks;
        c = active ? c : b.n_chunks - 1;
        XChunk<E> xc;
        load_x_lds<T>(xs, sums, c, xc);
#pragma unroll
        for (int r = 0; r < R; r++) {
            float t = chunk_dot<T>(u.raw[r], xc, c, 0.f);
            acc[r] += active ? t : 0.f;
        }
        if (ss + 1 == n_steps) {  // row group complete
            uint32_t j = 0;
            while (j + 1 < b.n_jobs && gg >= b.job[j + 1].rg_begin) j++;
            const uint32_t row0 = (gg - b.job[j].rg_begin) * R;
            const uint32_t rows = b.job[j].m.rows;
            float *y = b.job[j].y;
#pragma unroll
            for (int r = 0; r < R; r++) {
                float tot = wave_sum_dpp(acc[r]);
                if (lane == 63 && row0 + r < rows) y[row0 + r] = tot;
                acc[r] = 0.f;
            }
        }
    };
    auto advance = [&](uint32_t &gg, uint32_t &ss) {
        if (ss + 1 < n_steps) {
            ss++;
        } else {
            ss = 0;
            gg += total_waves;
        }
    };

    while (have_a) {
        uint32_t g2 = g, s2 = s;
        advance(g2, s2);
        const bool have_b = g2 < b.total_rgs;
        if (have_b) fetch(g2, s2, ub);
        consume(g, s, ua);
        if (!have_b) break;
        g = g2;
        s = s2;
        advance(g, s);
        have_a = g < b.total_rgs;
        if (have_a) fetch(g, s, ua);
        consume(g2, s2, ub);
    }
}

// ------------------------------------------------------------------ Q4_K GEMV: one lane per super-block
//
// VALU work per weight, not bytes in flight, is what bounds a 4-bit GEMV on this
// machine (64 non-packed f32 lanes per CU per clock against ~14 weights per CU
// per clock at full HBM rate), so the Q4_K kernel is laid out to keep that work
// minimal:
//   * a lane owns one whole 256-column super-block of one row, so the 16-byte
//     header is fetched once per 128 code bytes, d/dmin are converted once and
//     all sixteen 6-bit scale/min extractions use compile-time shifts;
//   * the code plane is stored piece-major (piece cc of block b at slot
//     cc * nb + b), so the 64 lanes of a wavefront still read consecutive
//     16-byte pieces of a row;
//   * nibbles become floats two at a time through the fp8 (E4M3) unpack: a byte
//     0x0n read as E4M3 is exactly n * 2^-9 (n < 8 subnormal, 8..15 first binade:
//     both linear), the factor is folded into d;
//   * the min term uses the per-sub-block sums of x, computed once per workgroup.
// LB lanes (a power of two) cover the nb blocks of a row and 64 / LB rows ride in
// one wavefront step.  Every wavefront streams on its own after the one barrier
// that publishes x: it keeps the next unit's 144 bytes per lane in flight while it
// does the arithmetic of the current one.

template <bool FP8> __device__ __forceinline__ float dot4_nib(uint32_t b4, const float *x, float acc) {
    if constexpr (FP8) {
        auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)b4, false);
        auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)b4, true);
        acc = fmaf(lo[0], x[0], acc);
        acc = fmaf(lo[1], x[1], acc);
        acc = fmaf(hi[0], x[2], acc);
        acc = fmaf(hi[1], x[3], acc);
        return acc;
    } else {
        return dot4_ub(b4, x, acc);
    }
}

template <int LB> __device__ __forceinline__ float group_sum_dpp(float v) {
#define NH_DPP_ADD(ctrl, rmask)                                                                              \
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, rmask, 0xf, false))
    if constexpr (LB >= 2) NH_DPP_ADD(0xb1, 0xf);    // quad_perm [1,0,3,2]
    if constexpr (LB >= 4) NH_DPP_ADD(0x4e, 0xf);    // quad_perm [2,3,0,1]
    if constexpr (LB >= 8) NH_DPP_ADD(0x141, 0xf);   // row_half_mirror
    if constexpr (LB >= 16) NH_DPP_ADD(0x140, 0xf);  // row_mirror
    if constexpr (LB >= 32) NH_DPP_ADD(0x142, 0xa);  // row_bcast15 into rows 1 and 3
    if constexpr (LB >= 64) NH_DPP_ADD(0x143, 0xc);  // row_bcast31 into rows 2 and 3
#undef NH_DPP_ADD
    return v;  // valid in the last lane of every group of LB lanes
}


// One unit of work of a lane: the header of its block and PL of its eight 16-byte code pieces.
template <int PL> struct Q4kUnit {
    uint4 hdr, q[PL];
};

// PL = 8: a lane owns a whole super-block.  PL = 4: two lanes share one (pieces 0..3 = sub-blocks
// 0..3, pieces 4..7 = sub-blocks 4..7), which doubles the wavefronts a short-row matrix gives the
// chip and halves the arithmetic left to do after a wavefront's last bytes have arrived.
// LB lanes cover a row: LB / (8 / PL) blocks, the first half of the lanes holding the first halves.
template <int LB, int NW, bool FP8, int PL>
__global__ __launch_bounds__(NW * 64, 4) void gemv_q4k_kernel(const GemvBatch b, const float nib_mul) {
    constexpr int GEMV_WAVES = NW;  // wavefronts per workgroup of this instantiation
    constexpr uint32_t RS = 64 / LB;       // rows per wavefront step = rows per row group
    constexpr uint32_t HALVES = 8 / PL;    // lanes per super-block
    constexpr uint32_t LBB = LB / HALVES;  // super-blocks per row and iteration
    static_assert(PL == 8 || PL == 4, "a lane owns a whole super-block or half of one");
    static_assert(LB >= HALVES, "too few lanes per row for half blocks");
    // LDS row of one (cc, i) slot: LB float4 plus one float4 of padding, so that the 16 slots
    // consecutive staging lanes write to fall into different banks.
    constexpr uint32_t XROW = LBB * 4 + 4;
    constexpr uint32_t XS_FLOATS = 64 * XROW;  // x region of one block iteration
    extern __shared__ __align__(16) float lds[];
    const uint32_t nb_all = b.job[0].m.nb;         // super-blocks per row: slot stride of the piece-major plane
    const uint32_t nb = b.units, cols = nb * 256;  // the window this launch covers
    const float *xw = b.x + (size_t)b.unit0 * 256;
    const uint32_t n_iter = (nb + LBB - 1) / LBB;  // always 1: the launcher cuts windows of at most LBB super-blocks
    // x, permuted so that lane blk reads piece i of code piece cc at a compile-time offset:
    //   float it * XS_FLOATS + (cc*8 + i) * XROW + (blk % LB) * 4 + e,   it = blk / LB
    float *xs = lds;
    float *ssum = lds + (size_t)n_iter * XS_FLOATS;  // [it][sub][blk % LB]: sum of x over a sub-block

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t total_waves = gridDim.x * GEMV_WAVES;
    const uint32_t sub_row = lane / LB, b0 = lane % LB;
    const uint32_t bl0 = b0 % LBB, half = b0 / LBB;  // block of the iteration, which half of it
    const uint32_t n_units = b.total_rgs * n_iter;  // unit u = (row group u / n_iter, iteration u % n_iter)

    struct Where {
        const uint8_t *p0, *p1;
        float *y;
        uint32_t s0, s1, rows, row0;
    };
    auto locate = [&](uint32_t g) {
        uint32_t j = 0;
        while (j + 1 < b.n_jobs && g >= b.job[j + 1].rg_begin) j++;
        Where w;
        w.p0 = b.job[j].m.p0;
        w.p1 = b.job[j].m.p1;
        w.y = b.job[j].y;
        w.s0 = b.job[j].m.s0;
        w.s1 = b.job[j].m.s1;
        w.rows = b.job[j].m.rows;
        w.row0 = (g - b.job[j].rg_begin) * RS;
        return w;
    };
    auto fetch = [&](uint32_t u, Q4kUnit<PL> &o) {
        const uint32_t g = u / n_iter, it = u - g * n_iter;
        const Where w = locate(g);
        uint32_t row = w.row0 + sub_row;
        row = row < w.rows ? row : w.rows - 1;
        uint32_t blk = it * LBB + bl0;
        blk = b.unit0 + (blk < nb ? blk : nb - 1);
        const uint32_t hoff = row * w.s1 + blk * 16, qoff = row * w.s0 + blk * 16;  // planes stay below 4 GB
        o.hdr = *reinterpret_cast<const uint4 *>(w.p1 + hoff);
#pragma unroll
        for (int c = 0; c < PL; c++)
            o.q[c] = *reinterpret_cast<const uint4 *>(w.p0 + (size_t)(half * PL + c) * nb_all * 16 + qoff);
    };

    uint32_t u = blockIdx.x * GEMV_WAVES + wave;
    Q4kUnit<PL> ua, ub;
    // Stage x once per workgroup; eight consecutive lanes hold one 32-column sub-block.
    // The x loads are issued before the first unit's weight loads, so they sit at the
    // head of the memory queue and the weights stream in behind them while x is
    // being written to LDS.
    auto stage = [&](uint32_t col, const float4 v) {
        const uint32_t blk = col >> 8, r = col & 255u, g = r >> 6, r2 = r & 63u, hi = r2 >> 5, r3 = r2 & 31u;
        const uint32_t cc = 2 * g + (r3 >> 4), t = hi * 16 + (r3 & 15u), it = blk / LBB, bl = blk % LBB;
        *reinterpret_cast<float4 *>(xs + (size_t)it * XS_FLOATS + (cc * 8 + (t >> 2)) * XROW + bl * 4) = v;
        float sm = (v.x + v.y) + (v.z + v.w);
#define NH_DPP_ADD(ctrl) sm += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sm), ctrl, 0xf, 0xf, false))
        NH_DPP_ADD(0xb1);
        NH_DPP_ADD(0x4e);
        NH_DPP_ADD(0x141);
#undef NH_DPP_ADD
        if ((lane & 7u) == 0) ssum[(it * 8 + (r >> 5)) * LBB + bl] = sm;
    };
    constexpr int NXV = (LBB * 64 + NW * 64 - 1) / (NW * 64);  // float4 per thread for LBB blocks of x
    if (n_iter == 1) {
        float4 xv[NXV];
#pragma unroll
        for (int k = 0; k < NXV; k++) {
            const uint32_t col = (tid + k * NW * 64) * 4;
            xv[k] = *reinterpret_cast<const float4 *>(xw + (col < cols ? col : 0));  // branch-free: stays first
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the x loads ahead of the weight loads in the queue
        fetch(u < n_units ? u : n_units - 1, ua);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < NXV; k++) {
            const uint32_t col = (tid + k * NW * 64) * 4;
            if (col < LBB * 256) stage(col, col < cols ? xv[k] : make_float4(0.f, 0.f, 0.f, 0.f));
        }
        __syncthreads();
    } else {
        for (uint32_t col = tid * 4; col < n_iter * LBB * 256; col += NW * 64 * 4)
            stage(col, col < cols ? *reinterpret_cast<const float4 *>(xw + col) : make_float4(0.f, 0.f, 0.f, 0.f));
        __syncthreads();
        if (u < n_units) fetch(u, ua);
    }

    float acc = 0.f;
    auto consume = [&](uint32_t uu, const Q4kUnit<PL> &q) {
        const uint32_t g = uu / n_iter, it = uu - g * n_iter;
        const bool active = it * LBB + bl0 < nb;
        // x rows of this lane's pieces: piece cc = half * PL + c starts at row cc * 8
        const float *xb = xs + (size_t)it * XS_FLOATS + bl0 * 4 + half * (PL * 8 * XROW);
        float t[PL];
#pragma unroll
        for (int k = 0; k < PL; k++) t[k] = 0.f;
#pragma unroll
        for (int c = 0; c < PL; c++) {
            float x[32];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float4 v = *reinterpret_cast<const float4 *>(xb + (c * 8 + i) * XROW);
                x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
            }
            const uint32_t w[4] = {q.q[c].x, q.q[c].y, q.q[c].z, q.q[c].w};
#pragma unroll
            for (int d = 0; d < 4; d++) {
                t[c & ~1] = dot4_nib<FP8>(w[d] & 0x0f0f0f0fu, x + 4 * d, t[c & ~1]);
                t[c | 1] = dot4_nib<FP8>((w[d] >> 4) & 0x0f0f0f0fu, x + 16 + 4 * d, t[c | 1]);
            }
        }
        const uint32_t h1 = q.hdr.y, h2 = q.hdr.z, h3 = q.hdr.w;
        float S = 0.f, Mn = 0.f;
        if constexpr (PL == 8) {
            const float *sp = ssum + (size_t)it * 8 * LBB + bl0;
#pragma unroll
            for (int k = 0; k < 4; k++) {  // langtax/src/quant.rs:8901-8912 with constant shifts
                const float sc_lo = (float)((h1 >> (8 * k)) & 63u), mn_lo = (float)((h2 >> (8 * k)) & 63u);
                const float sc_hi = (float)(((h3 >> (8 * k)) & 15u) | (((h1 >> (8 * k + 6)) & 3u) << 4));
                const float mn_hi = (float)(((h3 >> (8 * k + 4)) & 15u) | (((h2 >> (8 * k + 6)) & 3u) << 4));
                S = fmaf(sc_lo, t[k], S);
                S = fmaf(sc_hi, t[k + 4], S);
                Mn = fmaf(mn_lo, sp[k * LBB], Mn);
                Mn = fmaf(mn_hi, sp[(k + 4) * LBB], Mn);
            }
        } else {
            // sub-blocks 4 half .. 4 half + 3: the first half's pairs sit whole in the header, the
            // second half's are split over its three dwords
            const float *sp = ssum + ((size_t)it * 8 + 4 * half) * LBB + bl0;
            const uint32_t up = 0u - half;  // all ones in the second half
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t sc_lo = (h1 >> (8 * k)) & 63u, mn_lo = (h2 >> (8 * k)) & 63u;
                const uint32_t sc_hi = ((h3 >> (8 * k)) & 15u) | (((h1 >> (8 * k + 6)) & 3u) << 4);
                const uint32_t mn_hi = ((h3 >> (8 * k + 4)) & 15u) | (((h2 >> (8 * k + 6)) & 3u) << 4);
                S = fmaf((float)(sc_lo ^ ((sc_lo ^ sc_hi) & up)), t[k], S);
                Mn = fmaf((float)(mn_lo ^ ((mn_lo ^ mn_hi) & up)), sp[k * LBB], Mn);
            }
        }
        const float d = h2f((uint16_t)(q.hdr.x & 0xffffu)) * nib_mul, dmin = h2f((uint16_t)(q.hdr.x >> 16));
        const float part = fmaf(d, S, -(dmin * Mn));
        acc += active ? part : 0.f;
        if (it + 1 == n_iter) {  // row group complete
            const Where w = locate(g);
            const float tot = group_sum_dpp<LB>(acc);
            const uint32_t row = w.row0 + sub_row;
            if (b0 == LB - 1 && row < w.rows) w.y[row] = b.accumulate ? w.y[row] + tot : tot;
            acc = 0.f;
        }
    };

    while (u < n_units) {
        const uint32_t u2 = u + total_waves;
        if (u2 < n_units) fetch(u2, ub);
        consume(u, ua);
        if (u2 >= n_units) break;
        u = u2 + total_waves;
        if (u < n_units) fetch(u, ua);
        consume(u2, ub);
    }
}

// ------------------------------------------------------------------ Q6_K GEMV: one lane per super-block
//
// Same structure as the Q4_K kernel.  A lane owns one 256-column super-block of one
// row (128 bytes of ql, 64 of qh, 16 int8 scales, d); ql and qh are stored piece-major.
// Piece cc of ql (n = cc>>2, p = (cc>>1)&1, lh = cc&1) holds in its low nibbles 16
// codes of quarter p and in its high nibbles 16 codes of quarter p+2 of half n; their
// two high bits sit in qh piece 2n+lh at bit 2p resp. 2p+4 (langtax/src/quant.rs:8783-8853).
// The 6-bit codes are assembled four to a register, converted with v_cvt_f32_ubyte and
// brought back to -32..31 before the multiply; the sixteen int8 scales are applied per
// 16 columns.

struct Q6kUnit {
    uint4 ql[8], qh[4], sc;
    uint16_t d;
};

template <int LB, int NW>
__global__ __launch_bounds__(NW * 64, 4) void gemv_q6k_kernel(const GemvBatch b) {
    constexpr uint32_t RS = 64 / LB;
    constexpr uint32_t XROW = LB * 4 + 4;
    constexpr uint32_t XS_FLOATS = 64 * XROW;
    extern __shared__ __align__(16) float lds[];
    const uint32_t nb_all = b.job[0].m.nb;         // super-blocks per row: slot stride of the piece-major planes
    const uint32_t nb = b.units, cols = nb * 256;  // the window this launch covers
    const float *xw = b.x + (size_t)b.unit0 * 256;
    const uint32_t n_iter = (nb + LB - 1) / LB;
    float *xs = lds;                                  // as in the Q4_K kernel, with this dtype's column order

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t total_waves = gridDim.x * NW;
    const uint32_t sub_row = lane / LB, b0 = lane % LB;
    const uint32_t n_units = b.total_rgs * n_iter;

    struct Where {
        const uint8_t *p0, *p1, *p2, *p3;
        float *y;
        uint32_t s0, s1, s2, s3, rows, row0;
    };
    auto locate = [&](uint32_t g) {
        uint32_t j = 0;
        while (j + 1 < b.n_jobs && g >= b.job[j + 1].rg_begin) j++;
        Where w;
        w.p0 = b.job[j].m.p0; w.p1 = b.job[j].m.p1; w.p2 = b.job[j].m.p2; w.p3 = b.job[j].m.p3;
        w.s0 = b.job[j].m.s0; w.s1 = b.job[j].m.s1; w.s2 = b.job[j].m.s2; w.s3 = b.job[j].m.s3;
        w.y = b.job[j].y;
        w.rows = b.job[j].m.rows;
        w.row0 = (g - b.job[j].rg_begin) * RS;
        return w;
    };
    auto fetch = [&](uint32_t u, Q6kUnit &o) {
        const uint32_t g = u / n_iter, it = u - g * n_iter;
        const Where w = locate(g);
        uint32_t row = w.row0 + sub_row;
        row = row < w.rows ? row : w.rows - 1;
        uint32_t blk = it * LB + b0;
        blk = b.unit0 + (blk < nb ? blk : nb - 1);
        const uint8_t *ql = w.p0 + (size_t)row * w.s0 + (size_t)blk * 16;
        const uint8_t *qh = w.p1 + (size_t)row * w.s1 + (size_t)blk * 16;
#pragma unroll
        for (int cc = 0; cc < 8; cc++) o.ql[cc] = *reinterpret_cast<const uint4 *>(ql + (size_t)cc * nb_all * 16);
#pragma unroll
        for (int hc = 0; hc < 4; hc++) o.qh[hc] = *reinterpret_cast<const uint4 *>(qh + (size_t)hc * nb_all * 16);
        o.sc = *reinterpret_cast<const uint4 *>(w.p2 + (size_t)row * w.s2 + (size_t)blk * 16);
        o.d = *reinterpret_cast<const uint16_t *>(w.p3 + (size_t)row * w.s3 + (size_t)blk * 2);
    };

    // stage x: four consecutive lanes hold one 16-column group
    auto stage = [&](uint32_t col, const float4 v) {
        const uint32_t blk = col >> 8, r = col & 255u, n = r >> 7, quarter = (r >> 5) & 3u, l = r & 31u;
        const uint32_t cc = 4 * n + 2 * (quarter & 1u) + (l >> 4), t = (quarter >> 1) * 16 + (l & 15u);
        const uint32_t it = blk / LB, bl = blk % LB;
        *reinterpret_cast<float4 *>(xs + (size_t)it * XS_FLOATS + (cc * 8 + (t >> 2)) * XROW + bl * 4) = v;
    };
    for (uint32_t col = tid * 4; col < n_iter * LB * 256; col += NW * 64 * 4)
        stage(col, *reinterpret_cast<const float4 *>(xw + (col < cols ? col : 0)));
    __syncthreads();

    float acc = 0.f;
    Q6kUnit un;
    for (uint32_t u = blockIdx.x * NW + wave; u < n_units; u += total_waves) {
        fetch(u, un);
        const uint32_t g = u / n_iter, it = u - g * n_iter;
        const bool active = it * LB + b0 < nb;
        const float *xb = xs + (size_t)it * XS_FLOATS + b0 * 4;
        float t[16];
#pragma unroll
        for (int k = 0; k < 16; k++) t[k] = 0.f;
#pragma unroll
        for (int cc = 0; cc < 8; cc++) {
            constexpr int dummy = 0;
            (void)dummy;
            const int n = cc >> 2, p = (cc >> 1) & 1, lh = cc & 1;
            float x[32];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float4 v = *reinterpret_cast<const float4 *>(xb + (cc * 8 + i) * XROW);
                x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
            }
            const uint32_t lo[4] = {un.ql[cc].x, un.ql[cc].y, un.ql[cc].z, un.ql[cc].w};
            const uint4 hq = un.qh[2 * n + lh];
            const uint32_t hb[4] = {hq.x, hq.y, hq.z, hq.w};
            float tl = 0.f, th = 0.f;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                // Each byte becomes 4 (q - 32) as a signed byte: the 6-bit code in bits 2..7 with its top
                // bit flipped (q ^ 32 is q - 32 in 6-bit two's complement).  The 4 goes into the scale.
                const uint32_t two_lo = p == 0 ? (hb[d] << 6) : (hb[d] << 4);   // bits 2p..2p+1 moved to 6..7
                const uint32_t two_hi = p == 0 ? (hb[d] << 2) : hb[d];          // bits 2p+4..2p+5 moved to 6..7
                tl = dot4_sb((((lo[d] << 2) & 0x3c3c3c3cu) | (two_lo & 0xc0c0c0c0u)) ^ 0x80808080u, x + 4 * d, tl);
                th = dot4_sb((((lo[d] >> 2) & 0x3c3c3c3cu) | (two_hi & 0xc0c0c0c0u)) ^ 0x80808080u, x + 16 + 4 * d, th);
            }
            t[8 * n + 2 * p + lh] = tl;        // scale index 8n + lh + 2*quarter, quarter = p
            t[8 * n + 2 * (p + 2) + lh] = th;  // quarter = p + 2
        }
        const uint32_t scw[4] = {un.sc.x, un.sc.y, un.sc.z, un.sc.w};
        float S = 0.f;
#pragma unroll
        for (int k = 0; k < 16; k++) {
            // t index k = 8n + 2*quarter + lh is also the int8 scale index; the matching 16-column
            // group of x is (8n + 2*quarter + lh) in column order: group = r >> 4 with r = 128n + 32q + 16lh
            const float sc = (float)(int)(int8_t)(scw[k >> 2] >> (8 * (k & 3)));
            S = fmaf(sc, t[k], S);
        }
        const float part = (h2f(un.d) * 0.25f) * S;  // t holds 4 (q - 32) sums
        acc += active ? part : 0.f;
        if (it + 1 == n_iter) {
            const Where w = locate(g);
            const float tot = group_sum_dpp<LB>(acc);
            const uint32_t row = w.row0 + sub_row;
            if (b0 == LB - 1 && row < w.rows) w.y[row] = b.accumulate ? w.y[row] + tot : tot;
            acc = 0.f;
        }
    }
}

// ------------------------------------------------------------------ Q8_0 / Q4_0 / Q5_0 / Q5_1 GEMV: one lane per unit
//
// Same structure as the Q4_K kernel, for the dtypes with 32-column blocks.  A lane
// owns one unit of one row: 8 consecutive blocks (256 columns) of Q4_0/Q5_0/Q5_1 or
// 4 blocks (128 columns) of Q8_0, i.e. 8 code pieces of 16 bytes (piece-major, see
// matview.h) plus the unit's scales, which are contiguous in their plane.  x sits in
// LDS in column order, one float4 row per 4 columns of a unit, padded like the
// Q4_K kernel's.  Codes are brought to their signed value before the multiply
// (Q8_0: signed byte convert; Q4_0: signed 4-bit convert; Q5_0: minus 16); only Q5_1's
// offsets, which are separate terms of the weight, go through the per-block sums of x
// (langtax/src/quant.rs:7511-7541, 7734-7765, 7884-7950, 8046-8130).

template <uint32_t T> struct B32Geo {
    static constexpr int UC = T == T_Q8_0 ? 128 : 256;  // columns per unit
    static constexpr int NBLK = UC / 32;                // blocks per unit
    static constexpr int XV = UC / 32;                  // float4 of x per code piece
};
template <uint32_t T> struct B32Unit;
template <> struct B32Unit<T_Q8_0> { uint4 q[8]; uint2 d; };
template <> struct B32Unit<T_Q4_0> { uint4 q[8]; uint4 d; };
template <> struct B32Unit<T_Q5_0> { uint4 q[8]; uint4 qh[2]; uint4 d; };
template <> struct B32Unit<T_Q5_1> { uint4 q[8]; uint4 qh[2]; uint4 dm[2]; };

// I4: Q4_0 nibbles go through the signed 4-bit convert (else byte convert and subtract).
template <uint32_t T, int LB, int NW, bool I4>
__global__ __launch_bounds__(NW * 64, (T == T_Q5_0 || T == T_Q5_1) ? 3 : 4) void gemv_b32_kernel(const GemvBatch b) {
    using G = B32Geo<T>;
    constexpr uint32_t RS = 64 / LB;           // rows per wavefront step = rows per row group
    constexpr uint32_t XROW = LB * 4 + 4;      // floats per LDS row: LB float4 plus one of padding
    constexpr uint32_t XS_FLOATS = (G::UC / 4) * XROW;
    extern __shared__ __align__(16) float lds[];
    const uint32_t nu_all = b.job[0].m.cols / G::UC;  // units per row: slot stride of the piece-major plane
    const uint32_t nu = b.units, cols = nu * G::UC;   // the window this launch covers
    const float *xw = b.x + (size_t)b.unit0 * G::UC;
    const uint32_t n_iter = (nu + LB - 1) / LB;
    float *xs = lds;                                   // [it][column / 4 of the unit][unit % LB] float4
    float *ssum = lds + (size_t)n_iter * XS_FLOATS;    // [it][block of the unit][unit % LB]: sum of x over the block

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t total_waves = gridDim.x * NW;
    const uint32_t sub_row = lane / LB, b0 = lane % LB;
    // A wavefront takes whole row groups (every total_waves-th one) and walks the
    // n_iter unit columns of each in turn, so that a row's sum stays in one lane.
    struct Pos {
        uint32_t g, it;
    };
    auto advance = [&](Pos p) {
        p.it++;
        if (p.it == n_iter) {
            p.it = 0;
            p.g += total_waves;
        }
        return p;
    };
    auto valid = [&](const Pos &p) { return p.g < b.total_rgs; };

    struct Where {
        const MatView *m;
        float *y;
        uint32_t row0;
    };
    auto locate = [&](uint32_t g) {
        uint32_t j = 0;
        while (j + 1 < b.n_jobs && g >= b.job[j + 1].rg_begin) j++;
        Where w;
        w.m = &b.job[j].m;
        w.y = b.job[j].y;
        w.row0 = (g - b.job[j].rg_begin) * RS;
        return w;
    };
    auto fetch = [&](const Pos &p, B32Unit<T> &o) {
        const uint32_t it = p.it;
        const Where w = locate(p.g < b.total_rgs ? p.g : b.total_rgs - 1);
        const MatView &m = *w.m;
        uint32_t row = w.row0 + sub_row;
        row = row < m.rows ? row : m.rows - 1;
        uint32_t un = it * LB + b0;
        un = b.unit0 + (un < nu ? un : nu - 1);
        const uint8_t *q = m.p0 + (size_t)row * m.s0 + (size_t)un * 16;
#pragma unroll
        for (int cc = 0; cc < 8; cc++) o.q[cc] = *reinterpret_cast<const uint4 *>(q + (size_t)cc * nu_all * 16);
        if constexpr (T == T_Q8_0) {
            o.d = *reinterpret_cast<const uint2 *>(m.p1 + (size_t)row * m.s1 + (size_t)un * 8);
        } else if constexpr (T == T_Q4_0) {
            o.d = *reinterpret_cast<const uint4 *>(m.p1 + (size_t)row * m.s1 + (size_t)un * 16);
        } else {
            const uint4 *h = reinterpret_cast<const uint4 *>(m.p1 + (size_t)row * m.s1 + (size_t)un * 32);
            o.qh[0] = h[0];
            o.qh[1] = h[1];
            if constexpr (T == T_Q5_0) {
                o.d = *reinterpret_cast<const uint4 *>(m.p2 + (size_t)row * m.s2 + (size_t)un * 16);
            } else {
                const uint4 *dm = reinterpret_cast<const uint4 *>(m.p2 + (size_t)row * m.s2 + (size_t)un * 32);
                o.dm[0] = dm[0];
                o.dm[1] = dm[1];
            }
        }
    };

    Pos pa = {blockIdx.x * NW + wave, 0};
    B32Unit<T> ua, ub;
    // Stage x once per workgroup; eight consecutive lanes hold one 32-column block.
    auto stage = [&](uint32_t col, const float4 v) {
        const uint32_t un = col / G::UC, e = col % G::UC, it = un / LB, bl = un % LB;
        *reinterpret_cast<float4 *>(xs + (size_t)it * XS_FLOATS + (e >> 2) * XROW + bl * 4) = v;
        if constexpr (T == T_Q5_1) {  // the offsets m multiply the block sums of x
            float sm = (v.x + v.y) + (v.z + v.w);
#define NH_DPP_ADD(ctrl) sm += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sm), ctrl, 0xf, 0xf, false))
            NH_DPP_ADD(0xb1);
            NH_DPP_ADD(0x4e);
            NH_DPP_ADD(0x141);
#undef NH_DPP_ADD
            if ((lane & 7u) == 0) ssum[(it * G::NBLK + (e >> 5)) * LB + bl] = sm;
        }
    };
    constexpr int NXV = (LB * G::UC / 4 + NW * 64 - 1) / (NW * 64);  // float4 per thread for LB units of x
    if (n_iter == 1) {
        float4 xv[NXV];
#pragma unroll
        for (int k = 0; k < NXV; k++) {
            const uint32_t col = (tid + k * NW * 64) * 4;
            xv[k] = *reinterpret_cast<const float4 *>(xw + (col < cols ? col : 0));  // branch-free: stays first
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the x loads ahead of the weight loads in the queue
        fetch(pa, ua);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < NXV; k++) {
            const uint32_t col = (tid + k * NW * 64) * 4;
            if (col < LB * G::UC) stage(col, col < cols ? xv[k] : make_float4(0.f, 0.f, 0.f, 0.f));
        }
        __syncthreads();
    } else {
        for (uint32_t col = tid * 4; col < n_iter * LB * G::UC; col += NW * 64 * 4)
            stage(col, col < cols ? *reinterpret_cast<const float4 *>(xw + col) : make_float4(0.f, 0.f, 0.f, 0.f));
        __syncthreads();
        if (valid(pa)) fetch(pa, ua);
    }

    float acc = 0.f;
    auto consume = [&](const Pos &p, const B32Unit<T> &q) {
        const uint32_t g = p.g, it = p.it;
        const bool active = it * LB + b0 < nu;
        const float *xb = xs + (size_t)it * XS_FLOATS + b0 * 4;
        const float *sp = ssum + (size_t)it * G::NBLK * LB + b0;
        float t[G::NBLK];
#pragma unroll
        for (int k = 0; k < G::NBLK; k++) t[k] = 0.f;
        uint32_t qh[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr (T == T_Q5_0 || T == T_Q5_1) {
            qh[0] = q.qh[0].x; qh[1] = q.qh[0].y; qh[2] = q.qh[0].z; qh[3] = q.qh[0].w;
            qh[4] = q.qh[1].x; qh[5] = q.qh[1].y; qh[6] = q.qh[1].z; qh[7] = q.qh[1].w;
        }
#pragma unroll
        for (int cc = 0; cc < 8; cc++) {
            float x[4 * G::XV];
#pragma unroll
            for (int i = 0; i < G::XV; i++) {
                float4 v = *reinterpret_cast<const float4 *>(xb + (cc * G::XV + i) * XROW);
                x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
            }
            const uint32_t w[4] = {q.q[cc].x, q.q[cc].y, q.q[cc].z, q.q[cc].w};
#pragma unroll
            for (int d = 0; d < 4; d++) {
                if constexpr (T == T_Q8_0) {
                    t[cc >> 1] = dot4_sb(w[d], x + 4 * d, t[cc >> 1]);
                } else if constexpr (T == T_Q4_0) {
                    if constexpr (I4) {  // (n - 8) / 16 per nibble; the 16 goes into the block scale
                        const uint32_t wx = w[d] ^ 0x88888888u;
                        t[cc] = dot4_i4(wx, x + 4 * d, t[cc]);
                        t[cc] = dot4_i4(wx >> 4, x + 16 + 4 * d, t[cc]);
                    } else {
                        t[cc] = dot4_ub_biased(w[d] & 0x0f0f0f0fu, 8.f, x + 4 * d, t[cc]);
                        t[cc] = dot4_ub_biased((w[d] >> 4) & 0x0f0f0f0fu, 8.f, x + 16 + 4 * d, t[cc]);
                    }
                } else if constexpr (T == T_Q5_0) {
                    // bytes 8 (c - 16): the 5-bit code in bits 3..7 with its top bit flipped; the 8 goes into the scale
                    t[cc] = dot4_sb(q5_signed_bytes((w[d] << 3) & 0x78787878u, qh[cc], 4 * d), x + 4 * d, t[cc]);
                    t[cc] = dot4_sb(q5_signed_bytes((w[d] >> 1) & 0x78787878u, qh[cc], 16 + 4 * d), x + 16 + 4 * d, t[cc]);
                } else {
                    t[cc] = dot4_ub(q5_bytes(w[d] & 0x0f0f0f0fu, qh[cc], 4 * d), x + 4 * d, t[cc]);
                    t[cc] = dot4_ub(q5_bytes((w[d] >> 4) & 0x0f0f0f0fu, qh[cc], 16 + 4 * d), x + 16 + 4 * d, t[cc]);
                }
            }
        }
        float part = 0.f;
        if constexpr (T == T_Q8_0) {
            const uint32_t dd[2] = {q.d.x, q.d.y};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const float d = h2f((uint16_t)(dd[k >> 1] >> (16 * (k & 1))));
                part = fmaf(d, t[k], part);
            }
        } else if constexpr (T == T_Q4_0 || T == T_Q5_0) {
            const uint32_t dd[4] = {q.d.x, q.d.y, q.d.z, q.d.w};
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float d = h2f((uint16_t)(dd[k >> 1] >> (16 * (k & 1))));
                part = fmaf(T == T_Q5_0 ? d * 0.125f : (I4 ? d * 16.f : d), t[k], part);
            }
        } else {
            const uint32_t dm[8] = {q.dm[0].x, q.dm[0].y, q.dm[0].z, q.dm[0].w, q.dm[1].x, q.dm[1].y, q.dm[1].z, q.dm[1].w};
#pragma unroll
            for (int k = 0; k < 8; k++) {
                part = fmaf(h2f((uint16_t)(dm[k] & 0xffffu)), t[k], part);
                part = fmaf(h2f((uint16_t)(dm[k] >> 16)), sp[k * LB], part);
            }
        }
        acc += active ? part : 0.f;
        if (it + 1 == n_iter) {  // row group complete
            const Where w = locate(g);
            const float tot = group_sum_dpp<LB>(acc);
            const uint32_t row = w.row0 + sub_row;
            if (b0 == LB - 1 && row < w.m->rows) w.y[row] = b.accumulate ? w.y[row] + tot : tot;
            acc = 0.f;
        }
    };

    while (valid(pa)) {
        const Pos pb = advance(pa);
        if (valid(pb)) fetch(pb, ub);
        consume(pa, ua);
        if (!valid(pb)) break;
        pa = advance(pb);
        if (valid(pa)) fetch(pa, ua);
        consume(pb, ub);
    }
}

// ------------------------------------------------------------------ tiled GEMM (any token count)
//
// Eight consecutive decoded weights of one row starting at column k0 (k0 % 8 == 0).
template <uint32_t T> __device__ __forceinline__ void dequant8(const MatView &m, uint32_t row, uint32_t k0, float *w) {
    const size_t ro = (size_t)row;
    if constexpr (T == T_F32) {
        const float4 *p = reinterpret_cast<const float4 *>(m.p0 + ro * m.s0 + (size_t)k0 * 4);
        float4 a = p[0], b = p[1];
        w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w; w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w;
    } else if constexpr (T == T_F16) {
        uint4 q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + (size_t)k0 * 2);
        const uint32_t v[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[2 * i] = h2f((uint16_t)(v[i] & 0xffffu));
            w[2 * i + 1] = h2f((uint16_t)(v[i] >> 16));
        }
    } else if constexpr (T == T_Q8_0) {
        uint32_t b = k0 >> 5, j = k0 & 31;
        uint2 q = *reinterpret_cast<const uint2 *>(m.p0 + ro * m.s0 +
                                                   piece_offset(piece_major(T, m.cols), m.cols / unit_cols(T), 2 * b + (j >> 4)) + (j & 15));
        float d = h2f(*reinterpret_cast<const uint16_t *>(m.p1 + ro * m.s1 + (size_t)b * 2));
#pragma unroll
        for (int k = 0; k < 4; k++) {
            w[k] = sb(q.x, k) * d;
            w[4 + k] = sb(q.y, k) * d;
        }
    } else if constexpr (T == T_Q4_0 || T == T_Q5_0 || T == T_Q5_1) {
        // element e = j + i of block b: nibble of byte (e & 15), high nibble when e >= 16
        uint32_t b = k0 >> 5, j = k0 & 31, byte0 = j & 15;
        uint2 q = *reinterpret_cast<const uint2 *>(m.p0 + ro * m.s0 +
                                                   piece_offset(piece_major(T, m.cols), m.cols / unit_cols(T), b) + byte0);
        uint32_t sh = j >= 16 ? 4u : 0u;
        uint32_t n0 = (q.x >> sh) & 0x0f0f0f0fu, n1 = (q.y >> sh) & 0x0f0f0f0fu;
        if constexpr (T == T_Q4_0) {
            float d = h2f(*reinterpret_cast<const uint16_t *>(m.p1 + ro * m.s1 + (size_t)b * 2));
#pragma unroll
            for (int k = 0; k < 4; k++) {
                w[k] = (float)((int)((n0 >> (8 * k)) & 0xffu) - 8) * d;
                w[4 + k] = (float)((int)((n1 >> (8 * k)) & 0xffu) - 8) * d;
            }
        } else {
            uint32_t qh = *reinterpret_cast<const uint32_t *>(m.p1 + ro * m.s1 + (size_t)b * 4);
            uint32_t c0 = q5_bytes(n0, qh, j), c1 = q5_bytes(n1, qh, j + 4);
            if constexpr (T == T_Q5_0) {
                float d = h2f(*reinterpret_cast<const uint16_t *>(m.p2 + ro * m.s2 + (size_t)b * 2));
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    w[k] = (float)((int)((c0 >> (8 * k)) & 0xffu) - 16) * d;
                    w[4 + k] = (float)((int)((c1 >> (8 * k)) & 0xffu) - 16) * d;
                }
            } else {
                uint32_t dm = *reinterpret_cast<const uint32_t *>(m.p2 + ro * m.s2 + (size_t)b * 4);
                float d = h2f((uint16_t)(dm & 0xffffu)), mm = h2f((uint16_t)(dm >> 16));
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    w[k] = __fadd_rn(__fmul_rn((float)((c0 >> (8 * k)) & 0xffu), d), mm);
                    w[4 + k] = __fadd_rn(__fmul_rn((float)((c1 >> (8 * k)) & 0xffu), d), mm);
                }
            }
        }
    } else if constexpr (T == T_Q4_K) {
        uint32_t b = k0 >> 8, e = k0 & 255, sub = e >> 5, l = e & 31;
        const uint32_t cc = (sub >> 1) * 2 + (l >> 4);  // 16-byte piece of the block's codes
        uint2 q = *reinterpret_cast<const uint2 *>(m.p0 + ro * m.s0 + ((size_t)cc * m.nb + b) * 16 + (l & 15));
        uint4 hdr = *reinterpret_cast<const uint4 *>(m.p1 + ro * m.s1 + (size_t)b * 16);
        float d = h2f((uint16_t)(hdr.x & 0xffffu)), dmin = h2f((uint16_t)(hdr.x >> 16));
        float sc, mn;
        q4k_scale_min(hdr.y, hdr.z, hdr.w, (int)sub, sc, mn);
        float a = d * sc, bb = dmin * mn;
        uint32_t sh = (sub & 1) ? 4u : 0u;
        uint32_t n0 = (q.x >> sh) & 0x0f0f0f0fu, n1 = (q.y >> sh) & 0x0f0f0f0fu;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            w[k] = __fsub_rn(__fmul_rn(a, (float)((n0 >> (8 * k)) & 0xffu)), bb);
            w[4 + k] = __fsub_rn(__fmul_rn(a, (float)((n1 >> (8 * k)) & 0xffu)), bb);
        }
    } else if constexpr (T == T_Q6_K) {
        uint32_t b = k0 >> 8, e = k0 & 255, n = e >> 7, rr = e & 127, quarter = rr >> 5, l = rr & 31;
        const uint32_t qoff = n * 64 + (quarter & 1) * 32 + l, hoff = n * 32 + l;  // byte offsets inside the block
        uint2 lo = *reinterpret_cast<const uint2 *>(m.p0 + ro * m.s0 + ((size_t)(qoff >> 4) * m.nb + b) * 16 + (qoff & 15));
        uint2 hb = *reinterpret_cast<const uint2 *>(m.p1 + ro * m.s1 + ((size_t)(hoff >> 4) * m.nb + b) * 16 + (hoff & 15));
        int8_t s8 = *reinterpret_cast<const int8_t *>(m.p2 + ro * m.s2 + (size_t)b * 16 + n * 8 + quarter * 2 + (l >> 4));
        float ds = h2f(*reinterpret_cast<const uint16_t *>(m.p3 + ro * m.s3 + (size_t)b * 2)) * (float)(int)s8;
        uint32_t nsh = quarter >= 2 ? 4u : 0u, hsh = 2 * quarter;
        uint32_t c0 = ((lo.x >> nsh) & 0x0f0f0f0fu) | (((hb.x >> hsh) & 0x03030303u) << 4);
        uint32_t c1 = ((lo.y >> nsh) & 0x0f0f0f0fu) | (((hb.y >> hsh) & 0x03030303u) << 4);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            w[k] = ds * (float)((int)((c0 >> (8 * k)) & 0xffu) - 32);
            w[4 + k] = ds * (float)((int)((c1 >> (8 * k)) & 0xffu) - 32);
        }
    }
}

// Tile: 64 rows x 32 tokens per workgroup, 32 columns per pass through LDS,
// each thread owns 4 rows x 2 tokens and accumulates in f32 over all columns.
constexpr int GT_ROWS = 64, GT_TOK = 32, GT_K = 32;

template <uint32_t T>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(MatView m, const float *__restrict__ x, float *__restrict__ y,
                                                         uint32_t n_tokens) {
    __shared__ __align__(16) float ws[GT_K][GT_ROWS];
    __shared__ __align__(16) float xsm[GT_K][GT_TOK];
    const uint32_t tid = threadIdx.x;
    const uint32_t row_base = blockIdx.x * GT_ROWS, tok_base = blockIdx.y * GT_TOK;
    const uint32_t tx = tid & 15u, ty = tid >> 4;  // rows 4*tx.., tokens 2*ty..
    float acc[2][4];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = 0.f;

    const uint32_t w_row = tid & 63u, w_kg = tid >> 6;    // weight staging: row, 8-column group
    const uint32_t x_tok = tid & 31u, x_kg = tid >> 5;    // activation staging: token, 4-column group
    const uint32_t k_pad = (m.cols + 7u) & ~7u;
    const uint32_t g_row = row_base + w_row < m.rows ? row_base + w_row : m.rows - 1;
    const bool tok_ok = tok_base + x_tok < n_tokens;
    const float *xrow = x + (size_t)(tok_ok ? tok_base + x_tok : 0) * m.cols;

    for (uint32_t k0 = 0; k0 < k_pad; k0 += GT_K) {
        float w8[8];
        uint32_t kw0 = k0 + w_kg * 8;
        if (kw0 < k_pad) {
            dequant8<T>(m, g_row, kw0, w8);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) w8[i] = 0.f;
        }
#pragma unroll
        for (int i = 0; i < 8; i++) ws[w_kg * 8 + i][w_row] = w8[i];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t k = k0 + x_kg * 4 + i;
            xsm[x_kg * 4 + i][x_tok] = (tok_ok && k < m.cols) ? xrow[k] : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int k = 0; k < GT_K; k++) {
            float4 wv = *reinterpret_cast<const float4 *>(&ws[k][tx * 4]);
            float2 xv = *reinterpret_cast<const float2 *>(&xsm[k][ty * 2]);
            acc[0][0] = fmaf(wv.x, xv.x, acc[0][0]);
            acc[0][1] = fmaf(wv.y, xv.x, acc[0][1]);
            acc[0][2] = fmaf(wv.z, xv.x, acc[0][2]);
            acc[0][3] = fmaf(wv.w, xv.x, acc[0][3]);
            acc[1][0] = fmaf(wv.x, xv.y, acc[1][0]);
            acc[1][1] = fmaf(wv.y, xv.y, acc[1][1]);
            acc[1][2] = fmaf(wv.z, xv.y, acc[1][2]);
            acc[1][3] = fmaf(wv.w, xv.y, acc[1][3]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < 2; a++) {
        uint32_t t = tok_base + ty * 2 + a;
        if (t >= n_tokens) continue;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            uint32_t r = row_base + tx * 4 + b;
            if (r < m.rows) y[(size_t)t * m.rows + r] = acc[a][b];
        }
    }
}

// ------------------------------------------------------------------ MFMA GEMM (two or more tokens)
//
// Quantized dtypes only.  A weight is scale * code (+ offset) with an integer code
// of at most 8 bits, so the code is exact in bf16; an f32 activation is exactly
// the sum of three bf16 numbers (its 24 significand bits cut into 8 + 8 + 8).
// Per group of 16 columns that share a scale the kernel therefore forms
//     P[token, row] = sum_k x[token, k] * code[row, k]
// with three bf16 MFMAs whose products are exact and whose sums are f32, and
// then applies the f32 scale (and the offset times the group's sum of x) on the
// vector ALU:  y += scale * P + offset * Sx.  Nothing is quantized or rounded
// to fewer than 24 bits anywhere, so the result differs from the reference's
// (langtax/src/quant.rs:6746-6792, pool.rs:54-101) only in the order of f32 roundings.
//
// mm_xsplit_kernel cuts the activations once per call into the MFMA operand
// layout; gemm_mfma_kernel streams the weights: a workgroup owns 256 rows
// (one per thread for decoding, 64 per wavefront for the MFMAs) and 32 or 64
// tokens, walks its share of the columns in steps of 32, and, when the row and
// token tiles alone would not fill the chip, shares the columns of one tile
// between several workgroups whose partial sums mm_reduce_kernel adds in a
// fixed order.

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int MM_ROWS = TILE_ROWS;  // rows per workgroup = row tile of the tiled copy
constexpr int MM_MAX_JOBS = 8;

struct MmJob {
    MatView m;        // the tiled copy (matview.h)
    const float *x;   // tokens x cols
    float *y;         // tokens x rows
    float *part;      // ksplit x tokens x rows when ksplit > 1
    uint32_t tokens;
    uint32_t tok_off;    // first token slot of this job in the split activations
    uint32_t wg_begin;   // first workgroup of this job
    uint32_t tok_tiles;  // token tiles per row tile
    uint32_t ksplit;     // workgroups that share the columns of one tile
    uint32_t pad;
};
struct MmBatch {
    MmJob job[MM_MAX_JOBS];
    uint4 *xb;   // [group of 16 columns][part 0..2][half 0..1][token slot] x 8 bf16
    float *sx;   // [group of 16 columns][token slot]: sum of the group's activations
    uint32_t n_jobs, total_wgs, mpad, any_split;
    uint32_t nibble_bf16, pad0, pad1, pad2;  // nibble_bf16: the device converts nibble bytes straight to bf16 integers
};

template <uint32_t T> struct MmTraits {
    static constexpr bool OFFSET = (T == T_Q4_K || T == T_Q5_1);                       // W = scale * code + offset
    static constexpr bool SAME_SCALE = (T == T_Q4_0 || T == T_Q5_0 || T == T_Q5_1 || T == T_Q8_0);  // per 32 columns
};

// First of the 16 consecutive columns of group g (0 or 1) of step s.
template <uint32_t T> __device__ __forceinline__ uint32_t mm_group_col(uint32_t s, uint32_t g) {
    if constexpr (T == T_Q8_0) return s * 32 + g * 16;
    else return chunk_col<T>(s, (int)(16 * g));
}

__device__ __forceinline__ uint32_t bf16_pair(float lo, float hi) {
    // high halves of the two f32 patterns: exact for integers of at most 8 bits
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}
__device__ __forceinline__ uint4 bf16x8_of(const float *f) {
    return make_uint4(bf16_pair(f[0], f[1]), bf16_pair(f[2], f[3]), bf16_pair(f[4], f[5]), bf16_pair(f[6], f[7]));
}

template <uint32_t T>
__global__ __launch_bounds__(256) void mm_xsplit_kernel(const MmBatch b, uint32_t n_groups) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)n_groups * b.mpad) return;
    const uint32_t gi = (uint32_t)(idx / b.mpad), ts = (uint32_t)(idx % b.mpad);
    const float *src = nullptr;
    for (uint32_t j = 0; j < b.n_jobs; j++) {
        const MmJob &job = b.job[j];
        if (ts >= job.tok_off && ts - job.tok_off < job.tokens)
            src = job.x + (size_t)(ts - job.tok_off) * job.m.cols + mm_group_col<T>(gi >> 1, gi & 1u);
    }
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; i++) v[i] = src ? src[i] : 0.f;
    float sum = 0.f;
    float hi[16], mid[16], lo[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        sum += v[i];
        hi[i] = __uint_as_float(__float_as_uint(v[i]) & 0xffff0000u);
        const float r1 = v[i] - hi[i];  // exact
        mid[i] = __uint_as_float(__float_as_uint(r1) & 0xffff0000u);
        lo[i] = r1 - mid[i];            // exact, at most 8 significant bits
    }
    const size_t plane = (size_t)2 * b.mpad;  // one part: two halves
    uint4 *dst = b.xb + (size_t)gi * 3 * plane + ts;
    dst[0] = bf16x8_of(hi);
    dst[b.mpad] = bf16x8_of(hi + 8);
    dst[plane] = bf16x8_of(mid);
    dst[plane + b.mpad] = bf16x8_of(mid + 8);
    dst[2 * plane] = bf16x8_of(lo);
    dst[2 * plane + b.mpad] = bf16x8_of(lo + 8);
    b.sx[(size_t)gi * b.mpad + ts] = sum;
}

// Packed bytes of one 32-column step of one row.
template <uint32_t T> struct MmRaw { Raw<T> r; };
template <> struct MmRaw<T_Q8_0> { uint4 q0, q1; uint16_t d; };

// Step s of the row that thread `tid` of row tile `tile` decodes, from the tiled copy g
// (g.s0..s3 = units per row of each plane).
template <uint32_t T>
__device__ __forceinline__ void mm_load(const MatView &g, uint32_t tile, uint32_t tid, uint32_t s, MmRaw<T> &o) {
    auto at = [&](const uint8_t *p, uint32_t per_row, size_t i, size_t bytes) {
        return p + (((size_t)tile * per_row + i) * TILE_ROWS + tid) * bytes;
    };
    if constexpr (T == T_Q8_0) {
        o.q0 = *reinterpret_cast<const uint4 *>(at(g.p0, g.s0, 2 * (size_t)s, 16));
        o.q1 = *reinterpret_cast<const uint4 *>(at(g.p0, g.s0, 2 * (size_t)s + 1, 16));
        o.d = *reinterpret_cast<const uint16_t *>(at(g.p1, g.s1, s, 2));
    } else if constexpr (T == T_Q4_0) {
        o.r.q = *reinterpret_cast<const uint4 *>(at(g.p0, g.s0, s, 16));
        o.r.d = *reinterpret_cast<const uint16_t *>(at(g.p1, g.s1, s, 2));
    } else if constexpr (T == T_Q5_0) {
        o.r.q = *reinterpret_cast<const uint4 *>(at(g.p0, g.s0, s, 16));
        o.r.qh = *reinterpret_cast<const uint32_t *>(at(g.p1, g.s1, s, 4));
        o.r.d = *reinterpret_cast<const uint16_t *>(at(g.p2, g.s2, s, 2));
    } else if constexpr (T == T_Q5_1) {
        o.r.q = *reinterpret_cast<const uint4 *>(at(g.p0, g.s0, s, 16));
        o.r.qh = *reinterpret_cast<const uint32_t *>(at(g.p1, g.s1, s, 4));
        o.r.dm = *reinterpret_cast<const uint32_t *>(at(g.p2, g.s2, s, 4));
    } else if constexpr (T == T_Q4_K) {
        o.r.q = *reinterpret_cast<const uint4 *>(at(g.p0, g.s0, s, 16));
        o.r.hdr = *reinterpret_cast<const uint4 *>(at(g.p1, g.s1, s >> 3, 16));
    } else if constexpr (T == T_Q6_K) {
        const uint32_t blk = s >> 3, cc = s & 7u, n = cc >> 2, k = cc & 1u;
        o.r.ql = *reinterpret_cast<const uint4 *>(at(g.p0, g.s0, s, 16));
        o.r.qh = *reinterpret_cast<const uint4 *>(at(g.p1, g.s1, (size_t)blk * 4 + 2 * n + k, 16));
        o.r.sc = *reinterpret_cast<const uint2 *>(at(g.p2, g.s2, (size_t)blk * 2 + n, 8));
        o.r.d = *reinterpret_cast<const uint16_t *>(at(g.p3, g.s3, blk, 2));
    }
}

__device__ __forceinline__ void mm_codes4(uint32_t bytes, float bias, float *f) {
    f[0] = ub0(bytes) - bias;
    f[1] = ub1(bytes) - bias;
    f[2] = ub2(bytes) - bias;
    f[3] = ub3(bytes) - bias;
}

// Codes of the two groups of step s as bf16 (frag[g][half]), with scale[g] and
// offset[g]: W[row, col] = scale * code + offset.
template <uint32_t T, bool NIBBLE_BF16>
__device__ __forceinline__ void mm_decode(const MmRaw<T> &raw, uint32_t s, uint4 (&frag)[2][2], float (&scale)[2],
                                          float (&offset)[2]) {
    float f[2][16];
    offset[0] = offset[1] = 0.f;
    bool packed_done = false;  // frag already written by the fp8 -> bf16 path
    if constexpr (T == T_Q8_0) {
        const uint32_t w[8] = {raw.q0.x, raw.q0.y, raw.q0.z, raw.q0.w, raw.q1.x, raw.q1.y, raw.q1.z, raw.q1.w};
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int k = 0; k < 4; k++) f[i >> 2][4 * (i & 3) + k] = sb(w[i], k);
        scale[0] = scale[1] = h2f(raw.d);
    } else if constexpr (T == T_Q4_0) {
        const Raw<T> &r = raw.r;
        const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            mm_codes4(w[i] & 0x0f0f0f0fu, 8.f, f[0] + 4 * i);
            mm_codes4((w[i] >> 4) & 0x0f0f0f0fu, 8.f, f[1] + 4 * i);
        }
        scale[0] = scale[1] = h2f(r.d);
    } else if constexpr (T == T_Q5_0 || T == T_Q5_1) {
        const Raw<T> &r = raw.r;
        const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        constexpr float bias = T == T_Q5_0 ? 16.f : 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            mm_codes4(q5_bytes(w[i] & 0x0f0f0f0fu, r.qh, 4 * i), bias, f[0] + 4 * i);
            mm_codes4(q5_bytes((w[i] >> 4) & 0x0f0f0f0fu, r.qh, 16 + 4 * i), bias, f[1] + 4 * i);
        }
        if constexpr (T == T_Q5_0) {
            scale[0] = scale[1] = h2f(r.d);
        } else {
            scale[0] = scale[1] = h2f((uint16_t)(r.dm & 0xffffu));
            offset[0] = offset[1] = h2f((uint16_t)(r.dm >> 16));
        }
    } else if constexpr (T == T_Q4_K) {
        const Raw<T> &r = raw.r;
        const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        if constexpr (NIBBLE_BF16) {  // one convert per two codes, no f32 in between
            uint32_t o[2][8];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t lo = w[i] & 0x0f0f0f0fu, hi = (w[i] >> 4) & 0x0f0f0f0fu;
                o[0][2 * i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)lo, 512.0f, false));
                o[0][2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)lo, 512.0f, true));
                o[1][2 * i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)hi, 512.0f, false));
                o[1][2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)hi, 512.0f, true));
            }
#pragma unroll
            for (int g = 0; g < 2; g++) {
                frag[g][0] = make_uint4(o[g][0], o[g][1], o[g][2], o[g][3]);
                frag[g][1] = make_uint4(o[g][4], o[g][5], o[g][6], o[g][7]);
            }
            packed_done = true;
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                mm_codes4(w[i] & 0x0f0f0f0fu, 0.f, f[0] + 4 * i);
                mm_codes4((w[i] >> 4) & 0x0f0f0f0fu, 0.f, f[1] + 4 * i);
            }
        }
        // 6-bit (scale, min) pairs 2g and 2g+1 of the block, g = (s % 8) / 2 (langtax/src/quant.rs:8901-8912)
        const uint32_t g = (s & 7u) >> 1;
        const uint32_t sh = 16 * (g & 1u);  // pairs 2g, 2g+1 sit in bytes (2g % 4), (2g % 4) + 1 of each header dword
        const uint32_t a2 = (r.hdr.y >> sh) & 0xffffu, b2 = (r.hdr.z >> sh) & 0xffffu, c2 = (r.hdr.w >> sh) & 0xffffu;
        const uint32_t up = 0u - (g >> 1);  // all ones for pairs 4..7, which are split over the three dwords
        auto pick = [&](uint32_t lo, uint32_t hi) { return lo ^ ((lo ^ hi) & up); };
        const uint32_t s0 = pick(a2 & 63u, (c2 & 15u) | ((a2 >> 2) & 0x30u));
        const uint32_t s1 = pick((a2 >> 8) & 63u, ((c2 >> 8) & 15u) | ((a2 >> 10) & 0x30u));
        const uint32_t n0 = pick(b2 & 63u, ((c2 >> 4) & 15u) | ((b2 >> 2) & 0x30u));
        const uint32_t n1 = pick((b2 >> 8) & 63u, ((c2 >> 12) & 15u) | ((b2 >> 10) & 0x30u));
        const float d = h2f((uint16_t)(r.hdr.x & 0xffffu)), dmin = h2f((uint16_t)(r.hdr.x >> 16));
        const float sc0 = (float)s0, sc1 = (float)s1, m0 = (float)n0, m1 = (float)n1;
        scale[0] = d * sc0;
        scale[1] = d * sc1;
        offset[0] = -(dmin * m0);
        offset[1] = -(dmin * m1);
    } else if constexpr (T == T_Q6_K) {
        const Raw<T> &r = raw.r;
        const uint32_t lo[4] = {r.ql.x, r.ql.y, r.ql.z, r.ql.w};
        const uint32_t hb[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        const uint32_t cc = s & 7u, h = (cc >> 1) & 1u, k = cc & 1u;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t two_lo = (hb[i] >> (2 * h)) & 0x03030303u;
            const uint32_t two_hi = (hb[i] >> (2 * h + 4)) & 0x03030303u;
            mm_codes4((lo[i] & 0x0f0f0f0fu) | (two_lo << 4), 32.f, f[0] + 4 * i);
            mm_codes4(((lo[i] >> 4) & 0x0f0f0f0fu) | (two_hi << 4), 32.f, f[1] + 4 * i);
        }
        const int sh = (int)(8 * (2 * h + k));
        const float d = h2f(r.d);
        scale[0] = d * (float)(int)(int8_t)(r.sc.x >> sh);
        scale[1] = d * (float)(int)(int8_t)(r.sc.y >> sh);
    }
    if (!packed_done) {
#pragma unroll
        for (int g = 0; g < 2; g++) {
            frag[g][0] = bf16x8_of(f[g]);
            frag[g][1] = bf16x8_of(f[g] + 8);
        }
    }
}

// LDS of one pipeline stage: the split activations of one step of 32 columns for the
// workgroup's tokens (the weights never pass through LDS).
template <uint32_t T, int TT> struct MmStage {
    static constexpr bool OFFSET = MmTraits<T>::OFFSET;
    static constexpr int TOK = 32 * TT;
    static constexpr int XB_VEC = 12 * TOK;                             // [group][part][half][token] x 16 bytes
    static constexpr int XB_SLOTS = (XB_VEC + 255) / 256 * 256;        // every thread stores whole vectors, no tail branch
    static constexpr size_t XB = 0;
    static constexpr size_t SX = XB + (size_t)XB_SLOTS * 16;            // float [2][TOK], padded to one per thread
    static constexpr size_t BYTES = SX + (OFFSET ? (size_t)256 * 4 : 0);
};

// Lanes l and l + 32 exchange: a[l + 32] <-> b[l] (v_permlane32_swap).  Afterwards a holds, in
// both halves of the wavefront, what the lower half had (a's old lower half, b's old lower
// half) and b what the upper half had.
__device__ __forceinline__ void swap32(uint32_t &a, uint32_t &b) {
    const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    a = r[0];
    b = r[1];
}

// TT: token tiles of 32 per workgroup.  VQ: how many of a tile's four 8-token quads can hold
// tokens (a lane's accumulator v belongs to quad v / 4); the others are neither scaled nor stored.
// FB: nibble bytes go straight to bf16 with the packed fp8 convert (Q4_K, when the device probe allows).
//
// A wavefront owns 64 rows and decodes them itself, one row per lane: 16 codes per group as
// two halves of 8 bf16.  The MFMA wants, for the 32 rows of a row set, the first halves in
// lanes 0..31 and the second halves in lanes 32..63 - one v_permlane32_swap per register gives
// exactly that for both row sets at once (lower half: rows 0..31's first halves and rows
// 32..63's first halves; upper half: the second halves), so the weights never touch LDS and
// no barrier stands between a wavefront's decode and its MFMAs.  Only the split activations,
// which all four wavefronts read, go through LDS (two stages, one barrier per step).
template <uint32_t T, int TT, int VQ, bool FB>
__global__ __launch_bounds__(256, 2) void gemm_mfma_kernel(const MmBatch b) {
    constexpr int NV = 4 * VQ;
    using St = MmStage<T, TT>;
    constexpr bool OFFSET = St::OFFSET;
    constexpr bool SAME_SCALE = MmTraits<T>::SAME_SCALE;
    constexpr int TOK = St::TOK;
    constexpr int XR = (St::XB_VEC + 255) / 256;  // activation vectors each thread stages per step
    extern __shared__ __align__(16) uint8_t mm_lds[];

    uint32_t j = 0;
    for (uint32_t k = 1; k < b.n_jobs; k++)
        if (blockIdx.x >= b.job[k].wg_begin) j = k;
    const MmJob &job = b.job[j];
    const MatView &m = job.m;
    uint32_t local = blockIdx.x - job.wg_begin;
    const uint32_t ks = local % job.ksplit;
    local /= job.ksplit;
    const uint32_t tile_t = local % job.tok_tiles, tile_r = local / job.tok_tiles;

    // column shares are cut at multiples of 8 steps (a 256-column super-block)
    const uint32_t n_units = m.cols / 256;
    const uint32_t n_steps = m.cols / 32;
    const uint32_t s_begin = n_units ? 8 * (uint32_t)((uint64_t)n_units * ks / job.ksplit) : 0;
    const uint32_t s_end = n_units && ks + 1 < job.ksplit ? 8 * (uint32_t)((uint64_t)n_units * (ks + 1) / job.ksplit) : n_steps;

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t n = lane & 31u, kh = lane >> 5;
    const uint32_t row0 = tile_r * MM_ROWS;
    const uint32_t tok0 = tile_t * TOK;             // first token of the tile within the job
    const uint32_t slot0 = job.tok_off + tok0;      // same, as a slot of the split activations
    const size_t mpad = b.mpad;

    f32x16 acc[2][TT];
#pragma unroll
    for (int rs = 0; rs < 2; rs++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[rs][tt][v] = 0.f;

    // Global data of the next DEPTH steps, in registers while earlier steps compute: one
    // step of one workgroup is only a few KB, far too little to cover HBM latency.  The
    // 64-token tile has no registers to spare for four slots, and needs them less: its
    // steps take twice as long.
    constexpr int DEPTH = TT == 1 ? 4 : 2;
    // (named variables, not arrays: the ring must stay in registers)
    MmRaw<T> raw0, raw1, raw2, raw3;
    struct XbRegs { uint4 v0, v1, v2; };  // XR <= 3 vectors, as named members
    XbRegs xb0, xb1, xb2, xb3;
    static_assert(XR <= 3, "XbRegs holds three vectors");
    float sx0 = 0.f, sx1 = 0.f, sx2 = 0.f, sx3 = 0.f;

    // Every fetch issues the same loads whatever the step and the thread (indices
    // are clamped instead of branching), so that the number of loads in flight is
    // known at compile time and a wait for the oldest step does not wait for all.
    auto fetch_w = [&](uint32_t s_want, MmRaw<T> &raw) {
        const uint32_t s = s_want < s_end ? s_want : s_end - 1;
        mm_load<T>(m, tile_r, tid, s, raw);
    };
    // Offsets are applied once per 32 columns that share them: Q5_1 every step (one block),
    // Q4_K on even steps (a sub-block spans the same group of two consecutive steps).
    auto fetch_x = [&](uint32_t s_want, XbRegs &xbr, float &sxr) {
        const uint32_t s = s_want < s_end ? s_want : s_end - 1;
        const uint4 *src = b.xb + (size_t)s * 12 * mpad + slot0;
#pragma unroll
        for (int r = 0; r < XR; r++) {
            uint32_t v = tid + 256 * r;
            if (XR * 256 != St::XB_VEC) v = v < (uint32_t)St::XB_VEC ? v : (uint32_t)St::XB_VEC - 1;
            const uint4 val = src[(size_t)(v / TOK) * mpad + v % TOK];
            if (r == 0) xbr.v0 = val;
            if (r == 1) xbr.v1 = val;
            if (r == 2) xbr.v2 = val;
        }
        if constexpr (OFFSET) {
            const uint32_t g = (tid / TOK) & 1u, i = tid % TOK;
            const uint32_t se = T == T_Q5_1 ? s : s & ~1u;  // Q4_K: the pair of steps of one sub-block
            const size_t g0 = T == T_Q5_1 ? (size_t)2 * se : (size_t)2 * se + g;
            const size_t g1 = T == T_Q5_1 ? g0 + 1 : g0 + 2;
            sxr = b.sx[g0 * mpad + slot0 + i] + b.sx[g1 * mpad + slot0 + i];
        }
    };
    auto stage_x = [&](uint32_t buf, const XbRegs &xbr, const float &sxr) {
        uint8_t *st = mm_lds + (size_t)buf * St::BYTES;
        uint4 *xb_s = reinterpret_cast<uint4 *>(st + St::XB);
#pragma unroll
        for (int r = 0; r < XR; r++) {
            const uint32_t v = tid + 256 * r;
            xb_s[v] = r == 0 ? xbr.v0 : r == 1 ? xbr.v1 : xbr.v2;  // slots past XB_VEC are padding
        }
        if constexpr (OFFSET) reinterpret_cast<float *>(st + St::SX)[tid] = sxr;  // read on offset steps, entries [0, 2 TOK)
    };
    // even_step: s is even (known at compile time: shares of K-quant rows start at a multiple of 8 steps)
    auto compute = [&](uint32_t s, uint32_t buf, const MmRaw<T> &raw, auto even_step) {
        constexpr bool with_offset = OFFSET && (T == T_Q5_1 || decltype(even_step)::value);
        const uint8_t *st = mm_lds + (size_t)buf * St::BYTES;
        const uint4 *xb_s = reinterpret_cast<const uint4 *>(st + St::XB);
        const float *sx_s = reinterpret_cast<const float *>(st + St::SX);
        // this lane's row: 16 codes per group as two halves, scale and offset
        uint4 frag[2][2];
        float scr[2], ofr[2];
        mm_decode<T, FB>(raw, s, frag, scr, ofr);
        bf16x8 wf[2][2];
        float sc[2][2], of[2][2];
#pragma unroll
        for (int g = 0; g < 2; g++) {
            uint4 lo = frag[g][0], hi = frag[g][1];
            swap32(lo.x, hi.x);
            swap32(lo.y, hi.y);
            swap32(lo.z, hi.z);
            swap32(lo.w, hi.w);
            wf[g][0] = __builtin_bit_cast(bf16x8, lo);  // rows 0..31 of the wavefront's 64: halves by lane / 32
            wf[g][1] = __builtin_bit_cast(bf16x8, hi);  // rows 32..63
            uint32_t s0 = __float_as_uint(scr[g]), s1 = s0;
            swap32(s0, s1);
            sc[g][0] = __uint_as_float(s0);
            sc[g][1] = __uint_as_float(s1);
            if constexpr (OFFSET) {
                uint32_t o0 = __float_as_uint(ofr[g]), o1 = o0;
                swap32(o0, o1);
                of[g][0] = __uint_as_float(o0);
                of[g][1] = __uint_as_float(o1);
            } else {
                of[g][0] = of[g][1] = 0.f;
            }
        }
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
            // one token tile at a time: interleaving the tiles only lengthens live ranges
            if (tt > 0) __builtin_amdgcn_sched_barrier(0);
            bf16x8 xf[2][3];
#pragma unroll
            for (int g = 0; g < 2; g++)
#pragma unroll
                for (int p = 0; p < 3; p++)
                    xf[g][p] = __builtin_bit_cast(bf16x8, xb_s[(g * 6 + 2 * p + kh) * TOK + tt * 32 + n]);
            // sxv: sums of activations (over the 32 columns an offset covers) of the lane's 16 token rows
            auto load_sx = [&](int g, float (&sxv)[16]) {
#pragma unroll
                for (int q = 0; q < VQ; q++) {
                    const float4 t4 = *reinterpret_cast<const float4 *>(sx_s + g * TOK + tt * 32 + 8 * q + 4 * kh);
                    sxv[4 * q] = t4.x; sxv[4 * q + 1] = t4.y; sxv[4 * q + 2] = t4.z; sxv[4 * q + 3] = t4.w;
                }
            };
            if constexpr (SAME_SCALE) {
                float sxv[16];
                if constexpr (with_offset) load_sx(0, sxv);
#pragma unroll
                for (int rs = 0; rs < 2; rs++) {
                    f32x16 p;
#pragma unroll
                    for (int v = 0; v < 16; v++) p[v] = 0.f;
#pragma unroll
                    for (int g = 0; g < 2; g++) {
                        p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xf[g][2], wf[g][rs], p, 0, 0, 0);
                        p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xf[g][1], wf[g][rs], p, 0, 0, 0);
                        p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xf[g][0], wf[g][rs], p, 0, 0, 0);
                    }
#pragma unroll
                    for (int v = 0; v < NV; v++) acc[rs][tt][v] = fmaf(sc[0][rs], p[v], acc[rs][tt][v]);
                    if constexpr (with_offset) {
#pragma unroll
                        for (int v = 0; v < NV; v++) acc[rs][tt][v] = fmaf(of[0][rs], sxv[v], acc[rs][tt][v]);
                    }
                }
            } else {
#pragma unroll
                for (int g = 0; g < 2; g++) {
                    float sxv[16];
                    if constexpr (with_offset) load_sx(g, sxv);
#pragma unroll
                    for (int rs = 0; rs < 2; rs++) {
                        f32x16 p;
#pragma unroll
                        for (int v = 0; v < 16; v++) p[v] = 0.f;
                        p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xf[g][2], wf[g][rs], p, 0, 0, 0);
                        p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xf[g][1], wf[g][rs], p, 0, 0, 0);
                        p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xf[g][0], wf[g][rs], p, 0, 0, 0);
#pragma unroll
                        for (int v = 0; v < NV; v++) acc[rs][tt][v] = fmaf(sc[g][rs], p[v], acc[rs][tt][v]);
                        if constexpr (with_offset) {
#pragma unroll
                            for (int v = 0; v < NV; v++) acc[rs][tt][v] = fmaf(of[g][rs], sxv[v], acc[rs][tt][v]);
                        }
                    }
                }
            }
        }
    };

    if (s_begin < s_end) {
        // No branch inside a step: the compiler then knows how many loads are in flight and
        // waits only for the oldest ring slot.  Step s reads its activations from LDS stage
        // (s - s_begin) & 1; those of step s + 1 are written to the other stage meanwhile.
#define NH_MM_STEP(d, RAW, XBN, SXN)                                                          \
    {                                                                                          \
        stage_x((d + 1) & 1, XBN, SXN);                                                        \
        fetch_x(base + d + 1 + DEPTH, XBN, SXN);                                               \
        const MmRaw<T> cur = RAW;                                                              \
        fetch_w(base + d + DEPTH, RAW);                                                        \
        __builtin_amdgcn_sched_barrier(0);                                                     \
        compute(base + d, d & 1, cur, std::integral_constant<bool, ((d) & 1) == 0>{});         \
        __builtin_amdgcn_sched_barrier(0);                                                     \
        __syncthreads();                                                                       \
    }
        uint32_t base = s_begin;
        if constexpr (DEPTH == 4) {
            fetch_w(s_begin, raw0);
            fetch_w(s_begin + 1, raw1);
            fetch_w(s_begin + 2, raw2);
            fetch_w(s_begin + 3, raw3);
            fetch_x(s_begin, xb0, sx0);
            fetch_x(s_begin + 1, xb1, sx1);
            fetch_x(s_begin + 2, xb2, sx2);
            fetch_x(s_begin + 3, xb3, sx3);
            stage_x(0, xb0, sx0);
            fetch_x(s_begin + 4, xb0, sx0);
            __syncthreads();
            for (; base + 4 <= s_end; base += 4) {
                NH_MM_STEP(0, raw0, xb1, sx1)
                NH_MM_STEP(1, raw1, xb2, sx2)
                NH_MM_STEP(2, raw2, xb3, sx3)
                NH_MM_STEP(3, raw3, xb0, sx0)
            }
            // at most three steps left (column counts that are not a multiple of 128)
            if (base < s_end) NH_MM_STEP(0, raw0, xb1, sx1)
            if (base + 1 < s_end) NH_MM_STEP(1, raw1, xb2, sx2)
            if (base + 2 < s_end) NH_MM_STEP(2, raw2, xb3, sx3)
        } else {
            fetch_w(s_begin, raw0);
            fetch_w(s_begin + 1, raw1);
            fetch_x(s_begin, xb0, sx0);
            fetch_x(s_begin + 1, xb1, sx1);
            stage_x(0, xb0, sx0);
            fetch_x(s_begin + 2, xb0, sx0);
            __syncthreads();
            for (; base + 2 <= s_end; base += 2) {
                NH_MM_STEP(0, raw0, xb1, sx1)
                NH_MM_STEP(1, raw1, xb0, sx0)
            }
            if (base < s_end) NH_MM_STEP(0, raw0, xb1, sx1)
        }
#undef NH_MM_STEP
    }

    // D[i][j]: lane holds weight row j = lane % 32 and token rows i = 8 (v / 4) + 4 (lane / 32) + v % 4.
    float *out = job.ksplit > 1 ? job.part + (size_t)ks * job.tokens * m.rows : job.y;
#pragma unroll
    for (int rs = 0; rs < 2; rs++) {
        const uint32_t row = row0 + wave * 64 + rs * 32 + n;
        if (row >= m.rows) continue;
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int v = 0; v < NV; v++) {
                const uint32_t t = tok0 + tt * 32 + 8 * (v >> 2) + 4 * kh + (v & 3);
                if (t < job.tokens) out[(size_t)t * m.rows + row] = acc[rs][tt][v];
            }
    }
}

// y = sum over the column shares, in share order.  The loads of one element's
// shares are independent and issued eight at a time; the additions keep the order.
template <typename V> __device__ __forceinline__ V mm_add(V a, V b);
template <> __device__ __forceinline__ float mm_add<float>(float a, float b) { return a + b; }
template <> __device__ __forceinline__ float4 mm_add<float4>(float4 a, float4 b) {
    return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}
template <typename V>
__device__ __forceinline__ void mm_reduce_span(const V *part, V *y, size_t total, uint32_t ksplit, size_t first, size_t stride) {
    for (size_t i = first; i < total; i += stride) {
        V s = part[i];
        uint32_t k = 1;
        for (; k + 8 <= ksplit; k += 8) {
            V t[8];
#pragma unroll
            for (int u = 0; u < 8; u++) t[u] = part[(size_t)(k + u) * total + i];
#pragma unroll
            for (int u = 0; u < 8; u++) s = mm_add(s, t[u]);
        }
        for (; k < ksplit; k++) s = mm_add(s, part[(size_t)k * total + i]);
        y[i] = s;
    }
}
__global__ __launch_bounds__(256) void mm_reduce_kernel(const MmBatch b) {
    const MmJob &job = b.job[blockIdx.y];
    if (job.ksplit < 2) return;
    const size_t total = (size_t)job.tokens * job.m.rows;
    const size_t first = (size_t)blockIdx.x * 256 + threadIdx.x, stride = (size_t)gridDim.x * 256;
    if ((total & 3) == 0 && (reinterpret_cast<uintptr_t>(job.y) & 15) == 0)
        mm_reduce_span(reinterpret_cast<const float4 *>(job.part), reinterpret_cast<float4 *>(job.y), total / 4, job.ksplit,
                       first, stride);
    else
        mm_reduce_span(job.part, job.y, total, job.ksplit, first, stride);
}

// ------------------------------------------------------------------ launchers

static bool g_nibble_bf16 = false;  // the packed fp8 -> bf16 convert turns nibble bytes into the integers 0..15
static bool g_nibble_i4 = false;    // the signed 4-bit convert with a byte select gives (n - 8) / 16 for nibble n ^ 8
static int g_cu_count = 256;
static size_t g_lds_limit = 64 * 1024;

void set_device_limits(int cu_count, size_t lds_per_block) {
    if (cu_count > 0) g_cu_count = cu_count;
    if (lds_per_block > 0) g_lds_limit = lds_per_block;
}

// Jobs must share x, dtype and column count.  hipErrorInvalidValue = "does not fit this
// kernel" (x too long for LDS); the caller then uses the tiled kernel.
template <uint32_t T, int R>
static hipError_t launch_gemv_t(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n_jobs,
                                const float *x) {
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
    b.unit0 = b.units = b.accumulate = b.pad = 0;  // column windows are a lane-per-unit matter
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

hipError_t probe_fp8_nibble_unit(hipStream_t stream, float *unit_out) {
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
    g_nibble_bf16 = exact;
    exact = true;
    for (int n = 0; n < 16; n++)
        for (int k = 0; k < 8; k++) exact = exact && h[128 + 8 * n + k] == (float)(n - 8) / 16.0f;
    g_nibble_i4 = exact;
    return hipSuccess;
}

static float g_nib_mul = 0.f;  // 1 / (value of fp8 byte 0x01); 0 = fp8 unpack not usable
void set_fp8_nibble_unit(float unit) { g_nib_mul = unit > 0.f ? 1.0f / unit : 0.f; }

template <int LB, int NW, int PL>
static hipError_t launch_q4k_lb(hipStream_t stream, const GemvBatch &b, uint32_t units, size_t lds) {
    const bool fp8 = g_nib_mul != 0.f;
    const void *kern = fp8 ? reinterpret_cast<const void *>(gemv_q4k_kernel<LB, NW, true, PL>)
                           : reinterpret_cast<const void *>(gemv_q4k_kernel<LB, NW, false, PL>);
    static size_t configured[2] = {0, 0};
    if (lds > 48 * 1024 && lds > configured[fp8]) {
        hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)g_lds_limit);
        if (e != hipSuccess) return e;
        configured[fp8] = g_lds_limit;
    }
    size_t per_cu = g_lds_limit * 2 / (lds ? lds : 1);  // 160 KB of LDS per CU
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 16 / NW) per_cu = 16 / NW;             // 16 wavefronts per CU
    uint32_t grid = (uint32_t)((size_t)g_cu_count * per_cu);
    const uint32_t needed = (units + NW - 1) / NW;
    if (grid > needed) grid = needed;
    const float mul = fp8 ? g_nib_mul : 1.0f;
    if (fp8)
        hipLaunchKernelGGL((gemv_q4k_kernel<LB, NW, true, PL>), dim3(grid), dim3(NW * 64), lds, stream, b, mul);
    else
        hipLaunchKernelGGL((gemv_q4k_kernel<LB, NW, false, PL>), dim3(grid), dim3(NW * 64), lds, stream, b, mul);
    return hipGetLastError();
}

// Jobs of a lane-per-unit launch: lb lanes per row, 64 / lb rows per wavefront step.
static uint32_t fill_unit_jobs(GemvBatch &b, const MatView *mats, float *const *ys, uint32_t n_jobs, const float *x,
                               uint32_t lb) {
    const uint32_t rg_rows = 64 / lb;
    b.x = x;
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

static hipError_t launch_gemv_q4k(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n_jobs,
                                  const float *x) {
    const uint32_t nb = mats[0].nb;
    // one lane per super-block, at most 64 per row and launch: longer rows take several launches
    const UnitWindows win(nb, 64);
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
        b.accumulate = w > 0;
        const size_t lds = (size_t)(64 * (lbb * 4 + 4) + lbb * 8) * sizeof(float);
        if (lds > g_lds_limit) return hipErrorInvalidValue;
        hipError_t e;
        if (halves) {
            switch (lb) {
            case 2: e = launch_q4k_lb<2, 4, 4>(stream, b, rgs, lds); break;
            case 4: e = launch_q4k_lb<4, 4, 4>(stream, b, rgs, lds); break;
            case 8: e = launch_q4k_lb<8, 4, 4>(stream, b, rgs, lds); break;
            case 16: e = launch_q4k_lb<16, 4, 4>(stream, b, rgs, lds); break;
            default: e = launch_q4k_lb<32, 4, 4>(stream, b, rgs, lds); break;
            }
        } else {
            switch (lb) {
            // Short rows: small workgroups, so that even a 1024-row matrix spreads over every CU.
            case 1: e = launch_q4k_lb<1, 4, 8>(stream, b, rgs, lds); break;
            case 2: e = launch_q4k_lb<2, 4, 8>(stream, b, rgs, lds); break;
            case 4: e = launch_q4k_lb<4, 4, 8>(stream, b, rgs, lds); break;
            case 8: e = launch_q4k_lb<8, 4, 8>(stream, b, rgs, lds); break;
            case 16: e = launch_q4k_lb<16, 4, 8>(stream, b, rgs, lds); break;
            case 32: e = launch_q4k_lb<32, 8, 8>(stream, b, rgs, lds); break;
            default: e = launch_q4k_lb<64, 8, 8>(stream, b, rgs, lds); break;
            }
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
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
    if (per_cu > 16 / NW) per_cu = 16 / NW;
    uint32_t grid = (uint32_t)((size_t)g_cu_count * per_cu);
    const uint32_t needed = (units + NW - 1) / NW;
    if (grid > needed) grid = needed;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, stream, b);
    return hipGetLastError();
}

static hipError_t launch_gemv_q6k(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n_jobs,
                                  const float *x) {
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
        b.accumulate = w > 0;
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
        default: e = launch_q6k_lb<64, 8>(stream, b, rgs, lds); break;
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
    if (per_cu > 16 / NW) per_cu = 16 / NW;             // 16 wavefronts per CU
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
                                  const float *x) {
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
        b.accumulate = w > 0;
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
        default: e = launch_b32_lb<T, 64, 8>(stream, b, rgs, lds); break;
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
static hipError_t launch_multi_t(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n, const float *x) {
    if constexpr (T == T_Q4_K) return launch_gemv_q4k(stream, mats, ys, n, x);
    if constexpr (T == T_Q6_K) return launch_gemv_q6k(stream, mats, ys, n, x);
    if constexpr (T == T_Q8_0 || T == T_Q4_0 || T == T_Q5_0 || T == T_Q5_1) {
        hipError_t e = launch_gemv_b32<T>(stream, mats, ys, n, x);
        if (e != hipErrorInvalidValue) return e;
        (void)hipGetLastError();
    }
    // Rows per lane: four share the lane's activations, but a wavefront owns whole row groups, so
    // matrices with few rows take fewer rows per group to give every wavefront of the chip one.
    size_t rows = 0;
    for (uint32_t j = 0; j < n; j++) rows += mats[j].rows;
    const size_t wavefronts = (size_t)g_cu_count * 16;
    if (rows >= 4 * wavefronts) return launch_gemv_t<T, 4>(stream, mats, ys, n, x);
    if (rows >= 2 * wavefronts) return launch_gemv_t<T, 2>(stream, mats, ys, n, x);
    return launch_gemv_t<T, 1>(stream, mats, ys, n, x);
}

// ---- MFMA GEMM: planning and launch

static bool mm_type(uint32_t type) { return type != T_F32 && type != T_F16 && type_supported(type); }

struct MmPlan {
    MmBatch b;
    int tt;             // token tiles of 32 per workgroup (1 or 2)
    uint32_t max_tok;   // most tokens of any job
    uint32_t n_groups;  // groups of 16 columns
    size_t xb_bytes, sx_bytes, part_bytes;
};

static size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }

// Jobs share dtype and column count; every job has at least two tokens.
static void mm_plan(const MatView *mats, const uint32_t *tokens, const float *const *xs, float *const *ys, uint32_t n,
                    MmPlan &p) {
    MmBatch &b = p.b;
    uint32_t max_tok = 0, total_tok = 0;
    for (uint32_t j = 0; j < n; j++) max_tok = tokens[j] > max_tok ? tokens[j] : max_tok;
    p.tt = max_tok > 32 ? 2 : 1;
    p.max_tok = max_tok;
    const uint32_t tile_tok = 32u * (uint32_t)p.tt;
    uint32_t wgs = 0;
    bool any_split = false;
    const uint32_t n_steps = mats[0].cols / 32;
    // Columns are shared between workgroups only as far as the row and token tiles of the whole
    // launch leave CUs idle: every share costs a partial result written and read back.
    uint32_t launch_tiles = 0;
    for (uint32_t j = 0; j < n; j++)
        launch_tiles += ((tokens[j] + tile_tok - 1) / tile_tok) * ((mats[j].rows + MM_ROWS - 1) / MM_ROWS);
    uint32_t ks_launch = (uint32_t)(2 * g_cu_count) / (launch_tiles ? launch_tiles : 1);  // two workgroups per CU (measured best of 1..4)
    if (ks_launch > n_steps / 8) ks_launch = n_steps / 8;                                 // shares are whole 256-column units
    if (ks_launch > 32) ks_launch = 32;
    if (ks_launch < 1) ks_launch = 1;
    for (uint32_t j = 0; j < n; j++) {
        MmJob &job = b.job[j];
        job.m = mats[j];
        job.x = xs ? xs[j] : nullptr;
        job.y = ys ? ys[j] : nullptr;
        job.part = nullptr;
        job.tokens = tokens[j];
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
    b.mpad = total_tok + 64;  // a tile may read up to 63 slots past its job's last token
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

template <uint32_t T, int TT, int VQ, bool FB = false>
static hipError_t launch_mm_main(hipStream_t stream, const MmBatch &b) {
    if constexpr (T == T_Q4_K && !FB) {
        if (b.nibble_bf16) return launch_mm_main<T, TT, VQ, true>(stream, b);
    }
    constexpr size_t lds = 2 * MmStage<T, TT>::BYTES;  // two pipeline stages
    auto kern = gemm_mfma_kernel<T, TT, VQ, FB>;
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
    const size_t split_threads = (size_t)p.n_groups * b.mpad;
    hipLaunchKernelGGL(mm_xsplit_kernel<T>, dim3((unsigned)((split_threads + 255) / 256)), dim3(256), 0, stream, b,
                       p.n_groups);
    hipError_t e;
    if (p.tt == 2) e = launch_mm_main<T, 2, 4>(stream, b);
    else if (p.max_tok <= 8) e = launch_mm_main<T, 1, 1>(stream, b);
    else if (p.max_tok <= 16) e = launch_mm_main<T, 1, 2>(stream, b);
    else if (p.max_tok <= 24) e = launch_mm_main<T, 1, 3>(stream, b);
    else e = launch_mm_main<T, 1, 4>(stream, b);
    if (e != hipSuccess) return e;
    if (b.any_split) hipLaunchKernelGGL(mm_reduce_kernel, dim3(512, b.n_jobs), dim3(256), 0, stream, b);
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

// Single-token products, and F32/F16 products of any token count.
static hipError_t launch_plain(hipStream_t stream, const MatView &m, uint32_t tokens, const float *x, float *y) {
    auto run = [&](auto tag) -> hipError_t {
        constexpr uint32_t T = decltype(tag)::value;
        if (tokens == 1) {
            hipError_t e = launch_multi_t<T>(stream, &m, &y, 1, x);
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
static uint32_t mm_run(const MatView *mats, const uint32_t *tokens, uint32_t n, uint32_t g) {
    if (!mm_type(mats[g].type) || tokens[g] < 2) return 0;
    uint32_t run = 1;
    while (g + run < n && run < (uint32_t)MM_MAX_JOBS && tokens[g + run] >= 2 && mats[g + run].type == mats[g].type &&
           mats[g + run].cols == mats[g].cols)
        run++;
    return run;
}

size_t gemm_workspace_bytes(const MatView *mats, const uint32_t *tokens, uint32_t n) {
    size_t need = 0;
    for (uint32_t g = 0; g < n;) {
        if (tokens[g] == 0 || mats[g].rows == 0) { g++; continue; }
        const uint32_t run = mm_run(mats, tokens, n, g);
        if (run == 0) { g++; continue; }
        MmPlan p;
        mm_plan(mats + g, tokens + g, nullptr, nullptr, run, p);
        const size_t bytes = p.xb_bytes + p.sx_bytes + p.part_bytes;
        need = bytes > need ? bytes : need;
        g += run;
    }
    return need;
}

hipError_t launch_gemm_groups(hipStream_t stream, const MatView *mats, const MatView *tiled, const uint32_t *tokens,
                              const float *const *xs, float *const *ys, uint32_t n, void *ws, size_t ws_bytes) {
    for (uint32_t g = 0; g < n;) {
        if (tokens[g] == 0 || mats[g].rows == 0) { g++; continue; }
        const uint32_t run = mm_run(mats, tokens, n, g);
        hipError_t e;
        if (run == 0) {
            e = launch_plain(stream, mats[g], tokens[g], xs[g], ys[g]);
            g++;
        } else {
            MmPlan p;
            mm_plan(tiled + g, tokens + g, xs + g, ys + g, run, p);
            e = launch_mm(stream, p, ws, ws_bytes);
            g += run;
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
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

hipError_t launch_gemv_multi(hipStream_t stream, const MatView *mats, float *const *ys, uint32_t n, const float *x) {
    if (n == 0) return hipSuccess;
    if (n > GEMV_MAX_JOBS) return hipErrorInvalidValue;
    for (uint32_t j = 0; j < n; j++)
        if (mats[j].type != mats[0].type || mats[j].cols != mats[0].cols || mats[j].rows == 0) return hipErrorInvalidValue;
    switch (mats[0].type) {
    case T_F32: return launch_multi_t<T_F32>(stream, mats, ys, n, x);
    case T_F16: return launch_multi_t<T_F16>(stream, mats, ys, n, x);
    case T_Q4_0: return launch_multi_t<T_Q4_0>(stream, mats, ys, n, x);
    case T_Q5_0: return launch_multi_t<T_Q5_0>(stream, mats, ys, n, x);
    case T_Q5_1: return launch_multi_t<T_Q5_1>(stream, mats, ys, n, x);
    case T_Q8_0: return launch_multi_t<T_Q8_0>(stream, mats, ys, n, x);
    case T_Q4_K: return launch_multi_t<T_Q4_K>(stream, mats, ys, n, x);
    case T_Q6_K: return launch_multi_t<T_Q6_K>(stream, mats, ys, n, x);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gemm(hipStream_t stream, const MatView &m, const MatView &tiled, uint32_t tokens, const float *x,
                       float *y, void *ws, size_t ws_bytes) {
    return launch_gemm_groups(stream, &m, &tiled, &tokens, &x, &y, 1, ws, ws_bytes);
}

}  // namespace nh
