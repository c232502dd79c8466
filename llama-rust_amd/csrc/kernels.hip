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
    switch (v.type) {
    case T_Q8_0: {
        const uint8_t *s = src + r * src_row_bytes + b * 34;
        uint8_t *d = v.p1 + r * v.s1 + b * 2;
        d[0] = s[0];
        d[1] = s[1];
        uint8_t *q = v.p0 + r * v.s0 + b * 32;
        for (int i = 0; i < 32; i++) q[i] = s[2 + i];
        break;
    }
    case T_Q4_0: {
        const uint8_t *s = src + r * src_row_bytes + b * 18;
        uint8_t *d = v.p1 + r * v.s1 + b * 2;
        d[0] = s[0];
        d[1] = s[1];
        uint8_t *q = v.p0 + r * v.s0 + b * 16;
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
        uint8_t *q = v.p0 + r * v.s0 + b * 16;
        for (int i = 0; i < 16; i++) q[i] = s[6 + i];
        break;
    }
    case T_Q5_1: {
        const uint8_t *s = src + r * src_row_bytes + b * 24;
        uint8_t *d = v.p2 + r * v.s2 + b * 4;
        for (int i = 0; i < 4; i++) d[i] = s[i];
        uint8_t *h = v.p1 + r * v.s1 + b * 4;
        for (int i = 0; i < 4; i++) h[i] = s[4 + i];
        uint8_t *q = v.p0 + r * v.s0 + b * 16;
        for (int i = 0; i < 16; i++) q[i] = s[8 + i];
        break;
    }
    case T_Q4_K: {
        const uint8_t *s = src + r * src_row_bytes + b * 144;
        uint8_t *h = v.p1 + r * v.s1 + b * 16;
        for (int i = 0; i < 16; i++) h[i] = s[i];
        uint8_t *q = v.p0 + r * v.s0 + b * 128;
        for (int i = 0; i < 128; i++) q[i] = s[16 + i];
        break;
    }
    case T_Q6_K: {
        const uint8_t *s = src + r * src_row_bytes + b * 210;
        uint8_t *ql = v.p0 + r * v.s0 + b * 128;
        for (int i = 0; i < 128; i++) ql[i] = s[i];
        uint8_t *qh = v.p1 + r * v.s1 + b * 64;
        for (int i = 0; i < 64; i++) qh[i] = s[128 + i];
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
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + (size_t)c * 16);
        r.d = *reinterpret_cast<const uint16_t *>(m.p1 + ro * m.s1 + (size_t)(c >> 1) * 2);
    } else if constexpr (T == T_Q4_0) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + (size_t)c * 16);
        r.d = *reinterpret_cast<const uint16_t *>(m.p1 + ro * m.s1 + (size_t)c * 2);
    } else if constexpr (T == T_Q5_0) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + (size_t)c * 16);
        r.qh = *reinterpret_cast<const uint32_t *>(m.p1 + ro * m.s1 + (size_t)c * 4);
        r.d = *reinterpret_cast<const uint16_t *>(m.p2 + ro * m.s2 + (size_t)c * 2);
    } else if constexpr (T == T_Q5_1) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + (size_t)c * 16);
        r.qh = *reinterpret_cast<const uint32_t *>(m.p1 + ro * m.s1 + (size_t)c * 4);
        r.dm = *reinterpret_cast<const uint32_t *>(m.p2 + ro * m.s2 + (size_t)c * 4);
    } else if constexpr (T == T_Q4_K) {
        r.q = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + (size_t)c * 16);
        r.hdr = *reinterpret_cast<const uint4 *>(m.p1 + ro * m.s1 + (size_t)(c >> 3) * 16);
    } else if constexpr (T == T_Q6_K) {
        uint32_t blk = c >> 3, cc = c & 7, n = cc >> 2, k = cc & 1;
        r.ql = *reinterpret_cast<const uint4 *>(m.p0 + ro * m.s0 + (size_t)c * 16);
        r.qh = *reinterpret_cast<const uint4 *>(m.p1 + ro * m.s1 + (size_t)blk * 64 + n * 32 + k * 16);
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
            t = dot4_ub(w[i] & 0x0f0f0f0fu, x + 4 * i, t);
            t = dot4_ub((w[i] >> 4) & 0x0f0f0f0fu, x + 16 + 4 * i, t);
        }
        // sum (n - 8) x = sum n x - 8 sum x
        t = fmaf(-8.f, xc.s_lo + xc.s_hi, t);
        return fmaf(h2f(r.d), t, acc);
    } else if constexpr (T == T_Q5_0 || T == T_Q5_1) {
        const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            t = dot4_ub(q5_bytes(w[i] & 0x0f0f0f0fu, r.qh, 4 * i), x + 4 * i, t);
            t = dot4_ub(q5_bytes((w[i] >> 4) & 0x0f0f0f0fu, r.qh, 16 + 4 * i), x + 16 + 4 * i, t);
        }
        if constexpr (T == T_Q5_0) {
            t = fmaf(-16.f, xc.s_lo + xc.s_hi, t);
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
            tl = dot4_ub((lo[i] & 0x0f0f0f0fu) | (two_lo << 4), x + 4 * i, tl);
            th = dot4_ub(((lo[i] >> 4) & 0x0f0f0f0fu) | (two_hi << 4), x + 16 + 4 * i, th);
        }
        // codes are biased by 32: sum (q - 32) x = sum q x - 32 sum x
        tl = fmaf(-32.f, xc.s_lo, tl);
        th = fmaf(-32.f, xc.s_hi, th);
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
// One workgroup of NW wavefronts stages x in LDS once, then walks row tiles.
// Inside a tile, KW wavefronts split the columns of the same R rows (step s of
// the row belongs to wavefront s mod KW), RW = NW / KW such groups sit side by
// side on different rows.  Partial sums of the KW wavefronts meet in LDS and are
// added in a fixed order, so a result never depends on scheduling.

template <uint32_t T, int R, int NW>
__global__ __launch_bounds__(NW * 64) void gemv_kernel(MatView m, const float *__restrict__ x, float *__restrict__ y,
                                                        uint32_t n_chunks, uint32_t kw_count, uint32_t rw_count,
                                                        uint32_t x_pad) {
    constexpr int E = Geo<T>::E;
    extern __shared__ __align__(16) float lds[];
    float *xs = lds;                 // x_pad floats
    float *part = lds + x_pad;       // rw_count * R * kw_count floats

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    for (uint32_t i = tid; i < x_pad; i += NW * 64) xs[i] = i < m.cols ? x[i] : 0.f;
    __syncthreads();

    const uint32_t kw = wave % kw_count, rw = wave / kw_count;
    const uint32_t tile_rows = rw_count * R;
    const uint32_t n_tiles = (m.rows + tile_rows - 1) / tile_rows;
    const uint32_t n_steps = (n_chunks + 63u) / 64u;

    for (uint32_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const uint32_t row0 = tile * tile_rows + rw * R;
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = 0.f;
        if (rw < rw_count && row0 < m.rows) {
            for (uint32_t s = kw; s < n_steps; s += kw_count) {
                const uint32_t c = s * 64u + lane;
                if (c < n_chunks) {
                    Raw<T> raw[R];
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        uint32_t row = row0 + r < m.rows ? row0 + r : m.rows - 1;
                        load_raw<T>(m, row, c, raw[r]);
                    }
                    XChunk<E> xc;
                    load_x<T>(xs, c, xc);
#pragma unroll
                    for (int r = 0; r < R; r++) acc[r] = chunk_dot<T>(raw[r], xc, c, acc[r]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = wave_sum(acc[r]);
        if (lane == 0 && rw < rw_count) {
#pragma unroll
            for (int r = 0; r < R; r++) part[(rw * R + r) * kw_count + kw] = acc[r];
        }
        __syncthreads();
        if (tid < tile_rows) {
            uint32_t row = tile * tile_rows + tid;
            if (row < m.rows) {
                float s = 0.f;
                for (uint32_t k = 0; k < kw_count; k++) s += part[tid * kw_count + k];
                y[row] = s;
            }
        }
        __syncthreads();
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
        uint2 q = *reinterpret_cast<const uint2 *>(m.p0 + ro * m.s0 + (size_t)b * 32 + j);
        float d = h2f(*reinterpret_cast<const uint16_t *>(m.p1 + ro * m.s1 + (size_t)b * 2));
#pragma unroll
        for (int k = 0; k < 4; k++) {
            w[k] = sb(q.x, k) * d;
            w[4 + k] = sb(q.y, k) * d;
        }
    } else if constexpr (T == T_Q4_0 || T == T_Q5_0 || T == T_Q5_1) {
        // element e = j + i of block b: nibble of byte (e & 15), high nibble when e >= 16
        uint32_t b = k0 >> 5, j = k0 & 31, byte0 = j & 15;
        uint2 q = *reinterpret_cast<const uint2 *>(m.p0 + ro * m.s0 + (size_t)b * 16 + byte0);
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
        uint2 q = *reinterpret_cast<const uint2 *>(m.p0 + ro * m.s0 + (size_t)b * 128 + (sub >> 1) * 32 + l);
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
        uint2 lo = *reinterpret_cast<const uint2 *>(m.p0 + ro * m.s0 + (size_t)b * 128 + n * 64 + (quarter & 1) * 32 + l);
        uint2 hb = *reinterpret_cast<const uint2 *>(m.p1 + ro * m.s1 + (size_t)b * 64 + n * 32 + l);
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

// ------------------------------------------------------------------ launchers

static int g_cu_count = 256;
static size_t g_lds_limit = 64 * 1024;

void set_device_limits(int cu_count, size_t lds_per_block) {
    if (cu_count > 0) g_cu_count = cu_count;
    if (lds_per_block > 0) g_lds_limit = lds_per_block;
}

template <uint32_t T, int R, int NW>
static hipError_t launch_gemv_t(hipStream_t stream, const MatView &m, const float *x, float *y) {
    constexpr int E = Geo<T>::E;
    const uint32_t n_chunks = (m.cols + E - 1) / E;
    const uint32_t n_steps = (n_chunks + 63) / 64;
    uint32_t kw = n_steps < (uint32_t)NW ? n_steps : (uint32_t)NW;
    uint32_t rw = NW / kw;
    const uint32_t x_pad = n_chunks * E;
    const size_t lds = ((size_t)x_pad + (size_t)rw * R * kw) * sizeof(float);
    if (lds > g_lds_limit) return hipErrorInvalidValue;  // caller falls back to the tiled kernel
    auto kern = gemv_kernel<T, R, NW>;
    static size_t configured = 0;  // per instantiation
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)g_lds_limit);
        if (e != hipSuccess) return e;
        configured = g_lds_limit;
    }
    const uint32_t tile_rows = rw * R;
    const uint32_t n_tiles = (m.rows + tile_rows - 1) / tile_rows;
    size_t per_cu = g_lds_limit * 2 / (lds ? lds : 1);  // 160 KB of LDS per CU
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 4) per_cu = 4;
    uint32_t grid = (uint32_t)((size_t)g_cu_count * per_cu);
    if (grid > n_tiles) grid = n_tiles;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, stream, m, x, y, n_chunks, kw, rw, x_pad);
    return hipGetLastError();
}

template <uint32_t T>
static hipError_t launch_tiled_t(hipStream_t stream, const MatView &m, uint32_t tokens, const float *x, float *y) {
    dim3 grid((m.rows + GT_ROWS - 1) / GT_ROWS, (tokens + GT_TOK - 1) / GT_TOK);
    hipLaunchKernelGGL(gemm_tiled_kernel<T>, grid, dim3(256), 0, stream, m, x, y, tokens);
    return hipGetLastError();
}

template <uint32_t T>
static hipError_t launch_t(hipStream_t stream, const MatView &m, uint32_t tokens, const float *x, float *y) {
    if (tokens == 1) {
        hipError_t e = launch_gemv_t<T, 4, 8>(stream, m, x, y);
        if (e != hipErrorInvalidValue) return e;
        (void)hipGetLastError();
    }
    return launch_tiled_t<T>(stream, m, tokens, x, y);
}

hipError_t launch_gemm(hipStream_t stream, const MatView &m, uint32_t tokens, const float *x, float *y) {
    if (m.rows == 0 || tokens == 0) return hipSuccess;
    switch (m.type) {
    case T_F32: return launch_t<T_F32>(stream, m, tokens, x, y);
    case T_F16: return launch_t<T_F16>(stream, m, tokens, x, y);
    case T_Q4_0: return launch_t<T_Q4_0>(stream, m, tokens, x, y);
    case T_Q5_0: return launch_t<T_Q5_0>(stream, m, tokens, x, y);
    case T_Q5_1: return launch_t<T_Q5_1>(stream, m, tokens, x, y);
    case T_Q8_0: return launch_t<T_Q8_0>(stream, m, tokens, x, y);
    case T_Q4_K: return launch_t<T_Q4_K>(stream, m, tokens, x, y);
    case T_Q6_K: return launch_t<T_Q6_K>(stream, m, tokens, x, y);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace nh
