// Device-resident layout of one packed matrix and the per-dtype geometry.
//
// A GGUF tensor arrives as an array of self-contained blocks (scale(s) next to
// the codes they scale; 18/22/24/34/144/210 bytes each, only 2-byte aligned).
// That is the right layout for a CPU that walks one row with one thread, and
// the wrong one for a wavefront: 16-byte lane loads straddle block headers and
// every lane has to pick its codes out of a header/payload mix.  At upload the
// same bits are therefore re-laid into planes (structure of arrays), per row:
//
//   Q8_0 : codes[nb][32]                      | d[nb] f16
//   Q4_0 : codes[nb][16]                      | d[nb] f16
//   Q5_0 : codes[nb][16] | qh[nb] u32         | d[nb] f16
//   Q5_1 : codes[nb][16] | qh[nb] u32         | (d, m)[nb] 2 x f16
//   Q4_K : codes[nb][128]                     | header[nb][16] = d, dmin, scales[12]
//   Q6_K : ql[nb][128] | qh[nb][64] | sc[nb][16] int8 | d[nb] f16
//   F16 / F32 : the row itself, zero-padded to a multiple of 8 elements
//
// Nothing is expanded: the planes hold exactly the bits of the GGUF blocks
// (F16/F32 rows gain at most 7 elements of zero padding) and every code plane
// row starts 16-byte aligned.  One field is permuted inside its 32 bits: the
// fifth bits qh of a Q5 block are stored so that the four bits a code dword
// needs sit at the same bit of its four bytes (repack.inc, q5_permuted), and
// Q5_0's planes hold the complement of that word (its kernel wants the bit
// flipped).
//
// Code planes are stored piece-major.  The single-token kernels give one lane a
// "unit" of a row (a 256-column super-block; 8 consecutive blocks of Q4_0/Q5_x;
// 4 of Q8_0) whose codes are 8 pieces of 16 bytes (4 pieces for Q6_K's qh).
// Piece cc of unit u of a row is stored at slot cc * units_per_row + u, so that
// the lanes of a wavefront, which hold consecutive units and all fetch piece cc
// at the same time, read one contiguous run.  Rows of the 32-column dtypes whose
// length is not a whole number of units keep the block order (piece_major()).
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace nh {

enum : uint32_t {
    T_F32 = 0,
    T_F16 = 1,
    T_Q4_0 = 2,
    T_Q5_0 = 6,
    T_Q5_1 = 7,
    T_Q8_0 = 8,
    T_Q4_K = 12,
    T_Q6_K = 14
};

struct MatView {
    const uint8_t *p0, *p1, *p2, *p3;  // plane base pointers (device)
    uint32_t s0, s1, s2, s3;           // plane row strides in bytes
    uint32_t type, rows, cols, nb;     // nb = blocks per row
};

inline bool type_supported(uint32_t t) {
    return t == T_F32 || t == T_F16 || t == T_Q4_0 || t == T_Q5_0 || t == T_Q5_1 || t == T_Q8_0 ||
           t == T_Q4_K || t == T_Q6_K;
}
inline size_t block_elems(uint32_t t) {
    switch (t) {
    case T_F32:
    case T_F16: return 1;
    case T_Q4_0:
    case T_Q5_0:
    case T_Q5_1:
    case T_Q8_0: return 32;
    case T_Q4_K:
    case T_Q6_K: return 256;
    default: return 0;
    }
}
inline size_t block_bytes(uint32_t t) {
    switch (t) {
    case T_F32: return 4;
    case T_F16: return 2;
    case T_Q4_0: return 18;
    case T_Q5_0: return 22;
    case T_Q5_1: return 24;
    case T_Q8_0: return 34;
    case T_Q4_K: return 144;
    case T_Q6_K: return 210;
    default: return 0;
    }
}
// Bytes of one GGUF row, 0 when cols is not a whole number of blocks or on overflow.
inline size_t gguf_row_bytes(uint32_t t, size_t cols) {
    size_t qk = block_elems(t), bb = block_bytes(t);
    if (qk == 0 || cols % qk != 0) return 0;
    size_t nb = cols / qk;
    if (nb != 0 && bb > SIZE_MAX / nb) return 0;
    return nb * bb;
}

#if defined(__HIPCC__)
#define NH_HD __host__ __device__
#else
#define NH_HD
#endif

// Columns of the unit one lane of the single-token kernels owns.
NH_HD inline uint32_t unit_cols(uint32_t t) { return t == T_Q8_0 ? 128u : 256u; }
// Whether the code plane(s) of a matrix of this dtype and row length are piece-major.
NH_HD inline bool piece_major(uint32_t t, size_t cols) {
    switch (t) {
    case T_Q4_K:
    case T_Q6_K: return true;
    case T_Q4_0:
    case T_Q5_0:
    case T_Q5_1:
    case T_Q8_0: return cols % unit_cols(t) == 0;
    default: return false;
    }
}
// Byte offset, inside a row of a code plane with 8 pieces per unit, of the 16-byte piece that is
// number `piece` of the row in block order.
NH_HD inline size_t piece_offset(bool major, size_t units_per_row, size_t piece) {
    return major ? ((piece & 7) * units_per_row + (piece >> 3)) * 16 : piece * 16;
}

struct PlaneSpec {
    size_t stride[4];  // row strides
    size_t offset[4];  // plane offsets inside the allocation (256-byte aligned)
    size_t total;      // allocation size
};

inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Plane geometry for a rows x cols matrix of type t (cols already validated).
inline PlaneSpec plane_spec(uint32_t t, size_t rows, size_t cols) {
    PlaneSpec s = {};
    size_t nb = cols / block_elems(t);
    switch (t) {
    case T_F32: s.stride[0] = round_up(cols, 8) * 4; break;  // 8-element groups never leave the row
    case T_F16: s.stride[0] = round_up(cols, 8) * 2; break;
    case T_Q8_0: s.stride[0] = nb * 32; s.stride[1] = nb * 2; break;
    case T_Q4_0: s.stride[0] = nb * 16; s.stride[1] = nb * 2; break;
    case T_Q5_0: s.stride[0] = nb * 16; s.stride[1] = nb * 4; s.stride[2] = nb * 2; break;
    case T_Q5_1: s.stride[0] = nb * 16; s.stride[1] = nb * 4; s.stride[2] = nb * 4; break;
    case T_Q4_K: s.stride[0] = nb * 128; s.stride[1] = nb * 16; break;
    case T_Q6_K: s.stride[0] = nb * 128; s.stride[1] = nb * 64; s.stride[2] = nb * 16; s.stride[3] = nb * 2; break;
    default: break;
    }
    size_t off = 0;
    for (int i = 0; i < 4; i++) {
        s.offset[i] = off;
        // 64 bytes of slack after every plane: kernels may issue (masked-out) full-width
        // loads that start inside the last row.
        off = round_up(off + s.stride[i] * rows + 64, 256);
    }
    s.total = off;
    return s;
}

// Second copy of a quantized matrix for products of two or more tokens, where one
// thread decodes one row: rows are interleaved in tiles of 256 so that the 256
// threads of a workgroup, each fetching the same field of its own row, read
// one contiguous run.  Plane k holds units of unit[k] bytes, per_row[k] of them per
// row, unit i of row r at
//     ((r / 256 * per_row[k] + i) * 256 + r % 256) * unit[k].
//
//   Q8_0 : codes 16 B x 2 nb | d 2 B x nb
//   Q4_0 : codes 16 B x nb   | d 2 B x nb
//   Q5_0 : codes 16 B x nb   | qh 4 B x nb | d 2 B x nb
//   Q5_1 : codes 16 B x nb   | qh 4 B x nb | (d, m) 4 B x nb
//   Q4_K : codes 16 B x 8 nb | header 16 B x nb
//   Q6_K : ql 16 B x 8 nb    | qh 16 B x 4 nb | sc 8 B x 2 nb | d 2 B x nb
// (code units in the order of the GGUF block).  F32/F16 have no such copy.
constexpr uint32_t TILE_ROWS = 256;

// Products of at least this many tokens by a quantized matrix run on the matrix cores and read the tiled copy
// (two tokens are two single-token launches).
constexpr uint32_t MM_MIN_TOKENS = 3;
inline bool product_reads_tiled(uint32_t t, uint32_t tokens) {
    return tokens >= MM_MIN_TOKENS && t != T_F32 && t != T_F16 && type_supported(t);
}

struct TiledSpec {
    size_t unit[4], per_row[4];
    size_t offset[4];
    size_t total;  // 0: this dtype has no tiled copy
};

inline TiledSpec tiled_spec(uint32_t t, size_t rows, size_t cols) {
    TiledSpec s = {};
    if (t == T_F32 || t == T_F16 || !type_supported(t)) return s;
    const size_t nb = cols / block_elems(t);
    auto set = [&](int k, size_t unit, size_t per_row) { s.unit[k] = unit; s.per_row[k] = per_row; };
    switch (t) {
    case T_Q8_0: set(0, 16, 2 * nb); set(1, 2, nb); break;
    case T_Q4_0: set(0, 16, nb); set(1, 2, nb); break;
    case T_Q5_0: set(0, 16, nb); set(1, 4, nb); set(2, 2, nb); break;
    case T_Q5_1: set(0, 16, nb); set(1, 4, nb); set(2, 4, nb); break;
    case T_Q4_K: set(0, 16, 8 * nb); set(1, 16, nb); break;
    case T_Q6_K: set(0, 16, 8 * nb); set(1, 16, 4 * nb); set(2, 8, 2 * nb); set(3, 2, nb); break;
    default: break;
    }
    const size_t tiles = (rows + TILE_ROWS - 1) / TILE_ROWS;
    size_t off = 0;
    for (int k = 0; k < 4; k++) {
        s.offset[k] = off;
        off = round_up(off + tiles * s.per_row[k] * TILE_ROWS * s.unit[k], 256);
    }
    s.total = off;
    return s;
}

}  // namespace nh
