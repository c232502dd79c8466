"""Shared test inputs: the reference's closed-form fixtures, random block
generators with the distributions its tests draw from, and independent numpy
dequantizers written from the GGUF block definitions (they share no code with
the C oracle, which is what makes them a check on it)."""
import numpy as np

import oracle as O

F32, F16, Q4_0, Q5_0, Q5_1, Q8_0, Q4_K, Q6_K = O.ALL_TYPES
QK = {F32: 1, F16: 1, Q4_0: 32, Q5_0: 32, Q5_1: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256}
BLOCK = {F32: 4, F16: 2, Q4_0: 18, Q5_0: 22, Q5_1: 24, Q8_0: 34, Q4_K: 144, Q6_K: 210}
U = 2.0 ** -24


def row_bytes(ty, n_cols):
    assert n_cols % QK[ty] == 0
    return n_cols // QK[ty] * BLOCK[ty]


# ------------------------------------------------------------------ error bounds
# langtax/src/simd/tests.rs:70-91
def single_kernel_bound(n, abs_sum):
    k = n + 3.0
    g = k * U / (1.0 - k * U) if k * U < 0.5 else k * U
    return g * abs_sum


def observed_envelope_u(n):
    return max(8.0 * np.sqrt(n), 64.0)


def reference_tolerance_ok(actual, expected):
    """|a - e| <= 1e-4 + 1e-4|e|, both finite (native-cuda/src/lib.rs:37-53)."""
    a = np.asarray(actual, np.float64)
    e = np.asarray(expected, np.float64)
    return bool(np.all(np.isfinite(a)) and np.all(np.isfinite(e))
                and np.all(np.abs(a - e) <= 1e-4 + 1e-4 * np.abs(e)))


# ------------------------------------------------------------------ closed-form fixtures
# langtax/tests/native_cuda_parity.rs:27-34
def values(row, cols):
    col = np.arange(cols)
    return (((row * 7 + col * 11) % 31) - 15).astype(np.float32) / np.float32(16.0)


# native-cuda/src/main.rs:17-25
def selftest_weights(rows, cols):
    i = np.arange(rows * cols)
    return ((i % 23).astype(np.float32) - 11.0) / np.float32(16.0)


def selftest_input(tokens, cols, rnd):
    i = np.arange(tokens * cols)
    return (((i * 5 + rnd * 7) % 29).astype(np.float32) - 14.0) / np.float32(16.0)


# langtax/tests/native_cuda_parity.rs:36-122 (BF16 is outside the eight dtypes).
def _pack_row_f32(r):
    return O.pack_f32(values(r, 33))


def _pack_row_f16(r):
    return O.pack_f16(values(r, 33))


def _pack_row_q4_0(r):
    i = np.arange(32)
    return O.pack_q4_0_block(0.125, ((r * 3 + i * 7) % 16 - 8).astype(np.int8))


def _pack_row_q8_0(r):
    i = np.arange(32)
    return O.pack_q8_0_block(0.015625, ((r * 3 + i * 7) % 127 - 63).astype(np.int8))


def _pack_row_q4_k(r):
    i = np.arange(256)
    return O.pack_q4_k_block(0.03125, 0.015625, [1, 2, 3, 4, 5, 6, 7, 8], [2, 1, 0, 3, 1, 4, 2, 5],
                             ((r * 3 + i * 7) % 16).astype(np.uint8))


def _pack_row_q6_k(r):
    i = np.arange(256)
    return O.pack_q6_k_block(0.0078125, [1, 2, -3, 4, 5, -6, 7, 8, -1, 2, 3, -4, 5, 6, -7, 8],
                             ((r * 3 + i * 7) % 64 - 32).astype(np.int8))


# The reference's list has no Q5_0 / Q5_1 entry; these two follow the same
# recipe (dyadic scale, closed-form codes) so all eight dtypes are covered.
def _pack_row_q5_0(r):
    i = np.arange(32)
    return O.pack_q5_0_block(0.0625, ((r * 3 + i * 7) % 32).astype(np.uint8))


def _pack_row_q5_1(r):
    i = np.arange(32)
    return O.pack_q5_1_block(0.0625, -0.5, ((r * 5 + i * 3) % 32).astype(np.uint8))


class Format:
    def __init__(self, name, ty, cols, pack_row):
        self.name, self.ty, self.cols, self.pack_row = name, ty, cols, pack_row


def formats():
    return [
        Format("F32", F32, 33, _pack_row_f32),
        Format("F16", F16, 33, _pack_row_f16),
        Format("Q4_0", Q4_0, 32, _pack_row_q4_0),
        Format("Q8_0", Q8_0, 32, _pack_row_q8_0),
        Format("Q4_K", Q4_K, 256, _pack_row_q4_k),
        Format("Q6_K", Q6_K, 256, _pack_row_q6_k),
        Format("Q5_0", Q5_0, 32, _pack_row_q5_0),
        Format("Q5_1", Q5_1, 32, _pack_row_q5_1),
    ]


# ------------------------------------------------------------------ random packed rows
def _f16_bytes(a):
    """Encode finite f32 values as binary16 little-endian bytes (round to nearest)."""
    return np.asarray(a, np.float32).astype(np.float16).view(np.uint8)


def random_packed(ty, n_rows, n_cols, rng, signed=True, scale=0.05):
    """Random packed matrix with the distributions of the reference's SIMD tests
    (langtax/src/simd/tests.rs:459-486, 565-588, 663-681, 832-838, 1012-1033, 1176-1193):
    signed block scales, every code value, int8 including -128."""
    assert n_cols % QK[ty] == 0
    nb = n_cols // QK[ty]

    def sc(shape, s):
        v = rng.uniform(-s, s, size=shape) if signed else np.abs(rng.normal(0.0, s, size=shape))
        return v.astype(np.float32)

    if ty == F32:
        return rng.uniform(-1, 1, size=(n_rows, n_cols)).astype(np.float32).view(np.uint8).reshape(-1).copy()
    if ty == F16:
        return _f16_bytes(rng.uniform(-1, 1, size=(n_rows, n_cols))).reshape(-1).copy()
    blk = rng.integers(0, 256, size=(n_rows, nb, BLOCK[ty]), dtype=np.uint8)
    if ty in (Q8_0, Q4_0, Q5_0):
        blk[:, :, 0:2] = _f16_bytes(sc((n_rows, nb), scale * (2 if ty == Q8_0 else 1))).reshape(n_rows, nb, 2)
    elif ty == Q5_1:
        blk[:, :, 0:2] = _f16_bytes(sc((n_rows, nb), scale)).reshape(n_rows, nb, 2)
        blk[:, :, 2:4] = _f16_bytes(sc((n_rows, nb), 0.02)).reshape(n_rows, nb, 2)
    elif ty == Q4_K:
        blk[:, :, 0:2] = _f16_bytes(sc((n_rows, nb), scale)).reshape(n_rows, nb, 2)
        blk[:, :, 2:4] = _f16_bytes(sc((n_rows, nb), 0.02)).reshape(n_rows, nb, 2)
    elif ty == Q6_K:
        blk[:, :, 208:210] = _f16_bytes(sc((n_rows, nb), scale)).reshape(n_rows, nb, 2)
    return blk.reshape(-1).copy()


# ------------------------------------------------------------------ independent numpy dequantizers
def _h(b):
    """binary16 little-endian byte pairs -> f32, through numpy's own float16."""
    return np.ascontiguousarray(b).view(np.float16).astype(np.float32)[..., 0]


def np_dequant(ty, n_rows, n_cols, w):
    w = np.ascontiguousarray(w, np.uint8)
    if ty == F32:
        return w.view(np.float32).reshape(n_rows, n_cols).copy()
    if ty == F16:
        return w.view(np.float16).astype(np.float32).reshape(n_rows, n_cols)
    nb = n_cols // QK[ty]
    b = w.reshape(n_rows, nb, BLOCK[ty])
    f = np.float32
    if ty == Q8_0:
        d = _h(b[:, :, 0:2])[..., None]
        out = b[:, :, 2:].view(np.int8).astype(f) * d
    elif ty == Q4_0:
        d = _h(b[:, :, 0:2])[..., None]
        qs = b[:, :, 2:18].astype(np.int32)
        codes = np.concatenate([qs & 15, qs >> 4], axis=-1) - 8
        out = codes.astype(f) * d
    elif ty in (Q5_0, Q5_1):
        off = 2 if ty == Q5_0 else 4
        d = _h(b[:, :, 0:2])[..., None]
        qh = np.ascontiguousarray(b[:, :, off:off + 4]).view(np.uint32)  # (R, nb, 1)
        qs = b[:, :, off + 4:off + 20].astype(np.uint32)
        nib = np.concatenate([qs & 15, qs >> 4], axis=-1)
        fifth = (qh >> np.arange(32, dtype=np.uint32)) & 1
        codes = (nib | (fifth << 4)).astype(np.int32)
        if ty == Q5_0:
            out = (codes - 16).astype(f) * d
        else:
            m = _h(b[:, :, 2:4])[..., None]
            out = (codes.astype(f) * d) + m
    elif ty == Q4_K:
        d = _h(b[:, :, 0:2])[..., None]
        dmin = _h(b[:, :, 2:4])[..., None]
        s = b[:, :, 4:16].astype(np.uint32)
        sc = np.empty(s.shape[:-1] + (8,), np.uint32)
        mn = np.empty_like(sc)
        sc[..., :4] = s[..., 0:4] & 63
        mn[..., :4] = s[..., 4:8] & 63
        sc[..., 4:] = (s[..., 8:12] & 15) | ((s[..., 0:4] >> 6) << 4)
        mn[..., 4:] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
        qs = b[:, :, 16:144].reshape(n_rows, nb, 4, 32).astype(np.uint32)
        codes = np.stack([qs & 15, qs >> 4], axis=3).reshape(n_rows, nb, 8, 32)  # sub-block major
        a = (d * sc.astype(f))[..., None]
        bb = (dmin * mn.astype(f))[..., None]
        out = (a * codes.astype(f) - bb).reshape(n_rows, nb, 256)
    elif ty == Q6_K:
        d = _h(b[:, :, 208:210])[..., None]
        ql = b[:, :, 0:128].reshape(n_rows, nb, 2, 2, 32).astype(np.uint32)   # n, half, l
        qh = b[:, :, 128:192].reshape(n_rows, nb, 2, 32).astype(np.uint32)    # n, l
        sc = b[:, :, 192:208].view(np.int8).astype(f).reshape(n_rows, nb, 2, 4, 2)  # n, quarter, is
        lo0, lo1 = ql[:, :, :, 0, :], ql[:, :, :, 1, :]
        q = np.stack([(lo0 & 15) | ((qh & 3) << 4),
                      (lo1 & 15) | (((qh >> 2) & 3) << 4),
                      (lo0 >> 4) | (((qh >> 4) & 3) << 4),
                      (lo1 >> 4) | (((qh >> 6) & 3) << 4)], axis=3).astype(np.int32) - 32  # n, quarter, l
        ds = d[..., None, None] * sc                                    # n, quarter, is
        ds_l = np.repeat(ds, 16, axis=-1)                               # n, quarter, l
        out = (ds_l * q.astype(f)).reshape(n_rows, nb, 256)
    else:
        raise ValueError(ty)
    return np.ascontiguousarray(out.reshape(n_rows, n_cols), dtype=f)


def f64_product(ty, n_rows, n_cols, w, x):
    """Token-major f64 oracle from the independent numpy dequantizer."""
    wd = np_dequant(ty, n_rows, n_cols, w).astype(np.float64)
    xs = np.asarray(x, np.float32).reshape(-1, n_cols).astype(np.float64)
    return xs @ wd.T


def abs_product(ty, n_rows, n_cols, w, x):
    wd = np.abs(np_dequant(ty, n_rows, n_cols, w).astype(np.float64))
    xs = np.abs(np.asarray(x, np.float32).reshape(-1, n_cols).astype(np.float64))
    return xs @ wd.T
