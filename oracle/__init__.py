"""ctypes view of the CPU oracle (liboracle.so).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's cpu-baseline leg may import
this module; the product path never does.  `load()` builds the library with
`make` when it is missing.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")

F32, F16, Q4_0, Q5_0, Q5_1, Q8_0, Q4_K, Q6_K = 0, 1, 2, 6, 7, 8, 12, 14
ALL_TYPES = (F32, F16, Q4_0, Q5_0, Q5_1, Q8_0, Q4_K, Q6_K)
TYPE_NAMES = {F32: "F32", F16: "F16", Q4_0: "Q4_0", Q5_0: "Q5_0", Q5_1: "Q5_1",
              Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K"}

_lib = None


def build():
    subprocess.run(["make", "-C", HERE, "-s"], check=True)


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    lib = C.CDLL(LIB_PATH)
    u8p, f32p, f64p = C.c_void_p, C.c_void_p, C.c_void_p
    lib.lro_f16_to_f32.restype = C.c_float
    lib.lro_f16_to_f32.argtypes = [C.c_uint16]
    lib.lro_f32_to_f16.restype = C.c_uint16
    lib.lro_f32_to_f16.argtypes = [C.c_float]
    for name in ("lro_block_elems", "lro_block_bytes"):
        getattr(lib, name).restype = C.c_size_t
        getattr(lib, name).argtypes = [C.c_int]
    lib.lro_row_bytes.restype = C.c_size_t
    lib.lro_row_bytes.argtypes = [C.c_int, C.c_size_t]
    lib.lro_dequant_row.restype = C.c_int
    lib.lro_dequant_row.argtypes = [C.c_int, C.c_size_t, u8p, f32p]
    for name in ("lro_vec_dot_row", "lro_simd_dot_row"):
        getattr(lib, name).restype = C.c_float
        getattr(lib, name).argtypes = [C.c_int, C.c_size_t, u8p, f32p]
    for name in ("lro_row_dot_f64", "lro_row_abs_dot_f64"):
        getattr(lib, name).restype = C.c_double
        getattr(lib, name).argtypes = [C.c_int, C.c_size_t, u8p, f32p]
    lib.lro_gemm.restype = C.c_int
    lib.lro_gemm.argtypes = [C.c_int, C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t,
                             u8p, C.c_size_t, f32p, C.c_size_t, f32p, C.c_size_t]
    lib.lro_gemm_f64.restype = C.c_int
    lib.lro_gemm_f64.argtypes = [C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, u8p, f32p, f64p]
    lib.lro_gemm_f64_mag.restype = C.c_int
    lib.lro_gemm_f64_mag.argtypes = [C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, u8p, f32p, f64p, f64p]
    lib.lro_worker_count.restype = C.c_int
    lib.lro_worker_count.argtypes = [C.c_size_t]
    lib.lro_pack_q8_0_block.argtypes = [C.c_float, u8p, u8p]
    lib.lro_pack_q4_0_block.argtypes = [C.c_float, u8p, u8p]
    lib.lro_pack_q5_0_block.argtypes = [C.c_float, u8p, u8p]
    lib.lro_pack_q5_1_block.argtypes = [C.c_float, C.c_float, u8p, u8p]
    lib.lro_pack_q4_k_block.argtypes = [C.c_float, C.c_float, u8p, u8p, u8p, u8p]
    lib.lro_pack_q6_k_block.argtypes = [C.c_float, u8p, u8p, u8p]
    lib.lro_pack_f16.argtypes = [f32p, C.c_size_t, u8p]
    lib.lro_scale_min_k4.argtypes = [u8p, C.c_int, u8p, u8p]
    lib.lro_splitmix64.restype = C.c_uint64
    lib.lro_splitmix64.argtypes = [C.POINTER(C.c_uint64)]
    lib.lro_demo_q8_gemv.restype = C.c_uint64
    lib.lro_demo_q8_gemv.argtypes = [C.c_size_t, C.c_size_t, f32p]
    lib.lro_validate.restype = C.c_long
    lib.lro_validate.argtypes = [f32p, f64p, C.c_size_t]
    _lib = lib
    return lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _u8(a):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    return a


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def row_bytes(ty, n_cols):
    return load().lro_row_bytes(ty, n_cols)


def block_elems(ty):
    return load().lro_block_elems(ty)


def block_bytes(ty):
    return load().lro_block_bytes(ty)


def dequant_row(ty, n_cols, row):
    row = _u8(row)
    y = np.empty(n_cols, dtype=np.float32)
    rc = load().lro_dequant_row(ty, n_cols, _p(row), _p(y))
    if rc != 0:
        raise ValueError(f"dequant_row type {ty} n_cols {n_cols}: {rc}")
    return y


def dequant(ty, n_cols, w, n_rows):
    w = _u8(w)
    rb = row_bytes(ty, n_cols)
    return np.stack([dequant_row(ty, n_cols, w[r * rb:(r + 1) * rb]) for r in range(n_rows)]) \
        if n_rows else np.zeros((0, n_cols), np.float32)


def vec_dot_row(ty, n_cols, row, x, simd=False):
    row, x = _u8(row), _f32(x)
    fn = load().lro_simd_dot_row if simd else load().lro_vec_dot_row
    return np.float32(fn(ty, n_cols, _p(row), _p(x)))


def row_dot_f64(ty, n_cols, row, x):
    row, x = _u8(row), _f32(x)
    return load().lro_row_dot_f64(ty, n_cols, _p(row), _p(x))


def row_abs_dot_f64(ty, n_cols, row, x):
    row, x = _u8(row), _f32(x)
    return load().lro_row_abs_dot_f64(ty, n_cols, _p(row), _p(x))


def gemm(ty, n_cols, n_tokens, w, x, n_rows, simd=False, threads=1):
    """Token-major y[n_tokens, n_rows] from the scalar (or AVX2) CPU kernels."""
    w, x = _u8(w), _f32(x)
    y = np.empty(n_tokens * n_rows, dtype=np.float32)
    rc = load().lro_gemm(ty, 1 if simd else 0, threads, n_cols, n_tokens, n_rows, _p(w), w.size,
                         _p(x), x.size, _p(y), y.size)
    if rc != 0:
        raise ValueError(f"lro_gemm failed: {rc}")
    return y.reshape(n_tokens, n_rows)


def gemm_f64(ty, n_cols, n_tokens, w, x, n_rows):
    """Token-major f64 oracle over the dequantized weights."""
    w, x = _u8(w), _f32(x)
    y = np.empty(n_tokens * n_rows, dtype=np.float64)
    rc = load().lro_gemm_f64(ty, n_cols, n_tokens, n_rows, _p(w), _p(x), _p(y))
    if rc != 0:
        raise ValueError(f"lro_gemm_f64 failed: {rc}")
    return y.reshape(n_tokens, n_rows)


def gemm_f64_mag(ty, n_cols, n_tokens, w, x, n_rows):
    """(exact-ish f64 product, sum |w||x| per output), both token-major [n_tokens, n_rows]."""
    w, x = _u8(w), _f32(x)
    y = np.empty(n_tokens * n_rows, dtype=np.float64)
    mag = np.empty(n_tokens * n_rows, dtype=np.float64)
    rc = load().lro_gemm_f64_mag(ty, n_cols, n_tokens, n_rows, _p(w), _p(x), _p(y), _p(mag))
    if rc != 0:
        raise ValueError(f"lro_gemm_f64_mag failed: {rc}")
    return y.reshape(n_tokens, n_rows), mag.reshape(n_tokens, n_rows)


def validate(actual, expected):
    """Index of the first element failing |a-e| <= 1e-4 + 1e-4|e| (or non-finite), else -1."""
    a = _f32(actual).ravel()
    e = np.ascontiguousarray(expected, dtype=np.float64).ravel()
    assert a.size == e.size
    return load().lro_validate(_p(a), _p(e), a.size)


def pack_q8_0_block(d, qs):
    qs = np.ascontiguousarray(qs, dtype=np.int8)
    out = np.empty(34, np.uint8)
    load().lro_pack_q8_0_block(d, _p(qs), _p(out))
    return out


def pack_q4_0_block(d, v):
    v = np.ascontiguousarray(v, dtype=np.int8)
    out = np.empty(18, np.uint8)
    load().lro_pack_q4_0_block(d, _p(v), _p(out))
    return out


def pack_q5_0_block(d, q5):
    q5 = _u8(q5)
    out = np.empty(22, np.uint8)
    load().lro_pack_q5_0_block(d, _p(q5), _p(out))
    return out


def pack_q5_1_block(d, m, q5):
    q5 = _u8(q5)
    out = np.empty(24, np.uint8)
    load().lro_pack_q5_1_block(d, m, _p(q5), _p(out))
    return out


def pack_q4_k_block(d, dmin, sc, mn, q4):
    sc, mn, q4 = _u8(sc), _u8(mn), _u8(q4)
    out = np.empty(144, np.uint8)
    load().lro_pack_q4_k_block(d, dmin, _p(sc), _p(mn), _p(q4), _p(out))
    return out


def pack_q6_k_block(d, sc, q6):
    sc = np.ascontiguousarray(sc, dtype=np.int8)
    q6 = np.ascontiguousarray(q6, dtype=np.int8)
    out = np.empty(210, np.uint8)
    load().lro_pack_q6_k_block(d, _p(sc), _p(q6), _p(out))
    return out


def pack_f16(v):
    v = _f32(v)
    out = np.empty(2 * v.size, np.uint8)
    load().lro_pack_f16(_p(v), v.size, _p(out))
    return out


def pack_f32(v):
    return _f32(v).view(np.uint8).copy()


def scale_min_k4(scales, j):
    scales = _u8(scales)
    sc, mn = C.c_uint8(), C.c_uint8()
    load().lro_scale_min_k4(_p(scales), j, C.byref(sc), C.byref(mn))
    return sc.value, mn.value


class SplitMix64:
    def __init__(self, seed):
        self.state = C.c_uint64(seed)

    def next(self):
        return load().lro_splitmix64(C.byref(self.state))


def demo_q8_gemv(n_cols, n_rows):
    y = np.empty(n_rows, np.float32)
    h = load().lro_demo_q8_gemv(n_cols, n_rows, _p(y))
    return h, y
