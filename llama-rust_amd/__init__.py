"""native-hip: MI355X (gfx950) matrix executor for llama-rust's GGUF block-quantized
matrix products, seen from Python.

This module is a thin ctypes view of the C ABI in include/native_hip.h and a
mirror of the reference's executor interface (same names, argument meaning and
error behaviour), so that tests read like the reference's own:

  HipGemv / HipMatrix / Shape / validate   <- CudaGemv / CudaMatrix / Shape / validate
                                              (native-cuda/src/lib.rs:8-53, gpu.rs:125-418)
  gemv_<t>_f32 / gemm_<t>_f32               <- langtax/src/quant.rs:6144-6293, 6366-6478, 6891-7199

There is no CPU fallback anywhere: if the shared library is missing, loading
raises; if there is no gfx950 device, HipGemv() raises.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libnative_hip.so")
SOURCES = ["kernels.hip", "executor.cpp", "residency.cpp", "gguf.cpp", "llama_host.cpp"]
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-FP32 VALU forms are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]

F32, F16, Q4_0, Q5_0, Q5_1, Q8_0, Q4_K, Q6_K = 0, 1, 2, 6, 7, 8, 12, 14
ALL_TYPES = (F32, F16, Q4_0, Q5_0, Q5_1, Q8_0, Q4_K, Q6_K)
TYPE_NAMES = {F32: "f32", F16: "f16", Q4_0: "q4_0", Q5_0: "q5_0", Q5_1: "q5_1", Q8_0: "q8_0",
              Q4_K: "q4_k", Q6_K: "q6_k"}

OK, ERR_INVALID, ERR_DEVICE, ERR_OOM, ERR_FOREIGN, ERR_UNSUPPORTED = range(6)
PROLOGUE_NONE, PROLOGUE_RMSNORM, PROLOGUE_SWIGLU = 0, 1, 2
EPILOGUE_NONE, EPILOGUE_ADD_RMSNORM, EPILOGUE_SWIGLU, EPILOGUE_ADD_RMSNORM_DEFERRED = 0, 1, 2, 3


class NativeHipError(RuntimeError):
    """Err(String) of the reference's executor, plus the status code."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


def build(verbose=False):
    """Compile the HIP kernels and the C ABI for gfx950 into libnative_hip.so (in-tree)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-x", "hip"] + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


SELFTEST_SRC = os.path.join(os.path.dirname(HERE), "tests", "cpp", "selftest.cpp")
SELFTEST_BIN = os.path.join(os.path.dirname(HERE), "tests", "cpp", "selftest")


def build_selftest(verbose=False):
    """Compile the C++ self-test (host code only: the C++ mirror header over the C ABI)."""
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-Wall", "-Wextra", SELFTEST_SRC, "-o", SELFTEST_BIN,
           "-L" + HERE, "-lnative_hip", "-Wl,-rpath,$ORIGIN/../../llama-rust_amd"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return SELFTEST_BIN


_lib = None


def load_library():
    """Load the built library; never builds, never falls back."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeHipError(ERR_DEVICE, f"{LIB_PATH} is missing: build it first (python -c "
                                         "'import __graft_entry__ as g; g.build()'); there is no CPU fallback")
    lib = C.CDLL(LIB_PATH)
    vp, sz, u32 = C.c_void_p, C.c_size_t, C.c_uint32
    pvp = C.POINTER(C.c_void_p)
    psz = C.POINTER(C.c_size_t)
    sig = {
        "lnh_create": (C.c_int, [C.c_int, pvp]),
        "lnh_destroy": (None, [vp]),
        "lnh_memory_info": (C.c_int, [vp, psz, psz]),
        "lnh_last_error": (C.c_char_p, [vp]),
        "lnh_thread_error": (C.c_char_p, []),
        "lnh_upload_f32": (C.c_int, [vp, sz, sz, vp, sz, pvp]),
        "lnh_upload_packed": (C.c_int, [vp, u32, sz, sz, vp, sz, pvp]),
        "lnh_upload_packed_device": (C.c_int, [vp, u32, sz, sz, vp, sz, pvp]),
        "lnh_matrix_free": (None, [vp]),
        "lnh_matrix_info": (C.c_int, [vp, C.POINTER(u32), psz, psz, psz]),
        "lnh_matrix_prepare": (C.c_int, [vp, vp, sz]),
        "lnh_gemv": (C.c_int, [vp, vp, vp, sz, vp, sz]),
        "lnh_gemm": (C.c_int, [vp, vp, sz, vp, sz, vp, sz]),
        "lnh_gemv_once": (C.c_int, [vp, vp, sz, vp, sz, vp, sz]),
        "lnh_gemm_grouped": (C.c_int, [vp, sz, pvp, psz, vp, sz, vp, sz]),
        "lnh_gemm_shared": (C.c_int, [vp, sz, pvp, sz, vp, sz, vp, sz]),
        "lnh_gemm_device": (C.c_int, [vp, vp, sz, vp, vp, vp]),
        "lnh_gemm_grouped_device": (C.c_int, [vp, sz, pvp, psz, vp, vp, vp]),
        "lnh_gemm_device_noalloc": (C.c_int, [vp, vp, sz, vp, vp, vp]),
        "lnh_gemm_batch_device": (C.c_int, [vp, sz, pvp, psz, pvp, pvp, vp]),
        "lnh_gemv_shared_device": (C.c_int, [vp, sz, pvp, vp, pvp, C.c_int, vp]),
        "lnh_gemv_fused_device": (C.c_int, [vp, sz, pvp, vp, pvp, C.c_int, C.c_int, vp, C.c_float, vp]),
        "lnh_gemv_swiglu_device": (C.c_int, [vp, vp, vp, vp, vp, C.c_int, vp, C.c_float, vp]),
        "lnh_calibration_copy": (C.c_int, [vp, vp, vp, sz, vp]),
        "lnh_calibration_read": (C.c_int, [vp, vp, sz, vp]),
        "lnh_synchronize": (C.c_int, [vp]),
        "lnh_shape_checked": (C.c_int, [sz, sz, sz, sz, C.POINTER(u32), C.POINTER(u32)]),
        "lnh_validate": (C.c_int, [vp, sz, vp, sz]),
        "lnh_row_bytes": (sz, [u32, sz]),
        "lnh_resident_bytes": (sz, [u32, sz, sz, sz]),
        "lnq_gemv": (C.c_int, [u32, sz, vp, sz, vp, sz, vp, sz]),
        "lnq_gemm": (C.c_int, [u32, sz, sz, vp, sz, vp, sz, vp, sz]),
        "lnq_gemm_grouped": (C.c_int, [u32, sz, sz, sz, pvp, sz, psz, vp, sz, vp, sz]),
        "lnq_last_error": (C.c_char_p, []),
        "lnq_parse_cache_bytes": (C.c_int, [C.c_char_p, C.POINTER(C.c_int), psz]),
        "lnq_automatic_cache_bytes": (sz, [sz, sz]),
        "lnq_admission_requires_eviction": (C.c_int, [sz, sz, sz]),
        "lnq_cache_stats": (None, [psz, psz, psz, psz, psz]),
        "lnq_reset": (None, []),
        # include/native_hip_llama.h
        "lnm_last_error": (C.c_char_p, []),
        "lnm_load": (C.c_int, [C.c_char_p, pvp]),
        "lnm_load_bytes": (C.c_int, [vp, sz, pvp]),
        "lnm_free": (None, [vp]),
        "lnm_info": (C.c_int, [vp, vp]),
        "lnm_set_products": (C.c_int, [vp, C.c_int, vp, vp]),
        "lnm_session_new": (C.c_int, [vp, sz, vp, sz, pvp]),
        "lnm_session_new_device": (C.c_int, [vp, sz, vp, sz, sz, pvp]),
        "lnm_session_new_device_batch": (C.c_int, [vp, sz, sz, sz, pvp]),
        "lnm_batch_generate_greedy": (C.c_int, [vp, vp, vp, sz, vp, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
        "lnm_session_free": (None, [vp]),
        "lnh_act_create": (C.c_int, [vp, C.c_uint32, sz, sz, vp]),
        "lnh_act_free": (None, [vp]),
        "lnh_act_split_device": (C.c_int, [vp, vp, sz, vp, vp]),
        "lnh_gemm_act_device": (C.c_int, [vp, sz, vp, vp, sz, vp, C.c_int, vp, vp, C.c_float, vp, vp, vp]),
        "lnh_gemm_plain_act_device": (C.c_int, [vp, sz, vp, vp, sz, vp, C.c_int, vp, vp, C.c_float, vp, vp, vp]),
        "lnm_forward": (C.c_int, [vp, vp, sz, vp]),
        "lnm_prompt": (C.c_int, [vp, vp, sz, vp, vp]),
        "lnm_generate_greedy": (C.c_int, [vp, vp, sz, sz, vp, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
        "lnm_session_timing": (C.c_int, [vp, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_uint64)]),
        "lnm_dequant_row": (C.c_int, [u32, sz, vp, sz, vp]),
        "lnm_topk": (C.c_int, [vp, sz, sz, vp]),
        "lnm_router_weights": (C.c_int, [vp, vp, sz, C.c_int, vp]),
        "lnm_moe_ffn": (C.c_int, [vp, sz, sz, vp, vp]),
        "lnm_rmsnorm": (C.c_int, [vp, vp, sz, C.c_float]),
        "lnm_rope": (C.c_int, [vp, sz, sz, sz, C.c_float]),
        "lnm_softmax": (None, [vp, sz]),
        "lnm_argmax": (u32, [vp, sz]),
        "lnm_write_synthetic_llama": (C.c_int, [C.c_char_p, vp]),
        "lnm_gguf_inspect": (C.c_int, [vp, sz, psz, psz, psz]),
        "lnm_gguf_tensor": (C.c_int, [vp, sz, sz, C.c_char_p, sz, C.POINTER(u32), C.POINTER(C.c_uint64),
                                      C.POINTER(u32), psz, psz]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)  # AttributeError if the ABI lost a symbol
        fn.restype, fn.argtypes = res, args
    lib._signatures = sig
    _lib = lib
    return lib


def exported_symbols():
    """Every entry point include/native_hip.h and include/native_hip_llama.h declare (used by the ABI test)."""
    load_library()
    return sorted(_lib._signatures)


def _ptr(a):
    return C.c_void_p(a.ctypes.data) if a.size else C.c_void_p(0)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    return np.ascontiguousarray(a, dtype=np.uint8)


# ------------------------------------------------------------------ lib.rs mirror
class Shape:
    """native-cuda/src/lib.rs:8-34."""

    def __init__(self, rows, cols):
        self.rows, self.cols = rows, cols

    @staticmethod
    def checked(rows, cols, weights, input):
        lib = load_library()
        r, c = C.c_uint32(), C.c_uint32()
        rc = lib.lnh_shape_checked(rows, cols, weights, input, C.byref(r), C.byref(c))
        if rc != OK:
            raise NativeHipError(rc, lib.lnh_thread_error().decode())
        return Shape(r.value, c.value)


def validate(actual, expected):
    """native-cuda/src/lib.rs:37-53: raises on the first |a-e| > 1e-4 + 1e-4|e| or non-finite value."""
    lib = load_library()
    a = _f32(actual).ravel()
    e = np.ascontiguousarray(expected, dtype=np.float64).ravel()
    rc = lib.lnh_validate(_ptr(a), a.size, _ptr(e), e.size)
    if rc != OK:
        raise NativeHipError(rc, lib.lnh_thread_error().decode())


def row_bytes(ggml_type, cols):
    return load_library().lnh_row_bytes(ggml_type, cols)


def resident_bytes(ggml_type, rows, cols, tokens=1):
    """Device bytes a packed rows x cols matrix holds once it has met products of up to `tokens` tokens
    (0: no such matrix); what the residency layer charges before an upload."""
    return load_library().lnh_resident_bytes(ggml_type, rows, cols, tokens)


# ------------------------------------------------------------------ gpu.rs mirror
class HipMatrix:
    """Immutable matrix resident on the GPU (CudaMatrix, native-cuda/src/gpu.rs:125-130)."""

    def __init__(self, handle):
        self._h = handle

    def info(self):
        lib = load_library()
        t, r, c, b = C.c_uint32(), C.c_size_t(), C.c_size_t(), C.c_size_t()
        lib.lnh_matrix_info(self._h, C.byref(t), C.byref(r), C.byref(c), C.byref(b))
        return t.value, r.value, c.value, b.value

    def close(self):
        if self._h:
            load_library().lnh_matrix_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Act:
    """Split activations on the device (lnh_act)."""

    def __init__(self, lib, handle):
        self._lib, self._h = lib, handle

    def close(self):
        if getattr(self, "_h", None):
            self._lib.lnh_act_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class HipGemv:
    """The executor (CudaGemv, native-cuda/src/gpu.rs:132-418).  Errors raise; no CPU fallback."""

    def __init__(self, device_ordinal=0):
        self._lib = load_library()
        h = C.c_void_p()
        rc = self._lib.lnh_create(device_ordinal, C.byref(h))
        if rc != OK:
            raise NativeHipError(rc, self._lib.lnh_thread_error().decode())
        self._h = h

    def _check(self, rc):
        if rc != OK:
            raise NativeHipError(rc, self._lib.lnh_last_error(self._h).decode())

    def close(self):
        if getattr(self, "_h", None):
            self._lib.lnh_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def memory_info(self):
        f, t = C.c_size_t(), C.c_size_t()
        self._check(self._lib.lnh_memory_info(self._h, C.byref(f), C.byref(t)))
        return f.value, t.value

    def upload(self, rows, cols, weights):
        w = _f32(weights).ravel()
        m = C.c_void_p()
        self._check(self._lib.lnh_upload_f32(self._h, rows, cols, _ptr(w), w.size, C.byref(m)))
        return HipMatrix(m)

    def upload_packed(self, ggml_type, rows, cols, packed):
        w = _u8(packed).ravel()
        m = C.c_void_p()
        self._check(self._lib.lnh_upload_packed(self._h, ggml_type, rows, cols, _ptr(w), w.size, C.byref(m)))
        return HipMatrix(m)

    def upload_packed_device(self, ggml_type, rows, cols, device_ptr, nbytes):
        m = C.c_void_p()
        self._check(self._lib.lnh_upload_packed_device(self._h, ggml_type, rows, cols, C.c_void_p(device_ptr),
                                                       nbytes, C.byref(m)))
        return HipMatrix(m)

    def gemv_resident(self, matrix, input, output):
        """output is written in place; it is left untouched when the call fails."""
        x = _f32(input).ravel()
        assert output.dtype == np.float32 and output.flags.c_contiguous
        self._check(self._lib.lnh_gemv(self._h, matrix._h, _ptr(x), x.size, _ptr(output), output.size))

    def gemm_resident(self, matrix, tokens, input, output):
        x = _f32(input).ravel()
        assert output.dtype == np.float32 and output.flags.c_contiguous
        self._check(self._lib.lnh_gemm(self._h, matrix._h, tokens, _ptr(x), x.size, _ptr(output), output.size))

    def gemv(self, weights, input, output):
        w, x = _f32(weights).ravel(), _f32(input).ravel()
        assert output.dtype == np.float32 and output.flags.c_contiguous
        self._check(self._lib.lnh_gemv_once(self._h, _ptr(w), w.size, _ptr(x), x.size, _ptr(output), output.size))

    def gemm_grouped(self, matrices, tokens, input, output):
        x = _f32(input).ravel()
        n = len(matrices)
        mats = (C.c_void_p * n)(*[m._h for m in matrices])
        toks = (C.c_size_t * n)(*tokens)
        assert output.dtype == np.float32 and output.flags.c_contiguous
        self._check(self._lib.lnh_gemm_grouped(self._h, n, mats, toks, _ptr(x), x.size, _ptr(output), output.size))

    def gemm_shared(self, matrices, tokens, input, output):
        """Several matrices times one input of `tokens` rows; products back to back in `output`."""
        x = _f32(input).ravel()
        n = len(matrices)
        mats = (C.c_void_p * n)(*[m._h for m in matrices])
        assert output.dtype == np.float32 and output.flags.c_contiguous
        self._check(self._lib.lnh_gemm_shared(self._h, n, mats, tokens, _ptr(x), x.size, _ptr(output), output.size))

    def gemm_device(self, matrix, tokens, x_ptr, y_ptr, stream=0):
        self._check(self._lib.lnh_gemm_device(self._h, matrix._h, tokens, C.c_void_p(x_ptr), C.c_void_p(y_ptr),
                                              C.c_void_p(stream)))

    def prepare(self, matrix, max_tokens):
        """Makes now what products of up to max_tokens tokens by this matrix need beyond the upload (the multi-token
        layout of a quantized matrix), for callers that will run them where nothing may be allocated."""
        self._check(self._lib.lnh_matrix_prepare(self._h, matrix._h, max_tokens))

    def gemm_device_noalloc(self, matrix, tokens, x_ptr, y_ptr, stream=0):
        """gemm_device with the library's fixed device workspace: never allocates (include/native_hip.h)."""
        self._check(self._lib.lnh_gemm_device_noalloc(self._h, matrix._h, tokens, C.c_void_p(x_ptr), C.c_void_p(y_ptr),
                                                      C.c_void_p(stream)))

    def act_create(self, ggml_type, cols, max_tokens):
        """A device buffer for activations in the form the multi-token kernels read (include/native_hip.h)."""
        h = C.c_void_p()
        self._check(self._lib.lnh_act_create(self._h, ggml_type, cols, max_tokens, C.byref(h)))
        return Act(self._lib, h)

    def act_split_device(self, act, tokens, x_ptr, stream=0):
        self._check(self._lib.lnh_act_split_device(self._h, act._h, tokens, C.c_void_p(x_ptr), C.c_void_p(stream)))

    def gemm_act_device(self, matrices, act, tokens, y_ptrs=None, epilogue=EPILOGUE_NONE, residual_ptr=0, norm_w_ptr=0,
                        eps=0.0, xn_ptr=0, next_act=None, stream=0):
        """Products of split activations; with an epilogue the step after the product runs where its shares are summed
        and leaves its result split in next_act."""
        n = len(matrices)
        mats = (C.c_void_p * n)(*[m._h for m in matrices])
        ys = (C.c_void_p * n)(*y_ptrs) if y_ptrs is not None else None
        self._check(self._lib.lnh_gemm_act_device(self._h, n, mats, act._h, tokens, ys, epilogue, C.c_void_p(residual_ptr),
                                                  C.c_void_p(norm_w_ptr), eps, C.c_void_p(xn_ptr),
                                                  next_act._h if next_act is not None else None, C.c_void_p(stream)))

    def gemm_plain_act_device(self, matrices, x_ptr, tokens, y_ptrs=None, epilogue=EPILOGUE_NONE, residual_ptr=0, norm_w_ptr=0,
                              eps=0.0, xn_ptr=0, next_act=None, stream=0):
        """gemm_act_device with the product's own activations as plain f32 rows on the device."""
        n = len(matrices)
        mats = (C.c_void_p * n)(*[m._h for m in matrices])
        ys = (C.c_void_p * n)(*y_ptrs) if y_ptrs is not None else None
        self._check(self._lib.lnh_gemm_plain_act_device(self._h, n, mats, C.c_void_p(x_ptr), tokens, ys, epilogue,
                                                        C.c_void_p(residual_ptr), C.c_void_p(norm_w_ptr), eps, C.c_void_p(xn_ptr),
                                                        next_act._h if next_act is not None else None, C.c_void_p(stream)))

    def gemm_grouped_device(self, matrices, tokens, x_ptr, y_ptr, stream=0):
        n = len(matrices)
        mats = (C.c_void_p * n)(*[m._h for m in matrices])
        toks = (C.c_size_t * n)(*tokens)
        self._check(self._lib.lnh_gemm_grouped_device(self._h, n, mats, toks, C.c_void_p(x_ptr), C.c_void_p(y_ptr),
                                                      C.c_void_p(stream)))

    def make_batch(self, matrices, tokens, x_ptrs, y_ptrs):
        """Pre-marshalled argument arrays for gemm_batch_device (reused across calls)."""
        n = len(matrices)
        return (n, (C.c_void_p * n)(*[m._h for m in matrices]), (C.c_size_t * n)(*tokens),
                (C.c_void_p * n)(*x_ptrs), (C.c_void_p * n)(*y_ptrs))

    def gemm_batch_device(self, batch, stream=0):
        n, mats, toks, xs, ys = batch
        self._check(self._lib.lnh_gemm_batch_device(self._h, n, mats, toks, xs, ys, C.c_void_p(stream)))

    def gemv_shared_device(self, matrices, x_ptr, y_ptrs, accumulate=False, stream=0):
        """y_i = W_i x (accumulate: y_i += W_i x) for matrices that read the same device x, one launch."""
        n = len(matrices)
        mats = (C.c_void_p * n)(*[m._h for m in matrices])
        ys = (C.c_void_p * n)(*y_ptrs)
        self._check(self._lib.lnh_gemv_shared_device(self._h, n, mats, C.c_void_p(x_ptr), ys, int(accumulate),
                                                     C.c_void_p(stream)))

    def gemv_fused_device(self, matrices, x_ptr, y_ptrs, prologue, x2_ptr, eps=0.0, accumulate=False, stream=0):
        """The same with PROLOGUE_RMSNORM / PROLOGUE_SWIGLU applied to x as the kernel stages it."""
        n = len(matrices)
        mats = (C.c_void_p * n)(*[m._h for m in matrices])
        ys = (C.c_void_p * n)(*y_ptrs)
        self._check(self._lib.lnh_gemv_fused_device(self._h, n, mats, C.c_void_p(x_ptr), ys, int(accumulate), prologue,
                                                    C.c_void_p(x2_ptr), eps, C.c_void_p(stream)))

    def gemv_swiglu_device(self, gate, up, x_ptr, h_ptr, prologue=PROLOGUE_NONE, x2_ptr=0, eps=0.0, stream=0):
        """h = SiLU(gate x') * (up x') in one launch; x' = x or RMSNorm(x) * x2."""
        self._check(self._lib.lnh_gemv_swiglu_device(self._h, gate._h, up._h, C.c_void_p(x_ptr), C.c_void_p(h_ptr),
                                                     prologue, C.c_void_p(x2_ptr), eps, C.c_void_p(stream)))

    def calibration_copy(self, dst_ptr, src_ptr, nbytes, stream=0):
        self._check(self._lib.lnh_calibration_copy(self._h, C.c_void_p(dst_ptr), C.c_void_p(src_ptr), nbytes,
                                                   C.c_void_p(stream)))

    def calibration_read(self, src_ptr, nbytes, stream=0):
        self._check(self._lib.lnh_calibration_read(self._h, C.c_void_p(src_ptr), nbytes, C.c_void_p(stream)))

    def synchronize(self):
        self._check(self._lib.lnh_synchronize(self._h))


# ------------------------------------------------------------------ quant.rs mirror
def _q_check(rc):
    if rc != OK:
        raise NativeHipError(rc, load_library().lnq_last_error().decode())


def gemv(ggml_type, n_cols, w, x, y):
    """gemv_<t>_f32(n_cols, w, x, y): n_rows = len(y); y written in place, untouched on error."""
    w, x = _u8(w).ravel(), _f32(x).ravel()
    assert y.dtype == np.float32 and y.flags.c_contiguous
    _q_check(load_library().lnq_gemv(ggml_type, n_cols, _ptr(w), w.size, _ptr(x), x.size, _ptr(y), y.size))


def gemm(ggml_type, n_cols, n_tokens, w, x, y):
    """gemm_<t>_f32(n_cols, n_tokens, w, x, y): token-major x and y."""
    w, x = _u8(w).ravel(), _f32(x).ravel()
    assert y.dtype == np.float32 and y.flags.c_contiguous
    _q_check(load_library().lnq_gemm(ggml_type, n_cols, n_tokens, _ptr(w), w.size, _ptr(x), x.size, _ptr(y), y.size))


def gemm_grouped(ggml_type, n_cols, n_rows, parts, tokens, x, y):
    """One MoE projection: part g (bytes of expert g) times its tokens[g] packed rows of x."""
    parts = [_u8(p).ravel() for p in parts]
    n = len(parts)
    part_len = parts[0].size if n else 0
    assert all(p.size == part_len for p in parts)
    arr = (C.c_void_p * n)(*[p.ctypes.data for p in parts])
    toks = (C.c_size_t * n)(*tokens)
    x = _f32(x).ravel()
    assert y.dtype == np.float32 and y.flags.c_contiguous
    _q_check(load_library().lnq_gemm_grouped(ggml_type, n_cols, n_rows, n, arr, part_len, toks, _ptr(x), x.size,
                                             _ptr(y), y.size))


def _named(ty):
    def gemv_t(n_cols, w, x, y):
        return gemv(ty, n_cols, w, x, y)

    def gemm_t(n_cols, n_tokens, w, x, y):
        return gemm(ty, n_cols, n_tokens, w, x, y)

    return gemv_t, gemm_t


gemv_f32, gemm_f32 = _named(F32)
gemv_f16, gemm_f16 = _named(F16)
gemv_q4_0_f32, gemm_q4_0_f32 = _named(Q4_0)
gemv_q5_0_f32, gemm_q5_0_f32 = _named(Q5_0)
gemv_q5_1_f32, gemm_q5_1_f32 = _named(Q5_1)
gemv_q8_0_f32, gemm_q8_0_f32 = _named(Q8_0)
gemv_q4_k_f32, gemm_q4_k_f32 = _named(Q4_K)
gemv_q6_k_f32, gemm_q6_k_f32 = _named(Q6_K)


def cache_stats():
    lib = load_library()
    v = [C.c_size_t() for _ in range(5)]
    lib.lnq_cache_stats(*[C.byref(a) for a in v])
    return dict(zip(("entries", "bytes", "limit", "hits", "misses"), (a.value for a in v)))


def reset():
    load_library().lnq_reset()
