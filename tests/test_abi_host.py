"""Host-side checks that need no GPU: the C-ABI library loads and exports every
symbol the header declares, and the validation / residency-policy rules of the
reference hold (native-cuda/src/lib.rs:55-76, langtax/src/native_gpu.rs:217-360,
langtax/tests/native_cuda_parity.rs:409-431).  No compute call is made here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import cases as K

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
USIZE_MAX = (1 << 64) - 1


def test_library_exports_every_declared_symbol(pkg, lib):
    header = open(os.path.join(ROOT, "include", "native_hip.h")).read()
    header += open(os.path.join(ROOT, "include", "native_hip_llama.h")).read()
    declared = set(re.findall(r"\b(ln[hqm]_[a-z0-9_]+)\s*\(", header)) - {"lnm_matmul_fn"}
    assert len(declared) >= 46
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(pkg.exported_symbols())


def test_shape_checked_rejects_unsafe_shapes(pkg):
    """native-cuda/src/lib.rs:58-65."""
    for args in [(0, 2, 0, 2), (2, 3, 5, 3), (2, 3, 6, 2), (USIZE_MAX, 2, 0, 2)]:
        with pytest.raises(pkg.NativeHipError):
            pkg.Shape.checked(*args)
    s = pkg.Shape.checked(17, 33, 561, 33)
    assert (s.rows, s.cols) == (17, 33)
    with pytest.raises(pkg.NativeHipError, match="GEMV dimensions must be positive"):
        pkg.Shape.checked(0, 2, 0, 2)
    with pytest.raises(pkg.NativeHipError, match="GEMV shape overflow"):
        pkg.Shape.checked(USIZE_MAX, 2, 0, 2)
    with pytest.raises(pkg.NativeHipError, match="GEMV matrix exceeds u32 indexing"):
        pkg.Shape.checked(1 << 20, 1 << 20, 0, 1 << 20)
    with pytest.raises(pkg.NativeHipError, match="GEMV buffer lengths do not match shape"):
        pkg.Shape.checked(2, 3, 6, 2)


def test_validate_catches_nonfinite_and_wrong_results(pkg):
    """native-cuda/src/lib.rs:67-75."""
    for a, e in [([np.nan], [0.0]), ([np.inf], [np.inf]), ([1.0], [2.0]), ([], [0.0])]:
        with pytest.raises(pkg.NativeHipError):
            pkg.validate(np.array(a, np.float32), np.array(e, np.float64))
    pkg.validate(np.array([1.00001, -2.0], np.float32), np.array([1.0, -2.0]))
    with pytest.raises(pkg.NativeHipError, match="GEMV output length mismatch"):
        pkg.validate(np.zeros(0, np.float32), np.zeros(1))
    with pytest.raises(pkg.NativeHipError, match="GEMV mismatch at row 1"):
        pkg.validate(np.array([1.0, 5.0], np.float32), np.array([1.0, 2.0]))


def test_row_bytes(pkg):
    for ty in pkg.ALL_TYPES:
        for cols in (256, 4096, 14336):
            assert pkg.row_bytes(ty, cols) == K.row_bytes(ty, cols)
    assert pkg.row_bytes(pkg.Q8_0, 33) == 0
    assert pkg.row_bytes(pkg.Q6_K, 128) == 0
    assert pkg.row_bytes(pkg.F16, 33) == 66
    assert pkg.row_bytes(3, 256) == 0  # Q4_1 is outside the eight dtypes


def test_resident_bytes_is_the_packed_size_once_or_about_twice(pkg):
    """What a residency cache charges before an upload: every dtype holds its GGUF bytes once (plus plane alignment
    and row padding) while it only meets one or two tokens; a quantized matrix that meets three or more holds the
    second layout as well, F32 / F16 never do.  Nothing for shapes the packed kernels do not take."""
    for ty in pkg.ALL_TYPES:
        for rows, cols in ((4096, 4096), (1000, 14336), (3, 256)):
            packed = rows * K.row_bytes(ty, cols)
            one = pkg.resident_bytes(ty, rows, cols, 1)
            assert one == pkg.resident_bytes(ty, rows, cols, 2)
            assert packed <= one <= packed + 4 * (256 + 64) + 16 * rows
            many = pkg.resident_bytes(ty, rows, cols, 3)
            assert many == pkg.resident_bytes(ty, rows, cols, 512)
            if ty in (pkg.F32, pkg.F16):
                assert many == one
            else:
                tiled_rows = (rows + 255) // 256 * 256
                assert one + tiled_rows * K.row_bytes(ty, cols) <= many <= one + tiled_rows * K.row_bytes(ty, cols) + 4 * 256
    assert pkg.resident_bytes(pkg.Q4_K, 16, 100, 1) == 0      # not whole blocks
    assert pkg.resident_bytes(3, 16, 256, 1) == 0             # Q4_1 is outside the eight dtypes
    assert pkg.resident_bytes(pkg.Q8_0, 0, 32, 1) == 0
    assert pkg.resident_bytes(pkg.Q8_0, 1 << 33, 32, 1) == 0  # rows beyond u32


def test_cache_budget_env_grammar(lib):
    """langtax/src/native_gpu.rs:338-359: `auto` or decimal digits, nothing else."""
    is_auto, b = C.c_int(), C.c_size_t()

    def parse(v):
        return lib.lnq_parse_cache_bytes(v, C.byref(is_auto), C.byref(b))

    assert parse(None) == 0 and is_auto.value == 1
    assert parse(b"auto") == 0 and is_auto.value == 1
    assert parse(b"0") == 0 and is_auto.value == 0 and b.value == 0
    assert parse(b"1073741824") == 0 and b.value == 1 << 30
    for bad in (b"", b" 1", b"1 ", b"+1", b"-1", b"1k", b"0x10", b"1.5", b"AUTO"):
        assert parse(bad) != 0, bad
        assert b"must be auto or a nonnegative decimal byte count" in lib.lnq_last_error()
    assert parse(b"99999999999999999999999999") != 0
    assert b"exceeds addressable memory" in lib.lnq_last_error()


def test_automatic_budget_and_admission_arithmetic(lib):
    """langtax/src/native_gpu.rs:310-336."""
    MiB, GiB = 1 << 20, 1 << 30
    auto = lib.lnq_automatic_cache_bytes
    assert auto(0, 0) == 0
    assert auto(256 * MiB, 8 * GiB) == 0                       # less than the 512 MiB headroom
    assert auto(1 * GiB, 8 * GiB) == 512 * MiB                 # headroom floor wins below 2 GiB
    assert auto(8 * GiB, 8 * GiB) == 6 * GiB                   # a quarter stays free
    assert auto(16 * GiB, 8 * GiB) == 6 * GiB                  # inconsistent report clamps to total
    assert auto(USIZE_MAX, USIZE_MAX) == USIZE_MAX - USIZE_MAX // 4
    adm = lib.lnq_admission_requires_eviction
    assert adm(0, 10, 10) == 0
    assert adm(1, 10, 10) == 1
    assert adm(0, 11, 10) == 1
    assert adm(USIZE_MAX, 1, USIZE_MAX) == 1                   # no overflow
    assert adm(USIZE_MAX - 1, 1, USIZE_MAX) == 0


def test_invalid_matrix_operations_preserve_output_without_touching_the_device(pkg):
    """langtax/tests/native_cuda_parity.rs:409-431 - every rejected call leaves
    `output` as it was; all of these fail validation before any device work."""
    for fmt in K.formats():
        packed = fmt.pack_row(0)
        x = K.values(1, fmt.cols)
        gemv = lambda cols, w, xx, y, ty=fmt.ty: pkg.gemv(ty, cols, w, xx, y)
        gemm = lambda cols, n, w, xx, y, ty=fmt.ty: pkg.gemm(ty, cols, n, w, xx, y)
        out = np.array([123.5], np.float32)
        with pytest.raises(pkg.NativeHipError, match="W bytes size 0 != "):
            gemv(fmt.cols, np.zeros(0, np.uint8), x, out)
        with pytest.raises(pkg.NativeHipError, match="X F32 elems size 0 != "):
            gemv(fmt.cols, packed, np.zeros(0, np.float32), out)
        with pytest.raises(pkg.NativeHipError, match="must be positive and token-aligned"):
            gemm(fmt.cols, 0, packed, x, out)
        doubled = np.concatenate([x, x])
        with pytest.raises(pkg.NativeHipError, match="token-aligned"):
            gemm(fmt.cols, 2, packed, doubled, out)
        assert out[0] == np.float32(123.5)
        # empty rows succeed and do nothing
        gemv(fmt.cols, np.zeros(0, np.uint8), x, np.zeros(0, np.float32))
        gemm(fmt.cols, 2, np.zeros(0, np.uint8), doubled, np.zeros(0, np.float32))
    out = np.array([123.5], np.float32)
    # gemm_f32(usize::MAX, 2, &[], &[], &mut output) must fail cleanly
    assert pkg.load_library().lnq_gemm(pkg.F32, USIZE_MAX, 2, None, 0, None, 0, out.ctypes.data, 1) != 0
    assert pkg.load_library().lnq_gemm(pkg.F32, USIZE_MAX, 2, None, 0, None, 0, out.ctypes.data, 0) != 0
    assert out[0] == np.float32(123.5)
    # lengths that are right with a pointer that is not: refused before the device is touched
    x32, y1 = np.zeros(32, np.float32), np.array([123.5], np.float32)
    lib = pkg.load_library()
    assert lib.lnq_gemm(pkg.Q8_0, 32, 1, None, 34, x32.ctypes.data, 32, y1.ctypes.data, 1) != 0
    assert b"buffer pointer is null" in lib.lnq_last_error()
    w34 = np.zeros(34, np.uint8)
    assert lib.lnq_gemm(pkg.Q8_0, 32, 1, w34.ctypes.data, 34, None, 32, y1.ctypes.data, 1) != 0
    assert lib.lnq_gemm(pkg.Q8_0, 32, 1, w34.ctypes.data, 34, x32.ctypes.data, 32, None, 1) != 0
    assert y1[0] == np.float32(123.5)
    with pytest.raises(pkg.NativeHipError, match="n_cols 33 is not a multiple of 32"):
        pkg.gemv(pkg.Q8_0, 33, np.zeros(34, np.uint8), np.zeros(33, np.float32), np.zeros(1, np.float32))
    with pytest.raises(pkg.NativeHipError, match="unsupported GGUF dtype"):
        pkg.gemv(3, 32, np.zeros(20, np.uint8), np.zeros(32, np.float32), np.zeros(1, np.float32))


def test_cpp_mirror_header_compiles_against_the_c_abi(pkg, tmp_path):
    """include/native_hip.hpp (HipGemv, HipMatrix, Shape, validate over the C ABI) and the
    self-test that uses it compile and link with the host compiler alone; running it needs a GPU
    and is done by the GPU tests."""
    import shutil
    import subprocess
    cxx = shutil.which(os.environ.get("CXX", "g++"))
    if cxx is None:
        pytest.skip("no host C++ compiler")
    out = tmp_path / "selftest"
    subprocess.run([cxx, "-std=c++17", "-Wall", "-Wextra", "-Werror", pkg.SELFTEST_SRC, "-o", str(out), "-L" + pkg.HERE,
                    "-lnative_hip"], check=True)
    assert out.exists()
