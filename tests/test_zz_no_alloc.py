"""The allocation-free product entry point (lnh_gemm_device_noalloc) against the entry point it is a
variant of (lnh_gemm_device), through the C ABI on a real MI355X.

Both run the same kernels; the only difference is where the workspace of the multi-token kernels lives
(a fixed array in the library's device code instead of the executor's allocation), so the results must
be equal bit for bit.  Two calls in a row share the array, the second with a smaller product, which
would expose contents left behind by the first.  The outputs are also held against the CPU oracle
(float64 product of the dequantized weights) under the f32 summation bound of tests/test_gpu_parity.py.
"""
import importlib

import numpy as np
import pytest

import cases as K
import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu(pkg):
    g = pkg.HipGemv(0)
    yield g
    g.close()


@pytest.fixture(scope="module")
def hip():
    return importlib.import_module("llama-rust_amd.hiprt")


def _both(gpu, hip, m, ty, rows, cols, tokens, w, rng):
    x = rng.normal(0, 1, tokens * cols).astype(np.float32)
    xd = hip.DeviceBuffer.from_numpy(x)
    ya, yb = hip.DeviceBuffer(tokens * rows * 4), hip.DeviceBuffer(tokens * rows * 4)
    ya.fill_byte(0xff)
    yb.fill_byte(0xff)
    gpu.gemm_device_noalloc(m, tokens, xd.ptr, ya.ptr)
    gpu.synchronize()
    gpu.gemm_device(m, tokens, xd.ptr, yb.ptr)
    gpu.synchronize()
    a = ya.to_numpy(np.float32).reshape(tokens, rows)
    b = yb.to_numpy(np.float32).reshape(tokens, rows)
    for buf in (xd, ya, yb):
        buf.free()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"{O.TYPE_NAMES[ty]} {rows}x{cols} M={tokens}"
    exact, mag = O.gemm_f64_mag(ty, cols, tokens, w, x, rows)
    err = np.abs(a - exact)
    assert np.all(err <= K.single_kernel_bound(cols, mag))
    assert np.all(err <= 1e-4 * np.maximum(np.abs(exact), np.sqrt(np.mean(exact ** 2)) / 4))


@pytest.mark.parametrize("ty", [K.Q4_K, K.Q4_0, K.Q5_0, K.Q5_1, K.Q6_K, K.Q8_0])
def test_noalloc_equals_gemm_device_twice_in_a_row(gpu, hip, ty):
    """A larger product, then a smaller one through the same static workspace (column shares, 16-token
    and 32-token tiles), each equal to lnh_gemm_device bit for bit and inside the oracle's bound."""
    rng = np.random.default_rng(100 + ty)
    rows, cols = 1024, 2048
    w = K.random_packed(ty, rows, cols, rng, signed=False, scale=0.02)
    m = gpu.upload_packed(ty, rows, cols, w)
    rows2, cols2 = 300, 1024
    w2 = K.random_packed(ty, rows2, cols2, rng, signed=False, scale=0.02)
    m2 = gpu.upload_packed(ty, rows2, cols2, w2)
    try:
        # the entry point allocates nothing, so what the multi-token kernels read must exist before it is called
        gpu.prepare(m, 40)
        gpu.prepare(m2, 5)
        _both(gpu, hip, m, ty, rows, cols, 40, w, rng)
        _both(gpu, hip, m2, ty, rows2, cols2, 5, w2, rng)
        _both(gpu, hip, m, ty, rows, cols, 9, w, rng)
        _both(gpu, hip, m2, ty, rows2, cols2, 1, w2, rng)   # single token: no workspace at all
    finally:
        m.close()
        m2.close()


@pytest.mark.parametrize("ty", [K.F16, K.F32])
def test_noalloc_plain_dtypes_with_shared_columns(gpu, hip, ty):
    """F16 / F32 matrices with two or more tokens keep the partial sums of their column shares in the same static
    array: few rows and many columns, so that the columns are shared between workgroups; then a smaller product."""
    rng = np.random.default_rng(300 + ty)
    rows, cols = 96, 14336
    w = K.random_packed(ty, rows, cols, rng)
    m = gpu.upload_packed(ty, rows, cols, w)
    rows2, cols2 = 40, 4096
    w2 = K.random_packed(ty, rows2, cols2, rng)
    m2 = gpu.upload_packed(ty, rows2, cols2, w2)
    try:
        _both(gpu, hip, m, ty, rows, cols, 33, w, rng)
        _both(gpu, hip, m2, ty, rows2, cols2, 4, w2, rng)
        _both(gpu, hip, m, ty, rows, cols, 2, w, rng)
    finally:
        m.close()
        m2.close()


@pytest.mark.parametrize("ty,tokens", [(K.Q4_K, 24), (K.Q5_1, 7), (K.Q8_0, 70), (K.F16, 5)])
def test_noalloc_recorded_into_a_graph_and_replayed(gpu, hip, ty, tokens):
    """What the entry point is for: a call recorded while the stream is being captured (nothing may be allocated
    there), replayed several times with the program's own eager work and synchronisations between the replays, the
    input changed between replays; every replay equal bit for bit to lnh_gemm_device on the same input."""
    rng = np.random.default_rng(500 + ty)
    rows, cols = 640, 4096
    w = K.random_packed(ty, rows, cols, rng, signed=False, scale=0.02)
    m = gpu.upload_packed(ty, rows, cols, w)
    stream = hip.Stream()
    xd = hip.DeviceBuffer(tokens * cols * 4)
    ya, yb = hip.DeviceBuffer(tokens * rows * 4), hip.DeviceBuffer(tokens * rows * 4)
    graph = None
    try:
        gpu.prepare(m, tokens)   # before the capture: the capture itself may not allocate
        graph = hip.Graph(stream, lambda s: gpu.gemm_device_noalloc(m, tokens, xd.ptr, ya.ptr, s.ptr))
        for replay in range(3):
            x = rng.normal(0, 1, tokens * cols).astype(np.float32)
            xd.upload(x)
            ya.fill_byte(0xff)
            yb.fill_byte(0xff)
            hip.device_synchronize()
            graph.launch()
            stream.synchronize()
            gpu.gemm_device(m, tokens, xd.ptr, yb.ptr)   # eager work of the program between the replays
            gpu.synchronize()
            a, b = ya.to_numpy(np.float32), yb.to_numpy(np.float32)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"replay {replay}"
            exact, mag = O.gemm_f64_mag(ty, cols, tokens, w, x, rows)
            assert np.all(np.abs(a.reshape(tokens, rows) - exact) <= K.single_kernel_bound(cols, mag)), f"replay {replay}"
    finally:
        if graph is not None:
            graph.destroy()
        for buf in (xd, ya, yb):
            buf.free()
        m.close()


def test_noalloc_rejects_what_does_not_fit(gpu, hip, pkg):
    """A product whose workspace exceeds the fixed array fails before anything is launched; y untouched."""
    rng = np.random.default_rng(7)
    rows, cols = 256, 14336
    w = K.random_packed(K.Q4_0, rows, cols, rng, signed=False, scale=0.02)
    m = gpu.upload_packed(K.Q4_0, rows, cols, w)
    tokens = 2048   # split activations alone: 896 groups x 6 x (2048 + 64) x 16 B = 182 MB
    xd = hip.DeviceBuffer(tokens * cols * 4)
    yd = hip.DeviceBuffer(tokens * rows * 4)
    yd.fill_byte(0x5a)
    try:
        # a matrix that has only been uploaded has no multi-token layout yet, and this entry point may not make it
        with pytest.raises(pkg.NativeHipError) as ei:
            gpu.gemm_device_noalloc(m, 4, xd.ptr, yd.ptr)
        assert ei.value.code == pkg.ERR_INVALID and "lnh_matrix_prepare" in str(ei.value)
        single = m.info()[3]
        gpu.prepare(m, 1)                       # a single token needs nothing more
        assert m.info()[3] == single
        gpu.prepare(m, 4)
        assert m.info()[3] > single
        with pytest.raises(pkg.NativeHipError) as ei:
            gpu.gemm_device_noalloc(m, tokens, xd.ptr, yd.ptr)
        assert ei.value.code == pkg.ERR_INVALID and "allocation-free" in str(ei.value)
        gpu.synchronize()
        assert np.all(yd.to_numpy(np.uint8) == 0x5a)
        # the executor still works, and so does the entry point
        x = rng.normal(0, 1, 4 * cols).astype(np.float32)
        xs = hip.DeviceBuffer.from_numpy(x)
        gpu.gemm_device_noalloc(m, 4, xs.ptr, yd.ptr)
        gpu.synchronize()
        got = yd.to_numpy(np.float32, 4 * rows).reshape(4, rows)
        exact, mag = O.gemm_f64_mag(K.Q4_0, cols, 4, w, x, rows)
        assert np.all(np.abs(got - exact) <= K.single_kernel_bound(cols, mag))
        xs.free()
    finally:
        xd.free()
        yd.free()
        m.close()
