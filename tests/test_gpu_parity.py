"""Parity of the HIP executor with the CPU oracle, through the C ABI, on a real
MI355X.  The cases restate the reference's own executor self-test
(native-cuda/src/main.rs) and integration contract
(langtax/tests/native_cuda_parity.rs) and add random data at the benchmark
shapes.

Tolerances (floating point, f32 accumulation), all against an f64 product of the
dequantized weights:
  (i)   the reference's acceptance rule |a - e| <= 1e-4 + 1e-4|e|
        (native-cuda/src/lib.rs:37-53), literally, wherever the data are the
        reference's own closed-form fixtures (outputs of order one);
  (ii)  for every output of every case, the proven bound for any f32 summation
        order, |a - e| <= gamma(n+3) * sum|w x|, and the reference's observed
        envelope max(64, 8 sqrt n) * 2^-24 * sum|w x| (langtax/src/simd/tests.rs:18-91);
  (iii) for every output of every random case, the relative criterion
        |a - e| <= 1e-4 * max(|e|, rms(e)/4): 1e-4 relative error wherever the
        output is not a near-cancellation (a pure |a-e|/|e| bound is unbounded
        as e -> 0 for ANY f32 summation order, the reference's CPU kernels
        included, because the rounding error scales with sum|w x|, not with |e|).
"""
import importlib
import os

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


# One entry per named case: (case, outputs, max |a-e| / bound, max relative error away from zero, outputs near zero,
#  max error in u of sum|wx|, the last-but-two and the last figure again for the restated AVX2 CPU kernels on the same
#  inputs, max |a-e| over what tier (iii) allows).
REPORT = []


def _report_lines(entries):
    """The figures behind the tolerance tiers: one line per named case, then one per benchmark configuration (worst
    over its cases).  `literal` is the benchmark's own criterion read literally - max |a-e|/|e| over the outputs
    with |e| >= 1e-3 rms(e), against 1e-4 - for the GPU and for the reference's AVX2 order on the same inputs;
    `tier iii` is max |a-e| / (1e-4 max(|e|, rms(e)/4)), the criterion the tests assert (<= 1)."""
    head = ("case | outputs | max |a-e| / gamma(n+3) sum|wx| | literal: max |a-e|/|e| where |e| >= 1e-3 rms(e) (1e-4 asked) | "
            "outputs below that | tier iii: max |a-e| / (1e-4 max(|e|, rms/4)) | max |a-e| in u = 2^-24 of sum|wx| | "
            "CPU (AVX2 order) literal | CPU: max |a-e| in u")
    lines = [head]
    per_config = {}
    for name, n, r_bound, r_rel, n_small, r_u, c_rel, c_u, r_iii in entries:
        lines.append(f"{name} | {n} | {r_bound:.4f} | {r_rel:.3e} | {n_small} | {r_iii:.3f} | {r_u:.2f} | {c_rel:.3e} | {c_u:.2f}")
        key = " ".join(name.split()[:2])
        a = per_config.setdefault(key, [0, 0.0, 0.0, 0, 0.0, 0.0, 0.0, 0.0])
        a[0] += n
        a[3] += n_small
        for i, v in ((1, r_bound), (2, r_rel), (4, r_iii), (5, r_u), (6, c_rel), (7, c_u)):
            a[i] = max(a[i], v)
    lines.append("")
    lines.append("per configuration (worst over its cases):")
    for key, (n, r_bound, r_rel, n_small, r_iii, r_u, c_rel, c_u) in per_config.items():
        lines.append(f"{key} | {n} | {r_bound:.4f} | {r_rel:.3e} ({'meets' if r_rel <= 1e-4 else 'exceeds'} 1e-4) | {n_small} | "
                     f"{r_iii:.3f} | {r_u:.2f} | {c_rel:.3e} ({'meets' if c_rel <= 1e-4 else 'exceeds'} 1e-4) | {c_u:.2f}")
    return lines


@pytest.fixture(scope="module", autouse=True)
def parity_report():
    """After the module's tests: the report of _report_lines, printed and (when PARITY_REPORT names a file) written out."""
    yield
    if not REPORT:
        return
    text = "\n".join(_report_lines(REPORT))
    print("\n" + text)
    path = os.environ.get("PARITY_REPORT")
    if path:
        with open(path, "w") as f:
            f.write(text + "\n")


def check(actual, ty, n_cols, n_tokens, n_rows, w, x, name="", strict=False):
    """Tiers (ii) and (iii) always; the reference's literal rule (i) when strict."""
    exact, mag = O.gemm_f64_mag(ty, n_cols, n_tokens, w, x, n_rows)
    a = np.asarray(actual, np.float32).reshape(n_tokens, n_rows).astype(np.float64)
    assert np.all(np.isfinite(a)), name
    err = np.abs(a - exact)
    if strict:
        bad = O.validate(a.astype(np.float32), exact)
        assert bad == -1, f"{name}: output {bad}: expected {exact.ravel()[bad]}, got {a.ravel()[bad]}"
    bound = K.single_kernel_bound(n_cols, mag)
    worst = np.argmax(err - bound)
    assert np.all(err <= bound), f"{name}: output {worst} off by {err.ravel()[worst]} > bound {bound.ravel()[worst]}"
    env = K.observed_envelope_u(n_cols) * K.U * mag
    worst = np.argmax(err - env)
    assert np.all(err <= env), (f"{name}: output {worst} off by {err.ravel()[worst] / max(mag.ravel()[worst], 1e-300) / K.U:.1f} u "
                                f"of sum|wx|, envelope {K.observed_envelope_u(n_cols):.0f} u")
    rms = np.sqrt(np.mean(exact ** 2))
    allowed = 1e-4 * np.maximum(np.abs(exact), rms / 4)
    worst = np.argmax(err - allowed)
    assert np.all(err <= allowed), (f"{name}: output {worst}: |a-e| = {err.ravel()[worst]:.3e} > 1e-4 * max(|e|, rms/4) = "
                                    f"{allowed.ravel()[worst]:.3e}")
    if name:
        away = np.abs(exact) >= 1e-3 * rms
        cpu = O.gemm(ty, n_cols, n_tokens, w, x, n_rows, simd=True, threads=0).reshape(n_tokens, n_rows).astype(np.float64)
        cerr = np.abs(cpu - exact)
        REPORT.append((name, err.size, float(np.max(err / np.maximum(bound, 1e-300))),
                       float(np.max(err[away] / np.abs(exact[away]))) if away.any() else 0.0, int(err.size - away.sum()),
                       float(np.max(err / np.maximum(mag, 1e-300)) / K.U),
                       float(np.max(cerr[away] / np.abs(exact[away]))) if away.any() else 0.0,
                       float(np.max(cerr / np.maximum(mag, 1e-300)) / K.U),
                       float(np.max(err / np.maximum(allowed, 1e-300)))))
    return err, mag


# ------------------------------------------------------------------ native-cuda/src/main.rs
def test_cpp_selftest_through_the_mirror_header(pkg):
    """The same scenario from C++ (tests/cpp/selftest.cpp over include/native_hip.hpp): a
    maintainer's compiled host code reaches the kernels through the C ABI only."""
    import subprocess
    if not os.path.exists(pkg.SELFTEST_BIN):
        pkg.build_selftest()
    r = subprocess.run([pkg.SELFTEST_BIN], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and r.stdout.startswith("OK"), r.stdout + r.stderr


def test_executor_selftest_shapes_and_rounds(pkg, gpu):
    """native-cuda/src/main.rs:8-45: revisited shapes, alternating vector/batch launches,
    every equal-sized reuse changes all inputs, every output is checked."""
    shapes = [(r, c) for r in (1, 7, 9, 257) for c in (63, 64, 65, 129, 1025)] + [(17, 33), (1, 1), (257, 129), (17, 33)]
    for rows, cols in shapes:
        w = K.selftest_weights(rows, cols)
        m = gpu.upload(rows, cols, w)
        for rnd, tokens in enumerate([1, 1, 3, 3, 1, 7, 1]):
            x = K.selftest_input(tokens, cols, rnd)
            expected = x.reshape(tokens, cols).astype(np.float64) @ w.reshape(rows, cols).astype(np.float64).T
            actual = np.full(rows * tokens, np.nan, np.float32)
            if tokens == 1:
                gpu.gemv_resident(m, x, actual)
            else:
                gpu.gemm_resident(m, tokens, x, actual)
            pkg.validate(actual, expected.ravel())
        m.close()


def test_executor_rejects_bad_calls_and_recovers(pkg, gpu):
    """native-cuda/src/main.rs:46-68."""
    m = gpu.upload(2, 3, np.array([1.0, -2.0, 3.0, 4.0, 5.0, -6.0], np.float32))
    out = np.array([123.5, -456.0], np.float32)
    with pytest.raises(pkg.NativeHipError, match="HIP GEMV vector lengths do not match resident matrix"):
        gpu.gemv_resident(m, np.array([1.0, 2.0], np.float32), out)
    with pytest.raises(pkg.NativeHipError, match="HIP GEMM buffer lengths do not match shape"):
        gpu.gemm_resident(m, 0, np.zeros(0, np.float32), out)
    other = pkg.HipGemv(0)
    with pytest.raises(pkg.NativeHipError, match="HIP matrix belongs to a different executor") as ei:
        other.gemv_resident(m, np.array([1.0, 2.0, 3.0], np.float32), out)
    assert ei.value.code == pkg.ERR_FOREIGN
    other.close()
    assert np.array_equal(out, np.array([123.5, -456.0], np.float32))
    gpu.gemv_resident(m, np.array([1.0, 2.0, 3.0], np.float32), out)
    pkg.validate(out, [6.0, -4.0])
    # upload + product in one call (CudaGemv::gemv)
    out2 = np.zeros(2, np.float32)
    gpu.gemv(np.array([1.0, -2.0, 3.0, 4.0, 5.0, -6.0], np.float32), np.array([1.0, 2.0, 3.0], np.float32), out2)
    assert np.array_equal(out2, np.array([6.0, -4.0], np.float32))
    with pytest.raises(pkg.NativeHipError, match="GEMV buffer lengths do not match shape"):
        gpu.upload(2, 3, np.zeros(5, np.float32))
    free, total = gpu.memory_info()
    assert 0 < free <= total
    m.close()
    # device buffers a call reads are taken in 16-byte pieces: an address that is not a multiple of 16 is refused
    # before anything is launched, for one token and for several
    import importlib
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(3)
    mq = gpu.upload_packed(K.Q8_0, 64, 256, K.random_packed(K.Q8_0, 64, 256, rng))
    dx, dy = hip.DeviceBuffer(8 * 256 * 4 + 16), hip.DeviceBuffer(8 * 64 * 4)
    for tokens in (1, 8):
        with pytest.raises(pkg.NativeHipError, match="16-byte aligned") as ei:
            gpu.gemm_device(mq, tokens, dx.ptr + 4, dy.ptr)
        assert ei.value.code == pkg.ERR_INVALID
    with pytest.raises(pkg.NativeHipError, match="16-byte aligned"):
        gpu.gemv_shared_device([mq], dx.ptr + 8, [dy.ptr])
    mq.close(); dx.free(); dy.free()


# ------------------------------------------------------------------ langtax/tests/native_cuda_parity.rs
@pytest.mark.parametrize("fmt", K.formats(), ids=lambda f: f.name)
def test_quantized_dispatch_matches_cpu_row_oracle(pkg, fmt):
    """native_cuda_parity.rs:160-191: 257 rows, token counts [1,1,3,3,7,1] twice, then the
    first row overwritten in place: residency must follow content, not the pointer."""
    pkg.reset()
    rows = 257
    packed = np.concatenate([fmt.pack_row(r) for r in range(rows)])
    for pas in range(2):
        for rnd, tokens in enumerate([1, 1, 3, 3, 7, 1]):
            x = np.concatenate([K.values(t + rnd * 3 + pas, fmt.cols) for t in range(tokens)])
            actual = np.full(rows * tokens, np.nan, np.float32)
            if tokens == 1:
                pkg.gemv(fmt.ty, fmt.cols, packed, x, actual)
            else:
                pkg.gemm(fmt.ty, fmt.cols, tokens, packed, x, actual)
            check(actual, fmt.ty, fmt.cols, tokens, rows, packed, x, fmt.name, strict=True)
            # dyadic data: the product is exactly representable, so any correct kernel hits it
            exact = O.gemm_f64(fmt.ty, fmt.cols, tokens, packed, x, rows)
            assert np.array_equal(actual.reshape(tokens, rows).astype(np.float64), exact), fmt.name
        rb = packed.size // rows
        packed[:rb] = fmt.pack_row(rows + 5)  # same buffer, same shape and dtype, different bytes
    stats = pkg.cache_stats()
    assert stats["misses"] == 2 and stats["hits"] == 10 and stats["entries"] == 2


def test_warp_boundary_shapes_match_independent_f64_dots(pkg):
    """native_cuda_parity.rs:335-375."""
    for rows in (1, 7, 9, 257):
        for cols in (63, 64, 65, 129, 1025):
            w = np.concatenate([K.values(r, cols) / np.float32(1.3) for r in range(rows)]).astype(np.float32)
            packed = O.pack_f32(w)
            for rnd in range(2):
                for tokens in (1, 3):
                    x = np.concatenate([K.values(t + rnd * 17, cols) / np.float32(1.7) for t in range(tokens)])
                    x = x.astype(np.float32)
                    expected = x.reshape(tokens, cols).astype(np.float64) @ w.reshape(rows, cols).astype(np.float64).T
                    actual = np.full(rows * tokens, np.nan, np.float32)
                    if tokens == 1:
                        pkg.gemv_f32(cols, packed, x, actual)
                    else:
                        pkg.gemm_f32(cols, tokens, packed, x, actual)
                    pkg.validate(actual, expected.ravel())


@pytest.mark.parametrize("fmt", K.formats(), ids=lambda f: f.name)
def test_multi_block_quantized_batches_match_cpu_oracle(pkg, fmt):
    """native_cuda_parity.rs:377-407."""
    for blocks in (2, 3):
        cols = fmt.cols * blocks
        for rows in (1, 9):
            packed = np.concatenate([fmt.pack_row(r + b * 5) for r in range(rows) for b in range(blocks)])
            if fmt.ty in (K.F32, K.F16):
                # F32 / F16 rows are plain element arrays: concatenating 33-wide pieces is a 66/99-wide row
                assert packed.size == rows * K.row_bytes(fmt.ty, cols)
            for tokens in (1, 2, 7, 8, 9, 31, 32, 33):
                x = np.concatenate([K.values(t * 3 + 1, cols) for t in range(tokens)])
                actual = np.full(rows * tokens, np.nan, np.float32)
                pkg.gemm(fmt.ty, cols, tokens, packed, x, actual)
                check(actual, fmt.ty, cols, tokens, rows, packed, x, fmt.name, strict=True)


def test_invalid_operations_preserve_output_with_a_live_device(pkg):
    """native_cuda_parity.rs:409-431, this time after the device has been used."""
    for fmt in K.formats():
        packed, x = fmt.pack_row(0), K.values(1, fmt.cols)
        out = np.array([123.5], np.float32)
        ok = np.zeros(1, np.float32)
        pkg.gemv(fmt.ty, fmt.cols, packed, x, ok)  # brings the executor up
        for bad in (lambda: pkg.gemv(fmt.ty, fmt.cols, np.zeros(0, np.uint8), x, out),
                    lambda: pkg.gemv(fmt.ty, fmt.cols, packed, np.zeros(0, np.float32), out),
                    lambda: pkg.gemm(fmt.ty, fmt.cols, 0, packed, x, out),
                    lambda: pkg.gemm(fmt.ty, fmt.cols, 2, packed, np.concatenate([x, x]), out)):
            with pytest.raises(pkg.NativeHipError):
                bad()
            assert out[0] == np.float32(123.5)
        again = np.zeros(1, np.float32)
        pkg.gemv(fmt.ty, fmt.cols, packed, x, again)  # still usable, same answer
        assert again[0] == ok[0]


def test_workspace_growth_under_stream_capture_is_refused_not_recorded(pkg):
    """A multi-token product that would have to allocate cannot be captured into a HIP graph: while the matrix has
    no multi-token layout both entry points fail with nothing launched; once lnh_matrix_prepare has made it the
    allocation-free entry point can be captured at once and the ordinary one after one eager call (its workspace
    grows then); the capture stays usable throughout and replays of both equal the eager result bit for bit."""
    hip = importlib.import_module("llama-rust_amd.hiprt")
    g = pkg.HipGemv(0)  # a fresh executor: no workspace yet
    rng = np.random.default_rng(31)
    rows, cols, tokens = 512, 1024, 8
    w = K.random_packed(K.Q4_K, rows, cols, rng, signed=False, scale=0.02)
    m = g.upload_packed(K.Q4_K, rows, cols, w)
    x = rng.normal(0, 1, tokens * cols).astype(np.float32)
    xd = hip.DeviceBuffer.from_numpy(x)
    ya, yb, yc = (hip.DeviceBuffer(tokens * rows * 4) for _ in range(3))
    stream = hip.Stream()
    seen = {}
    unprepared = []

    def enqueue_unprepared(s):   # the matrix has only been uploaded: its multi-token layout does not exist yet
        for call in (g.gemm_device, g.gemm_device_noalloc):
            try:
                call(m, tokens, xd.ptr, ya.ptr, s.ptr)
            except pkg.NativeHipError as e:
                unprepared.append((e.code, str(e)))

    single = m.info()[3]
    hip.Graph(stream, enqueue_unprepared).destroy()
    assert [c for c, _ in unprepared] == [pkg.ERR_INVALID] * 2 and all("lnh_matrix_prepare" in t for _, t in unprepared)
    assert m.info()[3] == single                 # nothing was made under the capture
    g.prepare(m, tokens)
    assert m.info()[3] > single

    def enqueue(s):
        try:
            g.gemm_device(m, tokens, xd.ptr, ya.ptr, s.ptr)
        except pkg.NativeHipError as e:
            seen["code"], seen["text"] = e.code, str(e)
        g.gemm_device_noalloc(m, tokens, xd.ptr, yb.ptr, s.ptr)

    graph = hip.Graph(stream, enqueue)
    assert seen.get("code") == pkg.ERR_INVALID and "being captured" in seen["text"]
    g.gemm_device(m, tokens, xd.ptr, yc.ptr, stream.ptr)   # eager: grows the workspace
    stream.synchronize()
    want = yc.to_numpy(np.float32)
    check(want, K.Q4_K, cols, tokens, rows, w, x, "eager product before the replays")
    graph2 = hip.Graph(stream, lambda s: g.gemm_device(m, tokens, xd.ptr, ya.ptr, s.ptr))   # now it can be captured
    for _ in range(3):
        yb.fill_byte(0xff)
        ya.fill_byte(0xff)
        graph.launch()
        graph2.launch()
        stream.synchronize()
        assert np.array_equal(yb.to_numpy(np.float32).view(np.uint32), want.view(np.uint32))
        assert np.array_equal(ya.to_numpy(np.float32).view(np.uint32), want.view(np.uint32))
    graph.destroy()
    graph2.destroy()
    for b in (xd, ya, yb, yc):
        b.free()
    m.close()
    g.close()


def test_q4k_matrix_beyond_32_bit_plane_offsets_is_refused(pkg, gpu):
    """The Q4_K single-token kernel addresses a plane with 32-bit byte offsets: an upload whose code plane
    would reach 4 GiB is refused by shape, before any byte of it is read (the buffer here is a stub)."""
    stub = np.zeros(144, np.uint8)
    with pytest.raises(pkg.NativeHipError, match="exceeds 4 GiB of codes") as ei:
        gpu.upload_packed(K.Q4_K, 65536, 131072, stub)
    assert ei.value.code == pkg.ERR_INVALID
    m = gpu.upload_packed(K.Q4_K, 1, 256, stub)  # the executor is still usable
    m.close()


def test_a_failed_product_leaves_no_cache_entry_behind(pkg):
    """langtax/src/native_gpu.rs:190-211 keeps an uploaded matrix only after its product returned Ok."""
    pkg.reset()
    rng = np.random.default_rng(12)
    cols, rows = 64, 5
    w = K.random_packed(K.Q8_0, rows, cols, rng)
    x = rng.normal(0, 1, cols).astype(np.float32)
    y = np.zeros(rows, np.float32)
    pkg.gemv(K.Q8_0, cols, w, x, y)
    before = pkg.cache_stats()
    assert before["entries"] == 1 and before["misses"] == 1
    # tokens * rows beyond u32: passes native_matmul's checks, is uploaded, and the product is refused
    lib = pkg.load_library()
    w2 = K.random_packed(K.Q8_0, 1, 32, rng)
    huge = (1 << 32) + 8
    rc = lib.lnq_gemm(K.Q8_0, 32, huge, w2.ctypes.data, w2.size, x.ctypes.data, huge * 32, y.ctypes.data, huge)
    assert rc != 0 and b"exceeds u32" in lib.lnq_last_error()
    after = pkg.cache_stats()
    assert after["entries"] == 1 and after["bytes"] == before["bytes"] and after["misses"] == 2
    pkg.gemv(K.Q8_0, cols, w, x, y)  # the earlier entry is still there and still found
    assert pkg.cache_stats()["hits"] == before["hits"] + 1


# ------------------------------------------------------------------ random data, all dtypes
@pytest.mark.parametrize("ty", [K.F16, K.F32], ids=lambda t: O.TYPE_NAMES[t])
def test_plain_dtypes_on_the_matrix_cores_every_tile_and_share_shape(pkg, gpu, ty):
    """F16 / F32 weights with two or more tokens run on the f32 matrix instruction: 128-row and 32- or 64-token
    tiles, columns in steps of 32 shared between workgroups when rows and tokens alone leave CUs idle.  Shapes on
    both sides of every tile edge, rows that are not whole 16-byte groups (activations then load element by
    element), a single step, many shares, token counts across the 32 / 64 switch and beyond one tile."""
    rng = np.random.default_rng(4000 + ty)
    for rows, cols in ((127, 32), (128, 31), (129, 33), (1, 4096), (260, 1030), (96, 8192), (512, 14336), (31, 3)):
        w = K.random_packed(ty, rows, cols, rng)
        m = gpu.upload_packed(ty, rows, cols, w)
        for tokens in (2, 3, 31, 32, 33, 64, 65, 130):
            x = rng.normal(0, 1, tokens * cols).astype(np.float32)
            y = np.full(tokens * rows, np.nan, np.float32)
            gpu.gemm_resident(m, tokens, x, y)
            check(y, ty, cols, tokens, rows, w, x, f"{O.TYPE_NAMES[ty]} {rows}x{cols} M={tokens}")
            if tokens in (3, 65):   # row t of a batch is the product of token t alone, up to the order of the sums
                t = tokens - 1
                alone = np.full(rows, np.nan, np.float32)
                gpu.gemm_resident(m, 1, x[t * cols:(t + 1) * cols], alone)
                exact, mag = O.gemm_f64_mag(ty, cols, 1, w, x[t * cols:(t + 1) * cols], rows)
                assert np.all(np.abs(y.reshape(tokens, rows)[t] - alone) <= 2 * K.single_kernel_bound(cols, mag))
        m.close()


@pytest.mark.parametrize("ty", O.ALL_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_random_gemv_and_gemm_within_bounds(pkg, gpu, ty):
    """Signed scales, every code value, int8 -128, token counts across the kernel switch points."""
    rng = np.random.default_rng(1000 + ty)
    if K.QK[ty] == 1:
        shapes = [(5, 1), (33, 7), (64, 100), (130, 257), (19, 1000), (300, 4096), (64, 4100)]
    elif K.QK[ty] == 32:
        shapes = [(3, 32), (65, 64), (10, 96), (33, 2048), (257, 4096), (40, 14336), (16, 16416), (6, 28672)]
    else:
        shapes = [(3, 256), (65, 512), (9, 768), (33, 2048), (257, 4096), (40, 14336), (12, 16640), (6, 28672)]
    for rows, cols in shapes:
        w = K.random_packed(ty, rows, cols, rng)
        m = gpu.upload_packed(ty, rows, cols, w)
        for tokens in (1, 2, 5, 8, 13, 16, 17, 33):
            x = rng.normal(0, 1, tokens * cols).astype(np.float32)
            y = np.full(tokens * rows, np.nan, np.float32)
            gpu.gemm_resident(m, tokens, x, y)
            check(y, ty, cols, tokens, rows, w, x, f"{O.TYPE_NAMES[ty]} {rows}x{cols} M={tokens}")
        m.close()


@pytest.mark.parametrize("ty", [K.Q4_0, K.Q5_0, K.Q5_1, K.Q8_0, K.Q4_K, K.Q6_K], ids=lambda t: O.TYPE_NAMES[t])
def test_multi_token_products_of_random_shapes(pkg, gpu, ty):
    """Seeded sweep over what decides the launch of a multi-token product: rows around the 256-row tile, column
    counts that give odd and even step counts and from none to 32 column shares, token counts on both sides of the
    16-, 32- and 64-token tiles (the first two cut their activations themselves), alone and as grouped calls whose
    products share launches.  Every output against the f64 product of the dequantized weights."""
    rng = np.random.default_rng(4200 + ty)
    unit = K.QK[ty]
    for case in range(14):
        rows = int(rng.choice([1, 5, 63, 64, 65, 255, 256, 257, 300, 513]))
        cols = unit * int(rng.choice([1, 2, 3, 5, 8, 9, 16, 17, 40]) if unit == 256 else rng.choice([1, 3, 8, 16, 17, 33, 64, 130, 257]))
        tokens = int(rng.choice([3, 4, 7, 8, 9, 15, 16, 17, 23, 31, 32, 33, 47, 64, 65, 70]))
        w = K.random_packed(ty, rows, cols, rng)
        m = gpu.upload_packed(ty, rows, cols, w)
        x = rng.normal(0, 1, tokens * cols).astype(np.float32)
        y = np.full(tokens * rows, np.nan, np.float32)
        gpu.gemm_resident(m, tokens, x, y)
        check(y, ty, cols, tokens, rows, w, x)
        m.close()
    # grouped: four matrices of one column count, token counts that fall into different tile classes
    for case in range(4):
        cols = unit * int(rng.choice([2, 4, 9]) if unit == 256 else rng.choice([8, 16, 33, 72]))
        rows = [int(r) for r in rng.choice([40, 256, 257, 520], 4)]
        toks = [int(t) for t in rng.choice([0, 3, 9, 16, 17, 30, 33, 64], 4)]
        ws = [K.random_packed(ty, r, cols, rng) for r in rows]
        ms = [gpu.upload_packed(ty, r, cols, w) for r, w in zip(rows, ws)]
        x = rng.normal(0, 1, sum(toks) * cols).astype(np.float32)
        y = np.full(sum(t * r for t, r in zip(toks, rows)), np.nan, np.float32)
        gpu.gemm_grouped(ms, toks, x, y)
        xo = yo = 0
        for r, t, w in zip(rows, toks, ws):
            if t:
                check(y[yo:yo + t * r], ty, cols, t, r, w, x[xo:xo + t * cols])
            xo += t * cols
            yo += t * r
        for m in ms:
            m.close()


@pytest.mark.parametrize("ty", [K.Q4_0, K.Q5_0, K.Q5_1, K.Q8_0, K.Q4_K, K.Q6_K], ids=lambda t: O.TYPE_NAMES[t])
def test_adversarial_activations_keep_the_reference_bound(pkg, gpu, ty):
    """The multi-token kernels hand the f32 activations to the matrix cores as three bf16 numbers
    each.  That is only a faithful f32 product (the reference never rounds activations,
    langtax/src/quant.rs:6760-6888) if the three parts carry all 24 significand bits at every
    magnitude: full-mantissa values, 2^-60 .. 2^60 in one row, signed zeros, tiny values."""
    rng = np.random.default_rng(4242 + ty)
    rows, cols, tokens = 96, 2048, 6
    w = K.random_packed(ty, rows, cols, rng)
    m = gpu.upload_packed(ty, rows, cols, w)
    mant = rng.integers(0, 1 << 23, size=(tokens, cols)).astype(np.uint32)
    sign = rng.integers(0, 2, size=(tokens, cols)).astype(np.uint32) << 31
    x = np.empty((tokens, cols), np.float32)
    # token 0: every significand bit set, exponent 0;  token 1: random full mantissas
    x[0] = (np.uint32(0x3F800000) | np.uint32(0x7FFFFF) | sign[0]).view(np.float32)
    x[1] = (np.uint32(0x3F800000) | mant[1] | sign[1]).view(np.float32)
    # token 2: exponents spread over 2^-60 .. 2^60 within the row
    e2 = rng.integers(127 - 60, 127 + 61, size=cols).astype(np.uint32) << 23
    x[2] = (e2 | mant[2] | sign[2]).view(np.float32)
    # token 3: tiny but normal values (2^-100), token 4: zeros of both signs among ordinary values
    x[3] = ((np.uint32(27) << 23) | mant[3] | sign[3]).view(np.float32)
    x[4] = rng.normal(0, 1, cols).astype(np.float32)
    x[4, ::3] = 0.0
    x[4, 1::3] = -0.0
    # token 5: one large value among small ones (cancellation in the other columns must survive)
    x[5] = rng.normal(0, 1e-3, cols).astype(np.float32)
    x[5, 777] = 3.0e4
    exact, mag = O.gemm_f64_mag(ty, cols, tokens, w, x.reshape(-1), rows)
    # 6 tokens run on the 16-token tiles, the same 6 three times over (18) on the 32-token tiles
    for reps in (1, 3):
        xr = np.tile(x, (reps, 1))
        y = np.full(reps * tokens * rows, np.nan, np.float32)
        gpu.gemm_resident(m, reps * tokens, xr.reshape(-1), y)
        assert np.all(np.isfinite(y))
        for rep in range(reps):
            err = np.abs(y.reshape(reps, tokens, rows)[rep].astype(np.float64) - exact)
            # the reference's proven bound and its observed envelope, per output, relative to sum |w x|
            assert np.all(err <= K.single_kernel_bound(cols, mag)), f"{reps * tokens} tokens"
            assert np.all(err <= K.observed_envelope_u(cols) * K.U * mag), f"{reps * tokens} tokens"
    # the single-token kernels on the same rows: the same bounds (a code bias factored out
    # through the sum of x would fail here: one large activation under a zero weight)
    for t in range(tokens):
        y1 = np.full(rows, np.nan, np.float32)
        gpu.gemv_resident(m, x[t], y1)
        err1 = np.abs(y1.astype(np.float64) - exact[t])
        assert np.all(err1 <= K.single_kernel_bound(cols, mag[t])), f"token {t}"
        assert np.all(err1 <= K.observed_envelope_u(cols) * K.U * mag[t]), f"token {t}"
    m.close()


@pytest.mark.parametrize("ty", [K.Q4_0, K.Q5_0, K.Q5_1, K.Q8_0, K.Q4_K, K.Q6_K], ids=lambda t: O.TYPE_NAMES[t])
def test_zero_blocks_among_swept_f16_scales(pkg, gpu, ty):
    """langtax/src/simd/tests.rs:1481-1520: all-zero blocks (scale bits and codes zero) among blocks whose scales walk
    through every fifth finite binary16 pattern.  The whole sweep of langtax/src/simd/tests.rs:795-828, every pattern
    through every kernel family, is test_gpu_sweeps.py::test_every_finite_f16_scale_pattern_through_every_kernel_family."""
    rng = np.random.default_rng(7)
    bits = np.array([b for b in range(0, 65536, 5) if (b >> 10) & 0x1f != 31], np.uint16)
    per_row = 4096 // K.QK[ty]
    rows = bits.size // per_row
    bits = bits[:rows * per_row]
    w = K.random_packed(ty, rows, 4096, rng).reshape(rows * per_row, K.BLOCK[ty])
    off = 208 if ty == K.Q6_K else 0
    w[:, off:off + 2] = bits.view(np.uint8).reshape(-1, 2)
    if ty == K.Q6_K:
        w[:, 192:208] = rng.integers(-3, 4, (w.shape[0], 16)).astype(np.int8).view(np.uint8)  # keep |w| finite
    if ty in (K.Q4_K, K.Q5_1):
        w[:, 2:4] = 0  # min / offset scale zero: the swept field dominates
    w[5] = 0
    w = w.reshape(-1)
    x = rng.uniform(-1, 1, 4096).astype(np.float32) * np.float32(2.0 ** -6)
    m = gpu.upload_packed(ty, rows, 4096, w)
    y = np.full(rows, np.nan, np.float32)
    gpu.gemv_resident(m, x, y)
    exact, mag = O.gemm_f64_mag(ty, 4096, 1, w, x, rows)
    assert np.all(np.abs(y - exact[0]) <= K.single_kernel_bound(4096, mag[0]))
    m.close()


# ------------------------------------------------------------------ benchmark shapes
def _baseline_matrix(ty, rows, cols, rng):
    """Synthetic weights with the benchmark configurations' distributions: |N(0, 0.02)| block scales, uniform codes."""
    return K.random_packed(ty, rows, cols, rng, signed=False, scale=0.02)


def test_config1_q8_0_gemv_4096(pkg, gpu):
    rng = np.random.default_rng(42)
    w = _baseline_matrix(K.Q8_0, 4096, 4096, rng)
    x = rng.normal(0, 1, 4096).astype(np.float32)
    m = gpu.upload_packed(K.Q8_0, 4096, 4096, w)
    y = np.full(4096, np.nan, np.float32)
    gpu.gemv_resident(m, x, y)
    err, mag = check(y, K.Q8_0, 4096, 1, 4096, w, x, "config 1")
    # same inputs, the reference's scalar and AVX2 CPU orders: all three agree within twice the bound
    for simd in (False, True):
        cpu = O.gemm(K.Q8_0, 4096, 1, w, x, 4096, simd=simd, threads=0)[0]
        assert np.all(np.abs(cpu.astype(np.float64) - y) <= 2 * K.single_kernel_bound(4096, mag[0]))
    m.close()


@pytest.mark.parametrize("rows,cols", [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (4093, 14336), (13, 14336),
                                       (8, 14336), (1, 14336), (6150, 14336)])
def test_config2_q4_k_decode_shapes(pkg, gpu, rows, cols):
    rng = np.random.default_rng(rows + cols)
    w = _baseline_matrix(K.Q4_K, rows, cols, rng)
    x = rng.normal(0, 1, cols).astype(np.float32)
    m = gpu.upload_packed(K.Q4_K, rows, cols, w)
    y = np.full(rows, np.nan, np.float32)
    gpu.gemv_resident(m, x, y)
    check(y, K.Q4_K, cols, 1, rows, w, x, f"config 2 {rows}x{cols}")
    m.close()


def test_config2_q6_k_output_head(pkg, gpu):
    rows, cols = 128256, 4096
    rng = np.random.default_rng(6)
    w = _baseline_matrix(K.Q6_K, rows, cols, rng)
    x = rng.normal(0, 1, cols).astype(np.float32)
    m = gpu.upload_packed(K.Q6_K, rows, cols, w)
    y = np.full(rows, np.nan, np.float32)
    gpu.gemv_resident(m, x, y)
    check(y, K.Q6_K, cols, 1, rows, w, x, "config 2 head")
    # greedy decode takes the first maximum (langtax/src/decode.rs:12104-12114)
    exact = O.gemm_f64(K.Q6_K, cols, 1, w, x, rows)[0]
    top2 = np.sort(exact)[-2:]
    if top2[1] - top2[0] > 1e-3:
        assert int(np.argmax(y)) == int(np.argmax(exact))
    m.close()


@pytest.mark.parametrize("ty", [K.Q4_0, K.Q5_0, K.Q5_1], ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("rows,cols", [(4096, 14336), (14336, 4096)])
def test_config3_batched_gemm(pkg, gpu, ty, rows, cols):
    """M in {1, 8, 32, 128, 512}.  The oracle checks a fixed sample of weight rows at every M
    (all rows at M = 1); the rest is covered by a property that needs no oracle: row r of the
    batched product equals the GEMV of token r when the same token is repeated."""
    rng = np.random.default_rng(ty * 31 + rows)
    w = _baseline_matrix(ty, rows, cols, rng)
    m = gpu.upload_packed(ty, rows, cols, w)
    rb = K.row_bytes(ty, cols)
    sample = _edge_rows(rows, rng, 12)
    w_sample = np.concatenate([w[r * rb:(r + 1) * rb] for r in sample])
    x_all = rng.normal(0, 1, 512 * cols).astype(np.float32)
    for tokens in (1, 8, 32, 128, 512):
        x = x_all[:tokens * cols]
        y = np.full(tokens * rows, np.nan, np.float32)
        gpu.gemm_resident(m, tokens, x, y)
        y2 = y.reshape(tokens, rows)
        assert np.all(np.isfinite(y2))
        check(np.ascontiguousarray(y2[:, sample]), ty, cols, tokens, sample.size, w_sample, x,
              f"config 3 {O.TYPE_NAMES[ty]} M={tokens}")
        if tokens == 1:
            check(y, ty, cols, 1, rows, w, x, "config 3 M=1 all rows")
            y1 = y.copy()
        else:
            # token 0 is the M = 1 input: both kernels must agree within twice the f32 bound
            _, mag0 = O.gemm_f64_mag(ty, cols, 1, w_sample, x[:cols], sample.size)
            assert np.all(np.abs(y2[0, sample].astype(np.float64) - y1[sample]) <= 2 * K.single_kernel_bound(cols, mag0[0]))
    m.close()


def _edge_rows(rows, rng, n_random):
    """Rows to hold against the oracle when a product is too large to check whole: both sides of every kind
    of boundary the multi-token kernels have (16- and 32-row matrix-core sets, the 64 rows of a wavefront,
    the 256-row tile of a workgroup) at the start, in the middle and at the end of the matrix, plus a few
    random ones."""
    fixed = [0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 255, 256, 257]
    mid = (rows // 2) // 256 * 256
    fixed += [mid - 1, mid, mid + 63, mid + 64]
    last = (rows - 1) // 256 * 256
    fixed += [last - 1, last, last + 1, rows - 65, rows - 64, rows - 33, rows - 17, rows - 2, rows - 1]
    picks = np.concatenate([np.array(fixed), rng.integers(0, rows, n_random)])
    return np.unique(picks[(picks >= 0) & (picks < rows)])


def test_config5_expert_grouped_gemm(pkg, gpu):
    """Mixtral-shaped routing (8 experts, top-2, 64 tokens) over Q4_K expert matrices.  Full
    expert shapes for gate (14336x4096) and down (4096x14336); the oracle checks sampled rows."""
    rng = np.random.default_rng(5)
    n_exp, n_tok, d, ff = 8, 64, 4096, 14336
    logits = rng.normal(0, 1, (n_tok, n_exp)).astype(np.float32)
    # softmax -> top-2, ties to the lower index (langtax/src/decode.rs:11363-11379)
    order = np.argsort(-logits, axis=1, kind="stable")[:, :2]
    buckets = [[t for t in range(n_tok) if e in order[t]] for e in range(n_exp)]
    tokens = [len(b) for b in buckets]
    assert sum(tokens) == 2 * n_tok
    for rows, cols in ((ff, d), (d, ff)):
        experts = [_baseline_matrix(K.Q4_K, rows, cols, rng) for _ in range(n_exp)]
        mats = [gpu.upload_packed(K.Q4_K, rows, cols, w) for w in experts]
        xs = rng.normal(0, 1, (n_tok, cols)).astype(np.float32)
        x_packed = np.concatenate([xs[b].reshape(-1) for b in buckets])
        y = np.full(sum(tokens) * rows, np.nan, np.float32)
        gpu.gemm_grouped(mats, tokens, x_packed, y)
        rb = K.row_bytes(K.Q4_K, cols)
        sample = _edge_rows(rows, rng, 4)
        yo = 0
        for e in range(n_exp):
            ye = y[yo:yo + tokens[e] * rows].reshape(tokens[e], rows)
            yo += tokens[e] * rows
            ws = np.concatenate([experts[e][r * rb:(r + 1) * rb] for r in sample])
            check(np.ascontiguousarray(ye[:, sample]), K.Q4_K, cols, tokens[e], sample.size, ws,
                  xs[buckets[e]].reshape(-1), f"config 5 expert {e}")
            assert np.all(np.isfinite(ye))
        # one grouped call against the reference's sequence of per-expert calls: the same
        # products, but a launch shares out columns by its total size, so the f32 sums may
        # be formed in a different order
        y_seq = np.full_like(y, np.nan)
        yo = 0
        for e in range(n_exp):
            n = tokens[e] * rows
            gpu.gemm_resident(mats[e], tokens[e], xs[buckets[e]].reshape(-1), y_seq[yo:yo + n])
            yo += n
        rms = float(np.sqrt(np.mean(y_seq.astype(np.float64) ** 2)))
        assert np.max(np.abs(y.astype(np.float64) - y_seq)) <= 2e-5 * rms
        # and a repeated call is bit-identical (fixed summation order)
        y_again = np.full_like(y, np.nan)
        gpu.gemm_grouped(mats, tokens, x_packed, y_again)
        assert np.array_equal(y, y_again)
        for mm in mats:
            mm.close()


def test_grouped_gemm_with_empty_groups_and_dispatch_layer(pkg):
    """Experts nobody routed to are skipped (langtax/src/decode.rs:10043-10047)."""
    rng = np.random.default_rng(9)
    rows, cols = 96, 512
    parts = [K.random_packed(K.Q4_K, rows, cols, rng) for _ in range(4)]
    tokens = [3, 0, 1, 9]
    x = rng.normal(0, 1, sum(tokens) * cols).astype(np.float32)
    y = np.full(sum(tokens) * rows, np.nan, np.float32)
    pkg.reset()
    pkg.gemm_grouped(K.Q4_K, cols, rows, parts, tokens, x, y)
    assert pkg.cache_stats()["entries"] == 3  # the empty expert was never uploaded
    xo = yo = 0
    for e, t in enumerate(tokens):
        if t:
            check(y[yo:yo + t * rows], K.Q4_K, cols, t, rows, parts[e], x[xo:xo + t * cols], f"group {e}")
        xo += t * cols
        yo += t * rows


@pytest.mark.parametrize("ty", [K.Q4_0, K.Q5_1, K.Q8_0, K.Q4_K, K.Q6_K], ids=lambda t: O.TYPE_NAMES[t])
def test_grouped_call_with_token_counts_on_both_sides_of_every_kernel_switch(pkg, gpu, ty):
    """One grouped call whose products have 0, 1, 2, 3, 16, 17, 33 and 70 tokens: single-token launches
    (1 and 2), the 16-token tiles (3, 16; not Q6_K), the 32-token tiles (17) and the 64-token tiles (33, 70)
    inside one call, in an order that interleaves the classes.  Every group against the oracle, and bit for
    bit equal to the same product called on its own."""
    rng = np.random.default_rng(77 + ty)
    rows, cols = 160, 1024
    tokens = [17, 3, 0, 70, 1, 16, 2, 33]
    ws = [K.random_packed(ty, rows, cols, rng) for _ in tokens]
    mats = [gpu.upload_packed(ty, rows, cols, w) for w in ws]
    x = rng.normal(0, 1, sum(tokens) * cols).astype(np.float32)
    y = np.full(sum(tokens) * rows, np.nan, np.float32)
    gpu.gemm_grouped(mats, tokens, x, y)
    xo = yo = 0
    for g, t in enumerate(tokens):
        if t:
            yg, xg = y[yo:yo + t * rows], x[xo:xo + t * cols]
            check(yg, ty, cols, t, rows, ws[g], xg, f"{O.TYPE_NAMES[ty]} group {g} M={t}")
            alone = np.full(t * rows, np.nan, np.float32)
            gpu.gemm_resident(mats[g], t, xg, alone)
            if t <= 2:
                assert np.array_equal(yg, alone)  # the same single-token launches
            else:  # a launch shares out columns by its total size: the same products, another order of the f32 sums
                rms = float(np.sqrt(np.mean(alone.astype(np.float64) ** 2)))
                assert np.max(np.abs(yg.astype(np.float64) - alone)) <= 2e-5 * rms
        xo += t * cols
        yo += t * rows
    for m in mats:
        m.close()


def test_shared_input_products_equal_separate_calls(pkg, gpu):
    """q, k, v (and gate, up) read the same activations: one call, one input copy.  The values are those
    of the separate calls bit for bit (same kernels, same order of additions within each row)."""
    rng = np.random.default_rng(21)
    for ty, cols, rows_list in [(K.Q4_K, 4096, (4096, 1024, 1024)), (K.Q4_K, 14336, (100, 37, 4099)), (K.Q8_0, 1024, (256, 96)),
                                (K.Q6_K, 512, (64, 64, 64, 64)), (K.F16, 320, (33, 7))]:
        ws = [K.random_packed(ty, r, cols, rng) for r in rows_list]
        mats = [gpu.upload_packed(ty, r, cols, w) for r, w in zip(rows_list, ws)]
        for tokens in (1, 5, 40):
            x = rng.normal(0, 1, tokens * cols).astype(np.float32)
            y = np.full(tokens * sum(rows_list), np.nan, np.float32)
            gpu.gemm_shared(mats, tokens, x, y)
            off = 0
            for r, w, m in zip(rows_list, ws, mats):
                part = y[off:off + tokens * r]
                check(part, ty, cols, tokens, r, w, x, f"shared {pkg.TYPE_NAMES[ty]} rows {r} tokens {tokens}")
                alone = np.full(tokens * r, np.nan, np.float32)
                gpu.gemm_resident(m, tokens, x, alone)
                if tokens == 1:
                    assert part.view(np.uint32).tolist() == alone.view(np.uint32).tolist()
                else:  # the split of long rows over workgroups is sized by the whole launch
                    assert np.abs(part - alone).max() <= 2e-5 * np.sqrt(np.mean(alone.astype(np.float64) ** 2))
                off += tokens * r
        with pytest.raises(pkg.NativeHipError, match="buffer lengths"):
            gpu.gemm_shared(mats, 2, np.zeros(cols, np.float32), np.zeros(2 * sum(rows_list), np.float32))
        for m in mats:
            m.close()
    a = gpu.upload_packed(K.Q8_0, 32, 256, K.random_packed(K.Q8_0, 32, 256, rng))
    b = gpu.upload_packed(K.Q8_0, 32, 512, K.random_packed(K.Q8_0, 32, 512, rng))
    with pytest.raises(pkg.NativeHipError, match="same column count"):
        gpu.gemm_shared([a, b], 1, np.zeros(256, np.float32), np.zeros(64, np.float32))
    with pytest.raises(pkg.NativeHipError, match="at least one token"):
        gpu.gemm_shared([a], 0, np.zeros(0, np.float32), np.zeros(0, np.float32))


# ------------------------------------------------------------------ residency
def test_residency_lru_and_budget(pkg, monkeypatch):
    """langtax/src/native_gpu.rs:161-211: hit moves to the back, admission evicts from the front,
    an over-budget matrix runs once and is not kept, budget 0 disables residency but not the GPU."""
    rng = np.random.default_rng(11)
    rows, cols = 64, 256
    mats = [K.random_packed(K.Q8_0, rows, cols, rng) for _ in range(4)]
    x = rng.normal(0, 1, cols).astype(np.float32)

    def run(w):
        y = np.full(rows, np.nan, np.float32)
        pkg.gemv(K.Q8_0, cols, w, x, y)
        check(y, K.Q8_0, cols, 1, rows, w, x)

    g = pkg.HipGemv(0)
    probe = g.upload_packed(K.Q8_0, rows, cols, mats[0])
    entry = probe.info()[3] + mats[0].size  # device planes + host identity copy
    probe.close()
    g.close()

    monkeypatch.setenv("LLAMA_HIP_CACHE_BYTES", str(2 * entry + 8))
    pkg.reset()
    run(mats[0]); run(mats[1])
    assert pkg.cache_stats()["entries"] == 2 and pkg.cache_stats()["misses"] == 2
    run(mats[0])                                     # hit: 0 becomes most recent
    assert pkg.cache_stats()["hits"] == 1
    run(mats[2])                                     # evicts 1 (front), keeps 0
    s = pkg.cache_stats()
    assert s["entries"] == 2 and s["bytes"] == 2 * entry
    run(mats[0])
    assert pkg.cache_stats()["hits"] == 2
    run(mats[1])                                     # 1 was evicted: a miss again
    assert pkg.cache_stats()["misses"] == 4

    monkeypatch.setenv("LLAMA_HIP_CACHE_BYTES", str(entry - 1))
    pkg.reset()
    run(mats[3]); run(mats[3])                       # over budget: runs, never retained
    s = pkg.cache_stats()
    assert s["entries"] == 0 and s["bytes"] == 0 and s["misses"] == 2

    monkeypatch.setenv("LLAMA_HIP_CACHE_BYTES", "0")
    pkg.reset()
    run(mats[0])
    assert pkg.cache_stats()["entries"] == 0

    monkeypatch.setenv("LLAMA_HIP_CACHE_BYTES", "lots")
    pkg.reset()
    with pytest.raises(pkg.NativeHipError, match="must be auto or a nonnegative decimal byte count"):
        run(mats[0])
    monkeypatch.delenv("LLAMA_HIP_CACHE_BYTES")
    pkg.reset()
    run(mats[0])
    assert pkg.cache_stats()["limit"] > (1 << 30)    # automatic budget on a 288 GB device


def test_residency_charges_the_multi_token_layout_when_it_appears(pkg, monkeypatch):
    """A cached matrix is charged for what it holds on the device: the single-token layout from its upload, the
    multi-token layout from the first product of three or more tokens on (it is made then, not before).  A
    budget that takes the first and not both keeps the matrix while it only meets single tokens and drops it
    after the product that made it grow."""
    rng = np.random.default_rng(21)
    rows, cols = 256, 512
    w = K.random_packed(K.Q4_K, rows, cols, rng, signed=False, scale=0.02)
    g = pkg.HipGemv(0)
    probe = g.upload_packed(K.Q4_K, rows, cols, w)
    single = probe.info()[3]
    g.prepare(probe, 8)
    both = probe.info()[3]
    probe.close()
    g.close()
    assert both > single

    def run(tokens):
        x = rng.normal(0, 1, tokens * cols).astype(np.float32)
        y = np.full(tokens * rows, np.nan, np.float32)
        pkg.gemm(K.Q4_K, cols, tokens, w, x, y)
        check(y, K.Q4_K, cols, tokens, rows, w, x)

    monkeypatch.setenv("LLAMA_HIP_CACHE_BYTES", str(1 << 30))
    pkg.reset()
    run(1)
    assert pkg.cache_stats()["bytes"] == single + w.size
    run(2)                                            # two tokens are two single-token launches
    assert pkg.cache_stats()["bytes"] == single + w.size
    run(8)
    s = pkg.cache_stats()
    assert s["bytes"] == both + w.size and s["entries"] == 1 and s["hits"] == 2
    pkg.reset()
    run(8)                                            # a miss that is a multi-token product is charged in full at once
    assert pkg.cache_stats()["bytes"] == both + w.size

    monkeypatch.setenv("LLAMA_HIP_CACHE_BYTES", str(single + w.size + 16))
    pkg.reset()
    run(1); run(1)
    s = pkg.cache_stats()
    assert s["entries"] == 1 and s["hits"] == 1
    run(8)                                            # correct result, then over budget: not kept
    s = pkg.cache_stats()
    assert s["entries"] == 0 and s["bytes"] == 0
    run(8)                                            # over budget from the start: runs once, never retained
    assert pkg.cache_stats()["entries"] == 0
    monkeypatch.delenv("LLAMA_HIP_CACHE_BYTES")
    pkg.reset()


def test_edge_sample_collision_does_not_alias(pkg):
    """langtax/src/native_gpu.rs:217-260: same dtype, shape, first and last 32 bytes, different middle."""
    rng = np.random.default_rng(12)
    rows, cols = 8, 256
    a = K.random_packed(K.Q8_0, rows, cols, rng)
    b = a.copy()
    b[a.size // 2] ^= 0x55
    x = rng.normal(0, 1, cols).astype(np.float32)
    pkg.reset()
    ya, yb = np.zeros(rows, np.float32), np.zeros(rows, np.float32)
    pkg.gemv(K.Q8_0, cols, a, x, ya)
    pkg.gemv(K.Q8_0, cols, b, x, yb)
    check(ya, K.Q8_0, cols, 1, rows, a, x)
    check(yb, K.Q8_0, cols, 1, rows, b, x)
    assert not np.array_equal(ya, yb)
    assert pkg.cache_stats()["entries"] == 2


# ------------------------------------------------------------------ device-resident buffers
def test_device_pointer_entry_points_match_host_path(pkg, gpu):
    import importlib
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(13)
    stream = hip.Stream()
    for ty, rows, cols in ((K.Q4_K, 300, 1024), (K.Q8_0, 300, 1024), (K.F16, 70, 333)):
        w = K.random_packed(ty, rows, cols, rng)
        m_host = gpu.upload_packed(ty, rows, cols, w)
        wd = hip.DeviceBuffer.from_numpy(w)
        m_dev = gpu.upload_packed_device(ty, rows, cols, wd.ptr, w.size)
        wd.free()
        for tokens in (1, 6):
            x = rng.normal(0, 1, tokens * cols).astype(np.float32)
            y_host = np.zeros(tokens * rows, np.float32)
            gpu.gemm_resident(m_host, tokens, x, y_host)
            xd = hip.DeviceBuffer.from_numpy(x)
            yd = hip.DeviceBuffer(tokens * rows * 4)
            yd.fill_byte(0xff)
            for s in (stream.ptr, 0):          # caller's stream, then the executor's own
                gpu.gemm_device(m_dev, tokens, xd.ptr, yd.ptr, s)
                stream.synchronize()
                gpu.synchronize()
                assert np.array_equal(yd.to_numpy(np.float32), y_host)
                yd.fill_byte(0xff)
            xd.free()
            yd.free()
        m_host.close()
        m_dev.close()
    stream.destroy()


@pytest.mark.parametrize("ty", O.ALL_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_batch_entry_point_fuses_products_that_share_an_input(pkg, gpu, ty):
    """lnh_gemm_batch_device: products reading the same x (q/k/v, gate/up) go out as one launch;
    the result must be bit-identical to issuing them one by one."""
    import importlib
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(50 + ty)
    cols = 1024 if K.QK[ty] > 1 else 1000
    shapes = [(300, cols), (77, cols), (64, cols), (129, 512), (5, cols)]
    ws = [K.random_packed(ty, r, c, rng) for r, c in shapes]
    mats = [gpu.upload_packed(ty, r, c, w) for (r, c), w in zip(shapes, ws)]
    xa = rng.normal(0, 1, cols).astype(np.float32)
    xb = rng.normal(0, 1, 512).astype(np.float32)
    xa_d, xb_d = hip.DeviceBuffer.from_numpy(xa), hip.DeviceBuffer.from_numpy(xb)
    x_ptrs = [xa_d.ptr, xa_d.ptr, xa_d.ptr, xb_d.ptr, xa_d.ptr]   # first three fuse, then two singles
    ys = [hip.DeviceBuffer(r * 4) for r, _ in shapes]
    for y in ys:
        y.fill_byte(0xff)
    batch = gpu.make_batch(mats, [1] * len(mats), x_ptrs, [y.ptr for y in ys])
    gpu.gemm_batch_device(batch)
    gpu.synchronize()
    for (r, c), w, m, xp, y in zip(shapes, ws, mats, x_ptrs, ys):
        x = xa if xp == xa_d.ptr else xb
        got = y.to_numpy(np.float32)
        check(got, ty, c, 1, r, w, x, f"batch {O.TYPE_NAMES[ty]} {r}x{c}")
        alone = np.zeros(r, np.float32)
        gpu.gemv_resident(m, x, alone)
        assert np.array_equal(got, alone)
    for b in ys + [xa_d, xb_d]:
        b.free()
    for m in mats:
        m.close()


@pytest.mark.parametrize("ty", [K.Q4_K, K.Q6_K, K.Q8_0])
@pytest.mark.parametrize("tokens", [5, 20])
def test_deferred_norm_of_zero_rows_without_eps(pkg, gpu, ty, tokens):
    """LNH_EPILOGUE_ADD_RMSNORM_DEFERRED where the factor has its special case: a residual row that stays zero with
    eps = 0 (rms = 0: the row is scaled by 0, decode.rs:11498-11513), next to rows of very different magnitude; the
    reading product equals the one after LNH_EPILOGUE_ADD_RMSNORM bit for bit, and the zero row's outputs are 0."""
    import importlib
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(1300 + ty * 5 + tokens)
    d, ff = 1024, 256
    w_o, w_g = K.random_packed(ty, d, d, rng, signed=True, scale=0.05), K.random_packed(ty, ff, d, rng, signed=True, scale=0.05)
    m_o, m_g = gpu.upload_packed(ty, d, d, w_o), gpu.upload_packed(ty, ff, d, w_g)
    x0 = rng.normal(0, 1, (tokens, d)).astype(np.float32)
    res0 = (rng.normal(0, 1, (tokens, d)) * np.logspace(-6, 6, tokens)[:, None]).astype(np.float32)
    x0[1] = 0
    res0[1] = 0
    g = (1 + rng.normal(0, 0.05, d)).astype(np.float32)
    dev = lambda a: hip.DeviceBuffer.from_numpy(np.ascontiguousarray(a).reshape(-1))
    d_x0, d_g = dev(x0), dev(g)
    a_n = gpu.act_create(ty, d, tokens)
    outs = []
    for epilogue in (pkg.EPILOGUE_ADD_RMSNORM, pkg.EPILOGUE_ADD_RMSNORM_DEFERRED):
        d_res, d_y = dev(res0), hip.DeviceBuffer(tokens * ff * 4)
        gpu.gemm_plain_act_device([m_o], d_x0.ptr, tokens, None, epilogue, d_res.ptr, d_g.ptr, 0.0, 0, a_n)
        gpu.gemm_act_device([m_g], a_n, tokens, [d_y.ptr])
        gpu.synchronize()
        outs.append((d_res.to_numpy(np.float32), d_y.to_numpy(np.float32).reshape(tokens, ff)))
        d_res.free(); d_y.free()
    assert np.array_equal(outs[0][0], outs[1][0])
    assert np.array_equal(outs[0][1], outs[1][1])
    assert np.all(np.isfinite(outs[1][1])) and not np.any(outs[1][1][1]) and np.any(outs[1][1][0])
    a_n.close()
    for m in (m_o, m_g):
        m.close()
    for b in (d_x0, d_g):
        b.free()


@pytest.mark.parametrize("ty", [K.Q4_K, K.Q4_0, K.Q6_K, K.Q5_0, K.Q5_1, K.Q8_0])
@pytest.mark.parametrize("tokens", [3, 8, 16, 17, 24, 32, 40, 130])
def test_split_activations_chain_equals_separate_launches(pkg, gpu, ty, tokens):
    """lnh_act_* / lnh_gemm_act_device: a chain of three products (o-like with the residual + RMSNorm epilogue, a
    gate/up pair with the SiLU(gate) * up epilogue, a down-like product with a plain sum) whose activations stay in
    the split form, against the same chain through lnh_gemm_device with the element-wise steps on the host: the
    products and the residual bit for bit (same kernels, same order of additions), the steps whose host form uses
    other roundings (sum of squares, exp) through the next product within 2e-5 of its magnitude."""
    import importlib
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(900 + ty * 7 + tokens)
    d, ff = 512, 768
    w_o, w_g, w_u, w_d = (K.random_packed(ty, r, c, rng, signed=False, scale=0.05)
                          for r, c in ((d, d), (ff, d), (ff, d), (d, ff)))
    m_o, m_g, m_u, m_d = (gpu.upload_packed(ty, r, c, w) for (r, c), w in (((d, d), w_o), ((ff, d), w_g), ((ff, d), w_u), ((d, ff), w_d)))
    x0 = rng.normal(0, 1, (tokens, d)).astype(np.float32)
    res0 = rng.normal(0, 1, (tokens, d)).astype(np.float32)
    g = (1 + rng.normal(0, 0.05, d)).astype(np.float32)
    eps = 1e-5
    dev = lambda a: hip.DeviceBuffer.from_numpy(np.ascontiguousarray(a).reshape(-1))
    d_x0, d_res, d_g = dev(x0), dev(res0), dev(g)
    d_xn, d_y = hip.DeviceBuffer(tokens * d * 4), hip.DeviceBuffer(tokens * d * 4)
    a_o, a_gu, a_d = gpu.act_create(ty, d, tokens + 5), gpu.act_create(ty, d, tokens), gpu.act_create(ty, ff, 2 * tokens)
    gpu.act_split_device(a_o, tokens, d_x0.ptr)
    gpu.gemm_act_device([m_o], a_o, tokens, None, pkg.EPILOGUE_ADD_RMSNORM, d_res.ptr, d_g.ptr, eps, d_xn.ptr, a_gu)
    gpu.gemm_act_device([m_g, m_u], a_gu, tokens, None, pkg.EPILOGUE_SWIGLU, next_act=a_d)
    gpu.gemm_act_device([m_d], a_d, tokens, [d_y.ptr])
    gpu.synchronize()
    got_res = d_res.to_numpy(np.float32).reshape(tokens, d)
    got_xn = d_xn.to_numpy(np.float32).reshape(tokens, d)
    got_y = d_y.to_numpy(np.float32).reshape(tokens, d)

    def product(m, rows, x):
        dx, dy = dev(x), hip.DeviceBuffer(x.shape[0] * rows * 4)
        gpu.gemm_device(m, x.shape[0], dx.ptr, dy.ptr)
        gpu.synchronize()
        y = dy.to_numpy(np.float32).reshape(x.shape[0], rows)
        dx.free(); dy.free()
        return y

    # the o-like product and the residual addition: bit for bit
    want_res = res0 + product(m_o, d, x0)
    assert np.array_equal(got_res, want_res)
    # RMSNorm of the new residual: against float64
    r64 = want_res.astype(np.float64)
    xn64 = r64 / np.sqrt(np.mean(r64 * r64, axis=1, keepdims=True) + eps) * g.astype(np.float64)
    assert np.abs(got_xn - xn64).max() <= 4e-6 * np.abs(xn64).max()
    # what the gate/up pair read is the split of exactly those rows: the pair's products of got_xn, SiLU * up on
    # the host, the down-like product of that, against the chain's result
    gate, up = product(m_g, ff, got_xn), product(m_u, ff, got_xn)
    with np.errstate(over="ignore"):
        h = (gate.astype(np.float64) / (1 + np.exp(-gate.astype(np.float64))) * up.astype(np.float64)).astype(np.float32)
    want_y = product(m_d, d, h)
    _, mag = O.gemm_f64_mag(ty, ff, tokens, w_d, h.reshape(-1), d)
    assert np.all(np.abs(got_y - want_y) <= 2e-5 * np.asarray(mag).reshape(tokens, d) + 1e-30), \
        float(np.max(np.abs(got_y - want_y) / (np.asarray(mag).reshape(tokens, d) + 1e-30)))
    # a plain sum after split activations is the three-launch product itself
    d_y2 = hip.DeviceBuffer(tokens * ff * 4)
    gpu.act_split_device(a_gu, tokens, dev(got_xn).ptr)
    gpu.gemm_act_device([m_g], a_gu, tokens, [d_y2.ptr])
    gpu.synchronize()
    assert np.array_equal(d_y2.to_numpy(np.float32).reshape(tokens, ff), gate)
    # the same chain entered with plain rows (lnh_gemm_plain_act_device: up to 16 tokens the product's launch cuts
    # them itself, more are cut into the workspace first): the same bits as through lnh_act_split_device
    d_res2, d_xn2, d_y3 = dev(res0), hip.DeviceBuffer(tokens * d * 4), hip.DeviceBuffer(tokens * d * 4)
    gpu.gemm_plain_act_device([m_o], d_x0.ptr, tokens, None, pkg.EPILOGUE_ADD_RMSNORM, d_res2.ptr, d_g.ptr, eps, d_xn2.ptr, a_gu)
    gpu.gemm_act_device([m_g, m_u], a_gu, tokens, None, pkg.EPILOGUE_SWIGLU, next_act=a_d)
    gpu.gemm_act_device([m_d], a_d, tokens, [d_y3.ptr])
    gpu.synchronize()
    assert np.array_equal(d_res2.to_numpy(np.float32).reshape(tokens, d), got_res)
    assert np.array_equal(d_xn2.to_numpy(np.float32).reshape(tokens, d), got_xn)
    assert np.array_equal(d_y3.to_numpy(np.float32).reshape(tokens, d), got_y)
    d_y4, d_y5 = hip.DeviceBuffer(tokens * ff * 4), hip.DeviceBuffer(tokens * ff * 4)
    d_gxn = dev(got_xn)
    gpu.gemm_plain_act_device([m_g, m_u], d_gxn.ptr, tokens, [d_y4.ptr, d_y5.ptr])
    gpu.synchronize()
    assert np.array_equal(d_y4.to_numpy(np.float32).reshape(tokens, ff), gate)
    assert np.array_equal(d_y5.to_numpy(np.float32).reshape(tokens, ff), up)
    with pytest.raises(pkg.NativeHipError, match="one dtype and column count"):
        gpu.gemm_plain_act_device([m_g, m_d], d_gxn.ptr, tokens, [d_y4.ptr, d_y5.ptr])
    # the residual epilogue with its norm left to the reading product (up to 32 tokens): o-like -> gate/up -> down-like
    # -> a gate product of the second norm, the same bits as with the norm formed in the epilogue
    a_n = gpu.act_create(ty, d, tokens + 1)
    d_y6, d_y7 = hip.DeviceBuffer(tokens * ff * 4), hip.DeviceBuffer(tokens * ff * 4)
    d_res4 = dev(res0)
    gpu.gemm_plain_act_device([m_o], d_x0.ptr, tokens, None, pkg.EPILOGUE_ADD_RMSNORM, d_res4.ptr, d_g.ptr, eps, 0, a_gu)
    gpu.gemm_act_device([m_g, m_u], a_gu, tokens, None, pkg.EPILOGUE_SWIGLU, next_act=a_d)
    gpu.gemm_act_device([m_d], a_d, tokens, None, pkg.EPILOGUE_ADD_RMSNORM, d_res4.ptr, d_g.ptr, eps, 0, a_n)
    gpu.gemm_act_device([m_g], a_n, tokens, [d_y6.ptr])
    gpu.synchronize()
    if tokens <= 32:
        d_res3 = dev(res0)
        gpu.gemm_plain_act_device([m_o], d_x0.ptr, tokens, None, pkg.EPILOGUE_ADD_RMSNORM_DEFERRED, d_res3.ptr, d_g.ptr, eps, 0, a_gu)
        gpu.gemm_act_device([m_g, m_u], a_gu, tokens, None, pkg.EPILOGUE_SWIGLU, next_act=a_d)
        gpu.gemm_act_device([m_d], a_d, tokens, None, pkg.EPILOGUE_ADD_RMSNORM_DEFERRED, d_res3.ptr, d_g.ptr, eps, 0, a_n)
        gpu.gemm_act_device([m_g], a_n, tokens, [d_y7.ptr])
        gpu.synchronize()
        assert np.array_equal(d_res3.to_numpy(np.float32), d_res4.to_numpy(np.float32))
        assert np.array_equal(d_y7.to_numpy(np.float32), d_y6.to_numpy(np.float32))
        with pytest.raises(pkg.NativeHipError, match="another token count"):
            gpu.gemm_act_device([m_g], a_n, tokens + 1, [d_y7.ptr])
        with pytest.raises(pkg.NativeHipError, match="no plain normalised rows"):
            gpu.gemm_act_device([m_d], a_d, tokens, None, pkg.EPILOGUE_ADD_RMSNORM_DEFERRED, d_res3.ptr, d_g.ptr, eps, d_xn.ptr, a_n)
        # filling the activations any other way ends the deferral
        gpu.act_split_device(a_n, tokens, d_gxn.ptr)
        gpu.gemm_act_device([m_g], a_n, tokens, [d_y7.ptr])
        gpu.synchronize()
        assert np.array_equal(d_y7.to_numpy(np.float32).reshape(tokens, ff), gate)
    else:
        with pytest.raises(pkg.NativeHipError, match="at most 32 tokens"):
            gpu.gemm_act_device([m_d], a_d, tokens, None, pkg.EPILOGUE_ADD_RMSNORM_DEFERRED, d_res4.ptr, d_g.ptr, eps, 0, a_n)
    a_n.close()
    # refusals: fewer than three tokens, another dtype's activations, capacity
    with pytest.raises(pkg.NativeHipError, match="three or more tokens"):
        gpu.gemm_act_device([m_d], a_d, 2, [d_y.ptr])
    with pytest.raises(pkg.NativeHipError, match="another dtype or column count"):
        gpu.gemm_act_device([m_d], a_o, tokens, [d_y.ptr])
    with pytest.raises(pkg.NativeHipError, match="capacity"):
        gpu.act_split_device(a_gu, tokens + 1, d_x0.ptr)
    with pytest.raises(pkg.NativeHipError, match="block-quantized"):
        gpu.act_create(K.F16, d, tokens)
    for a in (a_o, a_gu, a_d):
        a.close()
    for m in (m_o, m_g, m_u, m_d):
        m.close()
