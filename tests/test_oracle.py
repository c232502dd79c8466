"""Pins the CPU oracle (oracle/) before anything is compared with it.

Each check is independent of the oracle's own formulas: published known
answers from the reference's files, byte-level layouts asserted by the
reference's tests, numpy's float16, dequantizers written separately in numpy,
exact rational arithmetic on the reference's closed-form fixtures, and the
error bound the reference proves for any f32 summation order.
"""
import json
import os
from fractions import Fraction

import numpy as np
import pytest

import cases as K
import oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_kats.json")
with open(GOLDEN) as fh:
    KAT = json.load(fh)

QUANT_TYPES = [K.Q4_0, K.Q5_0, K.Q5_1, K.Q8_0, K.Q4_K, K.Q6_K]


# ---------------------------------------------------------------- published known answers
def test_published_q8_gemv_checksum():
    """README.md:274-291: y_checksum and y0 of the 4096x4096 demo GEMV."""
    h, y = O.demo_q8_gemv(4096, 4096)
    assert f"{h:016x}" == KAT["q8_demo"]["y_checksum"]
    assert f"{y[0]:.6f}" == KAT["q8_demo"]["y0"]


def test_splitmix64_published_outputs():
    """langtax/src/sample.rs:566-575."""
    s = O.SplitMix64(0)
    for want in KAT["splitmix64"]["seed0"]:
        assert s.next() == int(want, 16)
    assert s.next() >> 40 == KAT["splitmix64"]["seed0_fourth_shr40"]
    assert O.SplitMix64(1).next() == int(KAT["splitmix64"]["seed1_first"], 16)


# ---------------------------------------------------------------- binary16
def _f16_definition(h):
    """The arithmetic definition (langtax/src/fp16.rs:71-103), in exact rationals."""
    sign = -1 if h & 0x8000 else 1
    e, m = (h >> 10) & 0x1f, h & 0x3ff
    if e == 0:
        return sign * Fraction(m, 1 << 24)
    return sign * (1 + Fraction(m, 1024)) * (Fraction(2) ** (e - 15))


def test_f16_decode_every_pattern():
    lib = O.load()
    bits = np.arange(65536, dtype=np.uint16)
    got = np.array([lib.lro_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    want = bits.view(np.float16).astype(np.float32)
    fin = np.isfinite(want)
    assert np.array_equal(got[fin].view(np.uint32), want[fin].view(np.uint32))
    assert np.array_equal(np.isinf(got), np.isinf(want))
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.signbit(got[~np.isnan(want)]), np.signbit(want[~np.isnan(want)]))
    # and against the definition itself, on a stride that covers every exponent
    for h in list(range(0, 65536, 37)) + [1, 0x3ff, 0x400, 0x8001, 0x7bff, 0xfbff]:
        if (h >> 10) & 0x1f == 31:
            continue
        assert Fraction(float(got[h])) == _f16_definition(h), hex(h)


def test_f16_encode_truncates_and_round_trips():
    lib = O.load()
    # every finite binary16 value encodes back to its own bits (incl. subnormals, -0)
    for h in range(0, 65536):
        if (h >> 10) & 0x1f == 31:
            continue
        f = np.array([h], np.uint16).view(np.float16).astype(np.float32)[0]
        assert lib.lro_f32_to_f16(float(f)) == h, hex(h)
    # round toward zero: |decode(encode(x))| <= |x| and within one binary16 step
    rng = np.random.default_rng(1)
    xs = np.concatenate([rng.normal(0, 1, 2000), rng.normal(0, 1e-3, 2000), rng.normal(0, 3e-6, 500),
                         [0.1, -0.1, 65504.0, 65519.9, 1e-8, 7e4, -7e4]]).astype(np.float32)
    for x in xs:
        h = lib.lro_f32_to_f16(float(x))
        back = float(np.array([h], np.uint16).view(np.float16)[0])
        if abs(x) >= 65536.0:
            assert h & 0x7fff == 0x7c00
            continue
        assert abs(back) <= abs(float(x))
        nxt = float(np.array([(h & 0x7fff) + 1], np.uint16).view(np.float16)[0])
        assert abs(float(x)) < nxt or not np.isfinite(nxt)
    # the reference's own byte-level example: 0.25 -> 0x3400
    assert lib.lro_f32_to_f16(0.25) == 0x3400


# ---------------------------------------------------------------- packers / layouts
def test_q5_0_pack_bytes_known_answer():
    """langtax/src/quant.rs:10907-10926."""
    qs = np.zeros(32, np.uint8)
    qs[0], qs[16], qs[7], qs[23] = 19, 28, 7, 15
    w = O.pack_q5_0_block(0.25, qs)
    assert w.size == 22
    assert w[6] == 0xc3 and w[13] == 0xf7
    qh = int(w[2:6].view(np.uint32)[0])
    assert qh & 0x00010001 == 0x00010001
    assert qh & ((1 << 7) | (1 << 23)) == 0
    x = np.zeros(32, np.float32)
    x[0], x[16], x[7], x[23] = 2.0, 4.0, 1.0, 3.0
    # (19-16)*.25*2 + (28-16)*.25*4 + (7-16)*.25*1 + (15-16)*.25*3
    assert O.vec_dot_row(K.Q5_0, 32, w, x) == np.float32(1.5 + 12.0 - 2.25 - 0.75)
    assert O.vec_dot_row(K.Q5_0, 32, w, x, simd=True) == np.float32(10.5)


def test_q5_1_pack_bytes_known_answer():
    """langtax/src/quant.rs:11028-11046: the reference's byte-level answers for a Q5_1 block, and its
    dot against values decoded here from those bytes (numpy float16), not by the oracle's dequantizer."""
    qs = np.zeros(32, np.uint8)
    qs[0], qs[16], qs[7], qs[23] = 19, 28, 7, 15
    w = O.pack_q5_1_block(25.0 / 100.0, 5.0 / 100.0, qs)
    assert w.size == 24
    assert w[8] == 0xc3                                   # low nibble y[0] = 19, high nibble y[16] = 28
    qh = int(w[4:8].view(np.uint32)[0])
    assert qh & 0x00010001 == 0x00010001                  # their fifth bits
    assert w[15] == 0xf7                                  # low nibble y[7] = 7, high nibble y[23] = 15
    assert qh & ((1 << 7) | (1 << 23)) == 0
    d, m = (float(v) for v in w[0:4].view(np.float16))
    assert d == 0.25 and abs(m - 0.05) < 2 ** -14 and m <= 0.05   # the encoder rounds toward zero
    x = np.zeros(32, np.float32)
    x[0], x[16], x[7], x[23] = 2.0, 4.0, 1.0, 3.0
    codes = np.zeros(32)
    codes[[0, 16, 7, 23]] = 19, 28, 7, 15
    expected = float(np.sum((codes * d + m) * x))
    for simd in (False, True):
        got = float(O.vec_dot_row(K.Q5_1, 32, w, x, simd=simd))
        assert abs(got - expected) / (1 + abs(expected)) < 1e-5
    row = O.dequant(K.Q5_1, 32, w, 1)[0]
    assert row.tolist() == (np.float32(codes) * np.float32(d) + np.float32(m)).tolist()   # two roundings, no FMA


def test_q4_0_low_and_high_nibbles_are_elements_j_and_j_plus_16():
    """langtax/src/gguf.rs:1130-1137: v[0] = 1, v[16] = 2 packed at scale 1 against x[0] = 3, x[16] = 4
    gives 11 (a kernel that read the nibbles as neighbours x[2j], x[2j+1] would give 3)."""
    v = np.zeros(32, np.int8)
    v[0], v[16] = 1, 2
    w = O.pack_q4_0_block(1.0, v)
    assert w[0:2].view(np.float16)[0] == 1.0
    assert w[2] == 0xa9                                   # (1 + 8) | (2 + 8) << 4
    assert np.all(w[3:] == 0x88)                          # zero codes carry the bias 8 in both nibbles
    x = np.zeros(32, np.float32)
    x[0], x[16] = 3.0, 4.0
    assert O.vec_dot_row(K.Q4_0, 32, w, x) == np.float32(11.0)
    assert O.vec_dot_row(K.Q4_0, 32, w, x, simd=True) == np.float32(11.0)
    row = O.dequant(K.Q4_0, 32, w, 1)[0]
    assert row[0] == 1.0 and row[16] == 2.0 and np.count_nonzero(row) == 2


def test_q4_k_scale_pack_round_trip_all_values():
    """Every 6-bit scale/min through pack -> scale_min_k4 (quant.rs:4852-4878, 8901-8912)."""
    rng = np.random.default_rng(7)
    for trial in range(64):
        sc = (np.arange(8) * 9 + trial) % 64
        mn = (np.arange(8) * 5 + 63 - trial) % 64
        blk = O.pack_q4_k_block(1.0, 1.0, sc, mn, np.zeros(256, np.uint8))
        s = blk[4:16]
        for j in range(8):
            # independent statement of ggml's get_scale_min_k4
            if j < 4:
                want = (s[j] & 63, s[j + 4] & 63)
            else:
                want = ((s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4), (s[j + 4] >> 4) | ((s[j] >> 6) << 4))
            assert O.scale_min_k4(s, j) == (int(want[0]), int(want[1])) == (int(sc[j]), int(mn[j]))


def test_q8_0_and_q4_0_pack_layout():
    q = (np.arange(32) * 7 % 256 - 128).astype(np.int8)
    b = O.pack_q8_0_block(0.5, q)
    assert bytes(b[:2]) == b"\x00\x38" and np.array_equal(b[2:].view(np.int8), q)
    v = ((np.arange(32) * 5) % 16 - 8).astype(np.int8)
    b4 = O.pack_q4_0_block(2.0, v)
    assert bytes(b4[:2]) == b"\x00\x40"
    for j in range(16):
        assert b4[2 + j] == ((int(v[j]) + 8) | ((int(v[j + 16]) + 8) << 4))


def test_q6_k_pack_layout_matches_definition():
    rng = np.random.default_rng(3)
    q = rng.integers(-32, 32, 256).astype(np.int8)
    sc = rng.integers(-128, 128, 16).astype(np.int8)
    b = O.pack_q6_k_block(0.5, sc, q)
    assert b.size == 210 and bytes(b[208:210]) == b"\x00\x38"
    assert np.array_equal(b[192:208].view(np.int8), sc)
    w = K.np_dequant(K.Q6_K, 1, 256, b)[0]
    want = np.float32(0.5) * np.repeat(sc.astype(np.float32), 16) * q.astype(np.float32)
    assert np.array_equal(w, want)


# ---------------------------------------------------------------- hand-computable cases
def test_q6_k_one_nonzero_is_eleven():
    """langtax/src/quant.rs:10321-10343."""
    q = np.zeros(256, np.int8)
    q[0], q[32] = 1, 2
    sc = np.zeros(16, np.int8)
    sc[0], sc[2] = 1, 1
    w = O.pack_q6_k_block(1.0, sc, q)
    x = np.zeros(256, np.float32)
    x[0], x[32] = 3.0, 4.0
    assert O.vec_dot_row(K.Q6_K, 256, w, x) == np.float32(11.0)
    assert O.vec_dot_row(K.Q6_K, 256, w, x, simd=True) == np.float32(11.0)
    assert float(np.dot(O.dequant_row(K.Q6_K, 256, w), x)) == 11.0


def test_q4_k_sparse_case():
    """langtax/src/quant.rs:10347-10367: 0.25*2*3*2 + 0.25*1*5*4 = 8."""
    q = np.zeros(256, np.uint8)
    q[0], q[32] = 3, 5
    w = O.pack_q4_k_block(0.25, 0.0, [2, 1, 1, 1, 1, 1, 1, 1], [0] * 8, q)
    x = np.zeros(256, np.float32)
    x[0], x[32] = 2.0, 4.0
    assert O.vec_dot_row(K.Q4_K, 256, w, x) == np.float32(8.0)
    assert O.vec_dot_row(K.Q4_K, 256, w, x, simd=True) == np.float32(8.0)


def test_q4_k_dense_fused_equals_dequant_then_sequential_dot_bitwise():
    """langtax/src/quant.rs:10373-10393."""
    q = (np.arange(256) % 16).astype(np.uint8)
    w = O.pack_q4_k_block(0.25, 0.01, [2, 3, 4, 5, 1, 2, 3, 4], [1, 0, 1, 0, 1, 0, 1, 0], q)
    x = (np.arange(256).astype(np.float32) * np.float32(0.01)) - np.float32(0.5)
    fused = O.vec_dot_row(K.Q4_K, 256, w, x)
    row = O.dequant_row(K.Q4_K, 256, w)
    s = np.float32(0.0)
    for a, b in zip(row, x):
        s = np.float32(s + np.float32(a * b))
    assert fused.view(np.uint32) == s.view(np.uint32)


def test_q4_k_doc_example():
    """langtax/src/quant.rs:48-79."""
    q = (np.arange(256) % 16).astype(np.uint8)
    row = O.pack_q4_k_block(0.05, 0.01, [12] * 8, [3] * 8, q)
    x = ((np.arange(256) % 7).astype(np.float32) - 3.0)
    y = O.vec_dot_row(K.Q4_K, 256, row, x)
    w = K.np_dequant(K.Q4_K, 1, 256, row)[0]
    assert abs(float(y) - float(np.dot(w.astype(np.float64), x))) < 1e-3


# ---------------------------------------------------------------- dequantizers vs independent numpy
@pytest.mark.parametrize("ty", O.ALL_TYPES)
def test_dequant_matches_independent_numpy(ty):
    rng = np.random.default_rng(100 + ty)
    n_cols = 3 * K.QK[ty] if K.QK[ty] > 1 else 77
    n_rows = 9
    w = K.random_packed(ty, n_rows, n_cols, rng)
    got = O.dequant(ty, n_cols, w, n_rows)
    want = K.np_dequant(ty, n_rows, n_cols, w)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("ty", QUANT_TYPES)
def test_dequant_every_f16_scale_pattern(ty):
    """Every finite binary16 pattern as a block scale, subnormals included
    (langtax/src/simd/tests.rs:795-828)."""
    rng = np.random.default_rng(5)
    bits = np.array([b for b in range(0, 65536, 3) if (b >> 10) & 0x1f != 31], np.uint16)
    nb = bits.size
    w = K.random_packed(ty, 1, nb * K.QK[ty], rng).reshape(nb, K.BLOCK[ty])
    off = 208 if ty == K.Q6_K else 0
    w[:, off:off + 2] = bits.view(np.uint8).reshape(nb, 2)
    got = O.dequant_row(ty, nb * K.QK[ty], w.reshape(-1))
    want = K.np_dequant(ty, 1, nb * K.QK[ty], w.reshape(-1))[0]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_all_zero_blocks_give_signed_zero_consistently():
    """langtax/src/simd/tests.rs:1481-1520."""
    for ty in QUANT_TYPES:
        n = 2 * K.QK[ty]
        w = np.zeros(K.row_bytes(ty, n), np.uint8)
        x = np.linspace(-1, 1, n).astype(np.float32)
        assert O.vec_dot_row(ty, n, w, x) == 0.0
        assert O.vec_dot_row(ty, n, w, x, simd=True) == 0.0
        assert np.all(O.dequant_row(ty, n, w) == 0.0)


# ---------------------------------------------------------------- closed-form fixtures, exact rationals
def _exact_row_dot(wrow, x):
    return sum(Fraction(float(a)) * Fraction(float(b)) for a, b in zip(wrow, x))


@pytest.mark.parametrize("fmt", K.formats(), ids=lambda f: f.name)
def test_closed_form_fixture_matches_exact_arithmetic(fmt):
    """langtax/tests/native_cuda_parity.rs:27-148: every datum is a small dyadic
    rational, so the exact dot is representable and every kernel must hit it."""
    rows = 23
    packed = np.concatenate([fmt.pack_row(r) for r in range(rows)])
    wd = K.np_dequant(fmt.ty, rows, fmt.cols, packed)
    assert np.array_equal(O.dequant(fmt.ty, fmt.cols, packed, rows), wd)
    x = np.concatenate([K.values(t + 3, fmt.cols) for t in range(3)])
    exact = np.array([[float(_exact_row_dot(wd[r], x[t * fmt.cols:(t + 1) * fmt.cols]))
                       for r in range(rows)] for t in range(3)])
    for simd in (False, True):
        y = O.gemm(fmt.ty, fmt.cols, 3, packed, x, rows, simd=simd)
        assert np.array_equal(y.astype(np.float64), exact), fmt.name
    assert np.array_equal(O.gemm_f64(fmt.ty, fmt.cols, 3, packed, x, rows), exact)


def test_selftest_fixture_f32():
    """native-cuda/src/main.rs:8-45."""
    for rows, cols in [(1, 63), (7, 64), (9, 65), (257, 129), (17, 33), (1, 1), (9, 1025)]:
        w = K.selftest_weights(rows, cols)
        for rnd, tokens in enumerate([1, 1, 3, 3, 1, 7, 1]):
            x = K.selftest_input(tokens, cols, rnd)
            want = x.reshape(tokens, cols).astype(np.float64) @ w.reshape(rows, cols).astype(np.float64).T
            y = O.gemm(K.F32, cols, tokens, O.pack_f32(w), x, rows)
            assert np.array_equal(y.astype(np.float64), want)


# ---------------------------------------------------------------- error bounds on random data
@pytest.mark.parametrize("ty", O.ALL_TYPES)
def test_scalar_and_simd_within_proven_bound(ty):
    """langtax/src/simd/tests.rs:18-162: each kernel within gamma(n+3)*sum|wx| of
    the f64 value, the two within twice that of each other, and the observed
    deviation under max(64, 8 sqrt n) u."""
    rng = np.random.default_rng(200 + ty)
    if K.QK[ty] == 1:
        sizes = [1, 2, 7, 8, 9, 15, 16, 17, 31, 33, 63, 64, 65, 127, 129, 255, 257, 511, 1000, 1024, 4096]
    elif K.QK[ty] == 32:
        sizes = [32 * b for b in (1, 2, 3, 4, 5, 7, 8, 9, 16, 128)]
    else:
        sizes = [256 * b for b in (1, 2, 3, 4, 5, 8, 16)]
    for n in sizes:
        w = K.random_packed(ty, 4, n, rng)
        x = rng.uniform(-1, 1, n).astype(np.float32)
        exact = K.f64_product(ty, 4, n, w, x)[0]
        mag = K.abs_product(ty, 4, n, w, x)[0]
        rb = K.row_bytes(ty, n)
        for r in range(4):
            row = w[r * rb:(r + 1) * rb]
            s = float(O.vec_dot_row(ty, n, row, x))
            v = float(O.vec_dot_row(ty, n, row, x, simd=True))
            bound = K.single_kernel_bound(n, mag[r])
            assert abs(s - exact[r]) <= bound, (n, r)
            assert abs(v - exact[r]) <= bound, (n, r)
            assert abs(s - v) <= 2 * bound
            if mag[r] > 0:
                assert abs(s - v) / mag[r] / K.U <= K.observed_envelope_u(n)
            assert abs(O.row_dot_f64(ty, n, row, x) - exact[r]) <= 1e-12 * max(mag[r], 1e-30)
            assert abs(O.row_abs_dot_f64(ty, n, row, x) - mag[r]) <= 1e-12 * max(mag[r], 1e-30)


def test_cancelling_and_wide_range_rows_stay_in_bound():
    """langtax/src/simd/tests.rs:1532-1595."""
    for n in (8, 64, 256, 4096):
        w = np.empty(n, np.float32)
        w[0::2], w[1::2] = 1000.0, -1000.0
        x = np.ones(n, np.float32)
        x[1::2] = np.float32(1.0 + 2.0 ** -20)
        exact = float(np.dot(w.astype(np.float64), x.astype(np.float64)))
        mag = float(np.dot(np.abs(w).astype(np.float64), np.abs(x).astype(np.float64)))
        for simd in (False, True):
            got = float(O.vec_dot_row(K.F32, n, O.pack_f32(w), x, simd=simd))
            assert abs(got - exact) <= K.single_kernel_bound(n, mag)
    n = 1024
    w = np.full(n, 1e-6, np.float32)
    w[n // 2] = 1e12
    x = np.ones(n, np.float32)
    exact = float(np.sum(w.astype(np.float64)))
    for simd in (False, True):
        got = float(O.vec_dot_row(K.F32, n, O.pack_f32(w), x, simd=simd))
        assert abs(got - exact) <= K.single_kernel_bound(n, exact)


# ---------------------------------------------------------------- GEMM layout, threading, validation
@pytest.mark.parametrize("ty", O.ALL_TYPES)
def test_gemm_is_repeated_gemv_token_major_and_thread_independent(ty):
    """langtax/src/quant.rs:6760-6888, 12297-12415; langtax/src/pool.rs:83-148."""
    rng = np.random.default_rng(300 + ty)
    n_cols = 2 * K.QK[ty] if K.QK[ty] > 1 else 65
    n_rows, n_tokens = 37, 5
    w = K.random_packed(ty, n_rows, n_cols, rng)
    x = rng.uniform(-1, 1, n_tokens * n_cols).astype(np.float32)
    rb = K.row_bytes(ty, n_cols)
    for simd in (False, True):
        y = O.gemm(ty, n_cols, n_tokens, w, x, n_rows, simd=simd, threads=1)
        for t in range(n_tokens):
            for r in (0, 1, 17, 36):
                want = O.vec_dot_row(ty, n_cols, w[r * rb:(r + 1) * rb], x[t * n_cols:(t + 1) * n_cols], simd=simd)
                assert y[t, r].view(np.uint32) == want.view(np.uint32)
        for threads in (0, 2, 3, 10):
            yt = O.gemm(ty, n_cols, n_tokens, w, x, n_rows, simd=simd, threads=threads)
            assert np.array_equal(yt.view(np.uint32), y.view(np.uint32))


def test_gemm_validation_and_empty_rows():
    lib = O.load()
    x = np.zeros(64, np.float32)
    y = np.full(1, 123.5, np.float32)
    w = np.zeros(34, np.uint8)

    def call(ty, n_cols, n_tokens, n_rows, w, x, y):
        return lib.lro_gemm(ty, 0, 1, n_cols, n_tokens, n_rows, w.ctypes.data, w.size, x.ctypes.data, x.size,
                            y.ctypes.data, y.size)

    assert call(K.Q8_0, 32, 0, 1, w, x[:32], y) < 0        # zero tokens
    assert call(K.Q8_0, 32, 1, 1, w, x[:31], y) < 0        # short input
    assert call(K.Q8_0, 32, 1, 1, w[:33], x[:32], y) < 0   # short weights
    assert call(K.Q8_0, 33, 1, 1, w, x[:33], y) < 0        # unaligned columns
    assert call(K.Q8_0, 32, 2, 1, w, x, y) < 0             # y not a multiple of tokens
    assert y[0] == np.float32(123.5)
    empty = np.zeros(0, np.float32)
    assert call(K.Q8_0, 32, 2, 0, np.zeros(0, np.uint8), x, empty) == 0
    assert O.load().lro_worker_count(1) == 1
    assert 1 <= O.load().lro_worker_count(100000) <= 10


def test_validate_follows_reference_rules():
    """native-cuda/src/lib.rs:66-75."""
    assert O.validate([np.nan], [0.0]) == 0
    assert O.validate([np.inf], [np.inf]) == 0
    assert O.validate([1.0], [2.0]) == 0
    assert O.validate([1.00001, -2.0], [1.0, -2.0]) == -1
    assert O.validate([6.0, -4.0], [6.0, -4.0]) == -1


def test_row_bytes_and_alignment():
    assert O.row_bytes(K.Q8_0, 4096) == 128 * 34
    assert O.row_bytes(K.Q4_K, 4096) == 16 * 144
    assert O.row_bytes(K.Q6_K, 4096) == 16 * 210
    assert O.row_bytes(K.Q4_0, 14336) == 448 * 18
    assert O.row_bytes(K.Q5_0, 14336) == 448 * 22
    assert O.row_bytes(K.Q5_1, 14336) == 448 * 24
    assert O.row_bytes(K.F16, 33) == 66 and O.row_bytes(K.F32, 33) == 132
    assert O.row_bytes(K.Q8_0, 33) == 0 and O.row_bytes(K.Q4_K, 128) == 0
