"""The reference's deterministic sweeps, run whole on the device through every kernel family (one token,
3..16 tokens, 17..32 tokens, more than 32 tokens), through the C ABI:

  * every code value in every position of a block, alone, the rest of the row zero
    (langtax/src/simd/tests.rs:755-787 Q4_0, 933-960 Q5_0, 1110-1137 Q5_1, 1272-1293 Q8_0): one exact
    term per output, so the result must EQUAL the closed form, not merely lie inside a bound;
  * every finite binary16 pattern as a block scale (langtax/src/simd/tests.rs:795-828 and the sweeps
    of the other dtypes built the same way);
  * the element counts that straddle every vector width for the plain dtypes
    (langtax/src/simd/tests.rs:190-193).

The rows are wide enough for the lane-per-unit kernels (a whole number of 256-column units) as well as
the reference's own one-block rows, which take the generic kernel.
"""
import numpy as np
import pytest

import cases as K
import oracle as O

pytestmark = pytest.mark.gpu

# one token, the 16-token tile, the 32-token tile, the 64-token tiles
TOKEN_COUNTS = (1, 16, 32, 64)


@pytest.fixture(scope="module")
def gpu(pkg):
    g = pkg.HipGemv(0)
    yield g
    g.close()


def _f16_bytes(v):
    return np.asarray(v, np.float16).view(np.uint8)


def blocks_from_codes(ty, codes, d=0.25):
    """GGUF blocks of 32 from stored codes (unsigned: nibble 0..15, 5-bit 0..31; Q8_0: int8), scale d, Q5_1's
    offset zero.  Written from the block definitions (langtax/src/quant.rs:7511-7541, 7734-7765, 7884-7950,
    8046-8130): low nibble of qs[j] = element j, high nibble = element j + 16, bit j of qh = fifth bit of element j."""
    codes = np.asarray(codes)
    n = codes.shape[0]
    assert codes.shape == (n, 32)
    out = np.zeros((n, K.BLOCK[ty]), np.uint8)
    out[:, 0:2] = _f16_bytes(np.full(n, d)).reshape(n, 2)
    if ty == K.Q8_0:
        out[:, 2:34] = codes.astype(np.int8).view(np.uint8)
        return out
    c = codes.astype(np.uint32)
    qs = ((c[:, :16] & 15) | ((c[:, 16:] & 15) << 4)).astype(np.uint8)
    if ty == K.Q4_0:
        out[:, 2:18] = qs
        return out
    qh = np.zeros(n, np.uint32)
    for j in range(32):
        qh |= ((c[:, j] >> 4) & 1) << j
    at = 2 if ty == K.Q5_0 else 4
    out[:, at:at + 4] = qh.view(np.uint8).reshape(n, 4)
    out[:, at + 4:at + 20] = qs
    return out


# stored code that dequantizes to zero, the codes the reference places, and the value of a stored code
ZERO_CODE = {K.Q4_0: 8, K.Q5_0: 16, K.Q5_1: 0, K.Q8_0: 0}
CODES = {K.Q4_0: np.arange(16), K.Q5_0: np.arange(32), K.Q5_1: np.arange(32),
         K.Q8_0: np.array([-128, -127, -1, 0, 1, 126, 127])}
BIAS = {K.Q4_0: 8, K.Q5_0: 16, K.Q5_1: 0, K.Q8_0: 0}


@pytest.mark.parametrize("cols", [32, 512])
@pytest.mark.parametrize("ty", [K.Q4_0, K.Q5_0, K.Q5_1, K.Q8_0], ids=lambda t: O.TYPE_NAMES[t])
def test_every_code_in_every_position_is_exact(pkg, gpu, ty, cols):
    """Row (position p, code c) holds code c at column p and zero everywhere else, scale 0.25; the activations are
    small integers times a power of two per token.  Every output has one nonzero term, (c - bias) * 0.25 * x[p],
    exact in binary32: the kernels must return exactly that, whichever position of a block, block of a unit or
    unit of the row the code sits in.  32 columns is the reference's own shape (one block per row: the generic
    single-token kernel), 512 columns two units of the lane-per-unit kernels."""
    codes = CODES[ty]
    rows = cols * codes.size
    pos = np.repeat(np.arange(cols), codes.size)
    code = np.tile(codes, cols)
    stored = np.full((rows, cols), ZERO_CODE[ty], np.int32)
    stored[np.arange(rows), pos] = code
    w = blocks_from_codes(ty, stored.reshape(rows * cols // 32, 32)).reshape(-1)
    # the construction against the oracle's dequantizer: exactly one nonzero weight per row, where it was placed
    want_w = np.zeros((rows, cols), np.float32)
    want_w[np.arange(rows), pos] = (code - BIAS[ty]) * 0.25
    assert np.array_equal(np.asarray(O.dequant(ty, cols, w, rows), np.float32).reshape(rows, cols), want_w)
    m = gpu.upload_packed(ty, rows, cols, w)
    for tokens in TOKEN_COUNTS:
        t = np.arange(tokens)[:, None]
        x = ((1 + (np.arange(cols)[None, :] + 3 * t) % 32) * 2.0 ** (t % 4 - 1)).astype(np.float32)
        y = np.full(tokens * rows, np.nan, np.float32)
        gpu.gemm_resident(m, tokens, x.reshape(-1), y)
        want = ((code - BIAS[ty]) * 0.25).astype(np.float32)[None, :] * x[:, pos]
        got = y.reshape(tokens, rows)
        bad = np.argwhere(got != want)
        assert bad.size == 0, (f"{O.TYPE_NAMES[ty]} {cols} columns, {tokens} tokens: token {bad[0][0]} position {pos[bad[0][1]]} "
                               f"code {code[bad[0][1]]}: {got[tuple(bad[0])]} != {want[tuple(bad[0])]} ({bad.shape[0]} outputs differ)")
    m.close()


@pytest.mark.parametrize("ty", [K.Q4_0, K.Q5_0, K.Q5_1, K.Q8_0, K.Q4_K, K.Q6_K], ids=lambda t: O.TYPE_NAMES[t])
def test_every_finite_f16_scale_pattern_through_every_kernel_family(pkg, gpu, ty):
    """All 63 488 finite binary16 patterns (subnormals, both zeros, both signs) as the block scale d, one pattern per
    block, random codes, through the single-token kernel and the 16-, 32- and 64-token tiles: every output inside the
    reference's proven summation bound around the float64 product of the dequantized weights.  The hardware's
    f16 -> f32 conversions must keep subnormal scales, in every kernel that decodes them."""
    rng = np.random.default_rng(70 + ty)
    bits = np.array([b for b in range(65536) if (b >> 10) & 0x1f != 31], np.uint16)
    assert bits.size == 63488
    cols = 4096
    per_row = cols // K.QK[ty]
    rows = bits.size // per_row
    assert rows * per_row == bits.size  # 63 488 = 496 * 128 = 3 968 * 16: every pattern is used
    w = K.random_packed(ty, rows, cols, rng).reshape(rows * per_row, K.BLOCK[ty])
    off = 208 if ty == K.Q6_K else 0
    w[:, off:off + 2] = bits.view(np.uint8).reshape(-1, 2)
    if ty == K.Q6_K:
        w[:, 192:208] = rng.integers(-3, 4, (w.shape[0], 16)).astype(np.int8).view(np.uint8)  # keep |w| finite in f32
    if ty in (K.Q4_K, K.Q5_1):
        w[:, 2:4] = 0  # min / offset scale zero: the swept field is the whole weight
    w = w.reshape(-1)
    m = gpu.upload_packed(ty, rows, cols, w)
    for tokens in TOKEN_COUNTS:
        x = rng.uniform(-1, 1, (tokens, cols)).astype(np.float32) * np.float32(2.0 ** -6)
        y = np.full(tokens * rows, np.nan, np.float32)
        gpu.gemm_resident(m, tokens, x.reshape(-1), y)
        exact, mag = O.gemm_f64_mag(ty, cols, tokens, w, x.reshape(-1), rows)
        err = np.abs(y.reshape(tokens, rows).astype(np.float64) - exact)
        assert np.all(np.isfinite(y)), f"{tokens} tokens"
        worst = np.unravel_index(np.argmax(err - K.single_kernel_bound(cols, mag)), err.shape)
        assert np.all(err <= K.single_kernel_bound(cols, mag)), (
            f"{O.TYPE_NAMES[ty]}, {tokens} tokens: token {worst[0]} row {worst[1]} (scale patterns "
            f"{int(bits[worst[1] * per_row]):#06x}..): off by {err[worst]:.3e}, bound {K.single_kernel_bound(cols, mag)[worst]:.3e}")
    m.close()


ELEM_LENGTHS = (1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 23, 24, 25, 31, 32, 33, 63, 64, 65, 127, 128,
                129, 255, 256, 257, 511, 1000, 1024, 4096)


@pytest.mark.parametrize("ty", [K.F32, K.F16], ids=lambda t: O.TYPE_NAMES[t])
def test_plain_dtypes_at_every_element_count_of_the_reference(pkg, gpu, ty):
    """langtax/src/simd/tests.rs:190-193: row lengths on both sides of every vector width and their tails (the
    length 0 of that list is no matrix here: Shape::checked refuses it, tested with the validation rules).  One
    token takes the generic kernel with its scalar tail, two and more the f32 matrix-core tiles; rows on both
    sides of a 4-row group and of a 128-row tile."""
    rng = np.random.default_rng(190 + ty)
    for cols in ELEM_LENGTHS:
        for rows in (1, 5, 130):
            w = K.random_packed(ty, rows, cols, rng)
            m = gpu.upload_packed(ty, rows, cols, w)
            for tokens in (1, 2, 16, 33, 64):
                x = rng.normal(0, 1, tokens * cols).astype(np.float32)
                y = np.full(tokens * rows, np.nan, np.float32)
                gpu.gemm_resident(m, tokens, x, y)
                exact, mag = O.gemm_f64_mag(ty, cols, tokens, w, x, rows)
                err = np.abs(y.reshape(tokens, rows).astype(np.float64) - exact)
                assert np.all(err <= K.single_kernel_bound(cols, mag)), f"{O.TYPE_NAMES[ty]} {rows}x{cols}, {tokens} tokens"
            m.close()
    with pytest.raises(pkg.NativeHipError):
        gpu.upload_packed(ty, 4, 0, np.zeros(0, np.uint8))
