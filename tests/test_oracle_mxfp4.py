"""Pins the MXFP4 / Hadamard oracle (CPU).  None of these checks re-types the oracle's formulas:
they use hand-derived answers, a nearest-value search over the e2m1 grid, the Sylvester matrix from
scipy and algebraic invariants."""
import numpy as np
import pytest
import scipy.linalg

from oracle import mxfp4

GRID = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def _quant_block(vals):
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, : len(vals)] = vals
    codes, scales = mxfp4.mxfp4_quant(x)
    return mxfp4.unpack_codes(codes)[0], int(scales[0, 0])


def test_e2m1_table_is_ocp_mx():
    # sign | 2-bit exponent (bias 1) | 1-bit mantissa, sub-normal step 0.5
    for code in range(16):
        s, e, m = code >> 3, (code >> 1) & 3, code & 1
        mag = m * 0.5 if e == 0 else (1 + m * 0.5) * 2.0 ** (e - 1)
        assert mxfp4.E2M1_VALUES[code] == (-mag if s else mag)
    assert np.signbit(mxfp4.E2M1_VALUES[8])


def test_unpack_low_nibble_first():
    assert list(mxfp4.unpack_codes(np.array([[0x21, 0xF7]], dtype=np.uint8))[0]) == [1, 2, 7, 15]


def test_e8m0_closed_form_and_specials():
    b = np.arange(1, 255, dtype=np.uint8)
    want = np.ldexp(1.0, b.astype(np.int64) - 127).astype(np.float32)
    assert np.array_equal(mxfp4.e8m0_to_f32(b), want)
    assert mxfp4.e8m0_to_f32(np.array([0], dtype=np.uint8)).view(np.uint32)[0] == 0x00400000  # 2**-127
    assert np.isnan(mxfp4.e8m0_to_f32(np.array([255], dtype=np.uint8))[0])


# (block contents, expected scale byte, expected codes of the listed values): derived by hand from
# "scale = 2**(floor(log2(round_pow2(amax))) - 2), code = nearest e2m1 of x/scale, ties away from 0"
KATS = [
    ([6.0, 2.5, 0.25, 0.75, -1.0, 0.0], 127, [7, 5, 1, 2, 0xA, 0]),
    ([7.0, 3.5], 128, [6, 4]),            # amax 7 = 1.75*4 rounds up to 8 -> scale 2; 3.5 -> 4, 1.75 -> 2
    ([1.74], 125, [7]),                   # below the 1.75 boundary: pow2 = 1 -> scale 1/4; 6.96 saturates to 6
    ([1.75], 126, [6]),                   # at the boundary: pow2 = 2 -> scale 1/2; 3.5 -> 4 (tie up)
    ([-6.0, 6.0], 127, [0xF, 7]),
]


def test_known_answers():
    for vals, want_scale, want_codes in KATS[:5]:
        codes, scale = _quant_block(vals)
        assert scale == want_scale, (vals, scale)
        assert list(codes[: len(vals)]) == want_codes, (vals, list(codes[: len(vals)]))
    # 448 = 1.75 * 2**8 rounds up to 2**9, e = 9 - 2 = 7, scale byte 134, q = 448/128 = 3.5 -> 4.0 (code 6)
    codes, scale = _quant_block([448.0, -448.0, 32.0])
    assert scale == 134 and list(codes[:3]) == [6, 0xE, 1]


def test_zero_block_and_extremes():
    codes, scale = _quant_block([0.0])
    assert scale == 0 and not codes.any()
    codes, scale = _quant_block([np.inf, -np.inf, 1.0])
    assert scale == 254 and list(codes[:3]) == [7, 0xF, 0]
    # largest finite fp32 (just under 2**128): the power-of-two rounding reaches the Inf exponent field, e clamps
    # to 127, q = max * 2**-127 is just under 2.0 -> code 4
    codes, scale = _quant_block([np.finfo(np.float32).max])
    assert scale == 254 and codes[0] == 4
    # tiny sub-normal block: exponent field rounds to 0 or 1 -> e clamps to -127 -> byte 0
    codes, scale = _quant_block([1e-45])
    assert scale == 0


def test_scale_exponent_against_frexp():
    rng = np.random.default_rng(0)
    amax = np.abs(rng.standard_normal(20000).astype(np.float32)) * np.float32(10.0) ** rng.integers(-20, 20, 20000).astype(np.float32)
    amax = amax[(amax > 1e-30) & np.isfinite(amax)]
    mant, exp = np.frexp(amax.astype(np.float64))       # amax = mant * 2**exp, mant in [0.5, 1)
    pow2 = np.where(mant * 2 >= 1.75, exp, exp - 1)     # round to a power of two, up from 1.75x
    assert np.array_equal(mxfp4.block_scale_exponent(amax), pow2 - 2)


def test_codes_are_nearest_grid_point_ties_away():
    """Brute force: for a dense sweep of scaled values the code must be the nearest e2m1 magnitude,
    the upper one on exact ties, saturating at 6."""
    q = np.concatenate([np.linspace(0, 8, 6401), np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 1e-3, 100.0])]).astype(np.float32)
    q = np.concatenate([q, -q])
    codes = mxfp4.f32_to_e2m1(q)
    for val, code in zip(q.tolist(), codes.tolist()):
        mag = abs(val)
        d = np.abs(GRID - mag)
        best = np.flatnonzero(d == d.min()).max()  # ties -> larger magnitude
        if mag >= 6:
            best = 7
        assert (code & 7) == best, (val, code)
        assert (code >> 3) == (1 if np.signbit(np.float32(val)) else 0)


def test_quant_dequant_error_bound():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    codes, scales = mxfp4.mxfp4_quant(x)
    back = mxfp4.dequant(codes, scales)
    s = np.repeat(mxfp4.e8m0_to_f32(scales), 32, axis=1)
    # inside the representable range the error is at most half the widest grid gap (1.0 * scale);
    # the block maximum may saturate from < 8*scale down to 6*scale
    assert np.all(np.abs(back - x) <= 2.0 * s + 1e-12)
    assert np.all(np.abs(back - x)[np.abs(x) <= 6 * s] <= 1.0 * s[np.abs(x) <= 6 * s])
    assert codes.shape == (64, 128) and scales.shape == (64, 8)


def test_hadamard_matches_sylvester_matrix():
    H = scipy.linalg.hadamard(32).astype(np.float64)
    rng = np.random.default_rng(2)
    x = rng.integers(-8, 9, size=(16, 96)).astype(np.float32)   # small integers: every butterfly is exact
    got = mxfp4.hadamard32(x).astype(np.float64)
    want = (x.reshape(16, 3, 32).astype(np.float64) @ H).reshape(16, 96) * float(mxfp4.INV_SQRT32)
    assert np.allclose(got, want, rtol=1e-7, atol=0)
    e0 = np.zeros((1, 32), dtype=np.float32)
    e0[0, 0] = 1
    assert np.array_equal(mxfp4.hadamard32(e0), np.full((1, 32), mxfp4.INV_SQRT32, dtype=np.float32))


def test_hadamard_involution_and_norm():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((8, 64)).astype(np.float32)
    y = mxfp4.hadamard32(x)
    assert np.allclose(np.linalg.norm(y, axis=1), np.linalg.norm(x, axis=1), rtol=1e-5)
    assert np.allclose(mxfp4.hadamard32(y), x, atol=1e-5)   # (H/sqrt32)^2 = I
    assert abs(float(mxfp4.INV_SQRT32) - 32 ** -0.5) < 1e-8


def test_rotated_gemm_preserved():
    rng = np.random.default_rng(4)
    a = rng.standard_normal((4, 64)).astype(np.float32)
    b = rng.standard_normal((5, 64)).astype(np.float32)
    assert np.allclose(mxfp4.hadamard32(a) @ mxfp4.hadamard32(b).T, a @ b.T, atol=1e-4)


def _reference_vectors():
    """tests/golden/mxfp4_quant_vectors.npz: outputs of the reference's own kernel
    (include/tritonblas/utils.py:646-789), run under Triton's CPU interpreter by
    tests/golden/make_mxfp4_quant_vectors.py."""
    import os
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mxfp4_quant_vectors.npz"))
    x32 = d["x_f32_bits"].view(np.float32)
    xbf = (d["x_bf16_bits"].astype(np.uint32) << 16).view(np.float32)
    return {"f32": (x32, d["codes_f32"], d["scales_f32"]), "bf16": (xbf, d["codes_bf16"], d["scales_bf16"])}


@pytest.mark.parametrize("name", ["f32", "bf16"])
def test_oracle_equals_reference_kernel_output(name):
    """Every code byte and scale byte of the reference kernel's output, including the cases its source
    leaves to the platform: scale bytes of negative exponents, all-zero blocks (byte 0), denormal block
    maxima, shift counts of 32 and more, infinities."""
    x, codes, scales = _reference_vectors()[name]
    got_c, got_s = mxfp4.mxfp4_quant(x)
    assert np.array_equal(got_s, scales)
    assert np.array_equal(got_c, codes)
    # the set is not trivial: many scale bytes on both sides of the bias, zero blocks, every code
    assert len(np.unique(scales)) > 60 and scales.min() == 0 and scales.max() > 250
    assert set(np.unique(mxfp4.unpack_codes(codes))) == set(range(16))
