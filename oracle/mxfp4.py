"""MXFP4 (e2m1 codes + E8M0 block-32 scales) oracle, numpy, bit-exact integer arithmetic.

Test infrastructure: see ``oracle/__init__.py``.

Follows the reference's Triton quantiser bit by bit
(include/tritonblas/utils.py:646-740) and its dequantisers
(include/tritonblas/utils.py:547-609 and :612-643).  The 32-point Hadamard
rotation has no counterpart in the reference; it is defined here by a pinned
butterfly order and checked against the Sylvester matrix.

Decisions for inputs whose treatment the reference's source leaves to the platform:
  * scale byte = (e + 127) mod 256, so an all-zero block stores byte 0;
  * shifts by >= 32 in the sub-normal mantissa path give 0;
  * log2/exp2 of powers of two are exact integer exponent arithmetic;
  * NaN inputs are unspecified.
The first three agree with what the reference kernel itself produces under Triton's CPU interpreter
(tests/golden/mxfp4_quant_vectors.npz holds such blocks, fp32 denormals and infinities included);
what a GPU build of the reference does there is not pinned by anything in the reference tree.
"""
import numpy as np

MX_BLOCK = 32

# include/tritonblas/utils.py:590-607 (OCP MX e2m1 value table)
E2M1_VALUES = np.array(
    [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
    dtype=np.float32,
)

# fp32 nearest to 1/sqrt(32)
INV_SQRT32_BITS = 0x3E3504F3
INV_SQRT32 = np.array([INV_SQRT32_BITS], dtype=np.uint32).view(np.float32)[0]


def unpack_codes(packed: np.ndarray) -> np.ndarray:
    """(..., N/2) uint8 -> (..., N) 4-bit codes; low nibble is the even element
    (include/tritonblas/utils.py:585-587)."""
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = packed & 0xF
    out[..., 1::2] = packed >> 4
    return out


def mxfp4_to_f32(packed: np.ndarray) -> np.ndarray:
    """include/tritonblas/utils.py:547-609."""
    return E2M1_VALUES[unpack_codes(packed).astype(np.int64)]


def e8m0_to_f32(scale: np.ndarray) -> np.ndarray:
    """include/tritonblas/utils.py:612-643: 2**(b-127); byte 0 -> bits 0x00400000 (2**-127),
    byte 255 -> NaN."""
    b = np.ascontiguousarray(scale, dtype=np.uint8).astype(np.uint32)
    bits = b << np.uint32(23)
    bits = np.where(b == 0, np.uint32(0x00400000), bits)
    bits = np.where(b == 0xFF, np.uint32(0x7F800001), bits)
    return bits.astype(np.uint32).view(np.float32)


def dequant(packed: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """Values represented by (codes, scales): tests/test_matmul_fp4.py:20-46."""
    v = mxfp4_to_f32(packed)
    s = np.repeat(e8m0_to_f32(scale), MX_BLOCK, axis=-1)
    return (v * s).astype(np.float32)


def block_scale_exponent(amax: np.ndarray) -> np.ndarray:
    """Unbiased E8M0 exponent for a block maximum (include/tritonblas/utils.py:683-689).

    amax is rounded to a power of two (up iff its mantissa >= 0x600000, i.e. >= 1.75 * 2**k), then
    e = log2(that) - 2, clamped to [-127, 127]."""
    bits = np.ascontiguousarray(amax, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = ((bits + 0x200000) & 0xFFFFFFFF) & 0xFF800000
    field = ((bits >> 23) & 0xFF).astype(np.int64)
    e = field - 127 - 2
    e = np.where(field == 0, -127, e)       # log2(0) = -inf -> clamp
    e = np.where(field == 255, 127, e)      # log2(inf) = inf -> clamp
    return np.clip(e, -127, 127).astype(np.int64)


def f32_to_e2m1(qx: np.ndarray) -> np.ndarray:
    """Scaled fp32 value -> 4-bit e2m1 code (include/tritonblas/utils.py:701-721).

    Round to nearest, ties away from zero in magnitude, saturate at 6.0 (Inf/NaN -> +-6)."""
    q = np.ascontiguousarray(qx, dtype=np.float32).view(np.uint32).astype(np.uint64)
    s = q & 0x80000000
    e = (q >> 23) & 0xFF
    m = q & 0x7FFFFF
    adj = np.where(e < 127, 126 - e.astype(np.int64), 0)
    den = np.where(adj >= 32, 0, (0x400000 | (m >> 1)) >> np.minimum(adj, 31).astype(np.uint64))
    m = np.where(e < 127, den, m)
    e = np.maximum(e, 126) - 126
    tmp = np.minimum((((e << 2) | (m >> 21)) + 1) >> 1, 7)
    return ((s >> 28) | tmp).astype(np.uint8)


def mxfp4_quant(x: np.ndarray):
    """fp32 (M, N) -> (codes (M, N/2) uint8, scales (M, N/32) uint8).

    include/tritonblas/utils.py:678-726 (kernel) and :743-789 (driver)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, N = x.shape
    assert N % MX_BLOCK == 0
    xb = x.reshape(M, N // MX_BLOCK, MX_BLOCK)
    amax = np.max(np.abs(xb), axis=2)
    e = block_scale_exponent(amax)
    qscale = np.ldexp(np.float32(1.0), (-e).astype(np.int32)).astype(np.float32)  # exact, sub-normal for e=127
    with np.errstate(over="ignore", invalid="ignore"):
        qx = (xb * qscale[:, :, None]).astype(np.float32)
    codes = f32_to_e2m1(qx).reshape(M, N)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    scales = ((e + 127) & 0xFF).astype(np.uint8)
    return packed, scales


def hadamard32(x: np.ndarray) -> np.ndarray:
    """x (.., N) fp32 -> x * (I (x) H32) / sqrt(32) along the last axis, blocks of 32.

    Pinned evaluation order (so that a GPU kernel can be bit-identical): radix-2 butterflies with
    strides h = 1, 2, 4, 8, 16; at each stage the pair (i, i+h), i & h == 0, becomes
    (x[i] + x[i+h], x[i] - x[i+h]) in fp32; afterwards one fp32 multiply by 0x3E3504F3."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    shp = x.shape
    assert shp[-1] % 32 == 0
    y = x.reshape(-1, 32)
    for h in (1, 2, 4, 8, 16):
        y = y.reshape(-1, 32 // (2 * h), 2, h)
        a = y[:, :, 0, :]
        b = y[:, :, 1, :]
        y = np.stack([(a + b).astype(np.float32), (a - b).astype(np.float32)], axis=2)
    y = y.reshape(-1, 32)
    return (y * INV_SQRT32).astype(np.float32).reshape(shp)


def hadamard_mxfp4_quant(x: np.ndarray):
    """Fused rotate + quantise: mxfp4_quant(hadamard32(x)); the rotated values stay in fp32."""
    return mxfp4_quant(hadamard32(x))
