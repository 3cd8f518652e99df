"""Bit-exact parity of the MXFP4 quantiser (with and without the Hadamard rotation) on the GPU
against the integer oracle."""
import numpy as np
import pytest
import torch

from oracle import mxfp4 as OM

pytestmark = pytest.mark.gpu


def _run(x: torch.Tensor, hadamard: bool):
    import tritonblas_amd as tb
    fn = tb.hadamard_mxfp4_quant if hadamard else tb.dynamic_mxfp4_quant
    codes, scales = fn(x.cuda())
    torch.cuda.synchronize()
    return codes.cpu().numpy(), scales.cpu().numpy()


def _oracle(x: torch.Tensor, hadamard: bool):
    xf = x.float().numpy()
    return OM.hadamard_mxfp4_quant(xf) if hadamard else OM.mxfp4_quant(xf)


def _assert_same(x, hadamard):
    got_c, got_s = _run(x, hadamard)
    want_c, want_s = _oracle(x, hadamard)
    assert np.array_equal(got_s, want_s), f"{(got_s != want_s).sum()} scale bytes differ"
    assert np.array_equal(got_c, want_c), f"{(got_c != want_c).sum()} code bytes differ"


@pytest.mark.parametrize("hadamard", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 32), (3, 64), (128, 256), (257, 4096), (1000, 96)])
def test_random(shape, dtype, hadamard):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(shape, generator=g)
    mask = torch.rand(shape, generator=g) < 1e-2
    x = torch.where(mask, x * 20, x).to(dtype)
    _assert_same(x, hadamard)


@pytest.mark.parametrize("hadamard", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 32), (3, 64), (257, 4096), (1000, 96), (37, 14336)])
def test_both_index_paths(shape, dtype, hadamard, tb_option):
    """Below 2^31 items the kernel splits an item index into (row, column) with a multiply-high by a
    reciprocal the host computes; the kernel for larger tensors divides.  Both are forced here on row
    lengths that are and are not powers of two, and must give the oracle's bytes."""
    g = torch.Generator().manual_seed(11)
    x = torch.randn(shape, generator=g).to(dtype)
    for div64 in (0, 1):
        tb_option("quant_div64", div64)
        _assert_same(x, hadamard)


@pytest.mark.parametrize("name", ["f32", "bf16"])
def test_reference_kernel_vectors(name):
    """The HIP quantiser against the committed outputs of the reference's own kernel
    (tests/golden/mxfp4_quant_vectors.npz, written by tests/golden/make_mxfp4_quant_vectors.py from
    include/tritonblas/utils.py:646-789 under Triton's CPU interpreter): bit for bit."""
    import os
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mxfp4_quant_vectors.npz"))
    if name == "f32":
        x = torch.from_numpy(d["x_f32_bits"].view(np.float32).copy())
    else:
        x = torch.from_numpy(d["x_bf16_bits"].view(np.int16).copy()).view(torch.bfloat16)
    got_c, got_s = _run(x, False)
    assert np.array_equal(got_s, d[f"scales_{name}"]), f"{(got_s != d[f'scales_{name}']).sum()} scale bytes differ"
    assert np.array_equal(got_c, d[f"codes_{name}"]), f"{(got_c != d[f'codes_{name}']).sum()} code bytes differ"


@pytest.mark.parametrize("hadamard", [False, True])
def test_every_bf16_bit_pattern(hadamard):
    """All 65536 bf16 encodings (NaNs replaced by zero) under several block maxima."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    bits = torch.where(torch.isnan(bits), torch.zeros_like(bits), bits)
    bits = torch.cat([bits, torch.zeros(31 - 65536 % 31, dtype=torch.bfloat16)])
    rows = []
    for amax in (0.0, 6.0, 7.0, 1.74, 1e-30, 3e38, float("inf")):
        blk = bits.reshape(-1, 31)
        col = torch.full((blk.shape[0], 1), amax, dtype=torch.bfloat16)
        rows.append(torch.cat([blk, col], dim=1))
    x = torch.cat(rows, dim=0)
    if hadamard:
        # sums of 32 huge values overflow and inf - inf inside the rotation is NaN: unspecified
        x = torch.where(x.float().abs() > 1e36, torch.zeros_like(x), x)
    _assert_same(x, hadamard)


@pytest.mark.parametrize("hadamard", [False, True])
def test_scale_rounding_boundaries_and_subnormals(hadamard):
    vals = []
    for e in range(-140, 128, 3):
        for frac in (1.0, 1.25, 1.5, 1.7499999, 1.75, 1.9999999):
            vals.append(frac * 2.0 ** e)
    x = torch.zeros(len(vals), 32, dtype=torch.float32)
    x[:, 5] = torch.tensor(vals, dtype=torch.float64).to(torch.float32)
    x[:, 9] = -x[:, 5] * 0.3
    _assert_same(x, hadamard)


def test_strided_rows():
    import tritonblas_amd as tb
    x = torch.randn(64, 512, generator=torch.Generator().manual_seed(1)).bfloat16()
    xs = x.cuda()[:, :256]          # row stride 512, 256 columns
    codes, scales = tb.hadamard_mxfp4_quant(xs)
    want_c, want_s = OM.hadamard_mxfp4_quant(x[:, :256].float().numpy())
    assert np.array_equal(codes.cpu().numpy(), want_c) and np.array_equal(scales.cpu().numpy(), want_s)


def test_misaligned_view_and_empty_input():
    """a view that starts off a 16-byte boundary (or whose rows do) is copied first; no rows: empty results"""
    import tritonblas_amd as tb
    x = torch.randn(40, 200, generator=torch.Generator().manual_seed(2)).bfloat16()
    xs = x.cuda()[:, 3:3 + 160]          # starts 6 bytes into a row, row stride 400 bytes
    codes, scales = tb.dynamic_mxfp4_quant(xs)
    want_c, want_s = OM.mxfp4_quant(x[:, 3:3 + 160].float().numpy())
    assert np.array_equal(codes.cpu().numpy(), want_c) and np.array_equal(scales.cpu().numpy(), want_s)
    # a CONTIGUOUS view that merely starts two bytes off a 16-byte boundary
    flat = torch.randn(1 + 24 * 128, generator=torch.Generator().manual_seed(3)).bfloat16()
    xv = flat.cuda()[1:].view(24, 128)
    assert xv.is_contiguous() and xv.data_ptr() % 16 == 2
    codes, scales = tb.dynamic_mxfp4_quant(xv)
    want_c, want_s = OM.mxfp4_quant(flat[1:].view(24, 128).float().numpy())
    assert np.array_equal(codes.cpu().numpy(), want_c) and np.array_equal(scales.cpu().numpy(), want_s)
    codes, scales = tb.hadamard_mxfp4_quant(torch.zeros(0, 64, dtype=torch.bfloat16, device="cuda"))
    assert codes.shape == (0, 32) and scales.shape == (0, 2)


def test_quant_then_gemm_roundtrip():
    """Rotating both operands leaves A @ B^T unchanged: the MXFP4 GEMM of the two rotated+quantised
    operands approximates the bf16 product (quantisation noise only)."""
    import tritonblas_amd as tb
    from oracle import gemm as OG
    g = torch.Generator().manual_seed(2)
    a = torch.randn(256, 1024, generator=g).bfloat16()
    b = torch.randn(192, 1024, generator=g).bfloat16()
    aq, as_ = tb.hadamard_mxfp4_quant(a.cuda())
    bq, bs = tb.hadamard_mxfp4_quant(b.cuda())
    c = torch.zeros(256, 192, dtype=torch.bfloat16, device="cuda")
    tb.matmul_fp4(aq, bq, c, as_, bs)
    want = OG.ref_gemm_fp4(aq.cpu(), bq.cpu(), as_.cpu(), bs.cpu(), return_fp32=True)
    assert OG.rel_fro_error(c.float().cpu(), want.to(torch.bfloat16).float()) <= 1e-2
    exact = a.float() @ b.float().T
    assert OG.rel_fro_error(c.float().cpu(), exact) < 0.2
