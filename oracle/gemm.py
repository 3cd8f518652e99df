"""GEMM oracles: fp32 CPU ``torch.matmul`` of the (dequantised) operands, then the fused epilogue.

Test infrastructure: see ``oracle/__init__.py``.

These are the reference's own oracles restated:
  * fp16/bf16: ``torch.matmul`` / ``torch.mm``   tests/test_matmul_correctness.py:44, tests/test_matmul_lt.py:60
  * a8w8:      fp32 matmul * (sa[:,None]*sb[None,:]) (+bias) -> clamp for fp8 out -> cast
               tests/test_matmul_a8w8_lt.py:11-38, benchmarks/tritonblas_matmul.py:62-76
  * MXFP4:     LUT x E8M0 dequant, ``torch.mm(x, w.T)``   tests/test_matmul_fp4.py:20-46
  * FP8 per-channel quantisation recipe   include/tritonblas/utils.py:340-377
The grouped (MoE) GEMM has no reference code; it is the concatenation of per-expert a8w8 closed forms.
"""
import numpy as np
import torch

from . import mxfp4


def _div_by_scalar_as_on_gpu(t: torch.Tensor, s: float) -> torch.Tensor:
    """``tensor / python_scalar`` as torch evaluates it on a GPU: one multiplication by the scalar's fp32
    reciprocal (its element-wise kernels fold the division), which differs from a true division by one
    unit in the last place for some inputs.  The reference's quantisation recipe only ever runs on the
    GPU, so this -- not CPU torch's true division -- is the arithmetic behind its scales."""
    return t * torch.tensor(1.0 / s, dtype=torch.float32)


def quantize_per_channel_fp8(x: torch.Tensor, axis: int, dtype=torch.float8_e4m3fn, min_scale: float = 1e-8):
    """include/tritonblas/utils.py:340-377: amax -> scale = amax/448 -> q = (x * (1/scale)).to(fp8)."""
    base = x.to(torch.float32)
    max_abs = torch.clamp(base.abs().amax(dim=axis, keepdim=True), min=min_scale)
    scale = _div_by_scalar_as_on_gpu(max_abs, torch.finfo(dtype).max)
    inv = 1.0 / scale
    q = (base * inv).to(dtype)
    return q, scale.squeeze(axis).to(torch.float32)


def quantize_per_channel_int8(x: torch.Tensor, axis: int, min_scale: float = 1e-8):
    """include/tritonblas/utils.py:364-375, int8 branch: amax -> scale = amax/127 ->
    q = clamp(round(x * (1/scale)), -127, 127).to(int8)."""
    base = x.to(torch.float32)
    max_abs = torch.clamp(base.abs().amax(dim=axis, keepdim=True), min=min_scale)
    scale = _div_by_scalar_as_on_gpu(max_abs, 127.0)
    q = torch.round(base * (1.0 / scale)).clamp_(-127.0, 127.0).to(torch.int8)
    return q, scale.squeeze(axis).to(torch.float32)


def ref_gemm_int8(a: torch.Tensor, b: torch.Tensor, out_dtype, a_scale=None, b_scale=None, bias=None):
    """int8 operands: exact integer sums (include/tritonblas/kernels/persistent_gemm.py:75), then the
    a8w8 epilogue in fp32 (tests/test_matmul_a8w8_lt.py:11-38).  out_dtype int8: the fp32 result is
    truncated toward zero and saturated to [-128, 127] -- a decision of this build: the reference
    converts with a bare float->int8 cast, which is undefined outside that range, its own (switched
    off) test clamps the expectation to +-127 and compares at atol 5; parity unpinned.
    Returns fp64 for float out types (the caller rounds) and int8 for int8."""
    acc = torch.matmul(a.to(torch.int64), b.to(torch.int64)).to(torch.float64)
    if a_scale is not None and b_scale is not None:
        acc = (acc.to(torch.float32) * (a_scale.to(torch.float32)[:, None] * b_scale.to(torch.float32)[None, :])).to(torch.float64)
    if bias is not None:
        acc = acc + bias.to(torch.float64)[None, :]
    if out_dtype == torch.int8:
        return torch.clamp(torch.trunc(acc.to(torch.float32)), -128, 127).to(torch.int8)
    return acc


def ref_gemm(a: torch.Tensor, b: torch.Tensor, out_dtype=None, a_scale=None, b_scale=None, bias=None):
    """C = cast((fp32(A) @ fp32(B)) * (sa[:,None]*sb[None,:]) + bias[None,:]).

    a: (M, K), b: (K, N), any strides, any float dtype that converts to fp32 (incl. float8_e4m3fn).
    Epilogue order follows tests/test_matmul_a8w8_lt.py:11-38; the bias is per output *column*
    (include/tritonblas/kernels/stages/matrix_view.py:194-208, tests/test_addmm_correctness.py:35)."""
    acc = torch.matmul(a.to(torch.float32), b.to(torch.float32))
    if a_scale is not None and b_scale is not None:
        acc = acc * (a_scale.to(torch.float32)[:, None] * b_scale.to(torch.float32)[None, :])
    if bias is not None:
        acc = acc + bias.to(torch.float32)[None, :]
    if out_dtype is None:
        out_dtype = a.dtype
    if out_dtype in (torch.float8_e4m3fn, torch.float8_e5m2):   # tests/test_matmul_a8w8_lt.py:27-32
        mx = torch.finfo(out_dtype).max
        acc = torch.clamp(acc, -mx, mx)
    return acc.to(out_dtype)


def ref_gemm_fp4(a_codes, b_codes, a_scales, b_scales, out_dtype=torch.bfloat16, return_fp32=False):
    """a_codes (M, K/2) u8, b_codes (N, K/2) u8, scales (M|N, K/32) u8 -> (M, N).

    tests/test_matmul_fp4.py:20-46."""
    A = torch.from_numpy(mxfp4.dequant(_np(a_codes), _np(a_scales)))
    B = torch.from_numpy(mxfp4.dequant(_np(b_codes), _np(b_scales)))
    acc = torch.mm(A, B.T)
    return acc if return_fp32 else acc.to(out_dtype)


def ref_grouped_gemm_fp8(a_q, w_q, a_scale, w_scale, offsets, out_dtype=torch.bfloat16, return_fp32=False):
    """a_q (M, K) fp8 rows sorted by expert; w_q (E, N, K) fp8; a_scale (M,), w_scale (E, N);
    offsets int (E+1,) row boundaries.  Rows of expert e: C[o[e]:o[e+1]] = a8w8 closed form with W[e]."""
    E, N, K = w_q.shape
    M = a_q.shape[0]
    out = torch.zeros(M, N, dtype=torch.float32)
    off = [int(v) for v in offsets]
    for e in range(E):
        lo, hi = off[e], off[e + 1]
        if hi <= lo:
            continue
        acc = torch.matmul(a_q[lo:hi].to(torch.float32), w_q[e].to(torch.float32).T)
        out[lo:hi] = acc * (a_scale[lo:hi].to(torch.float32)[:, None] * w_scale[e].to(torch.float32)[None, :])
    return out if return_fp32 else out.to(out_dtype)


def rel_fro_error(got: torch.Tensor, want: torch.Tensor) -> float:
    """||got - want||_F / ||want||_F in fp64 (the parity measure the tolerances are stated in)."""
    g = got.detach().to("cpu", torch.float64)
    w = want.detach().to("cpu", torch.float64)
    den = torch.linalg.norm(w).item()
    return torch.linalg.norm(g - w).item() / (den if den > 0 else 1.0)


def _np(t):
    if isinstance(t, torch.Tensor):
        return t.detach().cpu().contiguous().view(torch.uint8).numpy()
    return np.asarray(t, dtype=np.uint8)
