"""Quantisation helpers around the GEMM entry points (reference include/tritonblas/utils.py).

``dynamic_mxfp4_quant`` / ``hadamard_mxfp4_quant`` run the library's HIP kernel; the per-channel FP8
recipe and the two dequantisers are a handful of torch ops on whatever device the tensor is on.
"""
from typing import Tuple, Union

import torch

from . import _lib
from ._lib import C


def get_fp8_dtypes():
    """gfx950 uses the OCP FP8 formats (reference utils.py:46)."""
    return torch.float8_e4m3fn, torch.float8_e5m2


def quantize_tensor_per_channel(tensor: torch.Tensor, target_dtype: torch.dtype, axis: int, *,
                                min_scale: float = 1e-8) -> Tuple[torch.Tensor, torch.Tensor]:
    """amax along ``axis`` -> scale = amax / dtype_max -> q = (x * (1/scale)).to(dtype); returns
    (q, scale squeezed along axis, fp32).  int8: dtype_max = 127, q rounded to nearest and clamped
    to [-127, 127] first.  Reference utils.py:340-377."""
    if target_dtype not in (torch.float8_e4m3fn, torch.float8_e5m2, torch.int8):
        raise ValueError(f"Unsupported quantized dtype: {target_dtype}")
    base = tensor.to(torch.float32)
    max_abs = torch.clamp(base.abs().amax(dim=axis, keepdim=True), min=min_scale)
    dtype_max = 127.0 if target_dtype == torch.int8 else torch.finfo(target_dtype).max
    scale = max_abs / dtype_max
    q = base * (1.0 / scale)
    if target_dtype == torch.int8:
        q = torch.round(q).clamp_(-dtype_max, dtype_max)
    return q.to(target_dtype), scale.squeeze(axis).to(torch.float32)


_E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]


def mxfp4_to_f32(x: torch.Tensor) -> torch.Tensor:
    """Packed e2m1 (two codes per byte, low nibble first) -> fp32 (reference utils.py:547-609)."""
    x = x.view(torch.uint8)
    lo, hi = x & 0xF, x >> 4
    idx = torch.stack([lo, hi], dim=-1).reshape(*x.shape[:-1], x.shape[-1] * 2).long()
    return torch.tensor(_E2M1, dtype=torch.float32, device=x.device)[idx]


def e8m0_to_f32(scale_e8m0: torch.Tensor) -> torch.Tensor:
    """E8M0 byte -> 2**(b-127); 0 -> 2**-127, 255 -> NaN (reference utils.py:612-643)."""
    b = scale_e8m0.view(torch.uint8)
    bits = b.to(torch.int32) << 23
    bits = torch.where(b == 0, torch.full_like(bits, 0x00400000), bits)
    bits = torch.where(b == 0xFF, torch.full_like(bits, 0x7F800001), bits)
    return bits.view(torch.float32)


def _quant(x: torch.Tensor, hadamard: bool, out=None):
    assert x.ndim == 2, "Input must be 2D tensor"
    M, N = x.shape
    assert N % 32 == 0, f"N ({N}) must be divisible by 32"
    if not x.is_cuda:
        raise RuntimeError("tritonblas_amd: the MXFP4 quantiser runs on the GPU only")
    if x.stride(1) != 1 or x.data_ptr() % 16 or (x.stride(0) * x.element_size()) % 16:
        # the kernel reads rows with 16-byte loads (a contiguous view that merely starts off a 16-byte
        # boundary needs a real copy: .contiguous() would hand the same memory back)
        x = x.clone(memory_format=torch.contiguous_format)
    if out is None:
        codes = torch.empty((M, N // 2), dtype=torch.uint8, device=x.device)
        scales = torch.empty((M, N // 32), dtype=torch.uint8, device=x.device)
    else:
        codes, scales = out
        for t, cols in ((codes, N // 2), (scales, N // 32)):
            assert t.dtype == torch.uint8 and t.device == x.device and tuple(t.shape) == (M, cols) and t.stride(1) == 1, \
                "out must be (codes (M, N/2), scales (M, N/32)) uint8 tensors on x's device with unit column stride"
    if M == 0 or N == 0:
        return codes, scales
    d = _lib.tb_quant_desc()
    d.struct_bytes = C.sizeof(_lib.tb_quant_desc)
    d.x_type = _lib.tb_dtype(x.dtype)
    d.m, d.n = M, N
    d.x, d.x_stride_m = C.c_void_p(x.data_ptr()), x.stride(0)
    d.codes, d.codes_stride_m = C.c_void_p(codes.data_ptr()), codes.stride(0)
    d.scales, d.scales_stride_m = C.c_void_p(scales.data_ptr()), scales.stride(0)
    d.hadamard = int(hadamard)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().tb_hadamard_mxfp4_quant(d, _lib.stream_handle(x.device)), "tb_hadamard_mxfp4_quant")
    return codes, scales


def dynamic_mxfp4_quant(x: torch.Tensor, *, out=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """(M, N) fp32/fp16/bf16 -> (codes (M, N/2) uint8, E8M0 scales (M, N/32) uint8).
    Reference utils.py:743-789.  `out=(codes, scales)` writes into caller-owned tensors (no allocation)."""
    return _quant(x, hadamard=False, out=out)


def hadamard_mxfp4_quant(x: torch.Tensor, *, out=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Same, after rotating every block of 32 values along N by H32/sqrt(32) in the same kernel."""
    return _quant(x, hadamard=True, out=out)


def hadamard32(x: torch.Tensor) -> torch.Tensor:
    """Blockwise H32/sqrt(32) rotation with torch ops (to rotate a weight offline)."""
    n = x.shape[-1]
    assert n % 32 == 0
    h = torch.ones(1, 1, dtype=torch.float32, device=x.device)
    for _ in range(5):
        h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
    y = x.to(torch.float32).reshape(-1, 32) @ h
    return (y * (1.0 / 32 ** 0.5)).reshape(x.shape)


def generate_matmul_inputs(m, n, k, in_dtype, out_dtype=torch.float16, transA="T", transB="T", init_type="randn",
                           *, device="cuda", seed=None):
    """A (m,k), B (k,n), C, bias (+ scales for fp8 / "fp4") with the reference's layout convention
    (utils.py:390-538): transA="T" stores A as (m,k); "N" stores (k,m) and returns its transpose view;
    transB="T" stores B as (k,n); "N" stores (n,k) and returns its transpose view."""
    from types import SimpleNamespace

    def init(shape, s):
        g = torch.Generator(device=device)
        if s is not None:
            g.manual_seed(s)
        if init_type == "randn":
            return torch.randn(shape, dtype=torch.float32, device=device, generator=g)
        if init_type == "hpl":
            return torch.rand(shape, dtype=torch.float32, device=device, generator=g) - 0.5
        if init_type == "zeros":
            return torch.zeros(shape, dtype=torch.float32, device=device)
        if init_type == "trig_float":
            return torch.arange(0, shape[0] * shape[1], device=device, dtype=torch.float32).reshape(shape).sin()
        raise ValueError(f"Unsupported init_type: {init_type}")

    A = init((m, k), seed) if transA == "T" else init((k, m), seed).T
    b_seed = seed + 10000 if seed is not None else None
    B = init((k, n), b_seed) if transB == "T" else init((n, k), b_seed).T
    scaleA = scaleB = None
    if isinstance(in_dtype, str) and in_dtype.lower() == "fp4":
        A, scaleA = dynamic_mxfp4_quant(A.contiguous())
        Bq, scaleB = dynamic_mxfp4_quant(B.T.contiguous())
        B = Bq.T
    elif in_dtype in (torch.float8_e4m3fn, torch.float8_e5m2, torch.int8):
        A, scaleA = quantize_tensor_per_channel(A, in_dtype, axis=1)
        B, scaleB = quantize_tensor_per_channel(B, in_dtype, axis=0)
    else:
        A, B = A.to(in_dtype), B.to(in_dtype)
    Cm = torch.zeros((m, n), device=device, dtype=out_dtype)
    bias = torch.zeros((m,), device=device, dtype=out_dtype)
    return SimpleNamespace(A=A, B=B, C=Cm, bias=bias, scaleA=scaleA, scaleB=scaleB)
