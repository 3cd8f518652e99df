"""GEMM entry points with the reference's Python signatures (include/tritonblas/matmul.py).

Each launcher fills one C descriptor and calls the shared library on torch's current stream; nothing
here computes.  ``a`` is (M, K), ``b`` is (K, N) with arbitrary 2-D strides (transposes are views),
``c`` is written in place and returned.
"""
from typing import Optional

import torch

from . import _lib
from ._lib import C
from .config import MatmulConfig, matmul_preamble
from .origami import OrigamiMatmulSelector


_SELECTOR_CACHE = {}
_SELECTOR_CACHE_MAX = 4096
# Launch state for entry points that are called without a MatmulConfig (tb.matmul(..., enable_streamk=True)
# and friends): one workspace per (device, stream), grown on demand.  Epoch tags make zeroing between
# launches unnecessary, and launches on one stream are ordered, so they can share it.  Entries are never
# dropped: a launch captured into a HIP graph keeps the raw pointer of the workspace it was given.
_STREAM_CONFIGS = {}


def _stream_config(dev) -> MatmulConfig:
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(dev).cuda_stream)
    cfg = _STREAM_CONFIGS.get(key)
    if cfg is None:
        cfg = MatmulConfig(device=dev, workspace=None)
        _STREAM_CONFIGS[key] = cfg
    return cfg


def _make_matmul_selector(M, N, K, a_dtype, b_dtype, c_dtype, device, mx_block_size=0, streamk=False,
                          num_stages: int = 2):
    """Reference matmul.py:42-66, which scores the tiles again on every call; here a selector is a pure
    function of its arguments and is kept (the entry points that build their own selector call this)."""
    key = (M, N, K, a_dtype, b_dtype, c_dtype, str(device), mx_block_size, bool(streamk), num_stages)
    sel = _SELECTOR_CACHE.get(key)
    if sel is None:
        if len(_SELECTOR_CACHE) >= _SELECTOR_CACHE_MAX:
            _SELECTOR_CACHE.clear()
        sel = OrigamiMatmulSelector(M, N, K, a_dtype, b_dtype, c_dtype, device, mx_block_size=mx_block_size,
                                    streamk=streamk, num_stages=num_stages)
        _SELECTOR_CACHE[key] = sel
    return sel


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(dev):
    """Context that makes ``dev`` the current device for a launch; free when it already is."""
    if dev.index is None or torch.cuda.current_device() == dev.index:
        return _NO_SWITCH
    return torch.cuda.device(dev)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _check_device(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("tritonblas_amd: tensors must live on a GPU (there is no CPU path)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("tritonblas_amd: tensors are on different devices")
    return dev


def _empty_problem(M, N, K, c, bias=None) -> bool:
    """M, N or K of zero: torch.matmul's answer (nothing to write, or an empty sum = zeros plus the bias)
    without a launch.  True when the problem was such a one."""
    if M == 0 or N == 0:
        return True
    if K == 0:
        if bias is None:
            c.zero_()
        else:
            c.copy_(bias.reshape(1, N).to(torch.float32).expand(M, N))
        return True
    return False


def _launch_gemm(a, b, c, selector, config, schedule, bias=None, a_scale=None, b_scale=None, sk_grid=None):
    assert a.shape[1] == b.shape[0], "Incompatible Dimensions"
    M, K = a.shape
    _, N = b.shape
    assert c.shape[0] == M and c.shape[1] == N, "Incompatible Dimensions"
    dev = _check_device(a, b, c, bias, a_scale, b_scale)
    if _empty_problem(M, N, K, c, bias):
        return c
    lib = _lib.load()
    d = _lib.tb_gemm_desc()
    d.struct_bytes = C.sizeof(_lib.tb_gemm_desc)
    d.a_type, d.b_type, d.c_type = _lib.tb_dtype(a.dtype), _lib.tb_dtype(b.dtype), _lib.tb_dtype(c.dtype)
    d.m, d.n, d.k = M, N, K
    d.a_stride_m, d.a_stride_k = a.stride(0), a.stride(1)
    d.b_stride_k, d.b_stride_n = b.stride(0), b.stride(1)
    d.c_stride_m, d.c_stride_n = c.stride(0), c.stride(1)
    d.a, d.b, d.c = _ptr(a), _ptr(b), _ptr(c)
    if (a_scale is None) != (b_scale is None):
        raise RuntimeError("tritonblas_amd: a_scale and b_scale come together")
    if a_scale is not None:
        if a_scale.dtype != torch.float32 or b_scale.dtype != torch.float32:
            raise RuntimeError("tritonblas_amd: scales must be float32")
        a_scale, b_scale = a_scale.reshape(-1), b_scale.reshape(-1)
        if not (a_scale.is_contiguous() and b_scale.is_contiguous() and a_scale.numel() == M and b_scale.numel() == N):
            raise RuntimeError("tritonblas_amd: a_scale must be contiguous (M,) and b_scale contiguous (N,)")
        d.a_scale, d.b_scale = _ptr(a_scale), _ptr(b_scale)
    if bias is not None:
        if bias.numel() != N:
            raise AssertionError("Incompatible Dimensions")
        if bias.dim() != 1:
            bias = bias.reshape(-1)     # (1, N) and the like: one value per output column
        d.bias, d.bias_type, d.bias_stride = _ptr(bias), _lib.tb_dtype(bias.dtype), bias.stride(0)
    if selector is not None:
        d.block_m, d.block_n, d.block_k = selector.block_m, selector.block_n, selector.block_k
        d.group_m, d.num_xcds = selector.group_m, selector.num_sms
        d.counters_per_xcd = selector.COUNTERS_PER_XCD
    d.schedule = schedule
    streamk = schedule in (_lib.TB_SCHED_STREAMK, _lib.TB_SCHED_STREAMK_WS)
    if selector is not None and getattr(selector, "_total_cus", None) is not None and not streamk:
        # a selector built for a CU partition sizes the launch (reference matmul.py:113: grid = N_CU):
        # as many workgroups as that many CUs hold at once; a mask (below) makes it one per mask entry
        d.grid = selector._N_CU * max(1, selector.waves_per_eu)
    if schedule == _lib.TB_SCHED_WORK_STEALING and config is not None:
        # reference matmul.py:112-159: GLOBAL_ATOMIC from the config, the per-workgroup mask by program id
        if getattr(config, "hierarchical", False):
            # (the split is left to the library: it knows the tile the launch really runs, which is not
            # the selector's when the operands need the gather kernel)
            d.ws_mode = _lib.TB_WS_HIERARCHICAL
        elif config.global_atomic:
            d.ws_mode = _lib.TB_WS_GLOBAL_ATOMIC
        mask = config.active_mask()
        if mask is not None:
            if mask.dtype != torch.int32 or not mask.is_contiguous() or mask.device != dev:
                raise RuntimeError("tritonblas_amd: config.mask must be a contiguous int32 tensor on the GEMM's device")
            d.cu_mask, d.cu_mask_len = _ptr(mask), mask.numel()
            d.grid = 0
    if streamk:
        if sk_grid is not None:
            d.grid = int(sk_grid)
        elif selector is not None and selector.streamk:
            d.grid = selector.sk_grid
    if schedule != _lib.TB_SCHED_PERSISTENT:
        # 0 bytes: the library runs this problem with a kernel that needs no workspace (or refuses the
        # descriptor, which the launch below reports)
        need = lib.tb_workspace_bytes(d)
        if need > 0:
            if config is None:
                config = _stream_config(dev)
            ws = config.ensure(need)
            d.workspace, d.workspace_bytes = C.c_void_p(ws.data_ptr()), ws.numel()
            # (the workspace tags Stream-K launches with its own count: nothing in the descriptor changes from
            # call to call, so a launch captured in a graph can be replayed)
            d.epoch = _lib.TB_EPOCH_ON_DEVICE
            d.spin_limit = int(getattr(config, "spin_limit", 0) or 0)
    with _on_device(dev):
        _lib.check(lib.tb_gemm(d, _lib.stream_handle(dev)), "tb_gemm")
    return c


def persistent_matmul_lt(a, b, c, selector, config: Optional[MatmulConfig] = None, bias=None, a_scale=None,
                         b_scale=None, quantized: bool = False, work_stealing: bool = False):
    """Data-parallel launch, optionally through the work-stealing queues (reference matmul.py:69-200)."""
    sched = _lib.TB_SCHED_WORK_STEALING if (work_stealing and config is not None) else _lib.TB_SCHED_PERSISTENT
    return _launch_gemm(a, b, c, selector, config, sched, bias=bias,
                        a_scale=a_scale if quantized else None, b_scale=b_scale if quantized else None)


def streamk_matmul_lt(a, b, c, selector, config: Optional[MatmulConfig] = None, bias=None, sk_grid=None,
                      a_scale=None, b_scale=None, quantized: bool = False, work_stealing: bool = False):
    """Stream-K launch (reference matmul.py:202-366).  ``work_stealing``: the whole tiles in front of the
    Stream-K tail are drawn from the XCD x slot queues instead of being dealt out by workgroup id (reference
    matmul.py:279-323, kernels/streamk_gemm_work_stealing.py); the tail itself is the same, and so are the
    results.  A launch that shares the device with other work can run into the poll bound of the partial-tile
    exchange (NaN tiles + the workspace's status word): callers in that situation should call
    ``config.check()`` after synchronising."""
    sched = _lib.TB_SCHED_STREAMK_WS if work_stealing else _lib.TB_SCHED_STREAMK
    return _launch_gemm(a, b, c, selector, config, sched, bias=bias, sk_grid=sk_grid,
                        a_scale=a_scale if quantized else None, b_scale=b_scale if quantized else None)


def matmul_lt(a, b, c, selector, config: MatmulConfig = None, enable_streamk=False, work_stealing=False):
    """Reference matmul.py:368-378."""
    assert a.shape[1] == b.shape[0], "Incompatible Dimensions"
    if enable_streamk:
        return streamk_matmul_lt(a, b, c, selector, config, work_stealing=work_stealing)
    return persistent_matmul_lt(a, b, c, selector, config, work_stealing=work_stealing)


def matmul_a8w8_lt(a, b, a_scale, b_scale, c, selector, config: MatmulConfig = None, enable_streamk=False,
                   work_stealing=False):
    """Reference matmul.py:380-390."""
    assert a.shape[1] == b.shape[0], "Incompatible Dimensions"
    if enable_streamk:
        return streamk_matmul_lt(a, b, c, selector, config, a_scale=a_scale, b_scale=b_scale, quantized=True)
    return persistent_matmul_lt(a, b, c, selector, config, a_scale=a_scale, b_scale=b_scale, quantized=True,
                                work_stealing=work_stealing)


def _run(a, b, out, bias, enable_streamk, sk_grid, work_stealing, out_dtype_for_selector):
    M, K = a.shape
    _, N = b.shape
    if _empty_problem(M, N, K, out, bias):
        return out
    selector = _make_matmul_selector(M, N, K, a.dtype, b.dtype, out_dtype_for_selector, a.device,
                                     streamk=bool(enable_streamk))
    config = matmul_preamble(selector, a.device) if work_stealing else None
    if enable_streamk:
        return streamk_matmul_lt(a, b, out, selector, config, bias=bias, sk_grid=sk_grid, work_stealing=work_stealing)
    return persistent_matmul_lt(a, b, out, selector, config, bias=bias, work_stealing=work_stealing)


# ---- torch custom operators (reference matmul.py:393-472, 628-752) ----------------------------------
# Registered with torch.library so that autograd and torch.compile (fullgraph) see one opaque operator
# with a shape rule (fake implementation) instead of a ctypes call they cannot trace.  The reference
# registers the same four operators with triton_op; the namespace differs so that both packages can be
# imported side by side.
def _fake_new_output(a, b):
    assert a.shape[1] == b.shape[0], "Incompatible A-B Dimensions"
    return a.new_empty(a.shape[0], b.shape[1])


@torch.library.custom_op("tritonblas_amd::_matmul", mutates_args=())
def _matmul(a: torch.Tensor, b: torch.Tensor, enable_streamk: Optional[bool] = False, sk_grid: Optional[int] = None,
            work_stealing: Optional[bool] = False) -> torch.Tensor:
    assert a.shape[1] == b.shape[0], "Incompatible A-B Dimensions"
    out = a.new_empty(a.shape[0], b.shape[1])
    _run(a, b, out, None, enable_streamk, sk_grid, work_stealing, out.dtype)
    return out


@_matmul.register_fake
def _(a, b, enable_streamk=False, sk_grid=None, work_stealing=False):
    return _fake_new_output(a, b)


def _matmul_setup_context(ctx, inputs, output):
    a, b, enable_streamk, sk_grid, work_stealing = inputs
    ctx.save_for_backward(a, b)
    ctx.opts = (enable_streamk, sk_grid, work_stealing)


def _matmul_backward(ctx, grad_output):
    # two more library GEMMs: grad_a = g @ b^T, grad_b = a^T @ g
    a, b = ctx.saved_tensors
    sk, grid, ws = ctx.opts
    g = grad_output.contiguous()
    grad_a = matmul(g, b.T.contiguous(), enable_streamk=sk, sk_grid=grid, work_stealing=ws)
    grad_b = matmul(a.T.contiguous(), g, enable_streamk=sk, sk_grid=grid, work_stealing=ws)
    return grad_a, grad_b, None, None, None


_matmul.register_autograd(_matmul_backward, setup_context=_matmul_setup_context)


@torch.library.custom_op("tritonblas_amd::_matmul_out", mutates_args={"out"})
def _matmul_out(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor, enable_streamk: Optional[bool] = False,
                sk_grid: Optional[int] = None, work_stealing: Optional[bool] = False) -> None:
    assert a.shape[1] == b.shape[0], "Incompatible A-B Dimensions"
    _run(a, b, out, None, enable_streamk, sk_grid, work_stealing, out.dtype)


@_matmul_out.register_fake
def _(a, b, out, enable_streamk=False, sk_grid=None, work_stealing=False):
    assert a.shape[1] == b.shape[0], "Incompatible A-B Dimensions"
    return None


@torch.library.custom_op("tritonblas_amd::_addmm", mutates_args=())
def _addmm(bias: torch.Tensor, a: torch.Tensor, b: torch.Tensor, enable_streamk: Optional[bool] = False,
           sk_grid: Optional[int] = None, work_stealing: Optional[bool] = False) -> torch.Tensor:
    assert a.shape[1] == b.shape[0], "Incompatible A-B Dimensions"
    out = a.new_empty(a.shape[0], b.shape[1])
    _run(a, b, out, bias, enable_streamk, sk_grid, work_stealing, bias.dtype)
    return out


@_addmm.register_fake
def _(bias, a, b, enable_streamk=False, sk_grid=None, work_stealing=False):
    return _fake_new_output(a, b)


def _addmm_setup_context(ctx, inputs, output):
    bias, a, b, enable_streamk, sk_grid, work_stealing = inputs
    ctx.save_for_backward(a, b)
    ctx.opts = (enable_streamk, sk_grid, work_stealing)
    ctx.bias_shape = tuple(bias.shape)


def _addmm_backward(ctx, grad_output):
    a, b = ctx.saved_tensors
    sk, grid, ws = ctx.opts
    g = grad_output.contiguous()
    grad_a = matmul(g, b.T.contiguous(), enable_streamk=sk, sk_grid=grid, work_stealing=ws)
    grad_b = matmul(a.T.contiguous(), g, enable_streamk=sk, sk_grid=grid, work_stealing=ws)
    return grad_output.sum(dim=0).reshape(ctx.bias_shape), grad_a, grad_b, None, None, None


_addmm.register_autograd(_addmm_backward, setup_context=_addmm_setup_context)


@torch.library.custom_op("tritonblas_amd::_addmm_out", mutates_args={"out"})
def _addmm_out(bias: torch.Tensor, a: torch.Tensor, b: torch.Tensor, out: torch.Tensor,
               enable_streamk: Optional[bool] = False, sk_grid: Optional[int] = None,
               work_stealing: Optional[bool] = False) -> None:
    assert a.shape[1] == b.shape[0], "Incompatible A-B Dimensions"
    _run(a, b, out, bias, enable_streamk, sk_grid, work_stealing, bias.dtype)


@_addmm_out.register_fake
def _(bias, a, b, out, enable_streamk=False, sk_grid=None, work_stealing=False):
    assert a.shape[1] == b.shape[0], "Incompatible A-B Dimensions"
    return None


def matmul(a, b, out: Optional[torch.Tensor] = None, enable_streamk: Optional[bool] = False,
           sk_grid: Optional[int] = None, work_stealing: Optional[bool] = False) -> Optional[torch.Tensor]:
    """Reference matmul.py:475-495: out=None allocates and supports autograd; out=... writes in
    place, returns None and refuses tensors that require grad."""
    if out is None:
        return _matmul(a, b, enable_streamk, sk_grid, work_stealing)
    if torch.is_grad_enabled() and (a.requires_grad or b.requires_grad or out.requires_grad):
        raise RuntimeError(
            "tritonblas.matmul(): functions with out=... arguments don't support "
            "automatic differentiation, but one of the arguments requires grad."
        )
    return _matmul_out(a, b, out, enable_streamk, sk_grid, work_stealing)


def addmm(bias, a, b, out: Optional[torch.Tensor] = None, enable_streamk: Optional[bool] = False,
          sk_grid: Optional[int] = None, work_stealing: Optional[bool] = False) -> Optional[torch.Tensor]:
    """Reference matmul.py:727-752; the bias is added per output column."""
    if out is None:
        return _addmm(bias, a, b, enable_streamk, sk_grid, work_stealing)
    if torch.is_grad_enabled() and (bias.requires_grad or a.requires_grad or b.requires_grad or out.requires_grad):
        raise RuntimeError(
            "tritonblas.addmm(): functions with out=... arguments don't support "
            "automatic differentiation, but one of the arguments requires grad."
        )
    return _addmm_out(bias, a, b, out, enable_streamk, sk_grid, work_stealing)


def matmul_a8w8(a, b, a_scale, b_scale, c, enable_streamk=False, work_stealing=False, sk_grid=None):
    """Reference matmul.py:498-517."""
    assert a.shape[1] == b.shape[0], "Incompatible Dimensions"
    M, K = a.shape
    _, N = b.shape
    if _empty_problem(M, N, K, c):
        return c
    selector = _make_matmul_selector(M, N, K, a.dtype, b.dtype, c.dtype, a.device, streamk=bool(enable_streamk))
    config = matmul_preamble(selector, a.device) if work_stealing else None
    if enable_streamk:
        return streamk_matmul_lt(a, b, c, selector, config, sk_grid=sk_grid, a_scale=a_scale, b_scale=b_scale,
                                 quantized=True, work_stealing=work_stealing)
    return persistent_matmul_lt(a, b, c, selector, config, a_scale=a_scale, b_scale=b_scale, quantized=True,
                                work_stealing=work_stealing)


def matmul_fp4(a, b, c, a_scales, b_scales, block_m: int = None, block_n: int = None, block_k: int = None,
               group_size_m: int = 8, num_warps: int = 8, num_stages: int = 2):
    """MXFP4 GEMM (reference matmul.py:519-625).  a: (M, K/2) uint8, b: (N, K/2) uint8 (two e2m1
    codes per byte, low nibble first), scales (M|N, K/32) E8M0 bytes, c: (M, N) bf16/fp16.
    ``num_warps``/``num_stages`` are accepted for signature compatibility; the kernels fix them."""
    M, Kp = a.shape
    N = b.shape[0]
    K = Kp * 2
    assert b.shape[1] * 2 == K, f"Incompatible Dimensions: A has K={K}, B has K={b.shape[1] * 2}"
    for t in (a, b, a_scales, b_scales):
        if t.element_size() != 1:
            raise RuntimeError(f"tritonblas_amd: matmul_fp4 takes packed codes and E8M0 scales as one-byte elements, got {t.dtype}")
    if tuple(a_scales.shape) != (M, K // 32) or tuple(b_scales.shape) != (N, K // 32):
        raise RuntimeError(f"tritonblas_amd: matmul_fp4 scales must be (M, K/32) and (N, K/32), got {tuple(a_scales.shape)} and {tuple(b_scales.shape)}")
    dev = _check_device(a, b, c, a_scales, b_scales)
    if M == 0 or N == 0:
        return c
    a, b = a.view(torch.uint8), b.view(torch.uint8)
    a_scales, b_scales = a_scales.view(torch.uint8), b_scales.view(torch.uint8)
    if a.stride(1) != 1 or b.stride(1) != 1:
        raise RuntimeError("tritonblas_amd: matmul_fp4 needs K-contiguous packed operands")
    d = _lib.tb_gemm_fp4_desc()
    d.struct_bytes = C.sizeof(_lib.tb_gemm_fp4_desc)
    d.c_type = _lib.tb_dtype(c.dtype)
    d.m, d.n, d.k = M, N, K
    d.a, d.b, d.c = _ptr(a), _ptr(b), _ptr(c)
    d.a_stride_m, d.b_stride_n = a.stride(0), b.stride(0)
    d.c_stride_m, d.c_stride_n = c.stride(0), c.stride(1)
    d.a_scales, d.b_scales = _ptr(a_scales), _ptr(b_scales)
    d.a_scales_stride_m, d.a_scales_stride_k = a_scales.stride(0), a_scales.stride(1)
    d.b_scales_stride_n, d.b_scales_stride_k = b_scales.stride(0), b_scales.stride(1)
    if block_m is not None:
        assert block_k % 64 == 0, "BLOCK_K must be multiple of 64 for FP4"
        d.block_m, d.block_n, d.block_k = block_m, block_n, block_k
        d.group_m = group_size_m
    with _on_device(dev):
        _lib.check(_lib.load().tb_gemm_fp4(d, _lib.stream_handle(dev)), "tb_gemm_fp4")
    return c


def grouped_matmul_a8w8(a, w, a_scale, w_scale, c, group_offsets, block_m: int = None, block_n: int = None,
                        block_k: int = None, small_rows: int = 0, enable_streamk: bool = False,
                        config: MatmulConfig = None):
    """Grouped (MoE) FP8 GEMM: rows ``group_offsets[e]:group_offsets[e+1]`` of ``a`` (M, K) meet expert
    weight ``w[e]`` (N, K); ``c[rows] = cast((a[rows] @ w[e].T) * a_scale[rows, None] * w_scale[e][None, :])``.
    ``group_offsets`` is an int32 device tensor of E+1 ascending row offsets.  No host sync: the row counts
    are only read on the device.  An expert's last partial row block of at most ``small_rows`` rows goes to a
    second launch with a 32-row tile (0: the library's default of 64 rows, off when a tile is forced; -1: off).
    ``enable_streamk``: the tiles that do not fill whole rounds of the launch grid are cut into K ranges when the
    row counts make that cheaper than one more round (decided on the device; only those tiles' summation order
    changes).  The flags and partial tiles live in ``config``'s workspace, by default the one this package keeps
    per device and stream.  Off by default: exchanging 256x256 partial tiles costs about as much as 50 K steps, so it
    only pays for long K (beyond about 8192 for FP8), and the kernel that can cut tiles is 2-3 % slower when it
    does not."""
    M, K = a.shape
    E, N, K2 = w.shape
    assert K == K2 and c.shape[0] == M and c.shape[1] == N, "Incompatible Dimensions"
    assert group_offsets.numel() == E + 1 and group_offsets.dtype == torch.int32
    if a.dtype != torch.float8_e4m3fn or w.dtype != torch.float8_e4m3fn:
        raise RuntimeError(f"tritonblas_amd: grouped GEMM takes float8_e4m3fn operands, got {a.dtype} and {w.dtype}")
    dev = _check_device(a, w, c, a_scale, w_scale, group_offsets)
    if M == 0 or N == 0:
        return c
    if a.stride(1) != 1 or w.stride(2) != 1:
        raise RuntimeError("tritonblas_amd: grouped GEMM needs K-contiguous operands")
    d = _lib.tb_grouped_gemm_desc()
    d.struct_bytes = C.sizeof(_lib.tb_grouped_gemm_desc)
    d.c_type = _lib.tb_dtype(c.dtype)
    d.m_total, d.n, d.k, d.num_groups = M, N, K, E
    d.a, d.w, d.c = _ptr(a), _ptr(w), _ptr(c)
    d.a_stride_m, d.w_stride_g, d.w_stride_n = a.stride(0), w.stride(0), w.stride(1)
    d.c_stride_m, d.c_stride_n = c.stride(0), c.stride(1)
    if a_scale is not None:
        a_scale, w_scale = a_scale.reshape(-1), w_scale.reshape(E, N)
        if not (a_scale.is_contiguous() and w_scale.is_contiguous()):
            raise RuntimeError("tritonblas_amd: scales must be contiguous")
        d.a_scale, d.w_scale = _ptr(a_scale), _ptr(w_scale)
    d.group_offsets = _ptr(group_offsets)
    if block_m is not None:
        d.block_m, d.block_n, d.block_k = block_m, block_n, block_k
    d.small_rows = small_rows
    with _on_device(dev):
        lib = _lib.load()
        if enable_streamk:
            d.streamk = 1
            need = lib.tb_grouped_workspace_bytes(d)
            if need:
                cfg = config if config is not None else _stream_config(dev)
                ws = cfg.ensure(need)
                d.workspace, d.workspace_bytes = ws.data_ptr(), ws.numel()
                d.epoch, d.spin_limit = _lib.TB_EPOCH_ON_DEVICE, cfg.spin_limit
            else:
                d.streamk = 0
        _lib.check(lib.tb_grouped_gemm_fp8(d, _lib.stream_handle(dev)), "tb_grouped_gemm_fp8")
    return c
