"""GPU parity tests of the GEMM entry points against the CPU oracle (all launches go through the
C ABI).  Tolerances: relative Frobenius error <= 1e-3 for fp16/bf16 and <= 1e-2 for FP8/MXFP4,
measured against the oracle's fp32 GEMM of the (dequantised) operands rounded to the output type
the same way the kernel's epilogue rounds."""
import sys

import numpy as np
import pytest
import torch

from conftest import DTYPES, EDGE_CASE_DIMS, SKINNY_DIMS, STANDARD_DIMS
from oracle import gemm as OG
from oracle import inputs as OI
from oracle import mxfp4 as OM

pytestmark = pytest.mark.gpu

TOL_16 = 1e-3
TOL_Q = 1e-2


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _layout(x_cpu, trans):
    """Reference convention (utils.py:495-505): "T" keeps the logical shape contiguous, "N" stores
    the transpose and hands out a view."""
    x = x_cpu.cuda()
    if trans == "T":
        return x.contiguous()
    return x.T.contiguous().T


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _check(c_gpu, want_fp32, out_dtype, tol):
    want = want_fp32.to(out_dtype)
    err = OG.rel_fro_error(c_gpu.float(), want.float())
    assert err <= tol, f"relative Frobenius error {err:.3e} > {tol}"
    return err


@pytest.mark.parametrize("m,n,k", STANDARD_DIMS + EDGE_CASE_DIMS + SKINNY_DIMS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("transA,transB", [("T", "T"), ("N", "N"), ("T", "N"), ("N", "T")])
def test_matmul_16bit(m, n, k, dtype, transA, transB):
    import tritonblas_amd as tb
    _say(f"matmul {m}x{n}x{k} {dtype} {transA}{transB}")
    a_cpu, b_cpu = _rand((m, k), dtype, 0, 0.5), _rand((k, n), dtype, 10000, 0.5)
    a, b = _layout(a_cpu, transA), _layout(b_cpu, transB)
    c = tb.matmul(a, b)
    assert c.shape == (m, n) and c.dtype == dtype
    _check(c.cpu(), OG.ref_gemm(a_cpu, b_cpu, torch.float32), dtype, TOL_16)


@pytest.mark.parametrize("m,n,k", [(1024, 1024, 1024), (512, 768, 320), (300, 200, 192), (257, 129, 64)])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tile", [(256, 256, 64), (128, 128, 64), (64, 64, 64), (32, 128, 128)])
def test_every_16bit_tile_variant(m, n, k, dtype, tile):
    """Forces each built tile through matmul_lt (the selector would otherwise pick one)."""
    import tritonblas_amd as tb
    _say(f"matmul_lt {m}x{n}x{k} {dtype} tile={tile}")
    a_cpu, b_cpu = _rand((m, k), dtype, 1, 0.5), _rand((k, n), dtype, 10001, 0.5)
    want = OG.ref_gemm(a_cpu, b_cpu, torch.float32)
    for ta, tb_ in [("T", "T"), ("T", "N"), ("N", "T"), ("N", "N")]:
        a, b = _layout(a_cpu, ta), _layout(b_cpu, tb_)
        sel = tb.OrigamiMatmulSelector(m, n, k, dtype, dtype, dtype, a.device)
        sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = tile
        c = torch.zeros(m, n, dtype=dtype, device="cuda")
        out = tb.matmul_lt(a, b, c, sel, None)
        assert out is c
        _check(c.cpu(), want, dtype, TOL_16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
@pytest.mark.parametrize("stages", [3, 4])
@pytest.mark.parametrize("m,n,k", [(128, 512, 4096), (300, 200, 2304), (64, 64, 128), (512, 1024, 640)])
def test_deep_pipeline_variants_of_the_small_tile(dtype, stages, m, n, k, tb_option):
    """The 64x64 tile exists with 2, 3 and 4 copy stages; the library takes a deeper one while all tiles
    are resident at once.  Here every depth is forced (hook "waves" = waves_m, waves_n, stages), K both
    shorter and longer than the pipeline, ragged edges, Stream-K on top."""
    import tritonblas_amd as tb
    tb_option("waves", 220 + stages)
    tb_option("no_skinny", 1)
    _say(f"deep pipeline {dtype} stages={stages} {m}x{n}x{k}")
    quant = dtype == torch.float8_e4m3fn
    if quant:
        aq, bq, sa, sb = _a8w8_case(m, n, k, seed=61)
        a, b = aq.cuda(), bq.T.contiguous().cuda().T
        want, out_dtype, tol = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb), torch.bfloat16, TOL_Q
    else:
        a_cpu, b_cpu = _rand((m, k), dtype, 62, 0.5), _rand((k, n), dtype, 63, 0.5)
        a, b = a_cpu.cuda(), b_cpu.T.contiguous().cuda().T
        want, out_dtype, tol = OG.ref_gemm(a_cpu, b_cpu, torch.float32), dtype, TOL_16
    for sk in (False, True):
        sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, out_dtype, a.device, streamk=sk)
        sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 64, 64, (128 if quant else 64)
        cfg = tb.matmul_preamble(sel)
        c = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
        if quant:
            tb.matmul_a8w8_lt(a, b, sa.cuda(), sb.cuda(), c, sel, cfg, enable_streamk=sk)
        else:
            tb.matmul_lt(a, b, c, sel, cfg, enable_streamk=sk)
        _check(c.cpu(), want, out_dtype, tol)


def test_config1_fp16_1024():
    import tritonblas_amd as tb
    a_cpu, b_cpu = OI.c1_fp16()
    sel = tb.OrigamiMatmulSelector(1024, 1024, 1024, torch.float16, torch.float16, torch.float16, torch.device("cuda"))
    cfg = tb.matmul_preamble(sel)
    c = torch.empty(1024, 1024, dtype=torch.float16, device="cuda")
    tb.matmul_lt(a_cpu.cuda(), b_cpu.cuda(), c, sel, cfg)
    want32 = OG.ref_gemm(a_cpu, b_cpu, torch.float32)
    err = _check(c.cpu(), want32, torch.float16, TOL_16)
    # fp16 keeps 11 significant bits: the result also meets 1e-3 against the UNROUNDED fp32 GEMM (a bf16
    # result cannot: its own output rounding is 1.5e-3 of the norm)
    err_unrounded = OG.rel_fro_error(c.float().cpu(), want32)
    assert err_unrounded <= TOL_16, f"against the unrounded fp32 GEMM: {err_unrounded:.3e}"
    _say(f"config 1 fp16 1024^3 rel fro err {err:.2e} (unrounded oracle: {err_unrounded:.2e})")


def test_out_semantics_and_autograd():
    import tritonblas_amd as tb
    a = _rand((64, 128), torch.bfloat16, 3).cuda()
    b = _rand((128, 32), torch.bfloat16, 4).cuda()
    out = torch.empty(64, 32, dtype=torch.bfloat16, device="cuda")
    assert tb.matmul(a, b, out=out) is None
    assert torch.equal(out, tb.matmul(a, b))
    with pytest.raises(RuntimeError, match="differentiation"):
        tb.matmul(a.clone().requires_grad_(), b, out=out)
    with pytest.raises(AssertionError):
        tb.matmul(a, a)
    a32, b32 = a.float().requires_grad_(), b.float().requires_grad_()
    (a32 @ b32).sum().backward()
    ag, bg = a.clone().requires_grad_(), b.clone().requires_grad_()
    tb.matmul(ag, bg).sum().backward()
    assert OG.rel_fro_error(ag.grad.float().cpu(), a32.grad.cpu()) < 1e-2
    assert OG.rel_fro_error(bg.grad.float().cpu(), b32.grad.cpu()) < 1e-2


@pytest.mark.parametrize("m,n,k", [(128, 256, 512), (15, 17, 512), (512, 1024, 768)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_addmm_column_bias(m, n, k, dtype):
    import tritonblas_amd as tb
    a_cpu, b_cpu, bias_cpu = _rand((m, k), dtype, 5, 0.5), _rand((k, n), dtype, 6, 0.5), _rand((n,), dtype, 7)
    c = tb.addmm(bias_cpu.cuda(), a_cpu.cuda(), b_cpu.cuda())
    _check(c.cpu(), OG.ref_gemm(a_cpu, b_cpu, torch.float32, bias=bias_cpu), dtype, TOL_16)


def test_addmm_row_vector_bias_and_lone_scale():
    """a (1, N) bias is one value per column like an (N,) one; a scale vector without its partner is refused"""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import persistent_matmul_lt
    m, n, k = 64, 192, 256
    a_cpu, b_cpu, bias_cpu = _rand((m, k), torch.bfloat16, 5, 0.5), _rand((k, n), torch.bfloat16, 6, 0.5), _rand((n,), torch.bfloat16, 7)
    c = tb.addmm(bias_cpu.cuda().reshape(1, n), a_cpu.cuda(), b_cpu.cuda())
    _check(c.cpu(), OG.ref_gemm(a_cpu, b_cpu, torch.float32, bias=bias_cpu), torch.bfloat16, TOL_16)
    sel = tb.OrigamiMatmulSelector(m, n, k, torch.bfloat16, torch.bfloat16, torch.bfloat16, torch.device("cuda"))
    with pytest.raises(RuntimeError, match="come together"):
        persistent_matmul_lt(a_cpu.cuda(), b_cpu.cuda(), c, sel, None, a_scale=torch.ones(m, device="cuda"), quantized=True)


def test_empty_operands():
    """M, N or K of zero: nothing to compute, an untouched or zero-filled (plus bias) result as torch.matmul gives"""
    import tritonblas_amd as tb
    dev = torch.device("cuda")
    for m, n, k in ((0, 64, 128), (64, 0, 128)):
        a, b = torch.zeros(m, k, dtype=torch.bfloat16, device=dev), torch.zeros(k, n, dtype=torch.bfloat16, device=dev)
        assert tb.matmul(a, b).shape == (m, n)
    a, b = torch.zeros(32, 0, dtype=torch.bfloat16, device=dev), torch.zeros(0, 48, dtype=torch.bfloat16, device=dev)
    c = torch.full((32, 48), float("nan"), dtype=torch.bfloat16, device=dev)
    tb.matmul(a, b, out=c)
    assert torch.equal(c, torch.zeros_like(c))
    bias = torch.arange(48, dtype=torch.bfloat16, device=dev)
    assert torch.equal(tb.addmm(bias, a, b), bias.expand(32, 48))


# ---- FP8 a8w8 -----------------------------------------------------------------------------------
def _a8w8_case(m, n, k, seed=2):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=g).bfloat16()
    w = torch.randn(n, k, generator=torch.Generator().manual_seed(seed + 10000)).bfloat16()
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1)
    bq, sb = OG.quantize_per_channel_fp8(w.T, axis=0)   # B = (K, N) view of the (N, K) weight
    return aq, bq, sa, sb


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (512, 512, 512), (1024, 1024, 1024), (32, 1024, 2048), (100, 300, 640),
                                   (8, 128, 256), (2048, 1024, 512)])
@pytest.mark.parametrize("streamk", [False, True])
def test_a8w8(m, n, k, streamk):
    import tritonblas_amd as tb
    _say(f"a8w8 {m}x{n}x{k} streamk={streamk}")
    aq, bq, sa, sb = _a8w8_case(m, n, k)
    a = aq.cuda()
    b = bq.T.contiguous().cuda().T            # (K, N) view, K-contiguous like a stored (N, K) weight
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, c.dtype, a.device, streamk=streamk)
    cfg = tb.matmul_preamble(sel)
    tb.matmul_a8w8_lt(a, b, sa.cuda(), sb.cuda(), c, sel, cfg, enable_streamk=streamk)
    _check(c.cpu(), OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb), torch.bfloat16, TOL_Q)
    assert cfg.status() == 0


@pytest.mark.parametrize("tile", [(256, 256, 128), (128, 128, 128), (64, 64, 128), (32, 128, 256)])
def test_every_fp8_tile_variant(tile):
    import tritonblas_amd as tb
    m, n, k = 384, 640, 1024
    aq, bq, sa, sb = _a8w8_case(m, n, k, seed=7)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb)
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, torch.bfloat16, a.device)
    sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = tile
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    tb.matmul_a8w8_lt(a, b, sa.cuda(), sb.cuda(), c, sel, None)
    _check(c.cpu(), want, torch.bfloat16, TOL_Q)


@pytest.mark.parametrize("transA,transB", [("T", "T"), ("N", "N"), ("N", "T")])
def test_a8w8_other_layouts_take_the_gather_kernel(transA, transB):
    import tritonblas_amd as tb
    m, n, k = 192, 160, 320
    aq, bq, sa, sb = _a8w8_case(m, n, k, seed=9)
    a, b = _layout(aq.view(torch.uint8), transA).view(torch.float8_e4m3fn), _layout(bq.contiguous().view(torch.uint8), transB).view(torch.float8_e4m3fn)
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c)
    _check(c.cpu(), OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb), torch.bfloat16, TOL_Q)


# ---- schedules ----------------------------------------------------------------------------------
@pytest.mark.parametrize("m,n,k", [(768, 1024, 512), (512, 1024, 768), (2048, 1024, 512), (16, 16, 4096), (300, 200, 192)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_work_stealing_is_bit_identical_to_static(m, n, k, dtype):
    import tritonblas_amd as tb
    _say(f"work stealing {m}x{n}x{k} {dtype}")
    a, b = _rand((m, k), dtype, 11, 0.5).cuda(), _rand((k, n), dtype, 12, 0.5).cuda()
    sel = tb.OrigamiMatmulSelector(m, n, k, dtype, dtype, dtype, a.device)
    cfg = tb.matmul_preamble(sel)
    c0 = torch.zeros(m, n, dtype=dtype, device="cuda")
    tb.matmul_lt(a, b, c0, sel, cfg)
    for rep in range(3):   # the queues rearm themselves: no reset between launches
        c1 = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        tb.matmul_lt(a, b, c1, sel, cfg, work_stealing=True)
        assert torch.equal(c0, c1), f"launch {rep}"


@pytest.mark.parametrize("mode", ["global_atomic", "hierarchical"])
@pytest.mark.parametrize("m,n,k", [(768, 1024, 512), (2048, 2048, 256), (300, 200, 192), (16, 16, 4096), (4096, 4096, 128)])
def test_work_stealing_queue_modes_are_bit_identical_to_static(mode, m, n, k):
    """One shared counter, and XCD-local queues followed by a shared pool: every tile is computed exactly
    once whichever workgroup gets it, so C equals the static schedule's bit for bit; the counters
    (the pool's included) rearm themselves."""
    import tritonblas_amd as tb
    _say(f"work stealing {mode} {m}x{n}x{k}")
    dtype = torch.bfloat16
    a, b = _rand((m, k), dtype, 11, 0.5).cuda(), _rand((k, n), dtype, 12, 0.5).cuda()
    sel = tb.OrigamiMatmulSelector(m, n, k, dtype, dtype, dtype, a.device)
    cfg = tb.matmul_preamble(sel)
    setattr(cfg, mode, True)
    c0 = torch.zeros(m, n, dtype=dtype, device="cuda")
    tb.matmul_lt(a, b, c0, sel)
    for rep in range(3):
        c1 = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        tb.matmul_lt(a, b, c1, sel, cfg, work_stealing=True)
        assert torch.equal(c0, c1), f"launch {rep}"
    # the same workspace serves the other modes afterwards
    cfg.global_atomic = cfg.hierarchical = False
    c2 = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
    tb.matmul_lt(a, b, c2, sel, cfg, work_stealing=True)
    assert torch.equal(c0, c2)


@pytest.mark.parametrize("mode", ["queues", "global_atomic", "hierarchical"])
@pytest.mark.parametrize("active", [1, 7, 64, 200])
def test_work_stealing_with_masked_workgroups(mode, active):
    """active_cus < total_cus: the masked-out workgroups leave at once and the others take every tile
    (also the tiles of queues whose own workgroups are all masked out)."""
    import tritonblas_amd as tb
    m, n, k = 1024, 1536, 256
    _say(f"work stealing mask active={active} {mode}")
    dtype = torch.float16
    a, b = _rand((m, k), dtype, 21, 0.5).cuda(), _rand((k, n), dtype, 22, 0.5).cuda()
    sel = tb.OrigamiMatmulSelector(m, n, k, dtype, dtype, dtype, a.device, active_cus=active)
    cfg = tb.matmul_preamble(sel)
    assert cfg.mask.numel() == sel._N_CU and int(cfg.mask.sum()) == active and cfg.active_mask() is cfg.mask
    if mode != "queues":
        setattr(cfg, mode, True)
    c0 = torch.zeros(m, n, dtype=dtype, device="cuda")
    tb.matmul_lt(a, b, c0, sel)
    for rep in range(2):
        c1 = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        tb.matmul_lt(a, b, c1, sel, cfg, work_stealing=True)
        assert torch.equal(c0, c1), f"launch {rep}"
    # a caller-made mask with holes
    holes = torch.zeros(sel._N_CU, dtype=torch.int32)
    holes[3::5] = 1
    cfg.mask = holes.cuda()
    c2 = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
    tb.matmul_lt(a, b, c2, sel, cfg, work_stealing=True)
    assert torch.equal(c0, c2)


def test_work_stealing_bad_mask_and_split_are_refused():
    import ctypes as C
    import tritonblas_amd as tb
    from tritonblas_amd import _lib
    m = n = k = 512
    a, b = _rand((m, k), torch.float16, 1).cuda(), _rand((k, n), torch.float16, 2).cuda()
    c = torch.zeros(m, n, dtype=torch.float16, device="cuda")
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, a.dtype, a.dtype, a.device)
    cfg = tb.matmul_preamble(sel)
    cfg.mask = torch.ones(8, dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="int32"):
        tb.matmul_lt(a, b, c, sel, cfg, work_stealing=True)
    # through the C ABI: a grid larger than the mask, and a split that does not add up
    d = _lib.tb_gemm_desc()
    d.struct_bytes = C.sizeof(_lib.tb_gemm_desc)
    d.a_type = d.b_type = d.c_type = _lib.tb_dtype(torch.float16)
    d.m, d.n, d.k = m, n, k
    d.a_stride_m, d.a_stride_k, d.b_stride_k, d.b_stride_n, d.c_stride_m, d.c_stride_n = k, 1, n, 1, n, 1
    d.a, d.b, d.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
    d.schedule = _lib.TB_SCHED_WORK_STEALING
    ws = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    d.workspace, d.workspace_bytes = ws.data_ptr(), ws.numel()
    mask = torch.ones(16, dtype=torch.int32, device="cuda")
    d.cu_mask, d.cu_mask_len, d.grid = mask.data_ptr(), 16, 32
    lib = _lib.load()
    assert lib.tb_gemm(d, None) == -10          # TB_ERR_BAD_ARGUMENT
    d.grid = 0
    d.ws_mode, d.ws_local_tiles_per_xcd, d.ws_global_tiles = _lib.TB_WS_HIERARCHICAL, 1, 1
    assert lib.tb_gemm(d, None) == -7           # TB_ERR_BAD_SCHEDULE
    d.ws_mode = 5
    assert lib.tb_gemm(d, None) == -7
    torch.cuda.synchronize()


@pytest.mark.parametrize("m,n,k,grid", [(256, 256, 4096, 64), (128, 128, 8192, 256), (768, 1024, 512, 100), (300, 200, 1920, 37),
                                       (32, 512, 8192, 256), (64, 64, 64, 8)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_streamk_explicit_grid(m, n, k, grid, dtype):
    import tritonblas_amd as tb
    _say(f"stream-k {m}x{n}x{k} grid={grid} {dtype}")
    a_cpu, b_cpu = _rand((m, k), dtype, 13, 0.5), _rand((k, n), dtype, 14, 0.5)
    want = OG.ref_gemm(a_cpu, b_cpu, torch.float32)
    a, b = a_cpu.cuda(), b_cpu.cuda()
    for rep in range(2):   # the flags carry an epoch: a second launch needs no reset
        c = tb.matmul(a, b, enable_streamk=True, sk_grid=grid)
        _check(c.cpu(), want, dtype, TOL_16)


@pytest.mark.parametrize("m,n,k,grid", [(512, 512, 4096, 64), (300, 700, 8192, 200), (256, 256, 16384, 256)])
def test_streamk_workspace_reuse_with_new_data(m, n, k, grid):
    """Back-to-back Stream-K launches on ONE workspace with different operands each time: a partial tile
    or flag left behind by an earlier launch (in the workspace or in any cache on the way) must never
    reach a later result.  No synchronisation between the launches."""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import streamk_matmul_lt
    _say(f"stream-k workspace reuse {m}x{n}x{k} grid={grid}")
    dtype = torch.bfloat16
    sel = tb.OrigamiMatmulSelector(m, n, k, dtype, dtype, dtype, torch.device("cuda", 0), streamk=True)
    cfg = tb.matmul_preamble(sel)
    cases = []
    for rep in range(5):
        a_cpu, b_cpu = _rand((m, k), dtype, 100 + rep, 0.5), _rand((k, n), dtype, 200 + rep, 0.5)
        cases.append((a_cpu, b_cpu, a_cpu.cuda(), b_cpu.cuda(), torch.zeros(m, n, dtype=dtype, device="cuda")))
    torch.cuda.synchronize()
    for (_, _, a, b, c) in cases:
        streamk_matmul_lt(a, b, c, sel, cfg, sk_grid=grid)
    torch.cuda.synchronize()
    assert cfg.status() == 0
    for rep, (a_cpu, b_cpu, _, _, c) in enumerate(cases):
        _check(c.cpu(), OG.ref_gemm(a_cpu, b_cpu, torch.float32), dtype, TOL_16)


@pytest.mark.parametrize("kernel", ["streaming", "streamk"])
def test_decode_shape_small(kernel, tb_option):
    """The decode configuration's shape class (tiny M, long K) at a size the oracle finishes quickly:
    through the streaming skinny-M kernel and through the tile kernel's Stream-K fixup (the library
    picks between them by model time; the hooks "skinny" / "no_skinny" force the choice)."""
    import tritonblas_amd as tb
    tb_option("no_skinny" if kernel == "streamk" else "skinny", 1)
    m, n, k = 32, 1024, 7168
    aq, bq, sa, sb = _a8w8_case(m, n, k, seed=21)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, c.dtype, a.device, streamk=True)
    cfg = tb.matmul_preamble(sel)
    for _ in range(2):
        tb.matmul_a8w8_lt(a, b, sa.cuda(), sb.cuda(), c, sel, cfg, enable_streamk=True)
    _check(c.cpu(), OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb), torch.bfloat16, TOL_Q)
    assert cfg.status() == 0


@pytest.mark.parametrize("m,n,k", [(m, 1040, 2304) for m in (1, 5, 16, 17, 32, 33, 64)] +
                         [(m, 24576 + 40, 256) for m in (7, 32, 64)])   # wide N: 64-column workgroups
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
@pytest.mark.parametrize("forced", [True, False])
def test_skinny_rows(m, n, k, dtype, forced, tb_option):
    """Every row-block count of the streaming kernel and both column widths of its workgroups, ragged N,
    bias, all three element types; once forced onto the streaming kernel, once with the library's own
    choice between it and the tile kernels."""
    import tritonblas_amd as tb
    if forced:
        tb_option("skinny", 1)
    _say(f"skinny {m}x{n}x{k} {dtype} forced={forced}")
    if dtype == torch.float8_e4m3fn:
        aq, bq, sa, sb = _a8w8_case(m, n, k, seed=31)
        c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
        tb.matmul_a8w8(aq.cuda(), bq.T.contiguous().cuda().T, sa.cuda(), sb.cuda(), c)
        _check(c.cpu(), OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb), torch.bfloat16, TOL_Q)
    else:
        a_cpu, b_cpu, bias = _rand((m, k), dtype, 32, 0.5), _rand((k, n), dtype, 33, 0.5), _rand((n,), dtype, 34)
        b = b_cpu.T.contiguous().cuda().T
        c = tb.addmm(bias.cuda(), a_cpu.cuda(), b)
        _check(c.cpu(), OG.ref_gemm(a_cpu, b_cpu, torch.float32, bias=bias), dtype, TOL_16)


# ---- fp32 operands ------------------------------------------------------------------------------
TOL_32 = 1e-5   # full fp32 products and sums; a TF32-style 10-bit mantissa would sit near 5e-4


def _ref64(a_cpu, b_cpu, bias=None):
    acc = torch.matmul(a_cpu.double(), b_cpu.double())
    return acc if bias is None else acc + bias.double()[None, :]


@pytest.mark.parametrize("m,n,k", [(1024, 1024, 1024), (512, 768, 320), (300, 200, 192), (257, 129, 67), (16, 2048, 512),
                                   (2048, 64, 4096), (1, 1, 1)])
@pytest.mark.parametrize("transA,transB", [("T", "T"), ("N", "N"), ("T", "N"), ("N", "T")])
def test_matmul_fp32(m, n, k, transA, transB):
    """float32 in, float32 out (reference tests/test_matmul.py:23): K-contiguous operands run the
    LDS-direct kernels, every other layout the gather kernel."""
    import tritonblas_amd as tb
    _say(f"matmul fp32 {m}x{n}x{k} {transA}{transB}")
    a_cpu, b_cpu = _rand((m, k), torch.float32, 40, 0.5), _rand((k, n), torch.float32, 41, 0.5)
    a, b = _layout(a_cpu, transA), _layout(b_cpu, transB)
    c = tb.matmul(a, b)
    assert c.shape == (m, n) and c.dtype == torch.float32
    err = OG.rel_fro_error(c.cpu().double(), _ref64(a_cpu, b_cpu))
    assert err <= TOL_32, f"relative Frobenius error {err:.3e}"


@pytest.mark.parametrize("tile", [(256, 256, 32), (128, 128, 32), (64, 64, 32)])
@pytest.mark.parametrize("mode", ["persistent", "streamk", "work_stealing"])
def test_every_fp32_tile_variant_and_schedule(tile, mode):
    import tritonblas_amd as tb
    m, n, k = 640, 768, 1024
    _say(f"matmul_lt fp32 tile={tile} {mode}")
    a_cpu, b_cpu = _rand((m, k), torch.float32, 42, 0.5), _rand((k, n), torch.float32, 43, 0.5)
    a, b = a_cpu.cuda(), b_cpu.cuda().T.contiguous().T     # both K-contiguous
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, a.dtype, a.dtype, a.device, streamk=mode == "streamk")
    sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = tile
    cfg = tb.matmul_preamble(sel)
    for rep in range(2):
        c = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        tb.matmul_lt(a, b, c, sel, cfg, enable_streamk=mode == "streamk", work_stealing=mode == "work_stealing")
        err = OG.rel_fro_error(c.cpu().double(), _ref64(a_cpu, b_cpu))
        assert err <= TOL_32, f"relative Frobenius error {err:.3e} (launch {rep})"


def test_fp32_products_are_not_truncated():
    """Operands whose low mantissa bits carry the whole answer: (1 + e) * (1 - e) summed against -1."""
    import tritonblas_amd as tb
    k = 256
    e = 2.0 ** -12
    a = torch.full((64, k), 1.0 + e, dtype=torch.float32)
    b = torch.full((k, 64), 1.0 - e, dtype=torch.float32)
    c = tb.matmul(a.cuda(), b.cuda().T.contiguous().T).cpu()
    want = k * (1.0 - e * e)            # exact in fp32 arithmetic up to the final roundings
    assert torch.allclose(c, torch.full_like(c, want), rtol=0, atol=k * 2.0 ** -24 * 4)
    assert abs(float(c[0, 0]) - k) > k * e * e * 0.5   # a 10-bit-mantissa product would return exactly k


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_addmm_fp32(out_dtype):
    import tritonblas_amd as tb
    m, n, k = 384, 520, 264
    a_cpu, b_cpu, bias = _rand((m, k), torch.float32, 44, 0.5), _rand((k, n), torch.float32, 45, 0.5), _rand((n,), torch.float32, 46)
    if out_dtype == torch.float32:
        c = tb.addmm(bias.cuda(), a_cpu.cuda(), b_cpu.cuda())
    else:
        sel = tb.OrigamiMatmulSelector(m, n, k, torch.float32, torch.float32, out_dtype, torch.device("cuda"))
        c = torch.zeros(m, n, dtype=out_dtype, device="cuda")
        from tritonblas_amd.matmul import _launch_gemm
        from tritonblas_amd import _lib
        _launch_gemm(a_cpu.cuda(), b_cpu.cuda(), c, sel, None, _lib.TB_SCHED_PERSISTENT, bias=bias.cuda())
    want = _ref64(a_cpu, b_cpu, bias)
    err = OG.rel_fro_error(c.cpu().double(), want.to(out_dtype).double())
    assert err <= (TOL_32 if out_dtype == torch.float32 else TOL_16), f"{err:.3e}"


def test_streamk_grid_sized_for_another_tile():
    """The selector sizes its Stream-K grid for the tile it picked; operands that need the gather kernel
    run another tile with fewer co-resident workgroups.  The library then chooses the grid itself
    instead of refusing the launch."""
    import tritonblas_amd as tb
    m, n, k = 1261, 670, 2688
    a_cpu, b_cpu = _rand((m, k), torch.float32, 70, 0.5), _rand((k, n), torch.float32, 71, 0.5)
    a, b = a_cpu.cuda(), b_cpu.cuda()          # B is N-contiguous: no LDS-direct fp32 kernel for it
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, torch.float32, a.device, streamk=True)
    cfg = tb.matmul_preamble(sel)
    c = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    tb.matmul_lt(a, b, c, sel, cfg, enable_streamk=True)
    err = OG.rel_fro_error(c.cpu().double(), _ref64(a_cpu, b_cpu))
    assert err <= TOL_32, f"{err:.3e}"
    assert cfg.status() == 0


# ---- int8 operands -------------------------------------------------------------------------------
def _int8_case(m, n, k, seed):
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(seed))
    b = torch.randn(k, n, generator=torch.Generator().manual_seed(seed + 10000))
    aq, sa = OG.quantize_per_channel_int8(a, axis=1)
    bq, sb = OG.quantize_per_channel_int8(b, axis=0)
    return aq, bq, sa, sb


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (1024, 1024, 1024), (300, 200, 192), (257, 129, 67), (32, 2048, 4096), (1, 1, 1)])
@pytest.mark.parametrize("transA,transB", [("T", "N"), ("T", "T"), ("N", "N"), ("N", "T")])
def test_matmul_a8w8_int8_to_bf16(m, n, k, transA, transB):
    """int8 x int8 with per-row / per-column scales into bf16 (reference persistent_gemm.py:75 with a
    non-int8 C; the reference's own int8 test is switched off, tests/test_matmul_a8w8_lt.py:62)."""
    import tritonblas_amd as tb
    _say(f"a8w8 int8 {m}x{n}x{k} {transA}{transB}")
    aq, bq, sa, sb = _int8_case(m, n, k, 50)
    a, b = _layout(aq, transA), _layout(bq, transB)
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c)
    want = OG.ref_gemm_int8(aq, bq, torch.bfloat16, a_scale=sa, b_scale=sb)
    _check(c.cpu(), want.float(), torch.bfloat16, TOL_16)   # integer sums are exact: only the bf16 rounding is left


@pytest.mark.parametrize("tile", [(256, 256, 128), (128, 128, 128), (64, 64, 128)])
@pytest.mark.parametrize("mode", ["persistent", "streamk", "work_stealing"])
def test_int8_sums_are_exact_in_every_tile_and_schedule(tile, mode):
    """No scales, fp32 out: every output is an integer below 2^24 and must come out exactly."""
    import tritonblas_amd as tb
    from tritonblas_amd import _lib
    from tritonblas_amd.matmul import _launch_gemm
    m, n, k = 640, 768, 1024
    _say(f"int8 exact tile={tile} {mode}")
    g = torch.Generator().manual_seed(51)
    aq = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
    bq = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int8)
    want = torch.matmul(aq.to(torch.int64), bq.to(torch.int64).T)
    assert int(want.abs().max()) < 2 ** 24
    sel = tb.OrigamiMatmulSelector(m, n, k, torch.int8, torch.int8, torch.float32, torch.device("cuda"), streamk=mode == "streamk")
    sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = tile
    cfg = tb.matmul_preamble(sel)
    sched = {"persistent": _lib.TB_SCHED_PERSISTENT, "streamk": _lib.TB_SCHED_STREAMK, "work_stealing": _lib.TB_SCHED_WORK_STEALING}[mode]
    for rep in range(2):
        c = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        _launch_gemm(aq.cuda(), bq.cuda().T, c, sel, cfg, sched)
        assert torch.equal(c.cpu().to(torch.int64), want), f"launch {rep}"


def test_int8_output_truncates_and_saturates():
    import tritonblas_amd as tb
    m, n, k = 192, 320, 256
    aq, bq, sa, sb = _int8_case(m, n, k, 52)
    sa, sb = sa * 40.0, sb * 40.0          # push part of the results beyond +-127
    c = torch.zeros(m, n, dtype=torch.int8, device="cuda")
    tb.matmul_a8w8(aq.cuda(), bq.cuda().T.contiguous().T, sa.cuda(), sb.cuda(), c)
    want = OG.ref_gemm_int8(aq, bq, torch.int8, a_scale=sa, b_scale=sb)
    got = c.cpu()
    assert int((want == 127).sum()) > 0 and int((want == -128).sum()) > 0 and int((want.abs() < 100).sum()) > 0
    # the fp32 products acc*(sa*sb) of kernel and oracle agree to the last bit or the one before;
    # truncation can turn that into a difference of 1 right at an integer
    diff = (got.to(torch.int32) - want.to(torch.int32)).abs()
    assert int(diff.max()) <= 1 and float((diff > 0).float().mean()) < 1e-3


# ---- MXFP4 --------------------------------------------------------------------------------------
def _fp4_case(m, n, k, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.standard_normal((n, k)).astype(np.float32)
    xq, xs = OM.mxfp4_quant(x)
    wq, ws = OM.mxfp4_quant(w)
    return (torch.from_numpy(t) for t in (xq, wq, xs, ws))


@pytest.mark.parametrize("m,n,k", [(128, 128, 128), (256, 256, 256), (512, 512, 512), (1024, 1024, 1024), (100, 72, 640),
                                   (2048, 2048, 2048), (32, 256, 1024), (128, 128, 96)])
def test_matmul_fp4(m, n, k):
    import tritonblas_amd as tb
    _say(f"fp4 {m}x{n}x{k}")
    xq, wq, xs, ws = _fp4_case(m, n, k, 5)
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    tb.matmul_fp4(xq.cuda(), wq.cuda(), c, xs.cuda(), ws.cuda())
    _check(c.cpu(), OG.ref_gemm_fp4(xq, wq, xs, ws, return_fp32=True), torch.bfloat16, TOL_Q)


@pytest.mark.parametrize("tile", [(256, 256, 256), (128, 128, 256), (128, 128, 128), (64, 64, 256)])
def test_every_fp4_tile_variant(tile):
    import tritonblas_amd as tb
    m, n, k = 320, 448, 1024
    xq, wq, xs, ws = _fp4_case(m, n, k, 6)
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    tb.matmul_fp4(xq.cuda(), wq.cuda(), c, xs.cuda(), ws.cuda(), block_m=tile[0], block_n=tile[1], block_k=tile[2])
    _check(c.cpu(), OG.ref_gemm_fp4(xq, wq, xs, ws, return_fp32=True), torch.bfloat16, TOL_Q)


def test_fp4_scale_extremes():
    """Scale bytes far from 127 and per-block varying scales must be honoured exactly."""
    import tritonblas_amd as tb
    m, n, k = 64, 64, 256
    rng = np.random.default_rng(8)
    xq = torch.from_numpy(rng.integers(0, 256, (m, k // 2), dtype=np.uint8))
    wq = torch.from_numpy(rng.integers(0, 256, (n, k // 2), dtype=np.uint8))
    xs = torch.from_numpy(rng.integers(100, 150, (m, k // 32), dtype=np.uint8))
    ws = torch.from_numpy(rng.integers(100, 150, (n, k // 32), dtype=np.uint8))
    c = torch.zeros(m, n, dtype=torch.float32, device="cuda")
    tb.matmul_fp4(xq.cuda(), wq.cuda(), c, xs.cuda(), ws.cuda())
    _check(c.cpu(), OG.ref_gemm_fp4(xq, wq, xs, ws, return_fp32=True), torch.float32, 1e-5)


@pytest.mark.parametrize("tile", [(256, 256, 256), (128, 128, 256), (128, 128, 128), (64, 64, 256)])
@pytest.mark.parametrize("m,n,k", [(256, 256, 512), (320, 448, 1536), (512, 256, 4096)])
def test_fp4_fast_kernels_random_scales(tile, m, n, k):
    """The LDS-direct kernels (K a multiple of 512) stage the scale bytes through LDS group by group:
    random codes and random, widely varying scale bytes over several groups pin every byte's place."""
    import tritonblas_amd as tb
    _say(f"fp4 fast tile={tile} {m}x{n}x{k}")
    rng = np.random.default_rng(m + k)
    xq = torch.from_numpy(rng.integers(0, 256, (m, k // 2), dtype=np.uint8))
    wq = torch.from_numpy(rng.integers(0, 256, (n, k // 2), dtype=np.uint8))
    xs = torch.from_numpy(rng.integers(100, 150, (m, k // 32), dtype=np.uint8))
    ws = torch.from_numpy(rng.integers(100, 150, (n, k // 32), dtype=np.uint8))
    c = torch.zeros(m, n, dtype=torch.float32, device="cuda")
    tb.matmul_fp4(xq.cuda(), wq.cuda(), c, xs.cuda(), ws.cuda(), block_m=tile[0], block_n=tile[1], block_k=tile[2])
    _check(c.cpu(), OG.ref_gemm_fp4(xq, wq, xs, ws, return_fp32=True), torch.float32, 1e-5)


# ---- column split of a partial last round -----------------------------------------------------------
@pytest.mark.parametrize("kind", ["fp8", "bf16", "bias"])
@pytest.mark.parametrize("shape", [(2048, 28672, 512), (1536, 14336 + 40, 256), (1100, 20000, 384)])
def test_column_split(kind, shape, tb_option):
    """More tiles than the resident grid holds and a partial last round: the library may run the columns
    that fill whole rounds with the selected tile and the rest as a second launch with another tile.
    Forced here; every element of C must equal the one-launch result bit for bit (each output element
    sums its K range in the same order whatever tile it sits in), and a strip across the seam is
    checked against the oracle."""
    import tritonblas_amd as tb
    m, n, k = shape
    _say(f"column split {kind} {m}x{n}x{k}")
    g = torch.Generator().manual_seed(21)
    a = torch.randn(m, k, generator=g).bfloat16()
    w = torch.randn(n, k, generator=g).bfloat16()
    bias = torch.randn(n, generator=g).bfloat16() if kind == "bias" else None
    outs = {}
    for name, env in (("one", {"no_column_split": 1, "force_column_split": 0}), ("split", {"no_column_split": 0, "force_column_split": 1})):
        for key, val in env.items():
            tb_option(key, val)
        c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        # the tall tile named outright, so that the tile count (and with it the seam) is known
        import types
        sel = types.SimpleNamespace(block_m=256, block_n=256, block_k=128 if kind == "fp8" else 64, group_m=min(8, -(-m // 256)),
                                    num_sms=8, COUNTERS_PER_XCD=1, streamk=False, sk_grid=0, _total_cus=None, waves_per_eu=1)
        if kind == "fp8":
            aq, sa = OG.quantize_per_channel_fp8(a, axis=1)
            wq, sw = OG.quantize_per_channel_fp8(w, axis=1)
            tb.matmul_a8w8_lt(aq.cuda(), wq.cuda().T, sa.cuda(), sw.cuda(), c, sel, None)
        else:
            from tritonblas_amd.matmul import persistent_matmul_lt
            persistent_matmul_lt(a.cuda(), w.cuda().T, c, sel, None, bias=None if bias is None else bias.cuda())
        outs[name] = c.cpu()
    assert torch.isfinite(outs["split"].float()).all()
    assert torch.equal(outs["one"], outs["split"])
    cols = slice(n // 2, n)     # the seam lies in the right half (whole rounds come first)
    if kind == "fp8":
        want = OG.ref_gemm(aq, wq.T[:, cols], torch.float32, a_scale=sa, b_scale=sw[cols])
    else:
        want = OG.ref_gemm(a, w.T[:, cols], torch.float32, bias=None if bias is None else bias[cols])
    _check(outs["split"][:, cols], want, torch.bfloat16, TOL_Q if kind == "fp8" else TOL_16)


# ---- grouped MoE --------------------------------------------------------------------------------
@pytest.mark.parametrize("small_rows", [-1, 32, 64, 100])
@pytest.mark.parametrize("counts", [[300, 0, 700, 24], [1, 255, 256, 257, 0, 0, 31, 224], [1024], [0, 0, 5],
                                    [256 + 33, 512 + 64, 65, 32, 768 + 100, 101]])
def test_grouped_two_launches(counts, small_rows):
    """Tall tiles forced, last partial row blocks of at most small_rows rows left to the second launch
    with the 32-row tile: every row of C is written exactly once (C starts as NaN) with the oracle's
    values, for thresholds on both sides of the remainders."""
    import tritonblas_amd as tb
    _say(f"grouped two launches counts={counts} small_rows={small_rows}")
    E, n, k = len(counts), 384, 512
    m = sum(counts)
    offsets = torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(14)).bfloat16()
    w = torch.randn(E, n, k, generator=torch.Generator().manual_seed(10014)).bfloat16()
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1)
    wq, sw = OG.quantize_per_channel_fp8(w, axis=2)
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tb.grouped_matmul_a8w8(aq.cuda(), wq.cuda(), sa.cuda(), sw.cuda(), c, offsets.cuda(), 256, 256, 128, small_rows=small_rows)
    want = OG.ref_grouped_gemm_fp8(aq, wq, sa, sw, offsets, return_fp32=True)
    _check(c.cpu(), want, torch.bfloat16, TOL_Q)


@pytest.mark.parametrize("counts", [[300, 0, 700, 24], [1, 255, 256, 257, 0, 0, 31, 224], [1024], [0, 0, 5]])
def test_grouped_a8w8(counts):
    import tritonblas_amd as tb
    _say(f"grouped counts={counts}")
    E, n, k = len(counts), 384, 512
    m = sum(counts)
    offsets = torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(4)).bfloat16()
    w = torch.randn(E, n, k, generator=torch.Generator().manual_seed(10004)).bfloat16()
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1)
    wq, sw = OG.quantize_per_channel_fp8(w, axis=2)
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tb.grouped_matmul_a8w8(aq.cuda(), wq.cuda(), sa.cuda(), sw.cuda(), c, offsets.cuda())
    want = OG.ref_grouped_gemm_fp8(aq, wq, sa, sw, offsets, return_fp32=True)
    _check(c.cpu(), want, torch.bfloat16, TOL_Q)
    # permuting experts permutes the row blocks
    if E > 1:
        perm = list(reversed(range(E)))
        rows = torch.cat([torch.arange(int(offsets[e]), int(offsets[e + 1])) for e in perm])
        off2 = torch.tensor([0] + list(np.cumsum([counts[e] for e in perm])), dtype=torch.int32)
        c2 = torch.empty_like(c)
        tb.grouped_matmul_a8w8(aq[rows].cuda(), wq[perm].cuda(), sa[rows].cuda(), sw[perm].cuda(), c2, off2.cuda())
        assert torch.equal(c2.cpu(), c.cpu()[rows])


def _grouped_problem(counts, n, k, seed):
    E, m = len(counts), sum(counts)
    offsets = torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(seed)).bfloat16()
    w = torch.randn(E, n, k, generator=torch.Generator().manual_seed(10000 + seed)).bfloat16()
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1)
    wq, sw = OG.quantize_per_channel_fp8(w, axis=2)
    return offsets, aq, wq, sa, sw


@pytest.mark.parametrize("fix", [1, 64])
@pytest.mark.parametrize("grid", [8, 5, 12])
@pytest.mark.parametrize("counts", [[300, 0, 700, 24], [1, 255, 256, 257, 0, 0, 31, 224], [1024], [256, 256]])
def test_grouped_streamk_tail(counts, grid, fix, tb_option):
    """The tiles that do not fill whole rounds of the grid run as K ranges (Stream-K) on the 4-wave kernel: C
    (NaN before) holds the oracle's values, the whole tiles are bit-identical to the launch without a tail, two
    launches in a row share one workspace without a reset, and the configurations in which the device-side rule
    must cut tiles show published partial tiles in the workspace.  fix: what the rule charges per extra piece of a
    tile, in K steps (1: it cuts whenever a round is not full; 64: the library's value, which at this small K never cuts)."""
    import tritonblas_amd as tb
    from tritonblas_amd import _lib
    from tritonblas_amd.config import MatmulConfig
    _say(f"grouped streamk tail counts={counts} grid={grid} fix={fix}")
    n, k = 512, 2048
    tb_option("grid", grid)
    tb_option("grp_sk_fix", fix)
    offsets, aq, wq, sa, sw = _grouped_problem(counts, n, k, 24)
    want = OG.ref_grouped_gemm_fp8(aq, wq, sa, sw, offsets, return_fp32=True)
    args = (aq.cuda(), wq.cuda(), sa.cuda(), sw.cuda())
    m = sum(counts)
    plain = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tb.grouped_matmul_a8w8(*args, plain, offsets.cuda(), 256, 256, 128, small_rows=-1, enable_streamk=False)
    cfg = MatmulConfig(device=plain.device, workspace=None)
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tb.grouped_matmul_a8w8(*args, c, offsets.cuda(), 256, 256, 128, small_rows=-1, enable_streamk=True, config=cfg)
    assert cfg.status() == 0
    _check(c.cpu(), want, torch.bfloat16, TOL_Q)
    tiles = sum((r + 255) // 256 for r in counts) * (n // 256)
    launched = min(grid, ((m + 255) // 256 + len(counts)) * (n // 256))   # (the host only knows a bound of the table's length)
    cut = _lib.load().tb_streamk_tail_tiles(tiles, launched, k // 512, 4, fix)
    _, flags_off = _lib.workspace_layout()
    flags = cfg.workspace[flags_off:flags_off + 4 * grid].view(torch.int32).cpu()
    assert (int(flags.abs().sum()) > 0) == (cut > 0), (tiles, cut, flags)
    # whole tiles are the table's first tiles: expert by expert, row block fastest
    t, same = 0, 0
    for e, rows in enumerate(counts):
        mb = (rows + 255) // 256
        for local in range(mb * (n // 256)):
            if t < tiles - cut:
                r0 = int(offsets[e]) + (local % mb) * 256
                r1 = min(r0 + 256, int(offsets[e + 1]))
                c0 = (local // mb) * 256
                assert torch.equal(c[r0:r1, c0:c0 + 256], plain[r0:r1, c0:c0 + 256]), (e, local)
                same += 1
            t += 1
    assert same == tiles - cut
    # the same workspace again, other row counts, no reset
    counts2 = list(reversed(counts))
    offsets2, aq2, wq2, sa2, sw2 = _grouped_problem(counts2, n, k, 25)
    c2 = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tb.grouped_matmul_a8w8(aq2.cuda(), wq2.cuda(), sa2.cuda(), sw2.cuda(), c2, offsets2.cuda(), 256, 256, 128, small_rows=-1,
                           enable_streamk=True, config=cfg)
    assert cfg.status() == 0
    _check(c2.cpu(), OG.ref_grouped_gemm_fp8(aq2, wq2, sa2, sw2, offsets2, return_fp32=True), torch.bfloat16, TOL_Q)


def test_grouped_streamk_default_two_launch_plan(tb_option):
    """Default plan (the device chooses between one and two launches) with the Stream-K tail on (the workspace is the
    package's per-stream one): oracle values in every row."""
    import tritonblas_amd as tb
    _say("grouped streamk tail, default plan")
    tb_option("grid", 6)
    counts, n, k = [520, 30, 0, 300, 257], 512, 1024
    offsets, aq, wq, sa, sw = _grouped_problem(counts, n, k, 26)
    c = torch.full((sum(counts), n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tb_option("grp_sk_fix", 2)
    for _ in range(2):
        tb.grouped_matmul_a8w8(aq.cuda(), wq.cuda(), sa.cuda(), sw.cuda(), c, offsets.cuda(), enable_streamk=True)
    _check(c.cpu(), OG.ref_grouped_gemm_fp8(aq, wq, sa, sw, offsets, return_fp32=True), torch.bfloat16, TOL_Q)
