"""GPU tests of the hand-scheduled 4-wave 256x256 kernels (FP8 and MXFP4) and of the workspace rules.

The 4-wave kernels form every sum in the same order as the 8-wave kernels of the same tile (same MFMA
instruction, same K grouping), so the two must agree bit for bit; the 8-wave kernels are checked against
the CPU oracle throughout tests/test_gemm_gpu.py, and the cases here check the 4-wave ones against the
oracle as well.  All launches go through the C ABI."""
import ctypes as C
import sys

import numpy as np
import pytest
import torch

from oracle import gemm as OG
from oracle import mxfp4 as OM

pytestmark = pytest.mark.gpu
TOL_Q = 1e-2


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _fp8_case(m, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=g).bfloat16()
    w = torch.randn(n, k, generator=torch.Generator().manual_seed(seed + 10000)).bfloat16()
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1)
    bq, sb = OG.quantize_per_channel_fp8(w.T, axis=0)
    return aq, bq, sa, sb


def _run_fp8(aq, bq, sa, sb, waves, tb_option, out_dtype=torch.bfloat16, bias=None, work_stealing=False):
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import persistent_matmul_lt
    m, k = aq.shape
    n = bq.shape[1]
    tb_option("waves", waves)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, out_dtype, a.device)
    sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 256, 256, 128
    c = torch.full((m, n), float("nan"), device="cuda").to(out_dtype)
    cfg = tb.matmul_preamble(sel) if work_stealing else None
    persistent_matmul_lt(a, b, c, sel, cfg, bias=None if bias is None else bias.cuda(), a_scale=sa.cuda(), b_scale=sb.cuda(),
                         quantized=True, work_stealing=work_stealing)
    return c.cpu()


@pytest.mark.parametrize("m,n,k", [(256, 256, 512), (256, 256, 2048), (512, 768, 512), (300, 500, 768), (1, 257, 512),
                                   (1024, 2048, 1024), (2560, 2304, 512)])
def test_fp8_four_wave_kernel(m, n, k, tb_option):
    """Whole and ragged tiles, one to many tiles per workgroup (2560x2304 = 90 tiles): oracle parity and
    bit-equality with the 8-wave kernel."""
    _say(f"w4 fp8 {m}x{n}x{k}")
    aq, bq, sa, sb = _fp8_case(m, n, k, 71)
    new = _run_fp8(aq, bq, sa, sb, 22, tb_option)
    old = _run_fp8(aq, bq, sa, sb, 24, tb_option)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    assert OG.rel_fro_error(new.float(), want.float()) <= TOL_Q
    assert torch.equal(new.view(torch.int16), old.view(torch.int16))


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("with_bias", [False, True])
def test_fp8_four_wave_epilogue_variants(out_dtype, with_bias, tb_option):
    """fp16 / fp32 output and a per-column bias take the general epilogue of the 4-wave kernel."""
    m, n, k = 384, 640, 512
    aq, bq, sa, sb = _fp8_case(m, n, k, 72)
    bias = torch.randn(n, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16) if with_bias else None
    new = _run_fp8(aq, bq, sa, sb, 22, tb_option, out_dtype=out_dtype, bias=bias)
    old = _run_fp8(aq, bq, sa, sb, 24, tb_option, out_dtype=out_dtype, bias=bias)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb)
    if with_bias:
        want = want + bias.float()[None, :]
    assert OG.rel_fro_error(new.float(), want.to(out_dtype).float()) <= TOL_Q
    assert torch.equal(new, old)


def test_fp8_four_wave_work_stealing(tb_option):
    """The 4-wave kernel under the work-stealing schedule (tiles from the atomic queues, one tile looked
    ahead): bit-identical to its data-parallel result, three launches on one config without a reset."""
    m, n, k = 1536, 2304, 512
    aq, bq, sa, sb = _fp8_case(m, n, k, 73)
    static = _run_fp8(aq, bq, sa, sb, 22, tb_option)
    for rep in range(3):
        ws = _run_fp8(aq, bq, sa, sb, 22, tb_option, work_stealing=True)
        assert torch.equal(static.view(torch.int16), ws.view(torch.int16)), f"launch {rep}"


@pytest.mark.parametrize("k", [256, 384, 640])
def test_fp8_four_wave_needs_an_even_number_of_k_steps(k, tb_option):
    """K = 2, 3 or 5 steps of 128 (the 4-wave kernel runs an even number, at least four): the library must
    fall back to the 8-wave kernel by itself and stay correct."""
    m, n = 512, 512
    aq, bq, sa, sb = _fp8_case(m, n, k, 74)
    got = _run_fp8(aq, bq, sa, sb, 0, tb_option)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    assert OG.rel_fro_error(got.float(), want.float()) <= TOL_Q


def _fp4_case(m, n, k, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.standard_normal((n, k)).astype(np.float32)
    xq, xs = OM.mxfp4_quant(x)
    wq, ws = OM.mxfp4_quant(w)
    return torch.from_numpy(xq), torch.from_numpy(wq), torch.from_numpy(xs), torch.from_numpy(ws)


@pytest.mark.parametrize("m,n,k", [(256, 256, 1024), (256, 256, 4096), (512, 768, 1024), (300, 500, 1536), (2048, 1280, 2048),
                                   (300, 500, 3072), (768, 512, 5120)])
def test_fp4_four_wave_kernel(m, n, k, tb_option):
    """The 4-wave MXFP4 kernel against the oracle and, bit for bit, against the 8-wave kernel."""
    import tritonblas_amd as tb
    _say(f"w4 fp4 {m}x{n}x{k}")
    xq, wq, xs, ws = _fp4_case(m, n, k, 75)
    # scale bytes far from 127 in some blocks, different in every K block of a row: the E8M0 operands of the scaled
    # MFMA must be honoured, and a scale byte that ends up with the wrong K block must show
    xs[::3, ::2] = 120
    ws[1::4, 1::3] = 133
    xs[5::7, :] = (118 + torch.arange(k // 32) % 19).to(torch.uint8)
    ws[2::5, :] = (136 - torch.arange(k // 32) % 17).to(torch.uint8)
    outs = {}
    for waves in (22, 24):
        tb_option("waves", waves)
        c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        tb.matmul_fp4(xq.cuda(), wq.cuda(), c, xs.cuda(), ws.cuda(), block_m=256, block_n=256, block_k=256)
        outs[waves] = c.cpu()
    want = OG.ref_gemm_fp4(xq, wq, xs, ws, return_fp32=True).to(torch.bfloat16)
    assert OG.rel_fro_error(outs[22].float(), want.float()) <= TOL_Q
    assert torch.equal(outs[22].view(torch.int16), outs[24].view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (512, 768, 512), (300, 500, 384), (1, 300, 256), (2048, 1280, 1024)])
def test_16bit_four_wave_kernel(dtype, m, n, k, tb_option):
    """bf16 / fp16 with K-major operands (the TN layout): oracle parity, bit-equality with the 8-wave
    kernel, and a per-column bias through the general epilogue."""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import persistent_matmul_lt
    _say(f"w4 {dtype} {m}x{n}x{k}")
    g = torch.Generator().manual_seed(76)
    a_cpu = (torch.randn(m, k, generator=g) * 0.5).to(dtype)
    bt_cpu = (torch.randn(n, k, generator=g) * 0.5).to(dtype)
    bias = torch.randn(n, generator=g).to(dtype)
    a, b = a_cpu.cuda(), bt_cpu.cuda().T
    want = OG.ref_gemm(a_cpu, bt_cpu.T, torch.float32)
    for with_bias in (False, True):
        outs = {}
        for waves in (22, 24):
            tb_option("waves", waves)
            sel = tb.OrigamiMatmulSelector(m, n, k, dtype, dtype, dtype, a.device)
            sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 256, 256, 64
            c = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
            persistent_matmul_lt(a, b, c, sel, None, bias=bias.cuda() if with_bias else None)
            outs[waves] = c.cpu()
        ref = (want + bias.float()[None, :]) if with_bias else want
        assert OG.rel_fro_error(outs[22].float(), ref.to(dtype).float()) <= 1e-3
        assert torch.equal(outs[22].view(torch.int16), outs[24].view(torch.int16))


# ---- epilogue fused into the next tile's K loop -------------------------------------------------------------
def _launcher(kind, m, n, k, seed):
    """returns (run, want): run() launches the 256x256 tile kernel the hooks select and returns C on the host"""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import persistent_matmul_lt
    if kind in ("fp8", "i8"):
        if kind == "fp8":
            aq, bq, sa, sb = _fp8_case(m, n, k, seed)
        else:
            g = torch.Generator().manual_seed(seed)
            aq, sa = OG.quantize_per_channel_int8(torch.randn(m, k, generator=g), axis=1)
            bq, sb = OG.quantize_per_channel_int8(torch.randn(k, n, generator=g), axis=0)
        a, b, sad, sbd = aq.cuda(), bq.T.contiguous().cuda().T, sa.cuda(), sb.cuda()

        def run():
            sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, torch.bfloat16, a.device)
            sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 256, 256, 128
            c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            persistent_matmul_lt(a, b, c, sel, None, a_scale=sad, b_scale=sbd, quantized=True)
            return c.cpu()
        if kind == "i8":
            return run, OG.ref_gemm_int8(aq, bq, torch.bfloat16, a_scale=sa, b_scale=sb).to(torch.bfloat16)
        return run, OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    if kind == "fp4":
        xq, wq, xs, ws = _fp4_case(m, n, k, seed)
        xs[::3, ::2] = 121
        xd, wd, xsd, wsd = xq.cuda(), wq.cuda(), xs.cuda(), ws.cuda()

        def run():
            c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            tb.matmul_fp4(xd, wd, c, xsd, wsd, block_m=256, block_n=256, block_k=256)
            return c.cpu()
        return run, OG.ref_gemm_fp4(xq, wq, xs, ws, return_fp32=True).to(torch.bfloat16)
    g = torch.Generator().manual_seed(seed)
    a_cpu = (torch.randn(m, k, generator=g) * 0.5).bfloat16()
    bt_cpu = (torch.randn(n, k, generator=g) * 0.5).bfloat16()
    a, b = a_cpu.cuda(), bt_cpu.cuda().T

    def run():
        sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, torch.bfloat16, a.device)
        sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 256, 256, 64
        c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        persistent_matmul_lt(a, b, c, sel, None)
        return c.cpu()
    return run, OG.ref_gemm(a_cpu, bt_cpu.T, torch.float32).to(torch.bfloat16)


@pytest.mark.parametrize("kind,bk", [("fp8", 128), ("fp4", 256), ("bf16", 64), ("i8", 128)])
@pytest.mark.parametrize("m,n,steps,grid", [(512, 768, 4, 1), (512, 768, 6, 2), (300, 500, 8, 1), (1280, 768, 10, 3), (1100, 1300, 4, 2),
                                            (4096, 8192, 4, 0), (768, 1100, 12, 2), (1280, 768, 16, 3), (4096, 4096, 8, 0)])
def test_fused_epilogue(kind, bk, m, n, steps, grid, tb_option):
    """A workgroup that runs several tiles stores a full bf16 tile from inside the next tile's first K
    step.  With 1 to 3 workgroups for 6 to 30 tiles (and 512 tiles on the whole chip), whole and ragged
    tiles mixed, the result must equal, bit for bit, what the same kernel gives when every tile takes
    the compiled epilogue (hook lab = 4) and what the 8-wave kernel gives; twice in a row; and it must
    agree with the oracle."""
    k = steps * bk
    _say(f"fused epilogue {kind} {m}x{n}x{k} grid {grid}")
    run, want = _launcher(kind, m, n, k, 81)
    tb_option("grid", grid)
    tb_option("waves", 24)
    eight = run()
    tb_option("waves", 22)
    tb_option("lab", 4)
    compiled = run()
    tb_option("lab", 0)
    fused = run()
    again = run()
    assert OG.rel_fro_error(fused.float(), want.float()) <= (1e-3 if kind in ("bf16", "i8") else TOL_Q)
    assert torch.equal(compiled.view(torch.int16), eight.view(torch.int16))
    assert torch.equal(fused.view(torch.int16), compiled.view(torch.int16))
    assert torch.equal(again.view(torch.int16), fused.view(torch.int16))


@pytest.mark.parametrize("kind", ["fp8", "f16"])
@pytest.mark.parametrize("m,n,steps,grid", [(512, 768, 4, 1), (1280, 768, 6, 3), (1100, 1300, 8, 2), (4096, 4096, 4, 0)])
def test_fused_epilogue_fp16_output(kind, m, n, steps, grid, tb_option):
    """fp16 results take the fused epilogue too (its own conversion): the same bits as the compiled epilogue of
    the same kernel and as the 8-wave kernel, and the oracle's values."""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import persistent_matmul_lt
    bk = 128 if kind == "fp8" else 64
    k = steps * bk
    _say(f"fused epilogue, fp16 out, {kind} {m}x{n}x{k} grid {grid}")
    if kind == "fp8":
        aq, bq, sa, sb = _fp8_case(m, n, k, 87)
        sa = sa * 0.05          # keep the results inside fp16's range
        a, b = aq.cuda(), bq.T.contiguous().cuda().T
        kw = dict(a_scale=sa.cuda(), b_scale=sb.cuda(), quantized=True)
        want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).half()
        tol = TOL_Q
    else:
        g = torch.Generator().manual_seed(87)
        a_cpu = (torch.randn(m, k, generator=g) * 0.5).half()
        bt_cpu = (torch.randn(n, k, generator=g) * 0.5).half()
        a, b = a_cpu.cuda(), bt_cpu.cuda().T
        kw = {}
        want = OG.ref_gemm(a_cpu, bt_cpu.T, torch.float32).half()
        tol = 1e-3

    def run():
        sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, torch.float16, a.device)
        sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 256, 256, bk
        c = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        persistent_matmul_lt(a, b, c, sel, None, **kw)
        return c.cpu()
    tb_option("grid", grid)
    tb_option("waves", 24)
    eight = run()
    tb_option("waves", 22)
    tb_option("lab", 4)
    compiled = run()
    tb_option("lab", 0)
    fused = run()
    assert OG.rel_fro_error(fused.float(), want.float()) <= tol
    assert torch.equal(compiled.view(torch.int16), eight.view(torch.int16))
    assert torch.equal(fused.view(torch.int16), compiled.view(torch.int16))


def test_fused_epilogue_work_stealing(tb_option):
    """Tiles drawn from the work-stealing queues (which tile follows which is decided at run time) with
    two workgroups: same bits as the data-parallel launch."""
    m, n, k = 1280, 1024, 512
    aq, bq, sa, sb = _fp8_case(m, n, k, 82)
    tb_option("grid", 2)
    static = _run_fp8(aq, bq, sa, sb, 22, tb_option)
    for rep in range(2):
        ws = _run_fp8(aq, bq, sa, sb, 22, tb_option, work_stealing=True)
        assert torch.equal(static.view(torch.int16), ws.view(torch.int16)), f"launch {rep}"


# ---- workspace rules --------------------------------------------------------------------------------------
def test_streamk_then_work_stealing_on_one_config():
    """Stream-K flags and work-stealing counters live in disjoint regions of the workspace: a Stream-K
    launch whose workgroups 64, 128, 192 publish (explicit grid) followed by work stealing on the SAME
    config, and the other way round, both against the oracle."""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import streamk_matmul_lt
    dtype = torch.bfloat16
    m = n = k = 2048
    g = torch.Generator().manual_seed(81)
    a_cpu, b_cpu = (torch.randn(m, k, generator=g) * 0.5).to(dtype), (torch.randn(k, n, generator=g) * 0.5).to(dtype)
    want = OG.ref_gemm(a_cpu, b_cpu, torch.float32).to(dtype)
    a, b = a_cpu.cuda(), b_cpu.cuda()
    sel = tb.OrigamiMatmulSelector(m, n, k, dtype, dtype, dtype, a.device, streamk=True)
    cfg = tb.matmul_preamble(sel)
    for order in (("sk", "ws", "sk", "ws"), ("ws", "sk", "ws")):
        cfg.reset(streamk=True, work_stealing=True)
        for what in order:
            c = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
            if what == "sk":
                streamk_matmul_lt(a, b, c, sel, cfg, sk_grid=200)
            else:
                tb.matmul_lt(a, b, c, sel, cfg, work_stealing=True)
            err = OG.rel_fro_error(c.float().cpu(), want.float())
            assert err <= 1e-3, f"{order} at {what}: {err}"
        assert cfg.status() == 0


def test_streamk_epoch_zero_is_refused():
    """A zero-initialised descriptor (epoch 0) on a zeroed workspace would match every flag at once."""
    import tritonblas_amd as tb
    from tritonblas_amd import _lib
    lib = _lib.load()
    m, n, k = 256, 256, 4096
    a = torch.randn(m, k, device="cuda").half()
    b = torch.randn(k, n, device="cuda").half()
    c = torch.zeros(m, n, device="cuda").half()
    d = _lib.tb_gemm_desc()
    d.struct_bytes = C.sizeof(_lib.tb_gemm_desc)
    d.a_type = d.b_type = d.c_type = _lib.TB_F16
    d.m, d.n, d.k = m, n, k
    d.a_stride_m, d.a_stride_k = a.stride()
    d.b_stride_k, d.b_stride_n = b.stride()
    d.c_stride_m, d.c_stride_n = c.stride()
    d.a, d.b, d.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
    d.schedule, d.grid = _lib.TB_SCHED_STREAMK, 64
    need = lib.tb_workspace_bytes(d)
    assert need > 0
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    d.workspace, d.workspace_bytes = ws.data_ptr(), need
    d.epoch = 0
    assert lib.tb_gemm(d, _lib.stream_handle()) == _lib.TB_ERR_BAD_ARGUMENT
    d.epoch = 1
    assert lib.tb_gemm(d, _lib.stream_handle()) == _lib.TB_OK
    torch.cuda.synchronize()
    assert OG.rel_fro_error(c.float().cpu(), (a.float().cpu() @ b.float().cpu()).half().float()) <= 1e-3


def test_streamk_poll_bound_poisons_the_tile():
    """With a poll bound of one, owners give up before their partners publish (every kernel still ends
    normally): the tiles they could not finish must hold NaN, never stale memory, the status word must be
    set and MatmulConfig.check() must raise.  A later launch with the default bound is correct again."""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import streamk_matmul_lt
    dtype = torch.bfloat16
    m, n, k = 256, 256, 16384
    g = torch.Generator().manual_seed(82)
    a_cpu, b_cpu = (torch.randn(m, k, generator=g) * 0.5).to(dtype), (torch.randn(k, n, generator=g) * 0.5).to(dtype)
    want = OG.ref_gemm(a_cpu, b_cpu, torch.float32).to(dtype)
    a, b = a_cpu.cuda(), b_cpu.cuda()
    sel = tb.OrigamiMatmulSelector(m, n, k, dtype, dtype, dtype, a.device, streamk=True)
    cfg = tb.matmul_preamble(sel)
    cfg.spin_limit = 1
    c = torch.full((m, n), 7.0, dtype=dtype, device="cuda")
    streamk_matmul_lt(a, b, c, sel, cfg, sk_grid=256)
    torch.cuda.synchronize()
    got = c.float().cpu()
    if cfg.status() != 0:
        assert torch.isnan(got).any()
        ok = ~torch.isnan(got)
        assert torch.equal(got[ok], want.float()[ok]) or OG.rel_fro_error(got[ok], want.float()[ok]) <= 1e-3
        with pytest.raises(RuntimeError):
            cfg.check()
        assert cfg.status() == 0
    else:   # every partner happened to be early: then the result must simply be right
        assert OG.rel_fro_error(got, want.float()) <= 1e-3
    cfg.spin_limit = 0
    c2 = torch.zeros(m, n, dtype=dtype, device="cuda")
    streamk_matmul_lt(a, b, c2, sel, cfg, sk_grid=256)
    assert OG.rel_fro_error(c2.float().cpu(), want.float()) <= 1e-3
    cfg.check()


def test_streamk_poll_bound_two_tiles_one_workgroup():
    """Three workgroups share four tiles: the last workgroup owns a whole tile (no partner) and the tail of the
    tile before it (partner: workgroup 1).  With a poll bound of one, whatever it could not finish is NaN and
    everything else is right -- no tile of a workgroup that gave up is left as stale memory -- and with an e4m3
    result the poisoned tile reads as NaN bytes, not as a clamped finite value."""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import streamk_matmul_lt
    m, n, k = 512, 512, 8192
    aq, bq, sa, sb = _fp8_case(m, n, k, 83)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    for out_dtype in (torch.bfloat16, torch.float8_e4m3fn):
        want = OG.ref_gemm(aq, bq, out_dtype, a_scale=sa, b_scale=sb).float()
        sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, out_dtype, a.device, streamk=True)
        sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 256, 256, 128
        cfg = tb.matmul_preamble(sel)
        cfg.ensure(64 << 20)
        cfg.spin_limit = 1
        c = torch.full((m, n), 7.0, device="cuda").to(out_dtype)
        streamk_matmul_lt(a, b, c, sel, cfg, sk_grid=3, a_scale=sa.cuda(), b_scale=sb.cuda(), quantized=True)
        torch.cuda.synchronize()
        got = c.float().cpu()
        failed = cfg.status() != 0
        assert failed == bool(torch.isnan(got).any()), "NaN tiles and the status word go together"
        ok = ~torch.isnan(got)
        # (whole 256x256 tiles are poisoned, nothing else; no 7.0 of the initial fill survives anywhere)
        for ti in range(2):
            for tj in range(2):
                blk = ok[ti * 256:(ti + 1) * 256, tj * 256:(tj + 1) * 256]
                assert blk.all() or not blk.any()
        if out_dtype == torch.bfloat16:
            assert OG.rel_fro_error(got[ok], want[ok]) <= 1e-2
        else:
            torch.testing.assert_close(got[ok], want[ok], atol=2.0, rtol=0.2)
        cfg.clear_status()


# ---- e4m3 output ---------------------------------------------------------------------------------------------
def test_a8w8_fp8_output_keeps_nan():
    """torch.clamp keeps NaN (the reference's oracle, tests/test_matmul_a8w8_lt.py:11-38): a row whose scale is
    NaN must come out as e4m3 NaN bytes, a row whose scale is +Inf as +-448 (or NaN where the sum is zero)."""
    import tritonblas_amd as tb
    m, n, k = 256, 512, 512
    aq, bq, sa, sb = _fp8_case(m, n, k, 92)
    sa = sa.clone()
    sa[3] = float("nan")
    sa[100] = float("inf")
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    for streamk in (False, True):
        c = torch.zeros(m, n, dtype=torch.float8_e4m3fn, device="cuda")
        tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c, enable_streamk=streamk)
        want = OG.ref_gemm(aq, bq, torch.float8_e4m3fn, a_scale=sa, b_scale=sb).float()
        got = c.float().cpu()
        assert torch.isnan(want[3]).all() and torch.isnan(got[3]).all()
        assert torch.equal(torch.isnan(got), torch.isnan(want))
        assert torch.equal(got[100][~torch.isnan(got[100])], want[100][~torch.isnan(want[100])])
        fin = ~torch.isnan(want)
        torch.testing.assert_close(got[fin], want[fin], atol=2.0, rtol=0.2)


@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("m,n,k", [(512, 768, 512), (300, 500, 768), (1, 257, 512), (2048, 1280, 1024)])
def test_fp8_four_wave_kernel_e4m3_output(m, n, k, out_dtype, tb_option):
    """8-bit float results (e4m3, e5m2) straight from the 4-wave kernel's accumulators (eight bytes per lane and row
    block): the same bytes as the 8-wave kernel's, NaN kept, the reference's tolerance against the oracle (for e5m2
    widened to one unit in its last place, 25 %)."""
    aq, bq, sa, sb = _fp8_case(m, n, k, 93)
    sa = sa * (40.0 if out_dtype == torch.float8_e4m3fn else 5000.0)   # part of the result beyond the format's range
    sa[0] = float("nan")
    outs = {}
    for waves in (22, 24):
        outs[waves] = _run_fp8(aq, bq, sa, sb, waves, tb_option, out_dtype=out_dtype)
    want = OG.ref_gemm(aq, bq, out_dtype, a_scale=sa, b_scale=sb)
    assert torch.equal(outs[22].view(torch.uint8), outs[24].view(torch.uint8))
    got = outs[22].float()
    assert torch.isnan(got[0]).all() and not torch.isnan(got[1:]).any()
    # (the e5m2 case scales its sums 125 times as far up, and the absolute tolerance with them)
    e4 = out_dtype == torch.float8_e4m3fn
    torch.testing.assert_close(got[1:], want.float()[1:], atol=2.0 if e4 else 250.0, rtol=0.2 if e4 else 0.26)
    if m > 1:
        same = (outs[22][1:].view(torch.uint8) == want[1:].view(torch.uint8)).float().mean().item()
        assert same >= 0.99


@pytest.mark.parametrize("out_dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (100, 300, 640), (512, 1024, 512)])
@pytest.mark.parametrize("streamk", [False, True])
def test_a8w8_fp8_output(m, n, k, streamk, out_dtype):
    """a8w8 with an 8-bit float result: clamp to the format's largest finite value (448, 57344), round to nearest even
    -- the reference's oracle and tolerances for this case (tests/test_matmul_a8w8_lt.py:11-38, :108-112: atol 2.0,
    rtol 0.2; e5m2, whose steps are 25 % and whose case is scaled 125 times as far up, at rtol 0.26 and atol 250)."""
    import tritonblas_amd as tb
    aq, bq, sa, sb = _fp8_case(m, n, k, 91)
    e4 = out_dtype == torch.float8_e4m3fn
    sa = sa * (40.0 if e4 else 5000.0)   # push part of the result beyond the format's range so that the clamp is exercised
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    c = torch.zeros(m, n, dtype=out_dtype, device="cuda")
    tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c, enable_streamk=streamk)
    want = OG.ref_gemm(aq, bq, out_dtype, a_scale=sa, b_scale=sb)
    got = c.float().cpu()
    assert not torch.isnan(got).any() and not torch.isinf(got).any()
    lim = 448.0 if e4 else 57344.0
    assert got.abs().max() == lim, "the case is meant to reach the clamp"
    torch.testing.assert_close(got, want.float(), atol=2.0 if e4 else 250.0, rtol=0.2 if e4 else 0.26)
    # the rounding itself: at most one step away from the oracle's cast, and mostly identical
    same = (c.cpu().view(torch.uint8) == want.view(torch.uint8)).float().mean().item()
    assert same >= 0.99, f"only {same:.4f} of the codes match the oracle's"


# ---- Stream-K on the 4-wave kernels, and Stream-K with work stealing ------------------------------------------
def _launch_info(a, b, c, schedule, grid, tile, scales=False):
    from tritonblas_amd import _lib
    import ctypes as C
    d = _lib.tb_gemm_desc()
    d.struct_bytes = C.sizeof(_lib.tb_gemm_desc)
    d.a_type = d.b_type = _lib.tb_dtype(a.dtype)
    d.c_type = _lib.tb_dtype(c.dtype)
    d.m, d.k = a.shape
    d.n = b.shape[1]
    d.a_stride_m, d.a_stride_k = a.stride()
    d.b_stride_k, d.b_stride_n = b.stride()
    d.c_stride_m, d.c_stride_n = c.stride()
    d.a, d.b, d.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
    d.block_m, d.block_n, d.block_k = tile
    d.schedule, d.grid = schedule, grid
    info = _lib.tb_launch_info()
    assert _lib.load().tb_gemm_launch_info(d, C.byref(info)) == _lib.TB_OK
    return info


@pytest.mark.parametrize("kind,bk", [("fp8", 128), ("bf16", 64)])
@pytest.mark.parametrize("m,n,steps,grid", [(512, 512, 16, 12), (768, 512, 32, 7), (300, 500, 8, 5), (512, 768, 20, 9),
                                            (1024, 1024, 64, 256), (2304, 2048, 8, 64)])
@pytest.mark.parametrize("work_stealing", [False, True])
def test_four_wave_streamk(kind, bk, m, n, steps, grid, work_stealing, tb_option):
    """The Stream-K tail on the hand-scheduled kernels (K ranges cut at multiples of four K steps): oracle parity,
    the same bits in three launches on one config without reset, the launch really is the 4-wave kernel, and with
    the whole tiles drawn from the work-stealing queues the bits stay the same."""
    import tritonblas_amd as tb
    from tritonblas_amd import _lib
    from tritonblas_amd.matmul import streamk_matmul_lt
    k = steps * bk
    _say(f"w4 stream-k {kind} {m}x{n}x{k} grid {grid} ws {work_stealing}")
    if kind == "fp8":
        aq, bq, sa, sb = _fp8_case(m, n, k, 84)
        a, b = aq.cuda(), bq.T.contiguous().cuda().T
        scales = dict(a_scale=sa.cuda(), b_scale=sb.cuda(), quantized=True)
        want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
        tol = TOL_Q
    else:
        g = torch.Generator().manual_seed(84)
        a_cpu = (torch.randn(m, k, generator=g) * 0.5).bfloat16()
        bt_cpu = (torch.randn(n, k, generator=g) * 0.5).bfloat16()
        a, b = a_cpu.cuda(), bt_cpu.cuda().T
        scales = {}
        want = OG.ref_gemm(a_cpu, bt_cpu.T, torch.float32).to(torch.bfloat16)
        tol = 1e-3
    tb_option("waves", 22)
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, torch.bfloat16, a.device, streamk=True)
    sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 256, 256, bk
    c = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    sched = _lib.TB_SCHED_STREAMK_WS if work_stealing else _lib.TB_SCHED_STREAMK
    info = _launch_info(a, b, c, sched, grid, (256, 256, bk))
    tiles = ((m + 255) // 256) * ((n + 255) // 256)
    if tiles % min(grid, 256) != 0:
        assert info.four_wave == 1 and info.sk_unit == 4 and info.sk_tiles == tiles % info.grid
        assert info.sk_ws == (1 if work_stealing else 0)
    cfg = tb.matmul_preamble(sel)
    outs = []
    for rep in range(3):
        c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        streamk_matmul_lt(a, b, c, sel, cfg, sk_grid=grid, work_stealing=work_stealing, **scales)
        outs.append(c.cpu())
    cfg.check()
    assert OG.rel_fro_error(outs[0].float(), want.float()) <= tol
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    assert torch.equal(outs[0].view(torch.int16), outs[2].view(torch.int16))
    if work_stealing:
        cs = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        streamk_matmul_lt(a, b, cs, sel, cfg, sk_grid=grid, **scales)
        assert torch.equal(outs[0].view(torch.int16), cs.cpu().view(torch.int16)), "queues and static deal must give the same bits"


def test_streamk_work_stealing_eight_wave_kernel(tb_option):
    """The same schedule on a compiler-scheduled tile (128x128): whole tiles from the queues, Stream-K tail, same
    bits as the static deal, three launches without reset."""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import streamk_matmul_lt
    m, n, k = 1536, 1280, 2048
    g = torch.Generator().manual_seed(86)
    a_cpu = (torch.randn(m, k, generator=g) * 0.5).bfloat16()
    b_cpu = (torch.randn(k, n, generator=g) * 0.5).bfloat16()
    want = OG.ref_gemm(a_cpu, b_cpu, torch.float32).to(torch.bfloat16)
    a, b = a_cpu.cuda(), b_cpu.cuda()
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, torch.bfloat16, a.device, streamk=True)
    sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 128, 128, 64
    cfg = tb.matmul_preamble(sel)
    static = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    streamk_matmul_lt(a, b, static, sel, cfg, sk_grid=50)
    assert OG.rel_fro_error(static.float().cpu(), want.float()) <= 1e-3
    for rep in range(3):
        c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        streamk_matmul_lt(a, b, c, sel, cfg, sk_grid=50, work_stealing=True)
        assert torch.equal(c.view(torch.int16), static.view(torch.int16)), f"launch {rep}"
    cfg.check()
