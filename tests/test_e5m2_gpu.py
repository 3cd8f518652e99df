"""GPU tests of FP8 e5m2 operands, alone and mixed with e4m3 (the second type the reference's get_fp8_dtypes returns,
include/tritonblas/utils.py:46; its own a8w8 tests run e4m3 only).  Every kernel family that serves
e4m3 serves e5m2 with the other format field in its MFMAs: the hand-scheduled 4-wave kernel, the 8-wave
tile kernels, the gather kernel for operands the fast loaders cannot address, and the small-M streaming
kernel.  The oracle is the same for both formats: fp32 GEMM of the dequantised operands times the scale
vectors (oracle/gemm.py), with torch's own e5m2 -> fp32 conversion."""
import sys

import pytest
import torch

from oracle import gemm as OG

pytestmark = pytest.mark.gpu
E5 = torch.float8_e5m2
TOL_Q = 1e-2    # relative Frobenius error against the fp32 oracle rounded to the output type


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _case(m, n, k, seed):
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(seed)).bfloat16()
    w = torch.randn(n, k, generator=torch.Generator().manual_seed(seed + 10000)).bfloat16()
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1, dtype=E5)
    bq, sb = OG.quantize_per_channel_fp8(w.T, axis=0, dtype=E5)
    return aq, bq, sa, sb


def _run_tile(aq, bq, sa, sb, waves, tb_option, out_dtype=torch.bfloat16, work_stealing=False):
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import persistent_matmul_lt
    m, k = aq.shape
    n = bq.shape[1]
    tb_option("waves", waves)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, out_dtype, a.device)
    sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 256, 256, 128
    c = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
    cfg = tb.matmul_preamble(sel) if work_stealing else None
    persistent_matmul_lt(a, b, c, sel, cfg, a_scale=sa.cuda(), b_scale=sb.cuda(), quantized=True, work_stealing=work_stealing)
    return c.cpu()


def test_the_format_matters():
    """The oracle itself tells the formats apart: the same bytes read as e4m3 give another product."""
    aq, bq, sa, sb = _case(64, 64, 128, 3)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb)
    other = OG.ref_gemm(aq.view(torch.float8_e4m3fn), bq.view(torch.float8_e4m3fn), torch.float32, a_scale=sa, b_scale=sb)
    assert not torch.isfinite(other).all() or OG.rel_fro_error(other, want) > 0.5


@pytest.mark.parametrize("m,n,k", [(256, 256, 512), (512, 768, 512), (300, 500, 768), (1024, 2048, 1024), (2560, 2304, 512)])
def test_e5m2_four_wave_kernel(m, n, k, tb_option):
    """Whole and ragged tiles, one to many tiles per workgroup (fused epilogues from the second tile on):
    oracle parity and bit-equality with the 8-wave kernel of the same tile."""
    _say(f"w4 e5m2 {m}x{n}x{k}")
    aq, bq, sa, sb = _case(m, n, k, 171)
    new = _run_tile(aq, bq, sa, sb, 22, tb_option)
    old = _run_tile(aq, bq, sa, sb, 24, tb_option)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    assert OG.rel_fro_error(new.float(), want.float()) <= TOL_Q
    assert torch.equal(new.view(torch.int16), old.view(torch.int16))


def test_e5m2_four_wave_fused_epilogue_small_grid(tb_option):
    """Twelve tiles on three workgroups: every workgroup stores three tiles from inside the next tile's K loop."""
    m, n, k = 768, 1024, 1024
    aq, bq, sa, sb = _case(m, n, k, 172)
    tb_option("grid", 3)
    new = _run_tile(aq, bq, sa, sb, 22, tb_option)
    tb_option("lab", 4)     # compiled epilogues only
    plain = _run_tile(aq, bq, sa, sb, 22, tb_option)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    assert OG.rel_fro_error(new.float(), want.float()) <= TOL_Q
    assert torch.equal(new.view(torch.int16), plain.view(torch.int16))


@pytest.mark.parametrize("m,n,k", [(64, 64, 128), (128, 384, 256), (1000, 520, 640), (2048, 512, 4096), (33, 1100, 384)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_e5m2_matmul_a8w8(m, n, k, out_dtype):
    """The reference's entry point (matmul.py:498-517) with the library's own tile choice."""
    import tritonblas_amd as tb
    _say(f"a8w8 e5m2 {m}x{n}x{k} -> {out_dtype}")
    aq, bq, sa, sb = _case(m, n, k, 173)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    c = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
    tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(out_dtype)
    assert OG.rel_fro_error(c.cpu().float(), want.float()) <= TOL_Q


@pytest.mark.parametrize("schedule", ["streamk", "work_stealing"])
def test_e5m2_other_schedules(schedule):
    import tritonblas_amd as tb
    m, n, k = 1024, 1536, 2048
    aq, bq, sa, sb = _case(m, n, k, 174)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    if schedule == "streamk":
        tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c, enable_streamk=True, sk_grid=100)
    else:
        tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c, work_stealing=True)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    assert OG.rel_fro_error(c.cpu().float(), want.float()) <= TOL_Q


def test_e5m2_gather_kernel():
    """K not a multiple of the K step and an operand with a pitch the 16-byte loaders cannot use."""
    import tritonblas_amd as tb
    m, n, k = 200, 136, 200
    aq, bq, sa, sb = _case(m, n, k, 175)
    buf = torch.zeros(m, k + 3, dtype=torch.uint8, device="cuda")
    buf[:, :k] = aq.view(torch.uint8).cuda()
    a = buf[:, :k].view(E5)
    b = bq.T.contiguous().cuda().T
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    assert OG.rel_fro_error(c.cpu().float(), want.float()) <= TOL_Q


@pytest.mark.parametrize("m", [1, 16, 32, 48])
def test_e5m2_small_m_streaming_kernel(m, tb_option):
    import tritonblas_amd as tb
    n, k = 2048, 4096
    aq, bq, sa, sb = _case(m, n, k, 176)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    out = {}
    for name, opt in (("streaming", "skinny"), ("tiles", "no_skinny")):
        tb_option("skinny", 0)
        tb_option("no_skinny", 0)
        tb_option(opt, 1)
        c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c)
        out[name] = c.cpu()
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    for name, c in out.items():
        assert OG.rel_fro_error(c.float(), want.float()) <= TOL_Q, name


def test_e5m2_operands_e4m3_output():
    """The a8w8 oracle's 8-bit output (clamp to +-448, round to nearest even) with e5m2 operands, at the
    reference's tolerances (tests/test_matmul_a8w8_lt.py:108-112)."""
    import tritonblas_amd as tb
    m, n, k = 512, 512, 1024
    aq, bq, sa, sb = _case(m, n, k, 177)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    c = torch.zeros(m, n, dtype=torch.float8_e4m3fn, device="cuda")
    tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c)
    want = OG.ref_gemm(aq, bq, torch.float8_e4m3fn, a_scale=sa, b_scale=sb)
    torch.testing.assert_close(c.cpu().float(), want.float(), atol=2.0, rtol=0.2)
    assert (c.cpu().view(torch.uint8) == want.view(torch.uint8)).float().mean() >= 0.99


def test_other_mixed_operand_types_are_refused():
    """8-bit floats of the two formats mix (below); nothing else does."""
    import tritonblas_amd as tb
    aq, bq, sa, sb = _case(64, 64, 128, 178)
    a = aq.cuda()
    b = bq.T.contiguous().cuda().T.float().bfloat16()
    c = torch.zeros(64, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError):
        tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c)


# ---- A and B in different 8-bit float formats (reference origami.py:98-112, matmul.py:42-66 take the two types
# separately; its tests run no such case, so the oracle -- torch's own conversions of each operand to fp32 -- is the pin)
E4 = torch.float8_e4m3fn
MIXES = [(E4, E5), (E5, E4)]


def _mixed_case(m, n, k, seed, a_fmt, b_fmt):
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(seed)).bfloat16()
    w = torch.randn(n, k, generator=torch.Generator().manual_seed(seed + 10000)).bfloat16()
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1, dtype=a_fmt)
    bq, sb = OG.quantize_per_channel_fp8(w.T, axis=0, dtype=b_fmt)
    return aq, bq, sa, sb


def test_mixed_formats_the_assignment_matters():
    """The oracle tells the two mixtures apart: the same bytes with the formats swapped give another product."""
    aq, bq, sa, sb = _mixed_case(64, 64, 128, 5, E4, E5)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb)
    other = OG.ref_gemm(aq.view(E5), bq.view(E4), torch.float32, a_scale=sa, b_scale=sb)
    assert not torch.isfinite(other).all() or OG.rel_fro_error(other, want) > 0.5


@pytest.mark.parametrize("a_fmt,b_fmt", MIXES)
@pytest.mark.parametrize("m,n,k", [(256, 256, 512), (300, 500, 768), (1024, 2048, 1024), (2560, 2304, 512)])
def test_mixed_formats_four_wave_kernel(m, n, k, a_fmt, b_fmt, tb_option):
    """Whole and ragged tiles, fused epilogues from a workgroup's second tile on: oracle parity and bit-equality of the
    hand-scheduled kernel with the 8-wave kernel of the same tile."""
    _say(f"w4 {a_fmt} x {b_fmt} {m}x{n}x{k}")
    aq, bq, sa, sb = _mixed_case(m, n, k, 181, a_fmt, b_fmt)
    new = _run_tile(aq, bq, sa, sb, 22, tb_option)
    old = _run_tile(aq, bq, sa, sb, 24, tb_option)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    assert OG.rel_fro_error(new.float(), want.float()) <= TOL_Q
    assert torch.equal(new.view(torch.int16), old.view(torch.int16))


@pytest.mark.parametrize("a_fmt,b_fmt", MIXES)
@pytest.mark.parametrize("m,n,k", [(64, 64, 128), (128, 384, 256), (1000, 520, 640), (33, 1100, 384), (16, 2048, 4096)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32, torch.float8_e4m3fn])
def test_mixed_formats_matmul_a8w8(m, n, k, out_dtype, a_fmt, b_fmt):
    """The reference's entry point (matmul.py:498-517) with the library's own tile choice (small tiles, the 32-row
    tile; the small-M streaming kernel does not take mixtures), also with an 8-bit result."""
    import tritonblas_amd as tb
    _say(f"a8w8 {a_fmt} x {b_fmt} {m}x{n}x{k} -> {out_dtype}")
    aq, bq, sa, sb = _mixed_case(m, n, k, 183, a_fmt, b_fmt)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    c = torch.zeros(m, n, dtype=out_dtype, device="cuda")
    tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c)
    want = OG.ref_gemm(aq, bq, out_dtype, a_scale=sa, b_scale=sb)
    if out_dtype == torch.float8_e4m3fn:
        torch.testing.assert_close(c.cpu().float(), want.float(), atol=2.0, rtol=0.2)
        assert (c.cpu().view(torch.uint8) == want.view(torch.uint8)).float().mean() >= 0.99
    else:
        assert OG.rel_fro_error(c.cpu().float(), want.float()) <= TOL_Q


@pytest.mark.parametrize("a_fmt,b_fmt", MIXES)
@pytest.mark.parametrize("schedule", ["streamk", "streamk_w4", "work_stealing"])
def test_mixed_formats_other_schedules(schedule, a_fmt, b_fmt):
    """Stream-K (on the library's tile and, with K = 16 steps and a forced 256x256 tile, on the 4-wave kernel) and work
    stealing."""
    import tritonblas_amd as tb
    from tritonblas_amd.matmul import streamk_matmul_lt
    m, n, k = 1024, 1536, 2048
    aq, bq, sa, sb = _mixed_case(m, n, k, 184, a_fmt, b_fmt)
    a, b = aq.cuda(), bq.T.contiguous().cuda().T
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    if schedule == "streamk":
        tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c, enable_streamk=True, sk_grid=100)
    elif schedule == "streamk_w4":
        sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, c.dtype, a.device, streamk=True)
        sel._sel.block_m, sel._sel.block_n, sel._sel.block_k = 256, 256, 128
        cfg = tb.matmul_preamble(sel)
        cfg.ensure(64 << 20)
        streamk_matmul_lt(a, b, c, sel, cfg, sk_grid=20, a_scale=sa.cuda(), b_scale=sb.cuda(), quantized=True)
        assert cfg.status() == 0
    else:
        tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c, work_stealing=True)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    assert OG.rel_fro_error(c.cpu().float(), want.float()) <= TOL_Q


@pytest.mark.parametrize("a_fmt,b_fmt", MIXES)
def test_mixed_formats_gather_kernel(a_fmt, b_fmt):
    """K not a multiple of the K step and an operand with a pitch the 16-byte loaders cannot use."""
    import tritonblas_amd as tb
    m, n, k = 200, 136, 200
    aq, bq, sa, sb = _mixed_case(m, n, k, 185, a_fmt, b_fmt)
    buf = torch.zeros(m, k + 3, dtype=torch.uint8, device="cuda")
    buf[:, :k] = aq.view(torch.uint8).cuda()
    a = buf[:, :k].view(a_fmt)
    b = bq.T.contiguous().cuda().T
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tb.matmul_a8w8(a, b, sa.cuda(), sb.cuda(), c)
    want = OG.ref_gemm(aq, bq, torch.float32, a_scale=sa, b_scale=sb).to(torch.bfloat16)
    assert OG.rel_fro_error(c.cpu().float(), want.float()) <= TOL_Q


def test_product_quantiser_e5m2():
    """The product's per-channel quantiser for e5m2 (reference utils.py:340-377) against the oracle's recipe, bit for bit."""
    import tritonblas_amd.utils as U
    x = torch.randn(96, 160, generator=torch.Generator().manual_seed(9)).bfloat16()
    for axis in (0, 1):
        q, s = U.quantize_tensor_per_channel(x.cuda(), E5, axis=axis)
        qo, so = OG.quantize_per_channel_fp8(x, axis=axis, dtype=E5)
        assert torch.equal(q.cpu().view(torch.uint8), qo.view(torch.uint8))
        assert torch.equal(s.cpu(), so)
