"""Parity at the full sizes of the five benchmark configurations.

The CPU oracle cannot multiply these matrices in test time, so each case checks (1) a sample of
complete output rows (spread over the row tiles, every column tile) against the oracle's GEMM of
exactly those rows, and (2) a size-independent identity over the whole output: column sums,
sum_m C[m, :] = (sum_m s_a[m] A[m, :]) @ B * s_b, evaluated in fp64 on the host from the same
operands.  Inputs come from the seeded CPU generators of oracle/inputs.py."""
import numpy as np
import pytest
import torch

from oracle import gemm as OG
from oracle import inputs as OI
from oracle import mxfp4 as OM

pytestmark = pytest.mark.gpu


def _rows(m, count=12, seed=0):
    g = torch.Generator().manual_seed(seed)
    picks = torch.randint(0, m, (count,), generator=g)
    picks[0], picks[-1] = 0, m - 1
    return torch.unique(picks)


def _colsum_check(c_gpu, a32_weighted_sum, b32, col_scale, tol):
    """a32_weighted_sum: (K,) fp64 = sum over rows of (row scale * A row); b32: (K, N) fp32/any."""
    want = (a32_weighted_sum.double() @ b32.double())
    if col_scale is not None:
        want = want * col_scale.double()
    got = c_gpu.double().sum(dim=0).cpu()
    err = torch.linalg.norm(got - want) / torch.linalg.norm(want)
    assert err <= tol, f"column-sum identity off by {err:.3e}"


def test_c2_bf16_8192_tn():
    import tritonblas_amd as tb
    a, b = OI.c2_bf16()
    ad, bd = a.cuda(), b.T.contiguous().cuda().T
    c = torch.empty(8192, 8192, dtype=torch.bfloat16, device="cuda")
    sel = tb.OrigamiMatmulSelector(8192, 8192, 8192, a.dtype, b.dtype, c.dtype, ad.device)
    tb.matmul_lt(ad, bd, c, sel, None)
    rows = _rows(8192)
    want = OG.ref_gemm(a[rows], b, torch.float32).to(torch.bfloat16)
    assert OG.rel_fro_error(c[rows.cuda()].float().cpu(), want.float()) <= 1e-3
    # column sums: a sum of 8192 signed terms is a random walk, and so is the sum of their independent
    # bf16 output roundings (2^-9/sqrt(3) relative each): the identity holds to ~1.5e-3, not to 1e-3
    _colsum_check(c, a.double().sum(dim=0), b, None, 5e-3)
    # work stealing must reproduce the static schedule bit for bit at this size too
    cfg = tb.matmul_preamble(sel)
    c2 = torch.empty_like(c)
    tb.matmul_lt(ad, bd, c2, sel, cfg, work_stealing=True)
    assert torch.equal(c, c2)


def test_c3_fp8_prefill_and_decode():
    import tritonblas_amd as tb
    m, n, k = 8192, 28672, 8192
    a, w = OI.c3_fp8_source(m, n, k)
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1)
    wq, sw = OG.quantize_per_channel_fp8(w, axis=1)       # per output channel = per row of the (N, K) weight
    del a, w
    ad, wd, sad, swd = aq.cuda(), wq.cuda(), sa.cuda(), sw.cuda()
    c = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    sel = tb.OrigamiMatmulSelector(m, n, k, ad.dtype, wd.dtype, c.dtype, ad.device)
    tb.matmul_a8w8_lt(ad, wd.T, sad, swd, c, sel, None)
    rows = _rows(m, 8)
    want = OG.ref_gemm(aq[rows], wq.T, torch.float32, a_scale=sa[rows], b_scale=sw).to(torch.bfloat16)
    assert OG.rel_fro_error(c[rows.cuda()].float().cpu(), want.float()) <= 1e-2
    wsum = (aq.float() * sa[:, None]).double().sum(dim=0)
    _colsum_check(c, wsum, wq.T.float(), sw, 1e-2)
    del c
    # decode: 32 rows against the weight as (N, K) = (8192, 28672): reuse the first 8192*28672 weight bytes
    md, nd, kd = 32, 8192, 28672
    a2, w2 = OI.c3_fp8_source(md, nd, kd)
    aq2, sa2 = OG.quantize_per_channel_fp8(a2, axis=1)
    wq2, sw2 = OG.quantize_per_channel_fp8(w2, axis=1)
    cd = torch.empty(md, nd, dtype=torch.bfloat16, device="cuda")
    seld = tb.OrigamiMatmulSelector(md, nd, kd, aq2.dtype, wq2.dtype, cd.dtype, cd.device, streamk=True)
    cfg = tb.matmul_preamble(seld)
    tb.matmul_a8w8_lt(aq2.cuda(), wq2.cuda().T, sa2.cuda(), sw2.cuda(), cd, seld, cfg, enable_streamk=True)
    cols = torch.arange(0, nd, 7)
    want = OG.ref_gemm(aq2, wq2[cols].T, torch.float32, a_scale=sa2, b_scale=sw2[cols]).to(torch.bfloat16)
    assert OG.rel_fro_error(cd[:, cols.cuda()].float().cpu(), want.float()) <= 1e-2


def test_c4_grouped_moe():
    import tritonblas_amd as tb
    a, w, offsets = OI.c4_moe_source()
    assert int(offsets[-1]) == 8192
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1)
    wq, sw = OG.quantize_per_channel_fp8(w, axis=2)
    del a, w
    c = torch.full((8192, 14336), float("nan"), dtype=torch.bfloat16, device="cuda")
    tb.grouped_matmul_a8w8(aq.cuda(), wq.cuda(), sa.cuda(), sw.cuda(), c, offsets.cuda())
    assert not torch.isnan(c).any()
    # per expert: first, last and a middle row against the a8w8 closed form with that expert's weight
    for e in range(8):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        rows = torch.tensor(sorted({lo, (lo + hi) // 2, hi - 1}))
        want = OG.ref_gemm(aq[rows], wq[e].T, torch.float32, a_scale=sa[rows], b_scale=sw[e]).to(torch.bfloat16)
        assert OG.rel_fro_error(c[rows.cuda()].float().cpu(), want.float()) <= 1e-2, f"expert {e}"


def test_c5_mxfp4_quant_and_gemm():
    import tritonblas_amd as tb
    m, n, k = 8192, 8192, 16384
    a, b = OI.c5_mxfp4_source(m, n, k)
    ad, bd = a.cuda(), b.cuda()
    aq, as_ = tb.hadamard_mxfp4_quant(ad)
    bq, bs = tb.hadamard_mxfp4_quant(bd)
    # quantiser: bit-exact on sampled rows (the oracle takes ~1 s per 256 rows at K = 16384)
    rows = _rows(m, 64, seed=5)
    wc, ws = OM.hadamard_mxfp4_quant(a[rows].float().numpy())
    assert np.array_equal(aq[rows.cuda()].cpu().numpy(), wc) and np.array_equal(as_[rows.cuda()].cpu().numpy(), ws)
    # idempotence-style invariant over the whole tensor: dequantised values lie on the e2m1 grid
    # times the block scale and the largest magnitude of every block is 4 or 6 (amax maps into (3.5, 7]),
    # or the block is all zero
    codes = aq[:512].cpu().numpy()
    mags = OM.unpack_codes(codes) & 7
    blockmax = mags.reshape(512, -1, 32).max(axis=2)
    assert np.isin(blockmax, (0, 6, 7)).all()
    c = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    tb.matmul_fp4(aq, bq, c, as_, bs)
    r2 = _rows(m, 8, seed=6)
    want = OG.ref_gemm_fp4(aq[r2.cuda()].cpu(), bq.cpu(), as_[r2.cuda()].cpu(), bs.cpu(), return_fp32=True).to(torch.bfloat16)
    assert OG.rel_fro_error(c[r2.cuda()].float().cpu(), want.float()) <= 1e-2
    # the rotation cancels in A'B'^T: the MXFP4 product tracks the bf16 product up to quantisation noise
    exact = a[r2].float() @ b.float().T
    assert OG.rel_fro_error(c[r2.cuda()].float().cpu(), exact) < 0.25
