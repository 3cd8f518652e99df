"""Seeded random sweep over the GEMM entry points: element type x operand layouts x schedule x odd
shapes (any M, N, K including non-multiples of the vector width, slices with a row pitch), against
the CPU oracle.  Every launch goes through the C ABI.  TB_RANDOM_CASES / TB_RANDOM_SEED widen the sweep."""
import os
import random
import sys

import pytest
import torch

from oracle import gemm as OG

pytestmark = pytest.mark.gpu

TOL = {torch.float16: 1e-3, torch.bfloat16: 1e-3, torch.float32: 1e-5, torch.float8_e4m3fn: 1e-2, torch.int8: 1e-3}


def _cases(n, seed):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        dtype = rng.choice([torch.float16, torch.bfloat16, torch.float32, torch.float8_e4m3fn, torch.int8])
        big = rng.random() < 0.3
        m = rng.randint(1, 1500 if big else 300)
        nn = rng.randint(1, 1500 if big else 300)
        k = rng.choice([rng.randint(1, 2048), 32 * rng.randint(1, 64), 128 * rng.randint(1, 24)])
        out.append(dict(idx=i, dtype=dtype, m=m, n=nn, k=k, ta=rng.choice("TN"), tb=rng.choice("TN"),
                        sched=rng.choice(["persistent", "streamk", "ws", "ws_global", "ws_hier"]),
                        pitch=rng.choice([0, 0, 8, 3]), bias=rng.random() < 0.3, seed=rng.randint(0, 1 << 30)))
    return out


def _place(x_cpu, trans, pitch):
    """'T': the logical matrix is contiguous; 'N': its transpose is.  pitch > 0: rows sit in a wider buffer."""
    x = x_cpu.cuda()
    if trans == "N":
        x = x.T
    rows, cols = x.shape
    buf = torch.zeros(rows, cols + pitch, dtype=torch.uint8 if x.dtype == torch.float8_e4m3fn else x.dtype, device="cuda")
    if x.dtype == torch.float8_e4m3fn:
        buf = buf.view(torch.float8_e4m3fn)
        buf.view(torch.uint8)[:, :cols] = x.contiguous().view(torch.uint8)
    else:
        buf[:, :cols] = x
    v = buf[:, :cols]
    return v.T if trans == "N" else v


@pytest.mark.parametrize("case", _cases(int(os.environ.get("TB_RANDOM_CASES", "72")), int(os.environ.get("TB_RANDOM_SEED", "20241"))), ids=lambda c: f"{c['idx']}-{str(c['dtype']).split('.')[-1]}-{c['m']}x{c['n']}x{c['k']}-{c['ta']}{c['tb']}-{c['sched']}")
def test_random_case(case):
    import tritonblas_amd as tb
    print("random case", case, flush=True)
    sys.stdout.flush()
    dtype, m, n, k = case["dtype"], case["m"], case["n"], case["k"]
    g = torch.Generator().manual_seed(case["seed"])
    a32, b32 = torch.randn(m, k, generator=g) * 0.5, torch.randn(k, n, generator=g) * 0.5
    quant = dtype in (torch.float8_e4m3fn, torch.int8)
    out_dtype = torch.bfloat16 if quant else dtype
    bias = (torch.randn(n, generator=g).to(out_dtype) if case["bias"] and not quant else None)
    if dtype == torch.int8:
        a_cpu, sa = OG.quantize_per_channel_int8(a32, axis=1)
        b_cpu, sb = OG.quantize_per_channel_int8(b32, axis=0)
    elif quant:
        a_cpu, sa = OG.quantize_per_channel_fp8(a32, axis=1)
        b_cpu, sb = OG.quantize_per_channel_fp8(b32, axis=0)
    else:
        a_cpu, b_cpu, sa, sb = a32.to(dtype), b32.to(dtype), None, None
    a, b = _place(a_cpu, case["ta"], case["pitch"]), _place(b_cpu, case["tb"], case["pitch"])
    assert a.shape == (m, k) and b.shape == (k, n)
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, out_dtype, a.device, streamk=case["sched"] == "streamk")
    cfg = tb.matmul_preamble(sel)
    cfg.global_atomic, cfg.hierarchical = case["sched"] == "ws_global", case["sched"] == "ws_hier"
    ws, sk = case["sched"].startswith("ws"), case["sched"] == "streamk"
    c = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
    if quant:
        tb.matmul_a8w8_lt(a, b, sa.cuda(), sb.cuda(), c, sel, cfg, enable_streamk=sk, work_stealing=ws)
    elif bias is not None:
        from tritonblas_amd import _lib
        from tritonblas_amd.matmul import _launch_gemm
        sched = _lib.TB_SCHED_STREAMK if sk else (_lib.TB_SCHED_WORK_STEALING if ws else _lib.TB_SCHED_PERSISTENT)
        _launch_gemm(a, b, c, sel, cfg, sched, bias=bias.cuda())
    else:
        tb.matmul_lt(a, b, c, sel, cfg, enable_streamk=sk, work_stealing=ws)
    want = torch.matmul(a_cpu.double(), b_cpu.double())
    if quant:
        want = want * (sa.double()[:, None] * sb.double()[None, :])
    if bias is not None:
        want = want + bias.double()[None, :]
    got = c.cpu()
    assert torch.isfinite(got.float()).all(), "unwritten or non-finite outputs"
    err = OG.rel_fro_error(got.double(), want.float().to(out_dtype).double())
    assert err <= TOL[dtype], f"relative Frobenius error {err:.3e} > {TOL[dtype]}"


def _fp4_cases(n, seed):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        big = rng.random() < 0.3
        out.append(dict(idx=i, m=rng.randint(1, 900 if big else 200), n=rng.randint(1, 900 if big else 200),
                        k=32 * rng.choice([rng.randint(1, 40), 16 * rng.randint(1, 12), 16 * rng.randint(1, 12)]),
                        tile=rng.choice([None, None, (256, 256, 256), (128, 128, 256), (128, 128, 128), (64, 64, 256)]),
                        out=rng.choice([torch.bfloat16, torch.float16, torch.float32]), seed=rng.randint(0, 1 << 30)))
    return out


@pytest.mark.parametrize("case", _fp4_cases(max(8, int(os.environ.get("TB_RANDOM_CASES", "72")) // 3), 4242),
                         ids=lambda c: f"{c['idx']}-{c['m']}x{c['n']}x{c['k']}-{c['tile']}")
def test_random_fp4_case(case):
    """MXFP4: random codes and random, widely varying E8M0 scales; K any multiple of 32 (multiples of 512
    take the LDS-direct kernels, the rest the gather kernel), forced or selected tiles, three output types."""
    import numpy as np
    import tritonblas_amd as tb
    print("random fp4 case", case, flush=True)
    m, n, k = case["m"], case["n"], case["k"]
    rng = np.random.default_rng(case["seed"])
    xq = torch.from_numpy(rng.integers(0, 256, (m, k // 2), dtype=np.uint8))
    wq = torch.from_numpy(rng.integers(0, 256, (n, k // 2), dtype=np.uint8))
    hi = 129 if case["out"] == torch.float16 else 140      # (keep the sums inside the fp16 range)
    xs = torch.from_numpy(rng.integers(110, hi, (m, k // 32), dtype=np.uint8))
    ws = torch.from_numpy(rng.integers(110, hi, (n, k // 32), dtype=np.uint8))
    c = torch.full((m, n), float("nan"), dtype=case["out"], device="cuda")
    kw = {} if case["tile"] is None else dict(block_m=case["tile"][0], block_n=case["tile"][1], block_k=case["tile"][2])
    tb.matmul_fp4(xq.cuda(), wq.cuda(), c, xs.cuda(), ws.cuda(), **kw)
    want = OG.ref_gemm_fp4(xq, wq, xs, ws, return_fp32=True)
    got = c.cpu()
    assert torch.isfinite(got.float()).all()
    err = OG.rel_fro_error(got.double(), want.to(case["out"]).double())
    assert err <= (1e-5 if case["out"] == torch.float32 else 1e-3), f"relative Frobenius error {err:.3e}"


def _grouped_cases(n, seed):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        experts = rng.randint(1, 9)
        counts = [rng.choice([0, 1, rng.randint(1, 70), rng.randint(100, 600), 256, 257]) for _ in range(experts)]
        # plan: the library's own (0: one or two launches, priced on the device), one launch (-1), or the
        # tall tile forced and last row blocks of at most that many rows left to the second launch
        out.append(dict(idx=i, counts=counts, n=rng.choice([64, 200, 384, 1000]), k=rng.choice([128, 512, 1152, 1024]),
                        seed=rng.randint(0, 1 << 30), small_rows=rng.choice([0, 0, -1, 16, 32, 64, 100, 200])))
    return out


@pytest.mark.parametrize("case", _grouped_cases(max(6, int(os.environ.get("TB_RANDOM_CASES", "72")) // 6), 777),
                         ids=lambda c: f"{c['idx']}-{sum(c['counts'])}rows-{len(c['counts'])}experts-{c['n']}x{c['k']}")
def test_random_grouped_case(case):
    """Grouped FP8 GEMM over random per-expert row counts (empty experts, single rows, ragged blocks)."""
    import numpy as np
    import tritonblas_amd as tb
    print("random grouped case", case, flush=True)
    counts, n, k = case["counts"], case["n"], case["k"]
    m, E = sum(counts), len(counts)
    if m == 0:
        pytest.skip("no rows at all")
    offsets = torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32)
    g = torch.Generator().manual_seed(case["seed"])
    a = torch.randn(m, k, generator=g).bfloat16()
    w = torch.randn(E, n, k, generator=g).bfloat16()
    aq, sa = OG.quantize_per_channel_fp8(a, axis=1)
    wq, sw = OG.quantize_per_channel_fp8(w, axis=2)
    c = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    tile = (256, 256, 128) if case["small_rows"] > 0 else (None, None, None)
    tb.grouped_matmul_a8w8(aq.cuda(), wq.cuda(), sa.cuda(), sw.cuda(), c, offsets.cuda(), *tile, small_rows=case["small_rows"])
    want = OG.ref_grouped_gemm_fp8(aq, wq, sa, sw, offsets, return_fp32=True)
    got = c.cpu()
    assert torch.isfinite(got.float()).all()
    err = OG.rel_fro_error(got.double(), want.to(torch.bfloat16).double())
    assert err <= 1e-2, f"relative Frobenius error {err:.3e}"
