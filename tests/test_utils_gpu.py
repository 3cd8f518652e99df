"""GPU parity tests of the host-side helpers around the GEMMs (tritonblas_amd/utils.py, bench.py) against
the CPU oracle: the per-channel quantisation recipe as the product runs it on the GPU, the two
dequantisers on every byte value, the input generator's layout and seed rules, and the benchmark loop."""
import time

import numpy as np
import pytest
import torch

from oracle import gemm as OG
from oracle import mxfp4 as OM

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("shape", [(64, 96), (1000, 257), (2048, 4096)])
@pytest.mark.parametrize("src", [torch.float32, torch.bfloat16])
def test_quantize_per_channel_fp8_matches_oracle(shape, axis, src):
    """reference utils.py:340-377 (multiply by the reciprocal of the scale, then cast): the product's
    function on the GPU must give the oracle's (CPU) codes and scales bit for bit."""
    import tritonblas_amd.utils as U
    g = torch.Generator().manual_seed(3)
    x = torch.randn(shape, generator=g).to(src)
    x[5 % shape[0], :] = 0          # an all-zero channel along axis 1: the scale floor
    x[:, 7 % shape[1]] = 0          # ... and along axis 0
    q, s = U.quantize_tensor_per_channel(x.cuda(), torch.float8_e4m3fn, axis=axis)
    wq, ws = OG.quantize_per_channel_fp8(x, axis=axis)
    assert s.dtype == torch.float32 and tuple(s.shape) == tuple(ws.shape)
    assert torch.equal(s.cpu().view(torch.int32), ws.view(torch.int32))
    assert torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))


@pytest.mark.parametrize("axis", [0, 1])
def test_quantize_per_channel_int8_matches_oracle(axis):
    import tritonblas_amd.utils as U
    g = torch.Generator().manual_seed(4)
    x = torch.randn(513, 300, generator=g) * 3
    q, s = U.quantize_tensor_per_channel(x.cuda(), torch.int8, axis=axis)
    wq, ws = OG.quantize_per_channel_int8(x, axis=axis)
    assert torch.equal(s.cpu().view(torch.int32), ws.view(torch.int32))
    assert torch.equal(q.cpu(), wq)


def test_a8w8_gemm_with_the_products_quantiser():
    """The a8w8 path end to end as a caller runs it: the product's quantiser on the GPU feeds the GEMM;
    the oracle dequantises those very codes."""
    import tritonblas_amd as tb
    import tritonblas_amd.utils as U
    m, n, k = 512, 768, 1024
    g = torch.Generator().manual_seed(6)
    a = torch.randn(m, k, generator=g).bfloat16().cuda()
    w = torch.randn(n, k, generator=g).bfloat16().cuda()
    aq, sa = U.quantize_tensor_per_channel(a, torch.float8_e4m3fn, axis=1)
    bq, sb = U.quantize_tensor_per_channel(w.T, torch.float8_e4m3fn, axis=0)
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    tb.matmul_a8w8(aq, bq, sa, sb, c)
    want = OG.ref_gemm(aq.cpu(), bq.cpu(), torch.float32, a_scale=sa.cpu(), b_scale=sb.cpu()).to(torch.bfloat16)
    assert OG.rel_fro_error(c.float().cpu(), want.float()) <= 1e-2


def test_mxfp4_to_f32_every_byte():
    """reference utils.py:547-609: low nibble first, the 16-entry e2m1 table."""
    import tritonblas_amd.utils as U
    codes = torch.arange(256, dtype=torch.uint8).reshape(16, 16)
    got = U.mxfp4_to_f32(codes.cuda()).cpu().numpy()
    want = OM.mxfp4_to_f32(codes.numpy())
    assert got.shape == (16, 32)
    assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))   # (-0.0 included)


def test_e8m0_to_f32_every_byte():
    """reference utils.py:612-643: 2**(b-127), byte 0 -> 2**-127 (a denormal), byte 255 -> NaN."""
    import tritonblas_amd.utils as U
    b = torch.arange(256, dtype=torch.uint8)
    got = U.e8m0_to_f32(b.cuda()).cpu().numpy()
    want = OM.e8m0_to_f32(b.numpy()).astype(np.float32)
    assert np.isnan(got[255]) and np.isnan(want[255])
    assert np.array_equal(got[:255].view(np.uint32), want[:255].view(np.uint32))
    assert got[0] == np.ldexp(np.float32(1.0), -127) and got[127] == 1.0


@pytest.mark.parametrize("transA", ["T", "N"])
@pytest.mark.parametrize("transB", ["T", "N"])
def test_generate_matmul_inputs_layout_and_seeds(transA, transB):
    """reference utils.py:495-505: "T" keeps the logical shape contiguous, "N" stores the transpose and
    hands out a view; B is drawn with seed + 10000."""
    import tritonblas_amd.utils as U
    m, n, k, seed = 96, 160, 64, 42
    t = U.generate_matmul_inputs(m, n, k, torch.float16, torch.float16, transA, transB, "randn", seed=seed)
    assert tuple(t.A.shape) == (m, k) and tuple(t.B.shape) == (k, n) and tuple(t.C.shape) == (m, n)
    assert t.A.stride() == ((k, 1) if transA == "T" else (1, m))
    assert t.B.stride() == ((n, 1) if transB == "T" else (1, k))

    def draw(shape, s):
        g = torch.Generator(device="cuda")
        g.manual_seed(s)
        return torch.randn(shape, dtype=torch.float32, device="cuda", generator=g).half()

    assert torch.equal(t.A, draw((m, k), seed) if transA == "T" else draw((k, m), seed).T)
    assert torch.equal(t.B, draw((k, n), seed + 10000) if transB == "T" else draw((n, k), seed + 10000).T)
    again = U.generate_matmul_inputs(m, n, k, torch.float16, torch.float16, transA, transB, "randn", seed=seed)
    assert torch.equal(again.A, t.A) and torch.equal(again.B, t.B)


def test_generate_matmul_inputs_quantised():
    import tritonblas_amd.utils as U
    t = U.generate_matmul_inputs(128, 256, 512, torch.float8_e4m3fn, torch.bfloat16, "T", "N", seed=1)
    assert t.A.dtype == torch.float8_e4m3fn and t.scaleA.shape == (128,) and t.scaleB.shape == (256,)
    assert t.B.stride() == (1, 512)
    f = U.generate_matmul_inputs(64, 64, 256, "fp4", torch.bfloat16, seed=1)
    assert f.A.dtype == torch.uint8 and tuple(f.A.shape) == (64, 128) and tuple(f.scaleA.shape) == (64, 8)


def test_do_bench_shape_and_untimed_callbacks():
    """reference bench.py:64-131: warm-up + repeat calls, quantiles / modes, and the reset / preamble
    callbacks (and the cache flush) run outside the timed events."""
    import tritonblas_amd as tb
    x = torch.zeros(1 << 10, device="cuda")
    big = torch.randn(4096, 4096, device="cuda")
    calls = {"fn": 0, "reset": 0, "pre": 0}

    def fn():
        calls["fn"] += 1
        x.add_(1)

    def reset():
        calls["reset"] += 1
        for _ in range(4):
            torch.mm(big, big)      # milliseconds of GPU work that must not show up in the timings

    def pre():
        calls["pre"] += 1

    times = tb.do_bench(fn, reset_fn=reset, preamble_fn=pre, n_warmup=3, n_repeat=7, return_mode="all")
    assert len(times) == 7 and calls == {"fn": 10, "reset": 10, "pre": 10}
    assert max(times) < 1.0, f"a callback was timed: {times}"       # ms; four 4096^3 GEMMs take several ms
    q = tb.do_bench(fn, n_warmup=1, n_repeat=5, quantiles=[0.2, 0.5, 0.8])
    assert len(q) == 3 and q[0] <= q[1] <= q[2]
    for mode in ("min", "max", "mean", "median"):
        assert isinstance(tb.do_bench(fn, n_warmup=1, n_repeat=3, return_mode=mode, flush=False), float)
