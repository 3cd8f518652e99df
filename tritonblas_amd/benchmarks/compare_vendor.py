"""Side-by-side timing of this library and the vendor library PyTorch dispatches to (hipBLASLt through
torch.matmul / torch._scaled_mm) on the same tensors.

    python -m tritonblas_amd.benchmarks.compare_vendor [--shapes fp8,bf16,decode,mxfp4] [--steps 40] [--settle-ms 40]

Cases: "fp8" = a8w8 8192x28672x8192 with per-row / per-column scales (torch._scaled_mm row-wise is the
same operation; its tensor-wise form, one scale per tensor, is the simpler problem the vendor ships a
hand-written kernel for) and "bf16" = 8192^3 with K-major operands.  Every timing starts after
`settle-ms` of untimed launches of the same call (the engine clock needs tens of milliseconds of load
to settle) and is the average of `steps` back-to-back launches between two events.  "decode" = a8w8
32x8192x28672 (the 235 MB weight is the traffic): timed back to back and with the caches flushed before
every launch (do_bench), next to a plain device copy of as many bytes under the same flush.  "mxfp4" = the MXFP4
GEMM 8192x8192x16384 (e2m1 codes, one E8M0 scale per 32 values of K) against torch._scaled_mm on the same packed
operands and scale bytes (hipBLASLt's block-scaled kernel), with N(0,1) data and with all-zero codes (the second
shows what the kernels do when the engine clock is not held down by the power of the multipliers).  One JSON line per
case on stdout.  Run it under `rocprofv3 --kernel-trace --stats` or `--pmc` to see the kernels behind
each call.
"""
import argparse
import json
import sys
import time

import torch


def timed(fn, steps, settle_ms):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < settle_ms:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def case_fp8(steps, settle_ms, dev):
    import tritonblas_amd as tb
    import tritonblas_amd.utils as U
    m, n, k = 8192, 28672, 8192
    g = torch.Generator(device=dev).manual_seed(2)
    a = torch.randn(m, k, device=dev, generator=g).bfloat16()
    w = torch.randn(n, k, device=dev, generator=g).bfloat16()
    aq, sa = U.quantize_tensor_per_channel(a, torch.float8_e4m3fn, axis=1)
    wq, sw = U.quantize_tensor_per_channel(w, torch.float8_e4m3fn, axis=1)
    del a, w
    c = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    sel = tb.OrigamiMatmulSelector(m, n, k, aq.dtype, wq.dtype, c.dtype, dev)
    out = {"case": "fp8 a8w8 8192x28672x8192, bf16 out", "flops": 2.0 * m * n * k}
    out["this_library_ms"] = timed(lambda: tb.matmul_a8w8_lt(aq, wq.T, sa, sw, c, sel, None), steps, settle_ms)
    sa2, sw2 = sa.reshape(m, 1).contiguous(), sw.reshape(1, n).contiguous()
    try:
        ref = torch._scaled_mm(aq, wq.T, scale_a=sa2, scale_b=sw2, out_dtype=torch.bfloat16)
        out["vendor_rowwise_ms"] = timed(lambda: torch._scaled_mm(aq, wq.T, scale_a=sa2, scale_b=sw2, out_dtype=torch.bfloat16, out=c),
                                         steps, settle_ms)
        tb.matmul_a8w8_lt(aq, wq.T, sa, sw, c, sel, None)
        torch.cuda.synchronize()
        rows = slice(0, 512)
        out["rel_fro_between_the_two"] = float(((c[rows].float() - ref[rows].float()).norm() / ref[rows].float().norm()).item())
        del ref
    except Exception as e:   # (the row-wise form is not available in every PyTorch build)
        out["vendor_rowwise_error"] = str(e)[:200]
    one_a, one_w = torch.ones((), device=dev), torch.ones((), device=dev)
    try:
        out["vendor_tensorwise_ms"] = timed(lambda: torch._scaled_mm(aq, wq.T, scale_a=one_a, scale_b=one_w, out_dtype=torch.bfloat16, out=c),
                                            steps, settle_ms)
    except Exception as e:
        out["vendor_tensorwise_error"] = str(e)[:200]
    return out


def case_bf16(steps, settle_ms, dev):
    import tritonblas_amd as tb
    m = n = k = 8192
    g = torch.Generator(device=dev).manual_seed(3)
    a = (torch.rand(m, k, device=dev, generator=g) * 2 - 1).bfloat16()
    b = (torch.rand(n, k, device=dev, generator=g) * 2 - 1).bfloat16().T
    c = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, c.dtype, dev)
    out = {"case": "bf16 8192x8192x8192, K-major operands", "flops": 2.0 * m * n * k}
    out["this_library_ms"] = timed(lambda: tb.matmul_lt(a, b, c, sel, None), steps, settle_ms)
    out["vendor_ms"] = timed(lambda: torch.matmul(a, b, out=c), steps, settle_ms)
    return out


def case_decode(steps, settle_ms, dev):
    import tritonblas_amd as tb
    import tritonblas_amd.utils as U
    m, n, k = 32, 8192, 28672
    g = torch.Generator(device=dev).manual_seed(22)
    a = torch.randn(m, k, device=dev, generator=g).bfloat16()
    w = torch.randn(n, k, device=dev, generator=g).bfloat16()
    aq, sa = U.quantize_tensor_per_channel(a, torch.float8_e4m3fn, axis=1)
    wq, sw = U.quantize_tensor_per_channel(w, torch.float8_e4m3fn, axis=1)
    del a, w
    c = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    sel = tb.OrigamiMatmulSelector(m, n, k, aq.dtype, wq.dtype, c.dtype, dev, streamk=True)
    cfg = tb.matmul_preamble(sel, dev)
    ours = lambda: tb.matmul_a8w8_lt(aq, wq.T, sa, sw, c, sel, cfg, enable_streamk=True)
    sa2, sw2 = sa.reshape(m, 1).contiguous(), sw.reshape(1, n).contiguous()
    vendor = lambda: torch._scaled_mm(aq, wq.T, scale_a=sa2, scale_b=sw2, out_dtype=torch.bfloat16, out=c)
    nbytes = m * k + n * k + m * n * 2 + (m + n) * 4
    out = {"case": "fp8 a8w8 decode 32x8192x28672, bf16 out", "flops": 2.0 * m * n * k, "bytes": nbytes}
    out["this_library_ms"] = timed(ours, steps * 4, settle_ms / 4)
    out["this_library_flushed_ms"] = tb.do_bench(ours, n_warmup=5, n_repeat=40, return_mode="median")
    try:
        out["vendor_rowwise_ms"] = timed(vendor, steps * 4, settle_ms / 4)
        out["vendor_rowwise_flushed_ms"] = tb.do_bench(vendor, n_warmup=5, n_repeat=40, return_mode="median")
    except Exception as e:
        out["vendor_rowwise_error"] = str(e)[:200]
    x = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    y = torch.empty_like(x)
    out["plain_copy_of_as_many_bytes_flushed_ms"] = tb.do_bench(lambda: y.copy_(x), n_warmup=3, n_repeat=20, return_mode="median")
    return out


def case_mxfp4(steps, settle_ms, dev):
    import tritonblas_amd as tb
    import tritonblas_amd.utils as U
    m, n, k = 8192, 8192, 16384
    g = torch.Generator(device=dev).manual_seed(5)
    a = torch.randn(m, k, device=dev, generator=g).bfloat16()
    w = torch.randn(n, k, device=dev, generator=g).bfloat16()
    aq, sa = U.dynamic_mxfp4_quant(a)
    wq, sw = U.dynamic_mxfp4_quant(w)
    del a, w
    c = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    out = {"case": "mxfp4 8192x8192x16384, bf16 out", "flops": 2.0 * m * n * k}
    out["this_library_ms"] = timed(lambda: tb.matmul_fp4(aq, wq, c, sa, sw), steps, settle_ms)
    az, wz = torch.zeros_like(aq), torch.zeros_like(wq)
    s1a, s1w = torch.full_like(sa, 127), torch.full_like(sw, 127)
    out["this_library_zero_data_ms"] = timed(lambda: tb.matmul_fp4(az, wz, c, s1a, s1w), steps, settle_ms)
    try:
        f4, e8 = torch.float4_e2m1fn_x2, torch.float8_e8m0fnu
        va, vw, vsa, vsw = aq.view(f4), wq.view(f4), sa.view(e8), sw.view(e8)
        vendor = lambda x, y, p, q: torch._scaled_mm(x, y.t(), scale_a=p, scale_b=q, out_dtype=torch.bfloat16)
        ref = vendor(va, vw, vsa, vsw)
        tb.matmul_fp4(aq, wq, c, sa, sw)
        torch.cuda.synchronize()
        rows = slice(0, 512)
        out["rel_fro_between_the_two"] = float(((c[rows].float() - ref[rows].float()).norm() / ref[rows].float().norm()).item())
        del ref
        out["vendor_ms"] = timed(lambda: vendor(va, vw, vsa, vsw), steps, settle_ms)
        out["vendor_zero_data_ms"] = timed(lambda: vendor(az.view(f4), wz.view(f4), s1a.view(e8), s1w.view(e8)), steps, settle_ms)
    except Exception as e:   # (block-scaled FP4 through torch is not there in every PyTorch / hipBLASLt build)
        out["vendor_error"] = f"{type(e).__name__}: {str(e)[:200]}"
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--shapes", default="fp8,bf16")
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--settle-ms", type=float, default=40.0)
    args = ap.parse_args(argv)
    dev = torch.device("cuda", torch.cuda.current_device())
    for name in args.shapes.split(","):
        fn = {"fp8": case_fp8, "bf16": case_bf16, "decode": case_decode, "mxfp4": case_mxfp4}.get(name.strip())
        if fn is None:
            print(f"unknown case {name!r}", file=sys.stderr)
            return 2
        r = fn(args.steps, args.settle_ms, dev)
        for key in list(r):
            if key.endswith("_ms"):
                if "bytes" in r:
                    r[key.replace("_ms", "_TBps")] = round(r["bytes"] / r[key] / 1e9, 2)
                else:
                    r[key.replace("_ms", "_tflops")] = round(r["flops"] / r[key] / 1e9, 1)
                r[key] = round(r[key], 4)
        print(json.dumps(r), flush=True)
        torch.cuda.empty_cache()
    return 0


if __name__ == "__main__":
    sys.exit(main())
