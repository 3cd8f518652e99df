"""Headline benchmark: FP8 a8w8 GEMM 8192x28672x8192 (per-row / per-column scales, bf16 out) on one
MI355X, plus the MXFP4 GEMM 8192x8192x16384, the fused Hadamard+MXFP4 quantiser and the other
configurations as secondary figures on the same JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one launch of the FP8 GEMM with all operands resident in HBM.  The CPU baseline is
torch.matmul in fp32 on the host cores over the dequantised operands of a bounded row slice.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "mxfp4": 10100.0, "fp32": 157.3}
PEAK_HBM_GBPS = 8000.0


def timed(fn, steps, warmup, settle_ms=0.0):
    """K back-to-back launches between two events on the launch stream; returns ms per launch.
    settle_ms: keep launching (untimed) until that much time has passed after the warm-up launches --
    after an idle or memory-bound phase the engine clock takes tens of milliseconds of load to settle,
    and a short GEMM measured in that window reads 5-25 % slow (measured: MXFP4 8192x8192x16384
    0.45-0.53 ms over the first 13 launches, 0.418 ms from the 30th on)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    if settle_ms > 0:
        t_settle = time.perf_counter()
        while (time.perf_counter() - t_settle) * 1e3 < settle_ms:
            for _ in range(4):
                fn()
            torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(end) / steps, wall_ms


def timed_rotating(fns, steps, warmup):
    """HBM-bound kernels on cold data: back-to-back launches that cycle through several operand sets which together
    exceed the 256 MB memory-side cache (what one launch leaves there is gone when its set comes up again), with no
    flush in between whose write-back would share the memory bus with the timed kernel.  Returns ms per launch."""
    n = len(fns)
    for i in range(warmup):
        fns[i % n]()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        fns[i % n]()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def library_id():
    """First 12 hex digits of the SHA-256 of the shared library that is loaded: names the build a
    profile summary was taken from."""
    import hashlib
    from tritonblas_amd import _lib
    try:
        with open(_lib.LIB_PATH, "rb") as f:
            return hashlib.sha256(f.read()).hexdigest()[:12]
    except OSError:
        return None


def profile_summary(name):
    """A committed rocprofv3 summary (profiles/<name>.json) -- but only if it was taken from the very
    library build that is running now; a summary of another build says nothing about this one."""
    path = os.path.join(ROOT, "profiles", name + ".json")
    try:
        with open(path) as f:
            d = json.load(f)
    except (OSError, ValueError):
        return None
    return d if d.get("library_id") == library_id() else None


def host_us_per_call(fn, calls=300):
    """Host time of one call of an asynchronous launch: wall time of back-to-back calls before the
    synchronisation (the queue takes them faster than the GPU runs them, or the figure is the GPU's)."""
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(calls):
        fn()
    dt = time.perf_counter() - t0
    torch.cuda.synchronize()
    return dt / calls * 1e6


def fp8_inputs(m, n, k, dev, seed):
    import tritonblas_amd.utils as U
    g = torch.Generator(device=dev).manual_seed(seed)
    a = torch.randn(m, k, device=dev, generator=g, dtype=torch.float32).bfloat16()
    w = torch.randn(n, k, device=dev, generator=g, dtype=torch.float32).bfloat16()
    aq, sa = U.quantize_tensor_per_channel(a, torch.float8_e4m3fn, axis=1)
    wq, sw = U.quantize_tensor_per_channel(w, torch.float8_e4m3fn, axis=1)
    del a, w
    return aq, wq, sa, sw


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--skip-secondary", action="store_true")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (known HBM bytes) so that FETCH_SIZE / WRITE_SIZE "
                         "readings of a rocprofv3 --pmc run can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    import tritonblas_amd as tb
    import tritonblas_amd.utils as U
    from oracle import gemm as OG

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- headline: FP8 a8w8 prefill ------------------------------------------------------------
    M, N, K = 8192, 28672, 8192
    aq, wq, sa, sw = fp8_inputs(M, N, K, dev, 2)
    b = wq.T                                   # (K, N) view of the (N, K) weight: K-contiguous
    c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    sel = tb.OrigamiMatmulSelector(M, N, K, aq.dtype, b.dtype, c.dtype, dev)
    cfg = tb.matmul_preamble(sel, dev)
    step = lambda: tb.matmul_a8w8_lt(aq, b, sa, sw, c, sel, cfg)
    # (the W warm-up launches are followed by untimed launches until 40 ms have passed, so that a small W
    # does not put the timed launches into the window in which the engine clock is still settling)
    ms, wall_ms = timed(step, args.steps, args.warmup, settle_ms=40.0)
    flops = 2.0 * M * N * K
    tflops = flops / (ms * 1e-3) / 1e12

    # parity spot check on rows spread over the output (oracle on the host): against the oracle rounded
    # to bf16 like the kernel's epilogue rounds, and against the unrounded fp32 GEMM (that figure carries
    # the bf16 rounding of the output itself, about 1.5e-3)
    rows = torch.arange(0, M, 613)[:14]
    want32 = OG.ref_gemm(aq[rows].cpu(), b.cpu(), torch.float32, a_scale=sa[rows].cpu(), b_scale=sw.cpu())
    err = OG.rel_fro_error(c[rows].float().cpu(), want32.to(torch.bfloat16).float())
    err_unrounded = OG.rel_fro_error(c[rows].float().cpu(), want32)
    traffic = profile_summary("fp8_gemm_8192x28672x8192_hbm_traffic")
    clock = profile_summary("fp8_gemm_8192x28672x8192_mfma_busy")

    out = {
        "metric": "TFLOP/s & % MFMA peak: FP8 a8w8 8192x28672x8192; MXFP4 8192x8192x16384",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_ms_after_warmup": 40.0,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3", "data": "synthetic (seeded N(0,1) bf16, per-row/per-column amax/448 scales)",
        "config": {"workload": "FP8 a8w8 GEMM M=8192 N=28672 K=8192, bf16 out, scales in epilogue",
                   "tile": [sel.block_m, sel.block_n, sel.block_k], "schedule": "persistent"},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_TFLOPS["fp8"], "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_TFLOPS["fp8"], 4),
                     "traffic": traffic["hbm_bytes_per_launch"] if traffic else None,
                     "traffic_from": f"profiles/fp8_gemm_8192x28672x8192_hbm_traffic.json, library {traffic['library_id']}" if traffic
                                     else "no counter summary of this library build is committed",
                     # the part is power limited under this kernel: what the same work would be worth at the clock it sustained
                     "sustained_clock_ghz": clock["engine_clock_ghz"] if clock else None,
                     "frac_at_sustained_clock": round(tflops / (PEAK_TFLOPS["fp8"] * clock["engine_clock_ghz"] / 2.4), 4) if clock else None,
                     "mfma_busy_in_cycles": clock["mfma_busy"] if clock else None},
        "library_id": library_id(),
        "parity_rel_fro": float(f"{err:.3e}"),
        "parity_rel_fro_vs_unrounded_fp32": float(f"{err_unrounded:.3e}"),
        "wall_ms_per_step": round(wall_ms, 4),
        "device": {"name": props.name, "cus": props.multi_processor_count, "arch": getattr(props, "gcnArchName", ""),
                   "engine_clock_khz": int(sel._hardware._c.clock_khz), "memory_clock_khz": int(sel._hardware._c.mem_clock_khz),
                   "note": "peak clocks the runtime reports; the clock a kernel really ran at is in profiles/*_mfma_busy.txt"},
    }

    # ---- CPU baseline: torch.matmul fp32 over a bounded row slice of the same problem -----------
    if not args.skip_cpu:
        ms_rows = 8192
        a_s = aq[:ms_rows].cpu()
        b_cpu = b.cpu()
        a32, b32 = a_s.to(torch.float32), b_cpu.to(torch.float32)
        torch.matmul(a32[:64], b32)
        best = None
        for _ in range(5):      # (about 12 s of CPU work in all on the box's 16 threads)
            t0 = time.perf_counter()
            OG.ref_gemm(a_s, b_cpu, torch.float32, a_scale=sa[:ms_rows].cpu(), b_scale=sw.cpu())
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        out["cpu_baseline"] = {"value": round(2.0 * ms_rows * N * K / best / 1e12, 4), "unit": "TFLOP/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"rows 0..{ms_rows - 1} of the same GEMM ({ms_rows}x{N}x{K}), "
                                         f"oracle fp32 torch.matmul of the dequantised operands + scale epilogue, best of 5, "
                                         f"{best:.2f} s; os.cpu_count()={os.cpu_count()}"}
        del a32, b32, b_cpu
    del aq, wq, c, b

    # ---- secondary figures ----------------------------------------------------------------------
    if not args.skip_secondary:
        sec = {}
        steps2, warm2 = max(10, args.steps // 2), max(3, args.warmup // 2)
        # MXFP4: quantise A with the fused rotate+quant kernel (timed), B rotated + quantised the same way
        M4, N4, K4 = 8192, 8192, 16384
        g = torch.Generator(device=dev).manual_seed(5)
        def src(rows):
            x = torch.randn(rows, K4, device=dev, generator=g, dtype=torch.float32)
            mask = torch.rand(rows, K4, device=dev, generator=g) < 1e-3
            return torch.where(mask, x * 20.0, x).bfloat16()
        a4, b4 = src(M4), src(N4)
        qout = U.hadamard_mxfp4_quant(a4)
        qms, _ = timed(lambda: U.hadamard_mxfp4_quant(a4, out=qout), steps2 * 4, warm2)
        # HBM-bound kernels are timed a second time with the caches flushed before every launch (the
        # reference's benchmark loop, bench.py:64-131: 512 MiB rewritten outside the timed events); the
        # fraction of the HBM peak is the flushed figure, the back-to-back one is cache assisted
        qms_cold = tb.do_bench(lambda: U.hadamard_mxfp4_quant(a4, out=qout), n_warmup=5, n_repeat=40, return_mode="median")
        qbytes = M4 * K4 * 2 + M4 * K4 // 2 + M4 * K4 // 32
        # third way, and the one the HBM fraction is taken from: four operand sets in turn (4 x 340 MB against a 256 MB
        # memory-side cache), back to back, nothing flushed; a plain device copy that moves as many bytes, timed the
        # same way over four buffer pairs, is the yard-stick
        xsets = [a4] + [a4.roll(i + 1, 0) for i in range(3)]
        osets = [qout] + [(torch.empty_like(qout[0]), torch.empty_like(qout[1])) for _ in range(3)]
        qms_rot = timed_rotating([(lambda x=x, o=o: U.hadamard_mxfp4_quant(x, out=o)) for x, o in zip(xsets, osets)], steps2 * 4, 8)
        csrc = [torch.empty(qbytes // 2, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(4)]
        cdst = [torch.empty_like(x) for x in csrc]
        copy_rot = timed_rotating([(lambda x=x, y=y: y.copy_(x)) for x, y in zip(csrc, cdst)], steps2 * 4, 8)
        del xsets, osets, csrc, cdst
        sec["hadamard_mxfp4_quant_8192x16384"] = {"ms": round(qms_rot, 4), "GB/s": round(qbytes / qms_rot / 1e6, 1),
                                                  "frac_hbm_peak": round(qbytes / qms_rot / 1e6 / PEAK_HBM_GBPS, 4),
                                                  "timing": "four operand sets in turn (1.36 GB > the 256 MB memory-side cache), back to back, no flush",
                                                  "plain_copy_of_as_many_bytes_same_way_ms": round(copy_rot, 4),
                                                  "plain_copy_GB/s": round(qbytes / copy_rot / 1e6, 1),
                                                  "flushed_ms": round(qms_cold, 4), "flushed_GB/s": round(qbytes / qms_cold / 1e6, 1),
                                                  "hot_ms": round(qms, 4), "hot_GB/s": round(qbytes / qms / 1e6, 1),
                                                  "note": "bf16 in, codes + E8M0 scales out, outputs preallocated; flushed = the "
                                                          "reference's do_bench loop (512 MiB rewritten before every launch), hot = one set back to back"}
        aq4, as4 = qout
        bq4, bs4 = U.hadamard_mxfp4_quant(b4)
        a4_sample = a4[:128].float().cpu().numpy()
        del a4, b4
        c4 = torch.empty(M4, N4, dtype=torch.bfloat16, device=dev)
        fms, _ = timed(lambda: tb.matmul_fp4(aq4, bq4, c4, as4, bs4), steps2, warm2, settle_ms=40.0)
        tf4 = 2.0 * M4 * N4 * K4 / fms / 1e9
        clock4 = profile_summary("mxfp4_gemm_8192x8192x16384_mfma_busy")
        sec["mxfp4_gemm_8192x8192x16384"] = {
            "ms": round(fms, 4), "TFLOP/s": round(tf4, 1), "frac_mfma_peak": round(tf4 / PEAK_TFLOPS["mxfp4"], 4),
            "roofline": {"bound": "mfma", "achieved": round(tf4, 1), "peak": PEAK_TFLOPS["mxfp4"], "unit": "TFLOP/s",
                         "frac": round(tf4 / PEAK_TFLOPS["mxfp4"], 4),
                         "sustained_clock_ghz": clock4["engine_clock_ghz"] if clock4 else None,
                         "mfma_busy_in_cycles": clock4["mfma_busy"] if clock4 else None,
                         "counters_from": f"profiles/mxfp4_gemm_8192x8192x16384_mfma_busy.json, library {clock4['library_id']}" if clock4
                                          else "no counter summary of this library build is committed"}}
        # parity spot check and CPU baseline: the oracle's GEMM of the dequantised operands on rows spread over the output
        rows4 = torch.arange(0, M4, 4)[:2048] if not args.skip_cpu else torch.arange(0, M4, 613)[:14]
        a_rows, as_rows, b_cpu4, bs_cpu4 = aq4[rows4].cpu(), as4[rows4].cpu(), bq4.cpu(), bs4.cpu()
        best4, want4 = None, None
        for _ in range(1 if args.skip_cpu else 2):
            t0 = time.perf_counter()
            want4 = OG.ref_gemm_fp4(a_rows, b_cpu4, as_rows, bs_cpu4, return_fp32=True)
            dt = time.perf_counter() - t0
            best4 = dt if best4 is None else min(best4, dt)
        sec["mxfp4_gemm_8192x8192x16384"]["parity_rel_fro"] = float(f"{OG.rel_fro_error(c4[rows4].float().cpu(), want4.to(torch.bfloat16).float()):.3e}")
        if not args.skip_cpu:
            sec["mxfp4_gemm_8192x8192x16384"]["cpu_baseline"] = {
                "value": round(2.0 * len(rows4) * N4 * K4 / best4 / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"every fourth row, {len(rows4)} rows, of the same GEMM ({len(rows4)}x{N4}x{K4}): oracle dequantisation (numpy) of both "
                          f"operands + fp32 torch.mm, best of 2, {best4:.2f} s"}
        del a_rows, as_rows, b_cpu4, bs_cpu4, want4
        q_sample = (aq4[:128].cpu().numpy(), as4[:128].cpu().numpy())
        del aq4, bq4, c4
        # fp16 1024^3 (the plumbing configuration): launch bound, so the host's share of a call matters
        a1 = (torch.randn(1024, 1024, device=dev, generator=g) * 0.1).half()
        b1 = (torch.randn(1024, 1024, device=dev, generator=g) * 0.1).half()
        c1 = torch.empty(1024, 1024, dtype=torch.float16, device=dev)
        sel1 = tb.OrigamiMatmulSelector(1024, 1024, 1024, a1.dtype, b1.dtype, c1.dtype, dev)
        c1_call = lambda: tb.matmul_lt(a1, b1, c1, sel1, None)
        c1ms, _ = timed(c1_call, steps2 * 8, warm2)
        sec["fp16_gemm_1024x1024x1024"] = {"ms": round(c1ms, 5), "TFLOP/s": round(2.0 * 1024 ** 3 / c1ms / 1e9, 1),
                                           "host_us_per_call": round(host_us_per_call(c1_call), 2),
                                           "note": "matmul_lt through the Python wrapper and ctypes; host time = wall time of "
                                                   "back-to-back asynchronous calls before any synchronisation"}
        del a1, b1, c1
        # bf16 TN 8192^3
        a2 = (torch.rand(8192, 8192, device=dev, generator=g) * 2 - 1).bfloat16()
        b2 = (torch.rand(8192, 8192, device=dev, generator=g) * 2 - 1).bfloat16().T
        c2 = torch.empty(8192, 8192, dtype=torch.bfloat16, device=dev)
        sel2 = tb.OrigamiMatmulSelector(8192, 8192, 8192, a2.dtype, b2.dtype, c2.dtype, dev)
        bms, _ = timed(lambda: tb.matmul_lt(a2, b2, c2, sel2, None), steps2, warm2, settle_ms=40.0)
        tf2 = 2.0 * 8192 ** 3 / bms / 1e9
        sec["bf16_gemm_8192x8192x8192_TN"] = {"ms": round(bms, 4), "TFLOP/s": round(tf2, 1),
                                              "frac_mfma_peak": round(tf2 / PEAK_TFLOPS["bf16"], 4)}
        del a2, b2, c2
        # fp32 TN 8192^3 (16x16x4 fp32 MFMA: full fp32 products)
        a3 = (torch.rand(8192, 8192, device=dev, generator=g) * 2 - 1)
        b3 = (torch.rand(8192, 8192, device=dev, generator=g) * 2 - 1).T
        c3 = torch.empty(8192, 8192, dtype=torch.float32, device=dev)
        sel3 = tb.OrigamiMatmulSelector(8192, 8192, 8192, a3.dtype, b3.dtype, c3.dtype, dev)
        f32ms, _ = timed(lambda: tb.matmul_lt(a3, b3, c3, sel3, None), max(5, steps2 // 2), 2)
        tf3 = 2.0 * 8192 ** 3 / f32ms / 1e9
        sec["fp32_gemm_8192x8192x8192_TN"] = {"ms": round(f32ms, 4), "TFLOP/s": round(tf3, 1),
                                              "frac_mfma_peak": round(tf3 / PEAK_TFLOPS["fp32"], 4)}
        del a3, b3, c3
        # FP8 decode: for M <= 64 the library compares the model times of its streaming kernel and of the Stream-K tile kernel
        Md, Nd, Kd = 32, 8192, 28672
        aqd, wqd, sad, swd = fp8_inputs(Md, Nd, Kd, dev, 22)
        cd = torch.empty(Md, Nd, dtype=torch.bfloat16, device=dev)
        seld = tb.OrigamiMatmulSelector(Md, Nd, Kd, aqd.dtype, wqd.dtype, cd.dtype, dev, streamk=True)
        cfgd = tb.matmul_preamble(seld, dev)
        decode = lambda: tb.matmul_a8w8_lt(aqd, wqd.T, sad, swd, cd, seld, cfgd, enable_streamk=True)
        dms, _ = timed(decode, steps2 * 4, warm2)
        dms_cold = tb.do_bench(decode, n_warmup=5, n_repeat=40, return_mode="median")
        dbytes = Md * Kd + Nd * Kd + Md * Nd * 2 + (Md + Nd) * 4
        # cold data without a flush: four weight matrices in turn (4 x 235 MB against the 256 MB memory-side cache);
        # yard-stick: a plain device copy that moves as many bytes, four buffer pairs in turn
        wsets = [wqd] + [wqd.view(torch.uint8).roll(i + 1, 0).view(wqd.dtype) for i in range(3)]
        dms_rot = timed_rotating([(lambda w=w: tb.matmul_a8w8_lt(aqd, w.T, sad, swd, cd, seld, cfgd, enable_streamk=True)) for w in wsets],
                                 steps2 * 4, 8)
        csrc = [torch.empty(dbytes // 2, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(4)]
        cdst = [torch.empty_like(x) for x in csrc]
        dcopy_rot = timed_rotating([(lambda x=x, y=y: y.copy_(x)) for x, y in zip(csrc, cdst)], steps2 * 4, 8)
        del wsets, csrc, cdst
        sec["fp8_decode_32x8192x28672"] = {"ms": round(dms_rot, 4), "GB/s": round(dbytes / dms_rot / 1e6, 1),
                                           "frac_hbm_peak": round(dbytes / dms_rot / 1e6 / PEAK_HBM_GBPS, 4),
                                           "timing": "four weight matrices in turn (940 MB > the 256 MB memory-side cache), back to back, no flush",
                                           "plain_copy_of_as_many_bytes_same_way_ms": round(dcopy_rot, 4),
                                           "plain_copy_GB/s": round(dbytes / dcopy_rot / 1e6, 1),
                                           "flushed_ms": round(dms_cold, 4), "flushed_GB/s": round(dbytes / dms_cold / 1e6, 1),
                                           "hot_ms": round(dms, 4), "hot_GB/s": round(dbytes / dms / 1e6, 1),
                                           "host_us_per_call": round(host_us_per_call(decode), 2),
                                           "kernel": f"enable_streamk=True call; the library picks between the Stream-K tile kernel "
                                                     f"(selector: {seld.block_m}x{seld.block_n}x{seld.block_k} tiles, grid {seld.sk_grid}) "
                                                     f"and its streaming small-M kernel by model time"}
        del aqd, wqd, cd
        # grouped MoE FP8
        E, Ng, Kg, T = 8, 14336, 4096, 4096
        idx = torch.multinomial(torch.ones(T, E), 2, replacement=False, generator=torch.Generator().manual_seed(3))
        counts = torch.bincount(idx.flatten(), minlength=E)
        offs = torch.zeros(E + 1, dtype=torch.int32)
        offs[1:] = torch.cumsum(counts, 0).to(torch.int32)
        ag = torch.randn(2 * T, Kg, device=dev, generator=g).bfloat16()
        wg = torch.randn(E, Ng, Kg, device=dev, generator=g).bfloat16()
        agq, sag = U.quantize_tensor_per_channel(ag, torch.float8_e4m3fn, axis=1)
        wgq, swg = U.quantize_tensor_per_channel(wg, torch.float8_e4m3fn, axis=2)
        del ag, wg
        cg = torch.empty(2 * T, Ng, dtype=torch.bfloat16, device=dev)
        offs_d = offs.to(dev)
        gms, _ = timed(lambda: tb.grouped_matmul_a8w8(agq, wgq, sag, swg, cg, offs_d), steps2, warm2, settle_ms=40.0)
        tfg = 2.0 * 2 * T * Ng * Kg / gms / 1e9
        sec["grouped_moe_fp8_8x[rows x 4096]x[4096 x 14336]"] = {"ms": round(gms, 4), "TFLOP/s": round(tfg, 1),
                                                                 "frac_mfma_peak": round(tfg / PEAK_TFLOPS["fp8"], 4)}
        if not args.skip_cpu:
            # the oracle's numpy restatement of the same kernel on a bounded row sample: CPU baseline and bit-exact check
            from oracle import mxfp4 as OM
            rows_q = 128
            xs = a4_sample
            t0 = time.perf_counter()
            codes_ref, scales_ref = OM.hadamard_mxfp4_quant(xs)
            dtq = time.perf_counter() - t0
            same = bool((q_sample[0] == codes_ref).all() and (q_sample[1] == scales_ref).all())
            sec["hadamard_mxfp4_quant_8192x16384"]["cpu_baseline"] = {
                "value": round(rows_q * (K4 * 2 + K4 // 2 + K4 // 32) / dtq / 1e9, 5), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"rows 0..{rows_q - 1} of the same matrix, numpy restatement, {dtq:.2f} s", "bit_exact_vs_gpu": same}
        out["secondary"] = sec

    print(json.dumps(out))


if __name__ == "__main__":
    main()
