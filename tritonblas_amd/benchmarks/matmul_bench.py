"""Shape-list benchmark driver for the GEMM entry points.

    python -m tritonblas_amd.benchmarks.matmul_bench --input-yaml shapes.yaml --output-csv out.csv
        [--enable-streamk | --work-stealing] [--checkcorrectness] [--init_type randn|hpl|trig_float|zeros]
        [--shuffle-bench] [--csv-write-freq N] [--n-warmup W] [--n-repeat R]
        [--global-atomic | --hierarchical] [--counters-per-xcd C] [--cu-sweep [--cu-mask] [--cu-sweep-max-remove R]]

Input: a YAML list of {m, n, k, in_dtype, out_dtype, transA, transB} (in_dtype "fp4" selects the MXFP4
GEMM).  Output: one CSV row per case with the column set of the reference's driver
(benchmarks/tritonblas_matmul.py:287-293), so that result files of both can be compared directly.
Timing is the reference's do_bench loop (cache flush and workspace reset outside the timed region).
--checkcorrectness compares every case with torch on the GPU at the reference's tolerances
(benchmarks/tritonblas_matmul.py:78-111).
--cu-sweep repeats the shape list with 0, 1, 2, ... CUs per XCD taken away (benchmarks/tritonblas_matmul.py:381-412):
the selector is built with total_cus = active_cus = what is left, which sizes the launch grid, and with
--work-stealing the per-workgroup mask; rows gain a leading active_cus column.  That sweep runs in this process.
--cu-sweep --cu-mask fences the hardware instead, as the reference does: every step runs in a child process with
ROC_GLOBAL_CU_MASK set to the balanced mask of that step (benchmarks.common.build_balanced_hex_mask) and the library
sized for the whole device; the parent starts its children before it makes any GPU call of its own (it asks a first
child for the CU counts) and collects their rows as JSON.
"""
import argparse
import csv
import json
import os
import random
import subprocess
import sys

import torch
import yaml

FIELDNAMES = ["m", "n", "k", "mnk", "macro_tile", "bytes", "flops", "tritonblas_gflops", "a_type", "b_type", "c_type",
              "d_type", "compute_type", "in_dtype", "out_dtype", "init_type", "transA", "transB", "us", "alpha", "beta", "mode"]

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "float16": torch.float16, "fp16": torch.float16,
           "bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float8_e4m3fn": torch.float8_e4m3fn,
           "fp8": torch.float8_e4m3fn, "float8_e5m2": torch.float8_e5m2, "bf8": torch.float8_e5m2, "int8": torch.int8, "fp4": "fp4"}


def str_to_dtype(name):
    key = str(name).replace("torch.", "").lower()
    if key not in _DTYPES:
        raise ValueError(f"unsupported dtype {name!r}; this library runs float32, float16, bfloat16, float8_e4m3fn, float8_e5m2, int8 and fp4 inputs")
    return _DTYPES[key]


def _tolerances(in_dtype, out_dtype, quantized):
    if quantized:
        if out_dtype == torch.int8:
            return (2.0, 0.2)
        return (0.02, 1e-2) if out_dtype == torch.bfloat16 else (0.1, 0.05)
    return (0.5, 0.05)


def _make_case(m, n, k, in_dtype, out_dtype, transA, transB, init_type, enable_streamk, work_stealing, total_cus=None,
               active_cus=None, counters_per_xcd=None, global_atomic=False, hierarchical=False):
    """Returns (launch, reset, selector-or-None, inputs, reference-result function)."""
    import tritonblas_amd as tb
    from tritonblas_amd.utils import generate_matmul_inputs, mxfp4_to_f32, e8m0_to_f32
    inp = generate_matmul_inputs(m, n, k, in_dtype, out_dtype, transA, transB, init_type)
    if in_dtype == "fp4":
        bq = inp.B.T                                   # (n, k/2) packed, k-contiguous
        launch = lambda: tb.matmul_fp4(inp.A, bq, inp.C, inp.scaleA, inp.scaleB)

        def ref():
            a = mxfp4_to_f32(inp.A) * e8m0_to_f32(inp.scaleA).repeat_interleave(32, dim=1)
            b = mxfp4_to_f32(bq) * e8m0_to_f32(inp.scaleB).repeat_interleave(32, dim=1)
            return (a @ b.T).to(out_dtype)
        return launch, (lambda: None), None, inp, ref
    sel = tb.OrigamiMatmulSelector(m, n, k, inp.A.dtype, inp.B.dtype, inp.C.dtype, inp.A.device, streamk=enable_streamk,
                                   total_cus=total_cus, active_cus=active_cus)
    if counters_per_xcd is not None:
        sel.COUNTERS_PER_XCD = counters_per_xcd
    cfg = tb.matmul_preamble(sel)
    cfg.global_atomic, cfg.hierarchical = global_atomic, hierarchical
    if inp.scaleA is not None:
        launch = lambda: tb.matmul_a8w8_lt(inp.A, inp.B, inp.scaleA, inp.scaleB, inp.C, sel, cfg, enable_streamk,
                                           work_stealing=work_stealing)
        def ref():
            acc = (inp.A.float() @ inp.B.float()) * (inp.scaleA[:, None] * inp.scaleB[None, :])
            if out_dtype == torch.int8:   # (reference benchmarks/tritonblas_matmul.py:72-74)
                acc = torch.clamp(acc, -127.0, 127.0)
            return acc.to(out_dtype)
    else:
        launch = lambda: tb.matmul_lt(inp.A, inp.B, inp.C, sel, cfg, enable_streamk, work_stealing=work_stealing)
        ref = lambda: torch.matmul(inp.A, inp.B).to(out_dtype)
    reset = lambda: cfg.reset(streamk=enable_streamk, work_stealing=work_stealing)
    return launch, reset, sel, inp, ref


def _nbytes(*tensors):
    return sum(t.numel() * t.element_size() for t in tensors if t is not None)


def bench_matmul(input_yaml, init_type="randn", print_verbose=False, shuffle_benchmark=False, output_csv=None,
                 write_csv_freq=100, enable_streamk=False, work_stealing=False, check_correctness=False,
                 n_warmup=20, n_repeat=100, total_cus=None, active_cus=None, counters_per_xcd=None, global_atomic=False,
                 hierarchical=False):
    import tritonblas_amd as tb
    with open(input_yaml) as f:
        dataset = yaml.safe_load(f)
    cases = [(c["m"], c["n"], c["k"], str_to_dtype(c["in_dtype"]), str_to_dtype(c["out_dtype"]), c.get("transA", "T"),
              c.get("transB", "N")) for c in dataset]
    if shuffle_benchmark:
        random.shuffle(cases)
    mode = "work_stealing" if work_stealing else ("streamk" if enable_streamk else "persistent")
    results = []
    for count, (m, n, k, in_dtype, out_dtype, transA, transB) in enumerate(cases):
        launch, reset, sel, inp, ref = _make_case(m, n, k, in_dtype, out_dtype, transA, transB, init_type, enable_streamk,
                                                  work_stealing, total_cus, active_cus, counters_per_xcd, global_atomic,
                                                  hierarchical)
        ms = tb.do_bench(launch, reset_fn=reset, n_warmup=n_warmup, n_repeat=n_repeat)
        gflops = 2.0 * m * n * k * 1e-9 / (ms * 1e-3)
        tile = f"{sel.block_m}x{sel.block_n}x{sel.block_k}" if sel is not None else "library"
        if print_verbose:
            print(f"m={m}, n={n}, k={k}, in_dtype={in_dtype}, out_dtype={out_dtype}, init={init_type}, mode={mode}, "
                  f"perf={gflops:.1f}(GFLOPs) selected_tile={tile}", flush=True)
        results.append({
            "m": m, "n": n, "k": k, "mnk": m * n * k, "macro_tile": tile,
            "bytes": _nbytes(inp.A, inp.B, inp.C, inp.scaleA, inp.scaleB), "flops": 2 * m * n * k * 1e-12,
            "tritonblas_gflops": gflops, "a_type": str(inp.A.dtype), "b_type": str(inp.B.dtype), "c_type": str(inp.C.dtype),
            "d_type": str(inp.C.dtype), "compute_type": str(inp.C.dtype), "in_dtype": str(in_dtype), "out_dtype": str(out_dtype),
            "init_type": init_type, "transA": str(transA), "transB": str(transB), "us": ms * 1e3, "alpha": 1, "beta": 0,
            "mode": mode})
        if active_cus is not None:
            results[-1] = {"active_cus": active_cus, **results[-1]}
        if output_csv and count % write_csv_freq == 0:
            write_csv(output_csv, results)
        if check_correctness:
            inp.C.zero_()
            reset()
            launch()
            atol, rtol = _tolerances(in_dtype, out_dtype, inp.scaleA is not None)
            torch.testing.assert_close(inp.C.float(), ref().float(), atol=atol, rtol=rtol)
            print(f"SIZE M: {m}, N: {n}, K: {k}, trans: {transA}{transB} correct", flush=True)
    if output_csv:
        write_csv(output_csv, results)
    return results


def _fieldnames(results):
    # (reference benchmarks/tritonblas_matmul.py:294-295)
    return (["active_cus"] if results and "active_cus" in results[0] else []) + FIELDNAMES


def write_csv(filename, results):
    with open(filename, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=_fieldnames(results))
        w.writeheader()
        w.writerows(results)


def cu_sweep_steps(full_cus, num_xcds, cus_per_xcd, max_remove):
    """Active CU counts of the balanced sweep: r = 0..min(max_remove, cus_per_xcd - 1) CUs taken from every XCD
    (reference benchmarks/tritonblas_matmul.py:385-388)."""
    return [full_cus - r * num_xcds for r in range(min(max_remove, cus_per_xcd - 1) + 1)]


def _child(argv_tail, env=None):
    return subprocess.run([sys.executable, "-m", "tritonblas_amd.benchmarks.matmul_bench"] + argv_tail,
                          capture_output=True, text=True, env=env)


def masked_cu_sweep(args, argv):
    """Balanced CU-mask sweep (reference benchmarks/tritonblas_matmul.py:381-412): step r runs the shape list
    in a child process with the first r CUs of every XCD masked off by the runtime."""
    from .common import build_balanced_hex_mask
    info = _child(["--input-yaml", args.input_yaml, "--_cu-info"])
    if info.returncode != 0:
        raise RuntimeError("could not query the device: " + info.stderr[-500:])
    full_cus, num_xcds, cus_per_xcd = json.loads(info.stdout.strip().splitlines()[-1])
    # the child's arguments: everything but the sweep flags and the output file
    tail, skip = [], False
    for a in argv:
        if skip:
            skip = False
        elif a in ("--cu-sweep", "--cu-mask"):
            pass
        elif a in ("--output-csv", "--cu-sweep-max-remove"):
            skip = True
        elif a.startswith("--output-csv=") or a.startswith("--cu-sweep-max-remove="):
            pass
        else:
            tail.append(a)
    rows = []
    for r in range(min(args.cu_sweep_max_remove, cus_per_xcd - 1) + 1):
        active = full_cus - r * num_xcds
        env = os.environ.copy()
        mask = build_balanced_hex_mask(r, num_xcds, cus_per_xcd)
        if mask:
            env["ROC_GLOBAL_CU_MASK"] = mask
        else:
            env.pop("ROC_GLOBAL_CU_MASK", None)
        proc = _child(tail + ["--_active-cus", str(active)], env)
        print(f"[active_cus={active}] {proc.stderr[-300:]}", file=sys.stderr, flush=True)
        if proc.returncode != 0:
            print(f"[active_cus={active}] child failed with status {proc.returncode}", file=sys.stderr)
            continue
        rows += json.loads(proc.stdout.strip().splitlines()[-1])
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--input-yaml", required=True)
    ap.add_argument("--output-csv", default="")
    ap.add_argument("--init_type", default="randn", choices=["hpl", "trig_float", "zeros", "randn"])
    ap.add_argument("--shuffle-bench", action="store_true")
    ap.add_argument("--csv-write-freq", type=int, default=1000)
    ap.add_argument("--print-verbose", action="store_true")
    ap.add_argument("--checkcorrectness", action="store_true")
    ap.add_argument("--enable-streamk", action="store_true")
    ap.add_argument("--work-stealing", action="store_true")
    ap.add_argument("--n-warmup", type=int, default=20)
    ap.add_argument("--n-repeat", type=int, default=100)
    ap.add_argument("--cu-sweep", action="store_true", help="repeat the shape list with CUs taken away from every XCD")
    ap.add_argument("--cu-mask", action="store_true", help="with --cu-sweep: fence the hardware (ROC_GLOBAL_CU_MASK, one child "
                                                           "process per step) instead of sizing the launch")
    ap.add_argument("--cu-sweep-max-remove", type=int, default=34, help="most CUs to take from one XCD")
    # children of a --cu-mask sweep: print the CU counts / run the shape list and print the rows as JSON
    ap.add_argument("--_cu-info", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--_active-cus", type=int, default=None, help=argparse.SUPPRESS)
    ap.add_argument("--counters-per-xcd", type=int, default=None, help="work-stealing queues per XCD (default: the selector's)")
    ap.add_argument("--global-atomic", action="store_true", help="work stealing from one device-wide counter")
    ap.add_argument("--hierarchical", action="store_true", help="work stealing from XCD-local queues, then a shared pool")
    args = ap.parse_args(argv)
    if args.enable_streamk and args.work_stealing:
        ap.error("--enable-streamk and --work-stealing select different schedules; give one")
    if args.global_atomic and args.hierarchical:
        ap.error("--global-atomic and --hierarchical are different queue layouts; give one")
    if args.cu_mask and not args.cu_sweep:
        ap.error("--cu-mask is a mode of --cu-sweep")
    if args._cu_info:
        from .common import get_cu_info
        print(json.dumps(list(get_cu_info(torch.cuda.current_device()))))
        return
    if args.cu_sweep and args.cu_mask:
        # (no GPU call in this process: the children own the device, one at a time)
        res = masked_cu_sweep(args, argv if argv is not None else sys.argv[1:])
        if args.output_csv:
            write_csv(args.output_csv, res)
        else:
            w = csv.DictWriter(sys.stdout, fieldnames=_fieldnames(res))
            w.writeheader()
            w.writerows(res)
        return
    common = dict(init_type=args.init_type, print_verbose=args.print_verbose, shuffle_benchmark=args.shuffle_bench,
                  write_csv_freq=args.csv_write_freq, enable_streamk=args.enable_streamk, work_stealing=args.work_stealing,
                  check_correctness=args.checkcorrectness, n_warmup=args.n_warmup, n_repeat=args.n_repeat,
                  counters_per_xcd=args.counters_per_xcd, global_atomic=args.global_atomic, hierarchical=args.hierarchical)
    if args._active_cus is not None:
        # child of a masked sweep: the runtime fences the CUs, the library is sized for the whole device
        # (reference benchmarks/tritonblas_matmul.py:421: active_cus = total_cus under a CU mask)
        real_stdout, sys.stdout = sys.stdout, sys.stderr
        res = bench_matmul(args.input_yaml, output_csv=None, **common)
        sys.stdout = real_stdout
        print(json.dumps([{"active_cus": args._active_cus, **r} for r in res]))
        return
    if args.cu_sweep:
        from .common import get_cu_info
        res = []
        for active in cu_sweep_steps(*get_cu_info(torch.cuda.current_device()), args.cu_sweep_max_remove):
            res += bench_matmul(args.input_yaml, output_csv=None, total_cus=active, active_cus=active, **common)
        if args.output_csv:
            write_csv(args.output_csv, res)
    else:
        res = bench_matmul(args.input_yaml, output_csv=args.output_csv or None, **common)
    if not args.output_csv:
        w = csv.DictWriter(sys.stdout, fieldnames=_fieldnames(res))
        w.writeheader()
        w.writerows(res)


if __name__ == "__main__":
    main()
