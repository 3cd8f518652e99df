"""Shape-list benchmark driver for the GEMM entry points.

    python -m tritonblas_amd.benchmarks.matmul_bench --input-yaml shapes.yaml --output-csv out.csv
        [--enable-streamk | --work-stealing] [--checkcorrectness] [--init_type randn|hpl|trig_float|zeros]
        [--shuffle-bench] [--csv-write-freq N] [--n-warmup W] [--n-repeat R]
        [--global-atomic | --hierarchical] [--counters-per-xcd C] [--cu-sweep [--cu-sweep-max-remove R]]

Input: a YAML list of {m, n, k, in_dtype, out_dtype, transA, transB} (in_dtype "fp4" selects the MXFP4
GEMM).  Output: one CSV row per case with the column set of the reference's driver
(benchmarks/tritonblas_matmul.py:287-293), so that result files of both can be compared directly.
Timing is the reference's do_bench loop (cache flush and workspace reset outside the timed region).
--checkcorrectness compares every case with torch on the GPU at the reference's tolerances
(benchmarks/tritonblas_matmul.py:78-111).
--cu-sweep repeats the shape list with 0, 1, 2, ... CUs per XCD taken away (benchmarks/tritonblas_matmul.py:381-412):
the selector is built with total_cus = active_cus = what is left, which sizes the launch grid, and with
--work-stealing the per-workgroup mask; rows gain a leading active_cus column.  The sweep runs in this process;
to also fence the hardware, set the runtime's CU mask yourself (benchmarks.common.build_balanced_hex_mask
gives the balanced mask strings the reference uses).
"""
import argparse
import csv
import random
import sys

import torch
import yaml

FIELDNAMES = ["m", "n", "k", "mnk", "macro_tile", "bytes", "flops", "tritonblas_gflops", "a_type", "b_type", "c_type",
              "d_type", "compute_type", "in_dtype", "out_dtype", "init_type", "transA", "transB", "us", "alpha", "beta", "mode"]

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "float16": torch.float16, "fp16": torch.float16,
           "bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float8_e4m3fn": torch.float8_e4m3fn,
           "fp8": torch.float8_e4m3fn, "int8": torch.int8, "fp4": "fp4"}


def str_to_dtype(name):
    key = str(name).replace("torch.", "").lower()
    if key not in _DTYPES:
        raise ValueError(f"unsupported dtype {name!r}; this library runs float32, float16, bfloat16, float8_e4m3fn, int8 and fp4 inputs")
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
    ap.add_argument("--cu-sweep-max-remove", type=int, default=34, help="most CUs to take from one XCD")
    ap.add_argument("--counters-per-xcd", type=int, default=None, help="work-stealing queues per XCD (default: the selector's)")
    ap.add_argument("--global-atomic", action="store_true", help="work stealing from one device-wide counter")
    ap.add_argument("--hierarchical", action="store_true", help="work stealing from XCD-local queues, then a shared pool")
    args = ap.parse_args(argv)
    if args.enable_streamk and args.work_stealing:
        ap.error("--enable-streamk and --work-stealing select different schedules; give one")
    if args.global_atomic and args.hierarchical:
        ap.error("--global-atomic and --hierarchical are different queue layouts; give one")
    common = dict(init_type=args.init_type, print_verbose=args.print_verbose, shuffle_benchmark=args.shuffle_bench,
                  write_csv_freq=args.csv_write_freq, enable_streamk=args.enable_streamk, work_stealing=args.work_stealing,
                  check_correctness=args.checkcorrectness, n_warmup=args.n_warmup, n_repeat=args.n_repeat,
                  counters_per_xcd=args.counters_per_xcd, global_atomic=args.global_atomic, hierarchical=args.hierarchical)
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
