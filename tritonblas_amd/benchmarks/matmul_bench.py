"""Shape-list benchmark driver for the GEMM entry points.

    python -m tritonblas_amd.benchmarks.matmul_bench --input-yaml shapes.yaml --output-csv out.csv
        [--enable-streamk | --work-stealing] [--checkcorrectness] [--init_type randn|hpl|trig_float|zeros]
        [--shuffle-bench] [--csv-write-freq N] [--n-warmup W] [--n-repeat R]

Input: a YAML list of {m, n, k, in_dtype, out_dtype, transA, transB} (in_dtype "fp4" selects the MXFP4
GEMM).  Output: one CSV row per case with the column set of the reference's driver
(benchmarks/tritonblas_matmul.py:287-293), so that result files of both can be compared directly.
Timing is the reference's do_bench loop (cache flush and workspace reset outside the timed region).
--checkcorrectness compares every case with torch on the GPU at the reference's tolerances
(benchmarks/tritonblas_matmul.py:78-111).
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
           "fp8": torch.float8_e4m3fn, "fp4": "fp4"}


def str_to_dtype(name):
    key = str(name).replace("torch.", "").lower()
    if key not in _DTYPES:
        raise ValueError(f"unsupported dtype {name!r}; this library runs float16, bfloat16, float8_e4m3fn and fp4 inputs")
    return _DTYPES[key]


def _tolerances(in_dtype, out_dtype, quantized):
    if quantized:
        return (0.02, 1e-2) if out_dtype == torch.bfloat16 else (0.1, 0.05)
    return (0.5, 0.05)


def _make_case(m, n, k, in_dtype, out_dtype, transA, transB, init_type, enable_streamk, work_stealing):
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
    sel = tb.OrigamiMatmulSelector(m, n, k, inp.A.dtype, inp.B.dtype, inp.C.dtype, inp.A.device, streamk=enable_streamk)
    cfg = tb.matmul_preamble(sel)
    if inp.scaleA is not None:
        launch = lambda: tb.matmul_a8w8_lt(inp.A, inp.B, inp.scaleA, inp.scaleB, inp.C, sel, cfg, enable_streamk,
                                           work_stealing=work_stealing)
        ref = lambda: ((inp.A.float() @ inp.B.float()) * (inp.scaleA[:, None] * inp.scaleB[None, :])).to(out_dtype)
    else:
        launch = lambda: tb.matmul_lt(inp.A, inp.B, inp.C, sel, cfg, enable_streamk, work_stealing=work_stealing)
        ref = lambda: torch.matmul(inp.A, inp.B).to(out_dtype)
    reset = lambda: cfg.reset(streamk=enable_streamk, work_stealing=work_stealing)
    return launch, reset, sel, inp, ref


def _nbytes(*tensors):
    return sum(t.numel() * t.element_size() for t in tensors if t is not None)


def bench_matmul(input_yaml, init_type="randn", print_verbose=False, shuffle_benchmark=False, output_csv=None,
                 write_csv_freq=100, enable_streamk=False, work_stealing=False, check_correctness=False,
                 n_warmup=20, n_repeat=100):
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
                                                  work_stealing)
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


def write_csv(filename, results):
    with open(filename, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=FIELDNAMES)
        w.writeheader()
        w.writerows(results)


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
    args = ap.parse_args(argv)
    if args.enable_streamk and args.work_stealing:
        ap.error("--enable-streamk and --work-stealing select different schedules; give one")
    res = bench_matmul(args.input_yaml, args.init_type, args.print_verbose, args.shuffle_bench, args.output_csv or None,
                       args.csv_write_freq, args.enable_streamk, args.work_stealing, args.checkcorrectness,
                       args.n_warmup, args.n_repeat)
    if not args.output_csv:
        w = csv.DictWriter(sys.stdout, fieldnames=FIELDNAMES)
        w.writeheader()
        w.writerows(res)


if __name__ == "__main__":
    main()
