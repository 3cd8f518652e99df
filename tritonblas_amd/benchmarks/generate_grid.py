"""Writes YAML shape lists for matmul_bench.

    python -m tritonblas_amd.benchmarks.generate_grid --preset llm --in-dtype float8_e4m3fn --out-dtype bfloat16 -o shapes.yaml

Presets: "grid" (every (m, n, k) on a regular lattice, the reference's datasets/generate_grid.py),
"llm" (projection shapes of 8B/70B-class decoders for a few token counts), "fp4" (the production list
of the reference's datasets/generate_grid_fp4.py:12-36; k is kept a multiple of 32).
"""
import argparse
import itertools

import yaml

FP4_PRODUCTION = [(256, 2048, 8192), (2048, 8192, 8192), (16384, 16384, 16384)] + \
    [(b, 1280, 8192) for b in (1, 64, 128, 256, 512, 1024, 2048, 4096)] + \
    [(b, 8192, 1024) for b in (1, 64, 128, 256, 512, 1024, 2048, 4096)]


def shapes(preset, lo, hi, step):
    if preset == "grid":
        r = range(lo, hi + 1, step)
        return list(itertools.product(r, r, r))
    if preset == "fp4":
        return list(FP4_PRODUCTION)
    if preset == "llm":
        out = []
        for tokens in (32, 128, 512, 2048, 8192):
            for (n, k) in ((4096, 4096), (14336, 4096), (4096, 14336), (8192, 8192), (28672, 8192), (8192, 28672)):
                out.append((tokens, n, k))
        return out
    raise ValueError(preset)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--preset", default="grid", choices=["grid", "llm", "fp4"])
    ap.add_argument("--min", type=int, default=1024, dest="lo")
    ap.add_argument("--max", type=int, default=8192, dest="hi")
    ap.add_argument("--step", type=int, default=1024)
    ap.add_argument("--transA", default="T", choices=["N", "T"])
    ap.add_argument("--transB", default="N", choices=["N", "T"])
    ap.add_argument("--in-dtype", default="float16")
    ap.add_argument("--out-dtype", default="float16")
    ap.add_argument("-o", "--output", required=True)
    args = ap.parse_args(argv)
    in_dtype = "fp4" if args.preset == "fp4" else args.in_dtype
    cases = [{"m": m, "n": n, "k": k, "in_dtype": in_dtype, "out_dtype": args.out_dtype, "transA": args.transA,
              "transB": args.transB} for (m, n, k) in shapes(args.preset, args.lo, args.hi, args.step)
             if in_dtype != "fp4" or k % 32 == 0]
    with open(args.output, "w") as f:
        yaml.safe_dump(cases, f, sort_keys=False)
    print(f"{len(cases)} cases written to {args.output}")


if __name__ == "__main__":
    main()
