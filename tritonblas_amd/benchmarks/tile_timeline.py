"""When does every workgroup of the 4-wave GEMM kernel finish each of its tiles?

Needs a measurement build of the library whose 4-wave kernels record the constant 100 MHz counter at their
start, after every tile and at their end (-DW4_LAB_TS; one 64-bit word per event and workgroup):

    make -B -C tritonblas_amd/csrc LABFLAGS=-DW4_LAB_TS OUT=/tmp/lab/ts.so OBJDIR=/tmp/lab/obj -j16
    TRITONBLAS_AMD_LIB=/tmp/lab/ts.so python3 -m tritonblas_amd.benchmarks.tile_timeline [--n 28672] [--panel P]

Runs the FP8 a8w8 GEMM 8192 x N x 8192 (default N = 28672) until the clock has settled, then reads the
timestamps of the last launch: per XCD (workgroup id mod 8) the range of end times, per tile index the mean
duration over the workgroups and the spread of the end times.  --panel sets the column panel width of the
tile order (the library's own choice otherwise).
"""
import argparse
import ctypes as C
import sys
import time

import numpy as np
import torch


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--n", type=int, default=28672)
    ap.add_argument("--panel", type=int, default=-1)
    args = ap.parse_args(argv)
    import tritonblas_amd as tb
    import tritonblas_amd._lib as L
    lib = L.load()
    if not hasattr(lib, "tb_lab_timestamps"):
        print("this library build records no timestamps (build it with LABFLAGS=-DW4_LAB_TS)", file=sys.stderr)
        return 2
    if args.panel >= 0:
        L.check(lib.tb_debug_option(b"panel", args.panel), "tb_debug_option")
    dev = torch.device("cuda", torch.cuda.current_device())
    m, n, k = 8192, args.n, 8192
    g = torch.Generator(device=dev).manual_seed(1)
    aq = torch.randn(m, k, device=dev, generator=g).to(torch.float8_e4m3fn)
    wq = torch.randn(n, k, device=dev, generator=g).to(torch.float8_e4m3fn)
    sa, sw = torch.ones(m, device=dev), torch.ones(n, device=dev)
    c = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    sel = tb.OrigamiMatmulSelector(m, n, k, aq.dtype, aq.dtype, c.dtype, dev)
    if (sel.block_m, sel.block_n) != (256, 256):
        print(f"the selector picked a {sel.block_m}x{sel.block_n} tile: not the 4-wave kernel", file=sys.stderr)
        return 2
    fn = lambda: tb.matmul_a8w8_lt(aq, wq.T, sa, sw, c, sel, None)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.08:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
    for _ in range(10):
        fn()
    torch.cuda.synchronize()
    buf = (C.c_ulonglong * (1024 * 32))()
    lib.tb_lab_timestamps.argtypes = [C.c_void_p]
    lib.tb_lab_timestamps.restype = C.c_int
    if lib.tb_lab_timestamps(buf) != 0:
        print("reading the timestamps failed", file=sys.stderr)
        return 1
    grid = 256
    tiles_per_wg = (m // 256) * (n // 256) // grid
    ts = np.frombuffer(buf, dtype=np.uint64).reshape(1024, 32)[:grid].astype(np.int64)
    start, end, tile_end = ts[:, 0], ts[:, 31], ts[:, 1:1 + tiles_per_wg]
    us = lambda x: (x - start.min()) / 100.0
    print(f"FP8 a8w8 {m}x{n}x{k}, {tiles_per_wg} tiles per workgroup, panel {'default' if args.panel < 0 else args.panel}")
    print(f"kernel, first start to last end: {us(end.max()):.1f} us; mean end {us(end).mean():.1f} us; starts within {us(start.max()):.2f} us")
    xcd = np.arange(grid) % 8
    for x in range(8):
        e = us(end[xcd == x])
        print(f"  XCD {x}: workgroups end at {e.min():.1f} .. {e.max():.1f} us")
    prev = start
    for i in range(tiles_per_wg):
        e = tile_end[:, i]
        d = (e - prev) / 100.0
        within = max(us(e[xcd == x]).max() - us(e[xcd == x]).min() for x in range(8))
        print(f"  tile {i:2d}: mean duration {d.mean():6.2f} us (min {d.min():6.2f}, max {d.max():6.2f}); end times spread {us(e).max() - us(e).min():5.2f} us over "
              f"the chip, {within:5.2f} us within an XCD")
        prev = e
    return 0


if __name__ == "__main__":
    sys.exit(main())
