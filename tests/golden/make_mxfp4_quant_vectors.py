"""Writes tests/golden/mxfp4_quant_vectors.npz: inputs and the outputs of the reference's own MXFP4
quantiser for them.

The reference kernel (`_dynamic_mxfp4_quant_kernel`, include/tritonblas/utils.py:646-740, called through
`dynamic_mxfp4_quant`, :743-789) is a Triton kernel; here it runs under Triton's CPU interpreter
(TRITON_INTERPRET=1) on CPU tensors, loaded from the reference's utils.py by file path (the package's
__init__ needs a GPU and the `origami` module, neither of which exists in this container).  Only this
script ever touches the reference; the tests read the .npz.

Inputs (bf16 and fp32, stored as raw bit patterns): seeded N(0,1) with 20x outliers; every block
maximum mantissa around the round-up threshold of the scale (1.75 x 2^e) over a range of exponents;
all-zero blocks, negative zeros, denormals, values far below the block maximum (shift counts of 32
and more in the e2m1 rounding), the largest finite values and infinities.  No NaNs; no bf16 denormals
(see main()).

Usage (in the container that holds /root/reference):  python tests/golden/make_mxfp4_quant_vectors.py
"""
import importlib.util
import os
import sys

os.environ["TRITON_INTERPRET"] = "1"
import numpy as np
import torch

REF = "/root/reference/include/tritonblas/utils.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mxfp4_quant_vectors.npz")


def load_reference():
    # Triton 3.6's interpreter does not hand its builder to math functions called as tensor methods
    # (`x.floor()`, utils.py:688): route the method through the module-level function, which it patches.
    import triton.language as tl
    tl.tensor.floor = lambda self: tl.floor(self)
    spec = importlib.util.spec_from_file_location("reference_utils", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def inputs_fp32():
    g = torch.Generator().manual_seed(5)
    rows = []
    x = torch.randn(48, 128, generator=g)
    x = torch.where(torch.rand(48, 128, generator=g) < 0.02, x * 20, x)
    rows.append(x)
    # block maxima around the scale's round-up threshold, many exponents; the rest of the block spans the grid
    fill = torch.tensor([0.0, 0.03, 0.124, 0.125, 0.126, 0.2, 0.25, 0.3, 0.374, 0.375, 0.376, 0.5, 0.62, 0.625, 0.63,
                         0.75, 0.874, 0.875, 0.876, 1.0, 1.1, 1.2, 1.25, 1.3, 1.4, 1.5, 1.6, 1.7, -0.37, -0.8, -1.25])
    blocks = []
    for e in list(range(-140, -118)) + list(range(-20, 21, 3)) + list(range(100, 128)):
        for mant in (1.0, 1.25, 1.5, 1.7421875, 1.74609375, 1.75, 1.7578125, 1.875, 1.9921875):
            amax = torch.tensor(mant, dtype=torch.float64) * (2.0 ** e)
            b = torch.cat([(fill.double() * amax / 1.75), amax.reshape(1)]).float()
            blocks.append(b)
    n = len(blocks) - len(blocks) % 4
    rows.append(torch.stack(blocks[:n]).reshape(-1, 128))
    special = torch.zeros(8, 128)
    special[0, 32:64] = -0.0
    special[1, :32] = torch.tensor(np.frombuffer(np.arange(1, 33, dtype=np.uint32).tobytes(), dtype=np.float32).copy())  # fp32 denormals
    special[1, 32:64] = 1e-39
    special[2, :32] = torch.cat([torch.tensor([6.0]), 2.0 ** -torch.arange(1, 32).float() * 1.3])     # deep shifts
    special[2, 32:64] = torch.cat([torch.tensor([3.0e38]), 2.0 ** -torch.arange(20, 51).float()])
    special[3, :32] = torch.finfo(torch.float32).max
    special[3, 32:64] = torch.cat([torch.tensor([float("inf"), -float("inf")]), torch.linspace(-8, 8, 30)])
    special[4, :32] = torch.linspace(-6.5, 6.5, 32)
    special[4, 32:64] = torch.linspace(-0.26, 0.26, 32)
    special[5, :] = torch.linspace(-3.1, 3.1, 128)
    special[6, :64] = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0] * 8) * torch.tensor([1.0, -1.0]).repeat(32)
    rows.append(special)
    return torch.cat(rows, dim=0).contiguous()


def main():
    ref = load_reference()
    x32 = inputs_fp32()
    xbf = x32.bfloat16()
    # The interpreter's bf16 emulation mis-converts bf16 *denormal* inputs (its codes for them differ
    # from its own codes for the same values passed as fp32, which do agree with the bit-level reading
    # of the kernel): the bf16 set carries zeros in their place; the fp32 set keeps its denormals.
    bits = xbf.view(torch.int16)
    xbf = torch.where((bits & 0x7F80) == 0, torch.zeros_like(xbf), xbf)
    out = {}
    for name, x in (("f32", x32), ("bf16", xbf)):
        codes, scales = ref.dynamic_mxfp4_quant(x)
        out[f"x_{name}_bits"] = x.view(torch.int32).numpy().view(np.uint32) if name == "f32" else x.view(torch.int16).numpy().view(np.uint16)
        out[f"codes_{name}"] = codes.numpy()
        out[f"scales_{name}"] = scales.numpy()
        print(name, tuple(x.shape), "->", codes.shape, scales.shape)
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    sys.exit(main())
