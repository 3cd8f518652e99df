"""tritonblas_amd — hand-written gfx950 (MI355X) GEMM kernels behind the tritonBLAS Python API."""
from .matmul import matmul, matmul_a8w8
from .matmul import matmul_lt, matmul_a8w8_lt
from .matmul import matmul_fp4
from .matmul import addmm
from .matmul import grouped_matmul_a8w8
from .config import MatmulConfig, matmul_preamble
from .bench import do_bench
from .origami import OrigamiMatmulSelector
from .utils import dynamic_mxfp4_quant, hadamard_mxfp4_quant

__all__ = [
    "matmul", "matmul_a8w8", "matmul_lt", "matmul_a8w8_lt", "matmul_fp4", "addmm", "grouped_matmul_a8w8",
    "MatmulConfig", "matmul_preamble", "do_bench", "OrigamiMatmulSelector", "dynamic_mxfp4_quant",
    "hadamard_mxfp4_quant",
]
