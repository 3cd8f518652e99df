"""ctypes binding of ``libtritonblas_amd.so`` (the C ABI declared in ``include/tritonblas_amd.h``).

The library is built in-tree by ``make -C tritonblas_amd/csrc`` (``__graft_entry__.build()`` does
that).  There is no fallback: if the shared object is missing, importing any compute entry point
raises.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# TRITONBLAS_AMD_LIB names another build of the library (measurement builds of the kernels: see the
# W4GEN_LAB options of csrc/gen_w4.py); the default is the in-tree one
LIB_PATH = os.environ.get("TRITONBLAS_AMD_LIB") or os.path.join(_HERE, "lib", "libtritonblas_amd.so")

# ---- enums (mirrors of the header) -------------------------------------------------------------
TB_OK = 0
TB_EPOCH_ON_DEVICE = 0xFFFFFFFF   # tb_gemm_desc.epoch: the workspace counts its own Stream-K launches
TB_ERR_NULL_POINTER, TB_ERR_BAD_SHAPE, TB_ERR_BAD_DTYPE, TB_ERR_BAD_LAYOUT, TB_ERR_BAD_TILE = -1, -2, -3, -4, -5
TB_ERR_WORKSPACE, TB_ERR_BAD_SCHEDULE, TB_ERR_LAUNCH, TB_ERR_NO_DEVICE, TB_ERR_BAD_ARGUMENT = -6, -7, -8, -9, -10
TB_F16, TB_BF16, TB_FP8_E4M3, TB_FP4_E2M1, TB_F32, TB_I8, TB_FP8_E5M2 = 0, 1, 2, 3, 4, 5, 6
TB_SCHED_PERSISTENT, TB_SCHED_WORK_STEALING, TB_SCHED_STREAMK, TB_SCHED_STREAMK_WS = 0, 1, 2, 3
TB_WS_QUEUES, TB_WS_GLOBAL_ATOMIC, TB_WS_HIERARCHICAL = 0, 1, 2

EXPORTED_SYMBOLS = [
    "tb_abi_version", "tb_status_string", "tb_device_info", "tb_select", "tb_list_tiles", "tb_gemm",
    "tb_workspace_bytes", "tb_gemm_fp4", "tb_grouped_gemm_fp8", "tb_grouped_workspace_bytes", "tb_streamk_tail_tiles", "tb_hadamard_mxfp4_quant",
    "tb_tile_coords", "tb_default_panel", "tb_ws_queue_tile", "tb_hierarchical_split",
    "tb_workspace_layout", "tb_debug_option", "tb_gemm_static_workspace", "tb_static_workspace_status", "tb_gemm_launch_info",
]


class tb_hw(C.Structure):
    _fields_ = [("n_cu", C.c_int32), ("num_xcd", C.c_int32), ("cu_per_xcd", C.c_int32), ("lds_bytes", C.c_int32),
                ("l2_bytes", C.c_int32), ("clock_khz", C.c_int32), ("mem_clock_khz", C.c_int32),
                ("wave_size", C.c_int32), ("hbm_gbps", C.c_double), ("arch", C.c_char * 32)]


class tb_launch_info(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("block_m", "block_n", "block_k", "waves", "four_wave", "mode", "grid", "total_tiles",
                                         "sk_tiles", "sk_unit", "sk_ws", "skinny")]


class tb_problem(C.Structure):
    _fields_ = [("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64), ("a_type", C.c_int32), ("b_type", C.c_int32),
                ("c_type", C.c_int32), ("a_k_contiguous", C.c_int32), ("b_k_contiguous", C.c_int32),
                ("streamk", C.c_int32), ("num_groups", C.c_int32)]


class tb_selection(C.Structure):
    _fields_ = [("block_m", C.c_int32), ("block_n", C.c_int32), ("block_k", C.c_int32), ("group_m", C.c_int32),
                ("num_xcds", C.c_int32), ("occupancy", C.c_int32), ("num_stages", C.c_int32), ("sk_grid", C.c_int32),
                ("counters_per_xcd", C.c_int32), ("lds_bytes", C.c_int32), ("est_compute_us", C.c_double),
                ("est_memory_us", C.c_double), ("est_total_us", C.c_double)]


class tb_gemm_desc(C.Structure):
    _fields_ = [("struct_bytes", C.c_uint32), ("a_type", C.c_int32), ("b_type", C.c_int32), ("c_type", C.c_int32),
                ("bias_type", C.c_int32), ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64),
                ("a_stride_m", C.c_int64), ("a_stride_k", C.c_int64), ("b_stride_k", C.c_int64),
                ("b_stride_n", C.c_int64), ("c_stride_m", C.c_int64), ("c_stride_n", C.c_int64),
                ("a", C.c_void_p), ("b", C.c_void_p), ("c", C.c_void_p), ("a_scale", C.c_void_p),
                ("b_scale", C.c_void_p), ("bias", C.c_void_p), ("bias_stride", C.c_int64),
                ("block_m", C.c_int32), ("block_n", C.c_int32), ("block_k", C.c_int32), ("group_m", C.c_int32),
                ("num_xcds", C.c_int32), ("schedule", C.c_int32), ("grid", C.c_int32),
                ("counters_per_xcd", C.c_int32), ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
                ("epoch", C.c_uint32), ("spin_limit", C.c_uint32), ("cu_mask", C.c_void_p),
                ("cu_mask_len", C.c_int32), ("ws_mode", C.c_int32), ("ws_local_tiles_per_xcd", C.c_int32),
                ("ws_global_tiles", C.c_int32), ("column_split", C.c_int32)]


class tb_gemm_fp4_desc(C.Structure):
    _fields_ = [("struct_bytes", C.c_uint32), ("c_type", C.c_int32), ("m", C.c_int64), ("n", C.c_int64),
                ("k", C.c_int64), ("a", C.c_void_p), ("b", C.c_void_p), ("c", C.c_void_p),
                ("a_stride_m", C.c_int64), ("b_stride_n", C.c_int64), ("c_stride_m", C.c_int64),
                ("c_stride_n", C.c_int64), ("a_scales", C.c_void_p), ("b_scales", C.c_void_p),
                ("a_scales_stride_m", C.c_int64), ("a_scales_stride_k", C.c_int64),
                ("b_scales_stride_n", C.c_int64), ("b_scales_stride_k", C.c_int64),
                ("block_m", C.c_int32), ("block_n", C.c_int32), ("block_k", C.c_int32), ("group_m", C.c_int32),
                ("num_xcds", C.c_int32)]


class tb_grouped_gemm_desc(C.Structure):
    _fields_ = [("struct_bytes", C.c_uint32), ("c_type", C.c_int32), ("m_total", C.c_int64), ("n", C.c_int64),
                ("k", C.c_int64), ("num_groups", C.c_int32), ("a", C.c_void_p), ("w", C.c_void_p), ("c", C.c_void_p),
                ("a_stride_m", C.c_int64), ("w_stride_g", C.c_int64), ("w_stride_n", C.c_int64),
                ("c_stride_m", C.c_int64), ("c_stride_n", C.c_int64), ("a_scale", C.c_void_p),
                ("w_scale", C.c_void_p), ("group_offsets", C.c_void_p), ("block_m", C.c_int32),
                ("block_n", C.c_int32), ("block_k", C.c_int32), ("group_m", C.c_int32), ("num_xcds", C.c_int32),
                ("small_rows", C.c_int32), ("streamk", C.c_int32), ("epoch", C.c_uint32), ("spin_limit", C.c_uint32),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class tb_quant_desc(C.Structure):
    _fields_ = [("struct_bytes", C.c_uint32), ("x_type", C.c_int32), ("m", C.c_int64), ("n", C.c_int64),
                ("x", C.c_void_p), ("x_stride_m", C.c_int64), ("codes", C.c_void_p), ("codes_stride_m", C.c_int64),
                ("scales", C.c_void_p), ("scales_stride_m", C.c_int64), ("hadamard", C.c_int32)]


_lib = None


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C tritonblas_amd/csrc -j8` "
            "(or __graft_entry__.build()); there is no fallback path."
        )
    lib = C.CDLL(LIB_PATH)
    lib.tb_abi_version.restype = C.c_int
    lib.tb_status_string.restype = C.c_char_p
    lib.tb_status_string.argtypes = [C.c_int]
    lib.tb_device_info.argtypes = [C.c_int, C.POINTER(tb_hw)]
    lib.tb_select.argtypes = [C.POINTER(tb_problem), C.POINTER(tb_hw), C.POINTER(tb_selection)]
    lib.tb_list_tiles.argtypes = [C.c_int32, C.POINTER(C.c_int32), C.c_int32]
    lib.tb_gemm.argtypes = [C.POINTER(tb_gemm_desc), C.c_void_p]
    lib.tb_workspace_bytes.argtypes = [C.POINTER(tb_gemm_desc)]
    lib.tb_workspace_bytes.restype = C.c_size_t
    lib.tb_gemm_fp4.argtypes = [C.POINTER(tb_gemm_fp4_desc), C.c_void_p]
    lib.tb_grouped_gemm_fp8.argtypes = [C.POINTER(tb_grouped_gemm_desc), C.c_void_p]
    lib.tb_grouped_workspace_bytes.argtypes = [C.POINTER(tb_grouped_gemm_desc)]
    lib.tb_grouped_workspace_bytes.restype = C.c_size_t
    lib.tb_streamk_tail_tiles.argtypes = [C.c_int32] * 5
    lib.tb_hadamard_mxfp4_quant.argtypes = [C.POINTER(tb_quant_desc), C.c_void_p]
    lib.tb_tile_coords.argtypes = [C.c_int32] * 5 + [C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    lib.tb_default_panel.argtypes = [C.c_int32] * 3
    lib.tb_ws_queue_tile.argtypes = [C.c_int32] * 7 + [C.POINTER(C.c_int32)] * 2
    lib.tb_hierarchical_split.argtypes = [C.c_int64, C.c_int32, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    lib.tb_gemm_static_workspace.argtypes = [C.POINTER(tb_gemm_desc), C.c_void_p]
    lib.tb_gemm_launch_info.argtypes = [C.POINTER(tb_gemm_desc), C.POINTER(tb_launch_info)]
    lib.tb_static_workspace_status.argtypes = [C.POINTER(C.c_int), C.c_int]
    lib.tb_static_workspace_status.restype = C.c_int
    lib.tb_workspace_layout.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    lib.tb_debug_option.argtypes = [C.c_char_p, C.c_int]
    if lib.tb_abi_version() != 1:
        raise RuntimeError("libtritonblas_amd.so ABI version mismatch")
    _lib = lib
    return lib


def debug_option(name: str, value: int):
    """Set one of the library's tuning / test hooks (see ``tb_debug_option`` in the header)."""
    check(load().tb_debug_option(name.encode(), int(value)), "tb_debug_option")


def workspace_layout():
    """(counters_offset, flags_offset) of a workspace, in bytes."""
    a, b = C.c_size_t(), C.c_size_t()
    check(load().tb_workspace_layout(C.byref(a), C.byref(b)), "tb_workspace_layout")
    return int(a.value), int(b.value)


def status_string(status: int) -> str:
    return load().tb_status_string(status).decode()


def check(status: int, what: str = "tritonblas_amd"):
    """Map a status code to the exception the reference raises at the same point."""
    if status == TB_OK:
        return
    msg = status_string(status)
    if status == TB_ERR_BAD_SHAPE:
        raise AssertionError("Incompatible Dimensions")
    raise RuntimeError(f"{what}: {msg} (status {status})")


_DTYPES = {torch.float16: TB_F16, torch.bfloat16: TB_BF16, torch.float32: TB_F32, torch.float8_e4m3fn: TB_FP8_E4M3, torch.float8_e5m2: TB_FP8_E5M2,
           torch.int8: TB_I8}


def tb_dtype(dtype) -> int:
    if isinstance(dtype, str):
        if dtype.lower() in ("f4", "fp4"):
            return TB_FP4_E2M1
        raise RuntimeError(f"unsupported dtype {dtype!r}")
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise RuntimeError(f"tritonblas_amd: unsupported dtype {dtype}") from None


def stream_handle(device=None):
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)
