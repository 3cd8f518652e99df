"""Host-side logic that needs no GPU: the LDS model and Stream-K grid model restated from the
reference, the shared library's exports, the analytical selector, and argument validation."""
import ctypes as C
import os
import re

import pytest
import numpy as np
import torch

from oracle import selector as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# --- LDS model: the reference's known answers (tests/test_lds_estimation.py:44-150) --------------
@pytest.mark.parametrize("args,want", [
    ((128, 128, 64, 2, 2, 1), 128 * 64 * 2), ((256, 64, 64, 2, 2, 1), 256 * 64 * 2), ((64, 256, 64, 2, 2, 1), 64 * 256 * 2),
    ((128, 128, 64, 2, 2, 2), 32768), ((256, 256, 64, 2, 2, 2), 65536), ((128, 128, 64, 2, 2, 3), 65536),
    ((128, 64, 64, 2, 2, 2), 24576), ((256, 128, 64, 2, 2, 2), 49152), ((64, 64, 32, 2, 2, 2), 8192),
    ((128, 256, 64, 2, 2, 2), 49152), ((64, 64, 32, 4, 4, 2), 16384), ((128, 128, 32, 4, 4, 2), 32768),
    ((128, 128, 64, 4, 4, 2), 65536), ((128, 128, 64, 1, 2, 2), 24576), ((128, 128, 64, 0.5, 0.5, 2), 8192),
])
def test_lds_known_answers(args, want):
    from tritonblas_amd.origami import estimate_triton_lds_bytes
    assert O.estimate_lds_bytes(*args) == want
    assert estimate_triton_lds_bytes(*args) == want


def test_lds_capacity_known_answers():
    from tritonblas_amd.origami import check_triton_lds_capacity
    for fn in (O.check_lds_capacity, check_triton_lds_capacity):
        assert fn(64, 64, 32, 2, 2, 65536, 2) is True
        assert fn(256, 256, 64, 4, 4, 65536, 2) is False
        assert fn(256, 256, 64, 2, 2, 65536, 2) is True
        assert fn(128, 128, 64, 2, 2, 65536, 3) is True
        assert fn(128, 128, 64, 2, 2, 65536, 4) is False
        assert fn(128, 128, 64, 0.5, 0.5, 0, 2) is False


def test_reference_sk_grid_model_hand_checked():
    # 8192^2 output with 256^2 tiles on 256 CUs: 1024 tiles, first fraction gives 256, 1024 % 256 == 0
    assert O.compute_sk_grid(8192, 8192, 8192, 256, 256, 64, 256) == 256
    # decode shape with a 256-wide tile: 32 tiles < 256 CUs, k split by 8 -> 256 (divides? 32 % 256 != 0 -> tiles)
    assert O.compute_sk_grid(32, 8192, 28672, 256, 256, 128, 256) == 32
    # a non-divisor candidate falls back to the tile count
    assert O.compute_sk_grid(4864, 8192, 4160, 256, 256, 64, 256) == 19 * 32
    # 608 tiles on 304 CUs: the first fraction gives 304, which divides the tile count
    assert O.compute_sk_grid(4864, 8192, 4160, 256, 256, 64, 304) == 304
    # gfx942-only override: 1024 tiles on 304 CUs leave a last wave of 112 (< 128) -> 256
    assert O.compute_sk_grid(8192, 8192, 8192, 256, 256, 64, 304) == 256
    assert [O.ws_counters_per_xcd(t) for t in (1, 512, 513, 1536, 1537, 2048, 2049)] == [8, 8, 4, 4, 2, 2, 1]


# --- shared library ------------------------------------------------------------------------------
def _header_symbols():
    text = open(os.path.join(ROOT, "include", "tritonblas_amd.h")).read()
    return sorted(set(re.findall(r"\b(tb_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from tritonblas_amd import _lib
    lib = _lib.load()
    syms = _header_symbols()
    assert set(syms) == set(_lib.EXPORTED_SYMBOLS)
    for s in syms:
        assert hasattr(lib, s), s
    assert lib.tb_abi_version() == 1
    assert _lib.status_string(0) == "ok" and _lib.status_string(-2) == "Incompatible Dimensions"


def test_struct_sizes_match_the_header():
    """ctypes mirrors vs the C compiler's layout (compiled here with gcc)."""
    import subprocess
    import tempfile
    from tritonblas_amd import _lib
    src = '#include <stdio.h>\n#include "tritonblas_amd.h"\nint main(){printf("%zu %zu %zu %zu %zu %zu %zu\\n",' \
          'sizeof(tb_hw),sizeof(tb_problem),sizeof(tb_selection),sizeof(tb_gemm_desc),sizeof(tb_gemm_fp4_desc),' \
          'sizeof(tb_grouped_gemm_desc),sizeof(tb_quant_desc));return 0;}'
    with tempfile.TemporaryDirectory() as td:
        open(os.path.join(td, "s.c"), "w").write(src)
        subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), "-o", os.path.join(td, "s"), os.path.join(td, "s.c")])
        sizes = [int(v) for v in subprocess.check_output([os.path.join(td, "s")]).split()]
    mine = [C.sizeof(t) for t in (_lib.tb_hw, _lib.tb_problem, _lib.tb_selection, _lib.tb_gemm_desc, _lib.tb_gemm_fp4_desc,
                                  _lib.tb_grouped_gemm_desc, _lib.tb_quant_desc)]
    assert mine == sizes


def test_default_hardware_is_mi355x():
    from tritonblas_amd import _lib
    hw = _lib.tb_hw()
    assert _lib.load().tb_device_info(-1, hw) == 0
    assert (hw.n_cu, hw.num_xcd, hw.cu_per_xcd, hw.lds_bytes, hw.arch) == (256, 8, 32, 163840, b"gfx950")


def test_selector_properties_and_lds_fit():
    """Mirror of the reference's only selector pin (tests/test_lds_estimation.py:211-228): the chosen
    tile fits the LDS of the part; plus the attribute surface the launchers read."""
    import tritonblas_amd as tb
    from tritonblas_amd import _lib
    for shape, dt, bits in [((8192, 28672, 8192), torch.float8_e4m3fn, 8), ((8192, 8192, 8192), torch.bfloat16, 16),
                            ((1024, 1024, 1024), torch.float16, 16), ((8192, 8192, 16384), "f4", 4), ((15, 17, 512), torch.bfloat16, 16)]:
        for sk in (False, True):
            s = tb.OrigamiMatmulSelector(*shape, dt, dt, torch.bfloat16, torch.device("cuda"), streamk=sk)
            assert s._hardware.N_CU == 256 and s._hardware.NUM_XCD == 8 and s._hardware.lds_capacity == 163840
            assert s._hardware.arch.name == "gfx950" and s._N_CU == 256 and s._ACTIVE_CU == 256
            assert s._sel.lds_bytes <= s._hardware.lds_capacity
            n = _lib.load().tb_list_tiles(_lib.tb_dtype(dt), None, 0)
            buf = (C.c_int32 * (3 * n))()
            _lib.load().tb_list_tiles(_lib.tb_dtype(dt), buf, n)
            tiles = {(buf[3 * i], buf[3 * i + 1], buf[3 * i + 2]) for i in range(n)}
            assert (s.block_m, s.block_n, s.block_k) in tiles
            assert s.group_m == min(8, -(-shape[0] // s.block_m)) and s.num_sms == 8
            assert s.even_k == (shape[2] % s.block_k == 0)
            assert s.sk_grid >= 1 and s.num_stages >= 2 and s.waves_per_eu >= 1
            total = -(-shape[0] // s.block_m) * -(-shape[1] // s.block_n)
            assert s.COUNTERS_PER_XCD == O.ws_counters_per_xcd(total)


def test_streamk_whole_tiles_answer_survives_the_resident_clamp():
    """FP8 2048x14336x4096 with 256x256 tiles: 448 tiles on 256 resident workgroups, and the model says
    that a second round of whole tiles beats a shared tail (its answer is the tile count, 448).  A
    launch that asks for that grid, or for none, must then run whole tiles only -- which shows as a
    Stream-K descriptor that needs no workspace -- and not a 256-workgroup grid with 192 shared tiles."""
    import tritonblas_amd as tb
    from tritonblas_amd import _lib
    m, n, k = 2048, 14336, 4096
    s = tb.OrigamiMatmulSelector(m, n, k, torch.float8_e4m3fn, torch.float8_e4m3fn, torch.bfloat16, torch.device("cuda"), streamk=True)
    assert (s.block_m, s.block_n) == (256, 256) and s.sk_grid == 448
    for grid in (0, 448):
        d = _lib.tb_gemm_desc()
        d.struct_bytes = C.sizeof(_lib.tb_gemm_desc)
        d.a_type = d.b_type = _lib.tb_dtype(torch.float8_e4m3fn)
        d.c_type = _lib.tb_dtype(torch.bfloat16)
        d.m, d.n, d.k = m, n, k
        d.a_stride_m, d.a_stride_k, d.b_stride_n, d.b_stride_k, d.c_stride_m, d.c_stride_n = k, 1, k, 1, n, 1
        d.block_m, d.block_n, d.block_k = 256, 256, 128
        d.schedule, d.grid = _lib.TB_SCHED_STREAMK, grid
        assert _lib.load().tb_workspace_bytes(d) == 0
    d.grid = 256      # an explicit resident grid still shares the 192-tile tail
    assert _lib.load().tb_workspace_bytes(d) > 256 * 256 * 256 * 4


def test_argument_validation_without_a_gpu():
    from tritonblas_amd import _lib
    lib = _lib.load()
    assert lib.tb_gemm(None, None) == _lib.TB_ERR_NULL_POINTER
    d = _lib.tb_gemm_desc()
    assert lib.tb_gemm(d, None) == _lib.TB_ERR_BAD_ARGUMENT          # struct_bytes not set
    d.struct_bytes = C.sizeof(_lib.tb_gemm_desc)
    d.a_type, d.b_type = _lib.TB_F16, _lib.TB_BF16
    assert lib.tb_gemm(d, None) == _lib.TB_ERR_BAD_DTYPE
    d.b_type = _lib.TB_F16
    assert lib.tb_gemm(d, None) == _lib.TB_ERR_NULL_POINTER
    q = _lib.tb_quant_desc()
    q.struct_bytes = C.sizeof(_lib.tb_quant_desc)
    assert lib.tb_hadamard_mxfp4_quant(q, None) == _lib.TB_ERR_NULL_POINTER
    assert lib.tb_select(None, None, None) == _lib.TB_ERR_NULL_POINTER
    with pytest.raises(AssertionError, match="Incompatible Dimensions"):
        _lib.check(_lib.TB_ERR_BAD_SHAPE)
    with pytest.raises(RuntimeError):
        _lib.check(_lib.TB_ERR_BAD_TILE)


def test_grouped_descriptor_validation_and_workspace_size_without_a_gpu():
    """The grouped entry point's checks that need no device, and the workspace a Stream-K tail asks for: the flags
    and one fp32 256x256 partial tile per workgroup of a 256-CU grid when the 4-wave kernel can take it (K a
    multiple of 512), nothing otherwise."""
    from tritonblas_amd import _lib
    lib = _lib.load()
    g = _lib.tb_grouped_gemm_desc()
    assert lib.tb_grouped_gemm_fp8(g, None) == _lib.TB_ERR_BAD_ARGUMENT    # struct_bytes not set
    g.struct_bytes = C.sizeof(_lib.tb_grouped_gemm_desc)
    assert lib.tb_grouped_gemm_fp8(g, None) == _lib.TB_ERR_NULL_POINTER
    g.a = g.w = g.c = g.group_offsets = 256                                # (never dereferenced: the checks below fail first)
    g.c_type = _lib.TB_BF16
    g.m_total, g.n, g.k, g.num_groups = 8192, 14336, 4096, 8
    g.a_stride_m, g.w_stride_g, g.w_stride_n, g.c_stride_m, g.c_stride_n = 4096, 14336 * 4096, 4096, 14336, 1
    g.streamk = 2
    assert lib.tb_grouped_gemm_fp8(g, None) == _lib.TB_ERR_BAD_ARGUMENT
    g.streamk = 0
    g.small_rows = -2
    assert lib.tb_grouped_gemm_fp8(g, None) == _lib.TB_ERR_BAD_ARGUMENT
    g.small_rows = -1
    assert lib.tb_grouped_workspace_bytes(g) == 0                          # no Stream-K tail asked for
    g.streamk = 1
    _, flags_off = _lib.workspace_layout()
    assert lib.tb_grouped_workspace_bytes(g) == flags_off + 1024 + 256 * 256 * 256 * 4
    g.k = 4096 + 128                                                       # an odd number of K steps: 8-wave kernel, whole tiles
    g.a_stride_m = g.w_stride_n = g.k
    g.w_stride_g = 14336 * g.k
    assert lib.tb_grouped_workspace_bytes(g) == 0


def test_python_api_refuses_cpu_tensors():
    import tritonblas_amd as tb
    a = torch.zeros(16, 16, dtype=torch.float16)
    with pytest.raises(AssertionError, match="Incompatible Dimensions"):
        tb.matmul_lt(a, torch.zeros(8, 16, dtype=torch.float16), a, None, None)
    with pytest.raises(RuntimeError, match="GPU"):
        tb.matmul_lt(a, a, a.clone(), None, None)
    with pytest.raises(RuntimeError, match="differentiation"):
        tb.matmul(a.requires_grad_(), a, out=torch.zeros(16, 16, dtype=torch.float16))


# ---- tile order of the kernels (host evaluation through the C ABI) -------------------------------
import itertools


def _load():
    from tritonblas_amd import _lib
    return _lib.load()


def _coords(lib, t, tm, tn, gm, panel):
    pm, pn = C.c_int32(-1), C.c_int32(-1)
    assert lib.tb_tile_coords(t, tm, tn, gm, panel, C.byref(pm), C.byref(pn)) == 0
    return pm.value, pn.value


@pytest.mark.parametrize("tm,tn,gm", [(32, 112, 8), (4, 4, 8), (5, 7, 2), (1, 9, 8), (9, 1, 4), (13, 3, 8)])
def test_tile_order_without_panels_is_the_reference_swizzle(tm, tn, gm):
    from oracle import schedule as S
    lib = _load()
    for panel in (0, tn, tn + 5):
        assert [_coords(lib, t, tm, tn, gm, panel) for t in range(tm * tn)] == [S.tile_coords(t, tm, tn, gm) for t in range(tm * tn)]


@pytest.mark.parametrize("tm,tn,gm,panel", [(32, 112, 8, 16), (32, 112, 8, 32), (5, 7, 2, 3), (13, 30, 8, 4), (3, 9, 8, 1), (7, 10, 4, 9)])
def test_tile_order_with_panels_is_a_bijection_panel_by_panel(tm, tn, gm, panel):
    lib = _load()
    got = [_coords(lib, t, tm, tn, gm, panel) for t in range(tm * tn)]
    assert set(got) == set(itertools.product(range(tm), range(tn)))
    # panels are visited left to right, each completely before the next; inside a panel the order is
    # the reference swizzle of a (tm x width) problem
    from oracle import schedule as S
    pos = 0
    for first in range(0, tn, panel):
        width = min(panel, tn - first)
        want = [(m, first + n) for (m, n) in (S.tile_coords(t, tm, width, gm) for t in range(tm * width))]
        assert got[pos:pos + tm * width] == want
        pos += tm * width


def test_tile_coords_rejects_bad_arguments():
    from tritonblas_amd._lib import TB_ERR_BAD_ARGUMENT, TB_ERR_NULL_POINTER
    lib = _load()
    pm, pn = C.c_int32(), C.c_int32()
    assert lib.tb_tile_coords(12, 3, 4, 8, 0, C.byref(pm), C.byref(pn)) == TB_ERR_BAD_ARGUMENT
    assert lib.tb_tile_coords(0, 3, 4, 0, 0, C.byref(pm), C.byref(pn)) == TB_ERR_BAD_ARGUMENT
    assert lib.tb_tile_coords(0, 3, 4, 8, 0, None, C.byref(pn)) == TB_ERR_NULL_POINTER


def test_default_panel_is_a_near_square_multiple_of_the_xcd_block():
    lib = _load()
    assert lib.tb_default_panel(256, 32, 8) == 16     # 8 XCD blocks of 8x4 tiles -> rounds of 16x16
    assert lib.tb_default_panel(512, 64, 8) == 24
    assert lib.tb_default_panel(1, 1, 1) == 1
    assert lib.tb_default_panel(7, 1, 8) == 3


# ---- torch custom operators: registration and shape rules (no GPU needed) -------------------------
def test_custom_ops_are_registered_with_the_reference_signatures():
    import tritonblas_amd  # noqa: F401  (registers the operators)
    ops = torch.ops.tritonblas_amd
    assert str(ops._matmul.default._schema) == ("tritonblas_amd::_matmul(Tensor a, Tensor b, bool? enable_streamk=False, "
                                                "SymInt? sk_grid=None, bool? work_stealing=False) -> Tensor")
    assert "Tensor(a2!) out" in str(ops._matmul_out.default._schema) and str(ops._matmul_out.default._schema).endswith("-> ()")
    assert str(ops._addmm.default._schema).startswith("tritonblas_amd::_addmm(Tensor bias, Tensor a, Tensor b,")
    assert "Tensor(a3!) out" in str(ops._addmm_out.default._schema)


def test_custom_op_fake_implementations_propagate_shapes():
    import tritonblas_amd as tb
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        a = torch.empty(64, 32, device="cuda", dtype=torch.bfloat16)
        b = torch.empty(32, 48, device="cuda", dtype=torch.bfloat16)
        bias = torch.empty(48, device="cuda", dtype=torch.bfloat16)
        c = tb.matmul(a, b)
        assert tuple(c.shape) == (64, 48) and c.dtype == torch.bfloat16 and c.device.type == "cuda"
        assert tuple(tb.addmm(bias, a, b, enable_streamk=True).shape) == (64, 48)
        out = torch.empty(64, 48, device="cuda", dtype=torch.bfloat16)
        assert tb.matmul(a, b, out=out) is None and tb.addmm(bias, a, b, out=out) is None
        with pytest.raises(Exception, match="Incompatible A-B Dimensions"):
            tb.matmul(a, torch.empty(31, 48, device="cuda", dtype=torch.bfloat16))


# ---- work-stealing queues (host evaluation through the C ABI) ------------------------------------
from oracle import schedule as OS

TB_WS_QUEUES, TB_WS_GLOBAL_ATOMIC, TB_WS_HIERARCHICAL = 0, 1, 2


def _queue(lib, mode, q, total, X, S, local):
    cnt, tile = C.c_int32(-1), C.c_int32(-1)
    assert lib.tb_ws_queue_tile(mode, q, 0, total, X, S, local, C.byref(cnt), C.byref(tile)) == 0
    out = []
    for i in range(cnt.value):
        c2 = C.c_int32(-1)
        assert lib.tb_ws_queue_tile(mode, q, i, total, X, S, local, C.byref(c2), C.byref(tile)) == 0
        assert c2.value == cnt.value
        out.append(tile.value)
    assert lib.tb_ws_queue_tile(mode, q, cnt.value, total, X, S, local, C.byref(c2 if cnt.value else cnt), C.byref(tile)) == 0
    assert tile.value == -1
    return out


@pytest.mark.parametrize("total,X,S", [(1, 8, 4), (7, 8, 1), (64, 8, 8), (1000, 8, 4), (3584, 8, 1), (333, 4, 2), (50, 1, 3)])
def test_ws_flat_queues_follow_the_reference_ranges_and_cover_every_tile_once(total, X, S):
    lib = _load()
    seen = []
    for pid in range(X * S):   # workgroups 0..X*S-1 sit on distinct queues
        q, first, bound = OS.ws_slot_range(pid, total, X, S)
        got = _queue(lib, TB_WS_QUEUES, q, total, X, S, 0)
        assert got == list(range(first, first + bound))
        seen += got
    assert sorted(seen) == list(range(total))


@pytest.mark.parametrize("total,X", [(1, 8), (7, 8), (64, 8), (1001, 8), (333, 4), (50, 1)])
def test_ws_global_atomic_queue_is_the_chiplet_transform_of_the_counter(total, X):
    lib = _load()
    got = _queue(lib, TB_WS_GLOBAL_ATOMIC, 0, total, X, 4, 0)
    assert got == [OS.ws_global_atomic_tile(i, total, X) for i in range(total)]
    assert sorted(got) == list(range(total))
    # workgroup ids dealt round-robin to XCDs: consecutive counter values alternate between XCD runs
    if X > 1 and total >= 2 * X and total % X == 0:
        assert got[1] - got[0] == total // X


@pytest.mark.parametrize("total,X,local", [(1024, 8, 128), (1024, 8, 100), (9, 8, 1), (5, 8, 0), (3584, 8, 224), (77, 4, 10)])
def test_ws_hierarchical_queues(total, X, local):
    lib = _load()
    seen = []
    for xcd in range(X):
        got = _queue(lib, TB_WS_HIERARCHICAL, xcd, total, X, 4, local)
        assert got == [OS.ws_hierarchical_tile(xcd, i, 1, local, X) for i in range(local)]
        seen += got
    pool = _queue(lib, TB_WS_HIERARCHICAL, X, total, X, 4, local)
    assert pool == [OS.ws_hierarchical_tile(0, i, 2, local, X) for i in range(total - X * local)]
    assert sorted(seen + pool) == list(range(total))


def test_ws_queue_tile_rejects_bad_arguments():
    lib = _load()
    cnt, tile = C.c_int32(), C.c_int32()
    TB_ERR_NULL_POINTER, TB_ERR_BAD_ARGUMENT = -1, -10
    assert lib.tb_ws_queue_tile(3, 0, 0, 10, 8, 4, 0, C.byref(cnt), C.byref(tile)) == TB_ERR_BAD_ARGUMENT
    assert lib.tb_ws_queue_tile(0, 32, 0, 10, 8, 4, 0, C.byref(cnt), C.byref(tile)) == TB_ERR_BAD_ARGUMENT
    assert lib.tb_ws_queue_tile(1, 1, 0, 10, 8, 4, 0, C.byref(cnt), C.byref(tile)) == TB_ERR_BAD_ARGUMENT
    assert lib.tb_ws_queue_tile(2, 0, 0, 10, 8, 4, 2, C.byref(cnt), C.byref(tile)) == TB_ERR_BAD_ARGUMENT   # 8*2 > 10
    assert lib.tb_ws_queue_tile(0, 0, 0, 10, 8, 4, 0, None, C.byref(tile)) == TB_ERR_NULL_POINTER


def test_hierarchical_split_known_answers():
    # <= 4 tiles per CU: everything local; 14 tiles per CU and beyond: half
    assert OS.hierarchical_split(1024, 256, 8) == (128, 0)
    assert OS.hierarchical_split(512, 256, 8) == (64, 0)
    assert OS.hierarchical_split(3584, 256, 8) == (224, 1792)          # 14 per CU -> frac 0.5
    assert OS.hierarchical_split(256 * 20, 256, 8) == (320, 2560)      # floor at one half
    lp, g = OS.hierarchical_split(2048, 256, 8)                        # 8 per CU -> frac 0.8
    assert (lp, g) == (int(2048 * 0.8) // 8, 2048 - 8 * (int(2048 * 0.8) // 8))


@pytest.mark.parametrize("m,n,k", [(8192, 8192, 8192), (8192, 28672, 8192), (4096, 4096, 4096), (256, 256, 256), (16384, 16384, 1024)])
def test_selector_hierarchical_split_matches_the_reference_formula(m, n, k):
    import tritonblas_amd as tb
    sel = tb.OrigamiMatmulSelector(m, n, k, torch.bfloat16, torch.bfloat16, torch.bfloat16, "cpu")
    total = -(-m // sel.block_m) * -(-n // sel.block_n)
    hw = sel._hardware._c.num_xcd * sel._hardware._c.cu_per_xcd
    X = sel.num_sms
    want = OS.hierarchical_split(total, hw, X)
    got = sel.hierarchical_split(X)
    assert got[0] * X + got[1] == total and got[0] >= 0 and got[1] >= 0
    if want[1] >= 0:
        assert got == want
    else:   # fewer tiles than XCDs: the reference formula overshoots, the selector keeps the split valid
        assert got == (total // X, total - X * (total // X))


@pytest.mark.parametrize("remove,X,per", [(0, 8, 32), (1, 8, 32), (5, 8, 32), (31, 8, 32), (3, 4, 20), (2, 1, 7)])
def test_balanced_cu_mask(remove, X, per):
    from tritonblas_amd.benchmarks.common import build_balanced_hex_mask
    s = build_balanced_hex_mask(remove, X, per)
    assert s == OS.build_balanced_hex_mask(remove, X, per)
    if remove == 0:
        assert s == ""
        return
    v = int(s, 16)
    assert v < (1 << (X * per))
    for xcd in range(X):   # CU bit i sits on XCD i % X: every XCD loses exactly `remove` CUs, the lowest ones
        bits = [(v >> i) & 1 for i in range(xcd, X * per, X)]
        assert bits == [0] * remove + [1] * (per - remove)


def test_matmul_config_mask_rules():
    import tritonblas_amd as tb
    from tritonblas_amd.config import MatmulConfig
    cfg = MatmulConfig(device=torch.device("cpu"), workspace=None)
    assert cfg.mask is None and cfg.active_mask() is None and not cfg.global_atomic and not cfg.hierarchical
    m = torch.ones(8, dtype=torch.int32)
    cfg.mask = m            # a mask the caller assigns is used
    assert cfg.active_mask() is m
    cfg.mask = None
    assert cfg.active_mask() is None
    cfg2 = MatmulConfig(device=torch.device("cpu"), workspace=None, mask=m, use_mask=False)   # what matmul_preamble does with all CUs active
    assert cfg2.mask is m and cfg2.active_mask() is None


@pytest.mark.parametrize("total", [1, 5, 8, 9, 63, 512, 1024, 1100, 2048, 3584, 5120, 100000])
@pytest.mark.parametrize("hw_cus,xcds", [(256, 8), (304, 8), (64, 4), (32, 1)])
def test_library_hierarchical_split(total, hw_cus, xcds):
    lib = _load()
    l, g = C.c_int32(), C.c_int32()
    assert lib.tb_hierarchical_split(total, hw_cus, xcds, C.byref(l), C.byref(g)) == 0
    want = OS.hierarchical_split(total, hw_cus, xcds)
    assert l.value * xcds + g.value == total and l.value >= 0 and g.value >= 0
    if want[1] >= 0:
        assert (l.value, g.value) == want
    else:
        assert (l.value, g.value) == (total // xcds, total - xcds * (total // xcds))
    assert lib.tb_hierarchical_split(0, hw_cus, xcds, C.byref(l), C.byref(g)) == -10
    assert lib.tb_hierarchical_split(total, hw_cus, xcds, None, C.byref(g)) == -1


def test_grouped_gemm_refuses_other_operand_types():
    """the grouped entry point computes in FP8 e4m3 whatever it is handed: other types must not be read as that"""
    import tritonblas_amd as tb
    a = torch.zeros(8, 128, dtype=torch.float8_e5m2)
    w = torch.zeros(2, 16, 128, dtype=torch.float8_e5m2)
    c = torch.zeros(8, 16, dtype=torch.bfloat16)
    offs = torch.tensor([0, 4, 8], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="float8_e4m3fn"):
        tb.grouped_matmul_a8w8(a, w, None, None, c, offs)


def test_matmul_fp4_refuses_wrong_element_sizes_and_scale_shapes():
    import tritonblas_amd as tb
    a, b = torch.zeros(8, 64, dtype=torch.uint8), torch.zeros(16, 64, dtype=torch.uint8)
    c = torch.zeros(8, 16, dtype=torch.bfloat16)
    sa, sb = torch.zeros(8, 4, dtype=torch.uint8), torch.zeros(16, 4, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="one-byte"):
        tb.matmul_fp4(a.to(torch.bfloat16), b, c, sa, sb)
    with pytest.raises(RuntimeError, match="scales must be"):
        tb.matmul_fp4(a, b, c, sa.T.contiguous(), sb)


def _streamk_ranges(total, G, units, cut):
    """The K ranges the kernels give their workgroups for `cut` tiles at the end of a table (units of K per tile):
    workgroup i takes q units, the first `rem` workgroups one more, in the order of their ids."""
    first = (total - cut) * units
    q, rem = divmod(cut * units, G)
    return [(first + i * q + min(i, rem), first + (i + 1) * q + min(i + 1, rem)) for i in range(G)]


@pytest.mark.parametrize("G", [1, 5, 8, 12, 256])
def test_streamk_tail_rule_by_brute_force(G):
    """tb_streamk_tail_tiles against a walk of the ranges it implies: the answer is 0, the tail or the tail plus one
    round; the ranges cover every K unit of the cut tiles exactly once; no tile meets more ranges than the rule charged
    for; and among the three plans the answer is the cheapest by the critical path of that walk (whole rounds, then the
    longest range, then one exchange per extra piece of the most-cut tile)."""
    from tritonblas_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(G)
    for _ in range(300):
        total = int(rng.integers(1, 6 * G + 2))
        units = int(rng.integers(1, 17))
        unit_steps = int(rng.choice([1, 4]))
        fix = int(rng.integers(0, 40))
        cut = lib.tb_streamk_tail_tiles(total, G, units, unit_steps, fix)
        tail, rounds = total % G, total // G
        assert cut in {0, tail, tail + G} and cut <= total
        if tail == 0 or units < 2:
            assert cut == 0
            continue

        def walk_cost(c):
            if c == 0:
                return (rounds + 1) * units * unit_steps
            ranges = _streamk_ranges(total, G, units, c)
            cover = np.zeros(total * units, dtype=np.int32)
            pieces = {}
            for lo, hi in ranges:
                cover[lo:hi] += 1
                for t in range(lo // units, (hi + units - 1) // units if hi > lo else lo // units):
                    pieces[t] = pieces.get(t, 0) + 1
            assert (cover[(total - c) * units:] == 1).all() and (cover[:(total - c) * units] == 0).all()
            longest = max(hi - lo for lo, hi in ranges)
            return ((total - c) // G) * units * unit_steps + longest * unit_steps, max(pieces.values())

        options = [0, tail] + ([tail + G] if rounds >= 1 else [])
        costs = {}
        for c in options:
            if c == 0:
                costs[c] = walk_cost(0)
            else:
                base, most = walk_cost(c)
                # the rule's bound on the pieces of a tile is an upper bound of what the walk shows, and tight enough
                # that both agree on the price within one exchange
                q = (c * units) // G
                bound = min(units, ((units - 2) // max(q, 1) if units >= 2 else 0) + 2)
                assert most <= bound, (total, G, units, c, most, bound)
                costs[c] = base + (bound - 1) * fix
        assert costs[cut] == min(costs.values()), (total, G, units, unit_steps, fix, cut, costs)


def test_streamk_tail_rule_known_answers():
    """8 experts' 2072 tiles of 32 K steps on 256 workgroups: 8 whole rounds and 24 tiles.  Cutting the 24 tiles alone
    means eight pieces per tile; cutting them together with one whole round means two: with exchanges at 9 K steps the
    rule takes 280, at the library's 64 K steps it leaves the tiles whole, and with four times the K it cuts again."""
    from tritonblas_amd import _lib
    lib = _lib.load()
    assert lib.tb_streamk_tail_tiles(2072, 256, 8, 4, 9) == 280
    assert lib.tb_streamk_tail_tiles(2072, 256, 8, 4, 64) == 0
    assert lib.tb_streamk_tail_tiles(2072, 256, 32, 4, 64) == 280
    assert lib.tb_streamk_tail_tiles(2048, 256, 8, 4, 9) == 0          # whole rounds only
    assert lib.tb_streamk_tail_tiles(256 + 200, 256, 8, 4, 9) == 0     # a nearly full last round is cheaper whole
    assert lib.tb_streamk_tail_tiles(256 + 128, 256, 8, 4, 0) == 128   # free exchanges: always cut
    assert lib.tb_streamk_tail_tiles(100, 256, 8, 4, 9) in (0, 100)
    assert lib.tb_streamk_tail_tiles(10, 0, 8, 4, 9) == -10 and lib.tb_streamk_tail_tiles(10, 4, 8, 0, 9) == -10
