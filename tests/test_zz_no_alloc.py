"""tb_gemm_static_workspace: the entry point that allocates nothing (the Stream-K flags, partial tiles and
work-stealing counters live in a buffer inside the library's device image).  Called through the C ABI and
compared with tb_gemm on a caller-owned workspace: bit-equal results, two calls in a row, the second
with a smaller problem (the buffer keeps the first call's contents)."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _desc(_lib, a, b, c, schedule, grid):
    d = _lib.tb_gemm_desc()
    d.struct_bytes = C.sizeof(_lib.tb_gemm_desc)
    d.a_type = d.b_type = _lib.tb_dtype(a.dtype)
    d.c_type = _lib.tb_dtype(c.dtype)
    d.m, d.k = a.shape
    d.n = b.shape[1]
    d.a_stride_m, d.a_stride_k = a.stride()
    d.b_stride_k, d.b_stride_n = b.stride()
    d.c_stride_m, d.c_stride_n = c.stride()
    d.a, d.b, d.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
    d.schedule, d.grid = schedule, grid
    return d


@pytest.mark.parametrize("schedule", ["streamk", "work_stealing"])
def test_static_workspace_matches_caller_workspace(schedule):
    from tritonblas_amd import _lib
    lib = _lib.load()
    sched = _lib.TB_SCHED_STREAMK if schedule == "streamk" else _lib.TB_SCHED_WORK_STEALING
    g = torch.Generator(device="cuda").manual_seed(17)
    for (m, n, k, grid) in [(768, 1024, 2048, 100), (300, 200, 1920, 37)]:     # the second call is the smaller one
        a = (torch.randn(m, k, device="cuda", generator=g) * 0.5).bfloat16()
        b = (torch.randn(k, n, device="cuda", generator=g) * 0.5).bfloat16()
        want = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        d = _desc(_lib, a, b, want, sched, grid if schedule == "streamk" else 0)
        need = lib.tb_workspace_bytes(d)
        assert need > 0, "the case must use a workspace"
        ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
        d.workspace, d.workspace_bytes, d.epoch = ws.data_ptr(), need, 1
        assert lib.tb_gemm(d, _lib.stream_handle()) == _lib.TB_OK
        e = _desc(_lib, a, b, got, sched, grid if schedule == "streamk" else 0)
        assert lib.tb_gemm_static_workspace(e, _lib.stream_handle()) == _lib.TB_OK
        torch.cuda.synchronize()
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"{schedule} {m}x{n}x{k}"
        ref = (a.float() @ b.float()).bfloat16()
        assert ((got.float() - ref.float()).norm() / ref.float().norm()).item() <= 1e-3


def test_static_workspace_rejects_what_does_not_fit():
    """256 workgroups x 256x256 fp32 partial tiles = 64 MiB > the 16 MiB buffer: refused, nothing launched."""
    from tritonblas_amd import _lib
    lib = _lib.load()
    m, n, k = 4352, 4096, 4096    # 17 x 16 tiles of 256x256: a tail of 16 tiles shared by 256 workgroups
    a = torch.zeros(m, k, dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(k, n, dtype=torch.bfloat16, device="cuda")
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    d = _desc(_lib, a, b, c, _lib.TB_SCHED_STREAMK, 256)
    d.block_m, d.block_n, d.block_k = 256, 256, 64
    assert lib.tb_workspace_bytes(d) > 16 << 20
    assert lib.tb_gemm_static_workspace(d, _lib.stream_handle()) == _lib.TB_ERR_WORKSPACE


def test_static_workspace_status_word():
    """tb_static_workspace_status reads (and clears) the status word a poll-bound Stream-K launch sets in the
    library's own array.  The bound is forced from the host (one poll); every kernel still ends normally."""
    from tritonblas_amd import _lib
    lib = _lib.load()
    st = C.c_int(-1)
    assert lib.tb_static_workspace_status(C.byref(st), 1) == _lib.TB_OK
    assert lib.tb_static_workspace_status(C.byref(st), 0) == _lib.TB_OK and st.value == 0
    assert lib.tb_static_workspace_status(None, 0) == _lib.TB_ERR_NULL_POINTER
    m, n, k = 256, 256, 8192
    g = torch.Generator(device="cuda").manual_seed(5)
    a = (torch.randn(m, k, device="cuda", generator=g) * 0.5).bfloat16()
    b = (torch.randn(k, n, device="cuda", generator=g) * 0.5).bfloat16()
    c = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
    d = _desc(_lib, a, b, c, _lib.TB_SCHED_STREAMK, 16)
    d.block_m, d.block_n, d.block_k = 256, 256, 64
    d.spin_limit = 1
    assert lib.tb_gemm_static_workspace(d, _lib.stream_handle()) == _lib.TB_OK
    assert lib.tb_static_workspace_status(C.byref(st), 0) == _lib.TB_OK
    poisoned = bool(torch.isnan(c.float()).any())
    assert (st.value != 0) == poisoned
    assert lib.tb_static_workspace_status(C.byref(st), 1) == _lib.TB_OK
    assert lib.tb_static_workspace_status(C.byref(st), 0) == _lib.TB_OK and st.value == 0
    d.spin_limit = 0
    assert lib.tb_gemm_static_workspace(d, _lib.stream_handle()) == _lib.TB_OK
    torch.cuda.synchronize()
    ref = (a.float() @ b.float()).bfloat16()
    assert ((c.float() - ref.float()).norm() / ref.float().norm()).item() <= 1e-3
    assert lib.tb_static_workspace_status(C.byref(st), 0) == _lib.TB_OK and st.value == 0
