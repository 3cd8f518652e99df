"""Launches recorded into a HIP graph and replayed: the arguments of a replayed launch cannot change, so
nothing in them may have to (Stream-K partial tiles are tagged with a count the workspace keeps itself,
the work-stealing queues rearm themselves).  Every replay runs on new operand values, with eager work and
synchronisation in between, and is compared with the eager result of the same call."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("mode", ["streamk", "work_stealing", "persistent", "streamk+work_stealing"])
def test_python_launch_replays(mode):
    import tritonblas_amd as tb
    m, n, k = 512, 768, 4096
    _say(f"graph replay {mode}")
    g = torch.Generator(device="cuda").manual_seed(31)
    a = (torch.randn(m, k, device="cuda", generator=g) * 0.5).bfloat16()
    b = (torch.randn(k, n, device="cuda", generator=g) * 0.5).bfloat16()
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    sel = tb.OrigamiMatmulSelector(m, n, k, a.dtype, b.dtype, c.dtype, a.device, streamk="streamk" in mode)
    cfg = tb.matmul_preamble(sel)
    cfg_eager = tb.matmul_preamble(sel)
    kw = dict(enable_streamk="streamk" in mode, work_stealing="work_stealing" in mode)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):                      # plans, workspace and occupancy queries happen here, not under capture
            tb.matmul_lt(a, b, c, sel, cfg, **kw)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        tb.matmul_lt(a, b, c, sel, cfg, **kw)
    for rep in range(4):
        a.copy_((torch.randn(m, k, device="cuda", generator=g) * 0.5).bfloat16())
        c.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        want = torch.zeros_like(c)
        tb.matmul_lt(a, b, want, sel, cfg_eager, **kw)
        torch.cuda.synchronize()
        assert torch.equal(c.view(torch.int16), want.view(torch.int16)), f"replay {rep}"
        ref = (a.float() @ b.float())
        assert ((c.float() - ref).norm() / ref.norm()).item() <= 2e-3
    if "streamk" in mode:
        assert cfg.status() == 0


def test_static_workspace_streamk_replays():
    """The entry point that allocates nothing, Stream-K with an explicit grid, through the C ABI under capture."""
    from tritonblas_amd import _lib
    lib = _lib.load()
    m, n, k, grid = 768, 1024, 2048, 100
    g = torch.Generator(device="cuda").manual_seed(32)
    a = (torch.randn(m, k, device="cuda", generator=g) * 0.5).bfloat16()
    b = (torch.randn(k, n, device="cuda", generator=g) * 0.5).bfloat16()
    c = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")

    def desc(out):
        d = _lib.tb_gemm_desc()
        d.struct_bytes = C.sizeof(_lib.tb_gemm_desc)
        d.a_type = d.b_type = d.c_type = _lib.TB_BF16
        d.m, d.n, d.k = m, n, k
        d.a_stride_m, d.a_stride_k = a.stride()
        d.b_stride_k, d.b_stride_n = b.stride()
        d.c_stride_m, d.c_stride_n = out.stride()
        d.a, d.b, d.c = a.data_ptr(), b.data_ptr(), out.data_ptr()
        d.schedule, d.grid = _lib.TB_SCHED_STREAMK, grid
        return d

    d = desc(c)
    assert lib.tb_workspace_bytes(d) > 0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert lib.tb_gemm_static_workspace(d, _lib.stream_handle()) == _lib.TB_OK
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert lib.tb_gemm_static_workspace(d, _lib.stream_handle()) == _lib.TB_OK
    for rep in range(4):
        a.copy_((torch.randn(m, k, device="cuda", generator=g) * 0.5).bfloat16())
        c.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        want = torch.zeros_like(c)
        e = desc(want)
        ws = torch.zeros(lib.tb_workspace_bytes(e), dtype=torch.uint8, device="cuda")
        e.workspace, e.workspace_bytes, e.epoch = ws.data_ptr(), ws.numel(), 1
        assert lib.tb_gemm(e, _lib.stream_handle()) == _lib.TB_OK
        torch.cuda.synchronize()
        assert torch.equal(c.view(torch.int16), want.view(torch.int16)), f"replay {rep}"
