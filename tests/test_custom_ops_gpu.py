"""matmul / addmm as torch custom operators: autograd and torch.compile(fullgraph=True), following the
reference's tests/test_matmul_correctness.py and tests/test_addmm_correctness.py (forward and backward
against torch, out= semantics, persistent / Stream-K / work-stealing schedules, compiled and eager)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DIMS = [(128, 128, 128), (256, 512, 384), (96, 200, 72), (8, 8, 8), (1, 64, 32)]
TOL = dict(atol=1e-1, rtol=1e-1)   # the reference's tolerance for 16-bit types (test_matmul_correctness.py)


@pytest.fixture(autouse=True)
def _fresh_dynamo_cache():
    # every case compiles the same two Python functions with new shapes and flags: start each from an
    # empty cache instead of running into the recompile limit
    import torch._dynamo
    torch._dynamo.reset()
    yield


def _fn(fn, use_compile):
    # aot_eager: full Dynamo + AOTAutograd tracing (what needs the fake implementations and the autograd
    # registration) without depending on a code generator for the surrounding graph
    return torch.compile(fn, fullgraph=True, backend="aot_eager") if use_compile else fn


@pytest.mark.parametrize("use_compile", [False, True])
@pytest.mark.parametrize("schedule", ["persistent", "streamk", "work_stealing"])
@pytest.mark.parametrize("m,n,k", DIMS)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matmul_forward_backward(m, n, k, dtype, schedule, use_compile):
    import tritonblas_amd as tb
    print(f"custom op matmul {m}x{n}x{k} {dtype} {schedule} compile={use_compile}", flush=True)
    torch.manual_seed(42)
    kw = dict(enable_streamk=schedule == "streamk", work_stealing=schedule == "work_stealing")
    a = torch.randn(m, k, device="cuda", dtype=dtype, requires_grad=True)
    b = torch.randn(k, n, device="cuda", dtype=dtype, requires_grad=True)
    a_ref, b_ref = a.detach().clone().requires_grad_(True), b.detach().clone().requires_grad_(True)
    out = _fn(tb.matmul, use_compile)(a, b, **kw)
    ref = torch.matmul(a_ref, b_ref)
    torch.testing.assert_close(out, ref, **TOL)
    g = torch.randn_like(out)
    out.backward(g)
    ref.backward(g)
    torch.testing.assert_close(a.grad, a_ref.grad, **TOL)
    torch.testing.assert_close(b.grad, b_ref.grad, **TOL)


@pytest.mark.parametrize("use_compile", [False, True])
@pytest.mark.parametrize("schedule", ["persistent", "streamk"])
@pytest.mark.parametrize("m,n,k", DIMS)
def test_addmm_forward_backward(m, n, k, schedule, use_compile):
    import tritonblas_amd as tb
    print(f"custom op addmm {m}x{n}x{k} {schedule} compile={use_compile}", flush=True)
    torch.manual_seed(43)
    dtype = torch.bfloat16
    kw = dict(enable_streamk=schedule == "streamk")
    a = torch.randn(m, k, device="cuda", dtype=dtype, requires_grad=True)
    b = torch.randn(k, n, device="cuda", dtype=dtype, requires_grad=True)
    bias = torch.randn(n, device="cuda", dtype=dtype, requires_grad=True)
    refs = [t.detach().clone().requires_grad_(True) for t in (bias, a, b)]
    out = _fn(tb.addmm, use_compile)(bias, a, b, **kw)
    ref = torch.addmm(*refs)
    torch.testing.assert_close(out, ref, **TOL)
    g = torch.randn_like(out)
    out.backward(g)
    ref.backward(g)
    for got, want in zip((bias, a, b), refs):
        torch.testing.assert_close(got.grad, want.grad, **TOL)


@pytest.mark.parametrize("use_compile", [False, True])
def test_out_variants_write_in_place_and_refuse_autograd(use_compile):
    import tritonblas_amd as tb
    torch.manual_seed(44)
    a = torch.randn(64, 96, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(96, 80, device="cuda", dtype=torch.bfloat16)
    bias = torch.randn(80, device="cuda", dtype=torch.bfloat16)
    out = torch.zeros(64, 80, device="cuda", dtype=torch.bfloat16)
    assert _fn(tb.matmul, use_compile)(a, b, out=out) is None
    torch.testing.assert_close(out, torch.matmul(a, b), **TOL)
    out.zero_()
    assert _fn(tb.addmm, use_compile)(bias, a, b, out=out) is None
    torch.testing.assert_close(out, torch.addmm(bias, a, b), **TOL)
    a_g = a.clone().requires_grad_(True)
    with pytest.raises(RuntimeError, match="don't support automatic differentiation"):
        tb.matmul(a_g, b, out=out)
    with pytest.raises(RuntimeError, match="don't support automatic differentiation"):
        tb.addmm(bias, a_g, b, out=out)
    with torch.no_grad():
        assert tb.matmul(a_g, b, out=out) is None   # allowed when autograd is off (reference matmul.py:486)


def test_compiled_graph_mixes_custom_op_with_torch_ops():
    import tritonblas_amd as tb

    def f(x, w1, w2, bias):
        h = torch.relu(tb.addmm(bias, x, w1))
        return tb.matmul(h, w2).float().sum()

    torch.manual_seed(45)
    x = torch.randn(128, 64, device="cuda", dtype=torch.bfloat16)
    w1 = torch.randn(64, 256, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    w2 = torch.randn(256, 32, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    bias = torch.randn(256, device="cuda", dtype=torch.bfloat16)
    want = torch.matmul(torch.relu(torch.addmm(bias, x, w1)), w2).float().sum()
    got = torch.compile(f, fullgraph=True, backend="aot_eager")(x, w1, w2, bias)
    torch.testing.assert_close(got, want, rtol=2e-2, atol=2.0)
    got.backward()
    assert w1.grad is not None and w2.grad is not None and torch.isfinite(w1.grad).all()
