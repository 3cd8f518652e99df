"""Seeded synthetic inputs for the five benchmark configurations (CPU generator, so the CPU oracle
and the GPU consume identical bits; the reference draws on the GPU RNG, include/tritonblas/utils.py:297,
which cannot be reproduced off-GPU).  B's seed is A's seed + 10000 (include/tritonblas/utils.py:501).

Test infrastructure: see ``oracle/__init__.py``.
"""
import torch


def _g(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def c1_fp16(m=1024, n=1024, k=1024):
    a = (torch.randn(m, k, generator=_g(0)) * 0.1).half()
    b = (torch.randn(k, n, generator=_g(10000)) * 0.1).half()
    return a, b


def c2_bf16(m=8192, n=8192, k=8192):
    """TN: A (m,k) K-contiguous; B stored (n,k) K-contiguous, used as its transpose view."""
    a = (torch.rand(m, k, generator=_g(1)) * 2 - 1).bfloat16()
    bt = (torch.rand(n, k, generator=_g(10001)) * 2 - 1).bfloat16()
    return a, bt.T


def c3_fp8_source(m, n, k):
    a = torch.randn(m, k, generator=_g(2)).bfloat16()
    w = torch.randn(n, k, generator=_g(10002)).bfloat16()
    return a, w


def c4_moe_source(tokens=4096, experts=8, topk=2, n=14336, k=4096):
    idx = torch.multinomial(torch.ones(tokens, experts), topk, replacement=False, generator=_g(3))
    counts = torch.bincount(idx.flatten(), minlength=experts)
    offsets = torch.zeros(experts + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)
    a = torch.randn(tokens * topk, k, generator=_g(4)).bfloat16()
    w = torch.randn(experts, n, k, generator=_g(10004)).bfloat16()
    return a, w, offsets


def c5_mxfp4_source(m=8192, n=8192, k=16384):
    def one(rows, seed):
        g = _g(seed)
        x = torch.randn(rows, k, generator=g)
        mask = torch.rand(rows, k, generator=g) < 1e-3
        return torch.where(mask, x * 20.0, x).bfloat16()
    return one(m, 5), one(n, 10005)
