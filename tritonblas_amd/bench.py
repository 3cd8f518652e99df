"""Event-timed benchmark loop (reference include/tritonblas/bench.py:64-131): warm-up, then per
repetition: synchronise, reset/preamble callbacks, flush the caches by rewriting a 512 MiB buffer,
synchronise, time one call between two events."""
import torch

_CACHE_BYTES = 512 * 1024 * 1024
_cache = None


def _flush_cache(device):
    global _cache
    if _cache is None or _cache.device != device:
        _cache = torch.zeros(_CACHE_BYTES // 4, dtype=torch.int32, device=device)
    _cache.add_(1)


def do_bench(fn, reset_fn=lambda: None, preamble_fn=lambda: None, n_warmup=25, n_repeat=100, quantiles=None,
             return_mode="mean", flush=True):
    assert return_mode in ("min", "max", "mean", "median", "all")
    device = torch.device("cuda", torch.cuda.current_device())
    for _ in range(n_warmup):
        reset_fn()
        preamble_fn()
        fn()
    start = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    end = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for i in range(n_repeat):
        torch.cuda.synchronize()
        reset_fn()
        preamble_fn()
        if flush:
            _flush_cache(device)
        torch.cuda.synchronize()
        start[i].record()
        fn()
        end[i].record()
    torch.cuda.synchronize()
    times = torch.tensor([s.elapsed_time(e) for s, e in zip(start, end)], dtype=torch.float64)
    if quantiles is not None:
        return torch.quantile(times, torch.tensor(quantiles, dtype=torch.float64)).tolist()
    if return_mode == "all":
        return times.tolist()
    return getattr(torch, return_mode)(times).item()
