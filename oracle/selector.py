"""Host-side selector arithmetic that is fully specified inside the reference tree.

Test infrastructure: see ``oracle/__init__.py``.  The tile *choice* itself is made by an external
C++ library (origami, ROCm/rocm-libraries shared/origami @66af6cd8, fetched by setup.py:27-73) whose
source is not part of the reference tree: its parity is unpinned.
"""
from math import ceil


def estimate_lds_bytes(block_m, block_n, block_k, bytes_a, bytes_b, num_stages=2):
    """include/tritonblas/origami.py:9-43."""
    a = block_m * block_k * bytes_a
    b = block_k * block_n * bytes_b
    if num_stages <= 1:
        return max(a, b)
    return (num_stages - 1) * (a + b)


def check_lds_capacity(block_m, block_n, block_k, bytes_a, bytes_b, lds_capacity, num_stages=2):
    """include/tritonblas/origami.py:46-59."""
    return estimate_lds_bytes(block_m, block_n, block_k, bytes_a, bytes_b, num_stages) <= lds_capacity


def partial_tile_size(block_m, block_n, out_bits, sk_grid):
    """include/tritonblas/origami.py:418-437."""
    return block_m * block_n * (out_bits // 8) * sk_grid


def compute_sk_grid(M, N, K, block_m, block_n, block_k, cu_count, out_bits=16):
    """include/tritonblas/origami.py:349-416."""
    split_factors = [8, 6, 4, 3, 2, 1]
    tile_fractions = [0.0, 1.0 / 2.0, 1.0 / 8.0, 1.0 / 5.0, 1.0 / 4.0, 1.0 / 3.0]
    max_workspace = 128 * 1024 * 1024
    tiles = ceil(M / block_m) * ceil(N / block_n)
    sk_grid = tiles
    iters_per_tile = max(1, ceil(K / block_k))
    if tiles > cu_count:
        min_even_tiles = tiles / cu_count
        for frac in tile_fractions:
            frac_grid = int((tiles / (min_even_tiles + frac)) + 0.5)
            if tiles % frac_grid != 0 and partial_tile_size(block_m, block_n, out_bits, frac_grid) > max_workspace:
                continue
            if frac_grid <= cu_count:
                sk_grid = frac_grid
                break
    elif tiles < cu_count:
        for factor in split_factors:
            split_grid = tiles * factor
            iters_per_cu = iters_per_tile // factor
            if split_grid <= cu_count and iters_per_cu >= 8:
                sk_grid = split_grid
                break
    if tiles % sk_grid != 0:
        sk_grid = tiles
    if tiles >= cu_count:
        rem = tiles % cu_count
        if rem < 128 and rem > 0 and cu_count in [304, 80, 64]:
            sk_grid = 256 if cu_count == 304 else 64
    return sk_grid


def ws_counters_per_xcd(total_tiles):
    """include/tritonblas/origami.py:266-286."""
    if total_tiles <= 512:
        return 8
    if total_tiles <= 1536:
        return 4
    if total_tiles <= 2048:
        return 2
    return 1
