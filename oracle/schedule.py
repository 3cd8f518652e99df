"""Integer tile-schedule functions restated from the reference's device code (pure Python ints).

Test infrastructure: see ``oracle/__init__.py``.
"""


def cdiv(a, b):
    return -(-a // b)


def chiplet_transform(pid, num_workgroups, num_xcds):
    """include/tritonblas/kernels/stages/indexing/pid_transforms.py:6-16."""
    xcd = pid % num_xcds
    pos_in_xcd = pid // num_xcds
    min_per_xcd = num_workgroups // num_xcds
    extra = num_workgroups % num_xcds
    return xcd * min_per_xcd + min(xcd, extra) + pos_in_xcd


def chiplet_transform_chunked(pid, num_workgroups, num_xcds, chunk_size):
    """include/tritonblas/kernels/stages/indexing/pid_transforms.py:20-38 (note the strict '>')."""
    block = num_xcds * chunk_size
    if pid > (num_workgroups // block) * block:
        return pid
    local_pid = pid // num_xcds
    chunk_idx = local_pid // chunk_size
    pos_in_chunk = local_pid % chunk_size
    xcd = pid % num_xcds
    return chunk_idx * block + xcd * chunk_size + pos_in_chunk


def tile_coords(tile_id, num_pid_m, num_pid_n, group_m):
    """GROUP_M swizzle: include/tritonblas/kernels/stages/schedule.py:124-145."""
    num_pid_in_group = group_m * num_pid_n
    group_id = tile_id // num_pid_in_group
    first_pid_m = group_id * group_m
    gsz = min(num_pid_m - first_pid_m, group_m)
    pid_m = first_pid_m + ((tile_id % num_pid_in_group) % gsz)
    pid_n = (tile_id % num_pid_in_group) // gsz
    return pid_m, pid_n


def launch_chunk_size(group_m, total_programs, num_xcds):
    """include/tritonblas/matmul.py:105-110."""
    chunk = group_m * group_m
    if num_xcds > 0:
        chunk = min(chunk, max(1, total_programs // num_xcds))
    return chunk


def streamk_partition(total_tiles, grid):
    """include/tritonblas/matmul.py:238-241: tiles handled by the Stream-K tail."""
    return total_tiles % grid if grid > 0 else 0


def streamk_iter_range(pid, grid, total_tiles, sk_tiles, iters_per_tile):
    """include/tritonblas/kernels/stages/schedule.py:190-223 / streamk_gemm.py:175-181."""
    full = total_tiles - sk_tiles
    total_sk_iters = sk_tiles * iters_per_tile
    q, r = divmod(total_sk_iters, grid)
    start = full * iters_per_tile + pid * q + min(pid, r)
    end = full * iters_per_tile + (pid + 1) * q + min(pid + 1, r)
    return start, end


def streamk_segments(pid, grid, total_tiles, sk_tiles, iters_per_tile):
    """Segments [(tile, k_first, k_last_exclusive, is_tile_start)] one workgroup walks in its Stream-K
    range: include/tritonblas/kernels/streamk_gemm.py:184-187."""
    start, last = streamk_iter_range(pid, grid, total_tiles, sk_tiles, iters_per_tile)
    out = []
    while start < last:
        rem = start % iters_per_tile
        end = min(start + (iters_per_tile - rem), last)
        tile = start // iters_per_tile
        out.append((tile, rem, rem + (end - start), rem == 0))
        start = end
    return out


def streamk_walk_last_owner(wg, grid, total_tiles, sk_tiles, iters_per_tile):
    """The order in which the LIBRARY's Stream-K kernel walks the same iteration range (the range is the
    reference's, streamk_iter_range above; the walk is not: the reference's first segment owns the tile
    and spins on locks of later programs, streamk_gemm.py:248-324, which needs every program resident).
    Here `wg` is the raw workgroup id, the range is walked from its end, and the workgroup holding a
    tile's last iterations finishes it.  Returns [(tile, k_first, k_last_exclusive, kind, waits_for)]
    in processing order; kind is "publish" or "owner", waits_for the workgroup ids whose partials the
    owner adds, in that order."""
    start, last = streamk_iter_range(wg, grid, total_tiles, sk_tiles, iters_per_tile)
    q, r = divmod(sk_tiles * iters_per_tile, grid)
    out = []
    while start < last:
        tile = (last - 1) // iters_per_tile
        tile_first = tile * iters_per_tile
        begin = max(tile_first, start)
        if last != tile_first + iters_per_tile:
            out.append((tile, begin - tile_first, last - tile_first, "publish", []))
        else:
            waits, cur, nxt = [], begin, wg - 1
            while cur > tile_first:
                waits.append(nxt)
                cur -= q + (1 if nxt < r else 0)
                nxt -= 1
            out.append((tile, begin - tile_first, last - tile_first, "owner", waits))
        last = begin
    return out


def ws_slot_range(pid, total_tiles, num_xcds, counters_per_xcd):
    """Flat work-stealing queue a workgroup pulls from:
    include/tritonblas/kernels/persistent_gemm_work_stealing.py:296-314.
    Returns (counter_index, first_tile, bound)."""
    xcd = pid % num_xcds
    tiles_per_xcd = cdiv(total_tiles, num_xcds)
    slot = (pid // num_xcds) % counters_per_xcd
    xcd_base = xcd * tiles_per_xcd
    xcd_end = min(xcd_base + tiles_per_xcd, total_tiles)
    tiles_this_xcd = max(xcd_end - xcd_base, 0)
    tiles_per_slot = cdiv(tiles_this_xcd, counters_per_xcd)
    slot_base = slot * tiles_per_slot
    slot_end = min(slot_base + tiles_per_slot, tiles_this_xcd)
    return xcd * counters_per_xcd + slot, xcd_base + slot_base, max(slot_end - slot_base, 0)


def grouped_tile_lookup(tile_id, offsets, block_m, tiles_n):
    """Grouped (MoE) tile table: experts in order, each contributes cdiv(rows_e, block_m) * tiles_n
    tiles, m-block fastest.  Returns (expert, m_block, n_block) or None past the end.  New work, no
    reference counterpart."""
    acc = 0
    for e in range(len(offsets) - 1):
        rows = offsets[e + 1] - offsets[e]
        mb = cdiv(rows, block_m) if rows > 0 else 0
        cnt = mb * tiles_n
        if tile_id < acc + cnt:
            local = tile_id - acc
            return e, local % mb, local // mb
        acc += cnt
    return None


def grouped_two_launch_blocks(offsets, phase, big_m, small_rows, block_m):
    """Row blocks (expert, first_row, end_row) of a grouped GEMM split over two launches: phase 1
    tiles each expert's rows with big_m-row blocks but leaves a last partial block of at most
    small_rows rows to phase 2, which tiles exactly those rows with block_m-row blocks.  Listed in the
    table's order (experts ascending, blocks ascending).  New work, no reference counterpart."""
    out = []
    for e in range(len(offsets) - 1):
        lo, hi = offsets[e], offsets[e + 1]
        rows = max(hi - lo, 0)
        full, rem = divmod(rows, big_m)
        small = 0 < rem <= small_rows
        if phase == 1:
            mb = full + (1 if rem > 0 and not small else 0)
            lim = lo + full * big_m if small else hi
            out += [(e, lo + i * big_m, min(lo + (i + 1) * big_m, lim)) for i in range(mb)]
        else:
            base = lo + full * big_m
            mb = cdiv(rem, block_m) if small else 0
            out += [(e, base + i * block_m, min(base + (i + 1) * block_m, hi)) for i in range(mb)]
    return out


def grouped_split_pays(offsets, big_m, small_rows, small_m, tiles_n_big, tiles_n_small, grid_big, grid_small):
    """The verdict both launches of a grouped GEMM reach on the device from the row counts: split when
    4 * rounds(tall tiles of the split plan) + 3 * rounds(short tiles) < 4 * rounds(tall tiles of the
    one-launch plan) and there is a short block at all (a round of short tiles streams half a tall
    round's weight bytes but is bound by that stream: measured at three quarters of a tall round).
    New work, no reference counterpart."""
    one = len(grouped_two_launch_blocks(offsets, 1, big_m, 0, big_m))
    b1 = len(grouped_two_launch_blocks(offsets, 1, big_m, small_rows, big_m))
    b2 = len(grouped_two_launch_blocks(offsets, 2, big_m, small_rows, small_m))
    cost_one = 4 * cdiv(one * tiles_n_big, grid_big)
    cost_two = 4 * cdiv(b1 * tiles_n_big, grid_big) + 3 * cdiv(b2 * tiles_n_small, grid_small)
    return b2 > 0 and cost_two < cost_one


def ws_global_atomic_tile(raw_idx, total_tiles, num_xcds):
    """Tile a work-stealing workgroup gets for counter value raw_idx in GLOBAL_ATOMIC mode
    (reference kernels/persistent_gemm_work_stealing.py:292-295, 321)."""
    return chiplet_transform(raw_idx, total_tiles, num_xcds)


def ws_hierarchical_tile(xcd, raw_idx, level, local_tiles_per_xcd, num_xcds):
    """HIERARCHICAL mode (reference persistent_gemm_work_stealing.py:106-122, 211-216): level 1 takes
    from the XCD's own run of local_tiles_per_xcd tiles, level 2 from the pool behind all local runs."""
    if level == 1:
        return xcd * local_tiles_per_xcd + raw_idx
    return local_tiles_per_xcd * num_xcds + raw_idx


def hierarchical_split(total_tiles, hw_cus, num_xcds):
    """(local_per_xcd, global_tiles), reference origami.py:288-311 verbatim in arithmetic."""
    tiles_per_cu = total_tiles / max(hw_cus, 1)
    local_frac = max(0.5, 1.0 - max(0.0, tiles_per_cu - 4.0) * 0.05)
    local_per_xcd = int(total_tiles * local_frac) // num_xcds
    local_per_xcd = max(local_per_xcd, 1)
    return local_per_xcd, total_tiles - local_per_xcd * num_xcds


def build_balanced_hex_mask(remove_per_xcd, num_xcds, cus_per_xcd):
    """CU-mask string that removes remove_per_xcd CUs from every XCD (CU bit i belongs to XCD
    i % num_xcds; reference benchmarks/common.py:34-45)."""
    if remove_per_xcd == 0:
        return ""
    total = num_xcds * cus_per_xcd
    mask = (1 << total) - 1
    for i in range(remove_per_xcd):
        for xcd in range(num_xcds):
            mask &= ~(1 << (num_xcds * i + xcd))
    return f"0x{mask:x}"
