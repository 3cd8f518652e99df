"""Tile selector with the reference's ``OrigamiMatmulSelector`` surface
(include/tritonblas/origami.py:62-347), backed by the in-library analytical model (``tb_select``)
instead of the external origami package.
"""
from __future__ import annotations

from types import SimpleNamespace

import torch

from . import _lib


def estimate_triton_lds_bytes(block_m, block_n, block_k, bytes_a, bytes_b, num_stages: int = 2) -> float:
    """LDS footprint model of a software-pipelined tile (reference origami.py:9-43)."""
    a_bytes = block_m * block_k * bytes_a
    b_bytes = block_k * block_n * bytes_b
    if num_stages <= 1:
        return max(a_bytes, b_bytes)
    return (num_stages - 1) * (a_bytes + b_bytes)


def check_triton_lds_capacity(block_m, block_n, block_k, bytes_a, bytes_b, lds_capacity, num_stages: int = 2) -> bool:
    """Reference origami.py:46-59."""
    return estimate_triton_lds_bytes(block_m, block_n, block_k, bytes_a, bytes_b, num_stages) <= lds_capacity


def _dtype_bits(dtype) -> int:
    if isinstance(dtype, str):
        return 4
    try:
        return torch.finfo(dtype).bits
    except TypeError:
        return torch.iinfo(dtype).bits


def hardware_for_device(device_index) -> SimpleNamespace:
    """Hardware descriptor with the attribute names the reference reads (N_CU, NUM_XCD, CU_per_L2,
    lds_capacity, arch.name).  Without a GPU the MI355X defaults are returned."""
    lib = _lib.load()
    hw = _lib.tb_hw()
    idx = -1
    if device_index is not None and torch.cuda.is_available():
        idx = int(device_index)
    _lib.check(lib.tb_device_info(idx, hw), "tb_device_info")
    return SimpleNamespace(N_CU=hw.n_cu, NUM_XCD=hw.num_xcd, CU_per_L2=hw.cu_per_xcd, lds_capacity=hw.lds_bytes,
                           arch=SimpleNamespace(name=hw.arch.decode()), _c=hw)


class OrigamiMatmulSelector:
    """Same constructor and read-only properties as the reference (origami.py:98-347)."""

    estimate_triton_lds = staticmethod(estimate_triton_lds_bytes)
    COUNTERS_PER_XCD = 4

    def __init__(self, m: int, n: int, k: int, a_dtype, b_dtype, out_dtype, device, mx_block_size=0,
                 streamk=False, total_cus: int = None, active_cus: int = None, num_stages: int = 2):
        self._m, self._n, self._k = int(m), int(n), int(k)
        self.streamk = bool(streamk)
        self._mx_block_size = mx_block_size
        self._a_dtype, self._b_dtype, self._out_dtype = a_dtype, b_dtype, out_dtype
        self._a_dtype_bitsize = _dtype_bits(a_dtype)
        self._b_dtype_bitsize = _dtype_bits(b_dtype)
        self._out_dtype_bitsize = _dtype_bits(out_dtype)
        dev_index = None
        if device is not None:
            device = torch.device(device)
            if device.type == "cuda":
                dev_index = device.index if device.index is not None else (
                    torch.cuda.current_device() if torch.cuda.is_available() else None)
        self._hardware = hardware_for_device(dev_index)
        self._arch_name = self._hardware.arch.name
        if total_cus is not None:
            self._hardware.N_CU = total_cus
            self._hardware._c.n_cu = total_cus
        self._total_cus = total_cus
        self._N_CU = self._hardware.N_CU
        self._ACTIVE_CU = active_cus if active_cus is not None else self._N_CU
        self._active_cus = active_cus

        prob = _lib.tb_problem(m=self._m, n=self._n, k=self._k, a_type=_lib.tb_dtype(a_dtype),
                               b_type=_lib.tb_dtype(b_dtype), c_type=_lib.tb_dtype(out_dtype),
                               a_k_contiguous=1, b_k_contiguous=1, streamk=int(self.streamk), num_groups=0)
        sel = _lib.tb_selection()
        _lib.check(_lib.load().tb_select(prob, self._hardware._c, sel), "tb_select")
        self._sel = sel
        self._num_stages = sel.num_stages
        self._grid = sel.sk_grid if self.streamk else self._N_CU
        self._workgroup_mapping = sel.group_m
        self._xcc_workgroup_mapping = sel.num_xcds
        self.COUNTERS_PER_XCD = sel.counters_per_xcd

    block_m = property(lambda self: self._sel.block_m)
    block_n = property(lambda self: self._sel.block_n)
    block_k = property(lambda self: self._sel.block_k)
    group_m = property(lambda self: self._workgroup_mapping)
    num_sms = property(lambda self: self._xcc_workgroup_mapping)
    num_stages = property(lambda self: self._num_stages)
    waves_per_eu = property(lambda self: self._sel.occupancy)
    sk_grid = property(lambda self: self._grid)
    estimate_us = property(lambda self: self._sel.est_total_us)

    def hierarchical_split(self, num_xcds: int) -> tuple:
        """(local_tiles_per_xcd, global_tiles) of the hierarchical work-stealing mode (reference
        origami.py:288-311): up to 4 tiles per CU everything is XCD-local; above that the local share
        falls by 5 % per extra tile per CU down to one half, the rest goes to the pool every XCD
        steals from.  Uses the hardware CU count, not the active one.  Where the reference's formula
        hands out more local tiles than there are (fewer tiles than XCDs), the local queues get what
        divides evenly instead."""
        bm, bn = self.block_m, self.block_n
        total_tiles = ((self._m + bm - 1) // bm) * ((self._n + bn - 1) // bn)
        hw_cus = self._hardware._c.num_xcd * self._hardware._c.cu_per_xcd
        local, pool = _lib.C.c_int32(), _lib.C.c_int32()
        _lib.check(_lib.load().tb_hierarchical_split(total_tiles, hw_cus, int(num_xcds), _lib.C.byref(local), _lib.C.byref(pool)),
                   "tb_hierarchical_split")
        return local.value, pool.value

    @property
    def even_k(self):
        return self._k % self.block_k == 0

    def __repr__(self):
        return (f"OrigamiMatmulSelector({self._m}x{self._n}x{self._k}, tile={self.block_m}x{self.block_n}x{self.block_k}, "
                f"group_m={self.group_m}, xcds={self.num_sms}, sk_grid={self.sk_grid})")
