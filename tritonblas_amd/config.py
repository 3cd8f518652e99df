"""Launch state kept between calls: one device workspace that holds the work-stealing queue
counters or the Stream-K flags + partial tiles (reference include/tritonblas/config.py:10-134).

Layout of the workspace (bytes, ``tb_workspace_layout``): [0, 256) control words (status, done
counter); the work-stealing queue counters, one per 256-byte line; the Stream-K flags (one 32-bit word
per workgroup) followed by the fp32 partial tiles.  The regions are disjoint, so Stream-K and
work-stealing launches may share one config in any order.  Stream-K flags carry the launch epoch, so
nothing has to be cleared between launches; the work-stealing queues are rearmed by the kernel itself.
``reset()`` is still available after an aborted launch.

A Stream-K owner that waits for a partner's partial tile longer than ``spin_limit`` polls (the partner
is not resident: another kernel holds its CU, or the stream is CU-masked) gives up: it stores its tile as
NaN and sets the status word.  The launch itself cannot report this -- it is asynchronous -- so a caller
that shares the device calls ``check()`` (which synchronises) when it wants to know.
"""
import torch

from . import _lib

COUNTER_STRIDE = 64   # int32 between counters = 256 bytes
MAX_SK_TILES = 512
_CTL_BYTES = 256


class MatmulConfig:
    """``mask``: int32 per-workgroup enable mask of the work-stealing launch (1 = takes tiles, 0 = leaves
    at once; reference config.py:23).  A mask that ``matmul_preamble`` made for a selector with all CUs
    active is not handed to the kernel (the launch then keeps its default, occupancy-filling grid);
    a mask with masked-out entries, or one the caller assigns, is, and the launch has one workgroup
    per mask entry like the reference's.  ``global_atomic`` / ``hierarchical`` pick the single-counter
    and the XCD-local-then-shared-pool queueing of the reference's work-stealing kernel."""

    def __init__(self, device: torch.device, workspace: torch.Tensor, selector=None, mask: torch.Tensor = None,
                 global_atomic: bool = False, hierarchical: bool = False, use_mask: bool = None):
        self.device = device
        self.workspace = workspace
        self.selector = selector
        self._mask = mask
        self._use_mask = (mask is not None) if use_mask is None else use_mask
        self.global_atomic = global_atomic
        self.hierarchical = hierarchical
        self.epoch = 0
        self._retired = []      # outgrown workspaces (kept: a captured launch may still name them)
        self.spin_limit = 0     # Stream-K: polls per wait before an owner gives up (0: the library's 2**24)

    @property
    def mask(self):
        return self._mask

    @mask.setter
    def mask(self, value):
        self._mask = value
        self._use_mask = value is not None

    def active_mask(self):
        """The mask the kernel should look at, or None."""
        return self._mask if self._use_mask else None

    def ensure(self, nbytes: int):
        """Grow the workspace to at least nbytes (zero-initialised).  A workspace that has been handed to a
        launch is never freed: a launch captured into a HIP graph holds its raw pointer, so the buffers this
        config outgrows stay alive with it (a captured graph pins its config).  Under stream capture nothing
        may be allocated or cleared -- the fill would become a node of the graph -- so a call that would have
        to grow the workspace there raises: make the first call outside the capture."""
        if self.workspace is None or self.workspace.numel() < nbytes:
            if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
                raise RuntimeError("tritonblas_amd: this launch needs a larger workspace than its config holds, and "
                                   "the stream is being captured; run the call once outside the capture first")
            if self.workspace is not None:
                self._retired.append(self.workspace)
            self.workspace = torch.zeros(int(nbytes), dtype=torch.uint8, device=self.device)
            self.epoch = 0
        return self.workspace

    def next_epoch(self) -> int:
        """A host-side epoch for callers that drive tb_gemm themselves with this config's workspace (the
        package's own launches let the workspace count: _lib.TB_EPOCH_ON_DEVICE; do not mix the two on one
        workspace without reset()).  Epochs only count upwards; before they would wrap the workspace is cleared."""
        if self.epoch >= 0x7FFFFFFF:
            self.workspace.zero_()
            self.epoch = 0
        self.epoch += 1
        return self.epoch

    # views under the reference's attribute names (config.py:32-43) ---------------------------------
    # The reference keeps one buffer per purpose; here they are windows into the one workspace.  The
    # kernels do not use a global counter, per-iteration counters or "done" bytes: those names return
    # empty tensors so that code which only resets them keeps working.
    def _region(self, lo, hi, dtype=torch.int32):
        ws = self.workspace
        if ws is None or ws.numel() < hi:
            return torch.empty(0, dtype=dtype, device=self.device)
        return ws[lo:hi].view(dtype)

    @property
    def tile_counter(self):
        counters, flags = _lib.workspace_layout()
        return self._region(counters, flags)

    streamk_tile_counter = tile_counter

    @property
    def locks(self):
        _, flags = _lib.workspace_layout()
        grid = self.selector.sk_grid if self.selector is not None else 0
        return self._region(flags, flags + 4 * grid)

    sk_locks = locks

    @property
    def P(self):
        sel = self.selector
        grid = sel.sk_grid
        _, flags = _lib.workspace_layout()
        off = flags + ((grid * 4 + 255) // 256) * 256
        blk = sel.block_m * sel.block_n
        return self._region(off, off + grid * blk * 4, torch.float32).view(-1, blk)

    sk_P = P

    @property
    def global_counter(self):
        return torch.empty(0, dtype=torch.int32, device=self.device)

    sk_iter_counter = global_counter
    sk_done = global_counter

    def status(self) -> int:
        """Control word 0: non-zero after a Stream-K wait ran into its poll bound (synchronises)."""
        return int(self.workspace[:4].view(torch.int32).item())

    def clear_status(self):
        self.workspace[:4].zero_()

    def check(self):
        """Raise if a Stream-K launch on this config gave up waiting for a partial tile (it then wrote
        NaN tiles).  Synchronises with the device; clears the status."""
        if self.workspace is not None and self.status() != 0:
            self.clear_status()
            raise RuntimeError("tritonblas_amd: a Stream-K launch ran into its poll bound (a partner workgroup was "
                               "not resident); the tiles it could not finish hold NaN")

    def reset(self, streamk: bool = False, work_stealing: bool = False):
        """Clear mutable state (reference config.py:54-75)."""
        if (streamk or work_stealing) and self.workspace is not None:
            self.workspace.zero_()
            self.epoch = 0

    def __repr__(self):
        n = 0 if self.workspace is None else self.workspace.numel()
        return f"MatmulConfig(device={self.device!r}, workspace_bytes={n}, epoch={self.epoch})"


def workspace_bytes_for(selector, m=None, n=None, k=None) -> int:
    """Bytes that cover both the work-stealing and the Stream-K schedule for the selector's tile."""
    lib = _lib.load()
    need = 0
    for sched, grid in ((_lib.TB_SCHED_WORK_STEALING, 0), (_lib.TB_SCHED_STREAMK, selector.sk_grid if selector.streamk else 0)):
        d = _lib.tb_gemm_desc()
        d.struct_bytes = _lib.C.sizeof(_lib.tb_gemm_desc)
        d.a_type = d.b_type = _lib.tb_dtype(selector._a_dtype)
        d.c_type = _lib.tb_dtype(selector._out_dtype)
        d.m, d.n, d.k = selector._m, selector._n, selector._k
        d.a_stride_m, d.a_stride_k = selector._k, 1
        d.b_stride_k, d.b_stride_n = 1, selector._k
        d.c_stride_m, d.c_stride_n = selector._n, 1
        d.block_m, d.block_n, d.block_k = selector.block_m, selector.block_n, selector.block_k
        d.schedule, d.grid = sched, grid
        d.counters_per_xcd = selector.COUNTERS_PER_XCD
        need = max(need, lib.tb_workspace_bytes(d))
    return int(need)


def matmul_preamble(selector, device: torch.device = None) -> MatmulConfig:
    """Allocate the launch state for a selector (reference config.py:86-134)."""
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    need = max(workspace_bytes_for(selector), _CTL_BYTES)
    workspace = torch.zeros(need, dtype=torch.uint8, device=device)
    n_cu, active = selector._N_CU, selector._ACTIVE_CU
    mask = torch.ones(n_cu, dtype=torch.int32, device=device)
    if active < n_cu:
        mask[active:] = 0
    return MatmulConfig(device=device, workspace=workspace, selector=selector, mask=mask, use_mask=active < n_cu)
