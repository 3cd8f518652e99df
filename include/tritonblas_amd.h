/*
 * tritonblas_amd — C ABI of the MI355X (gfx950) GEMM library.
 *
 * The reference (ROCm/tritonBLAS) has no FFI: its boundary is a Python API whose launchers start
 * Triton kernels.  Each entry point below replaces one of those launch sites; the Python package
 * binds them with ctypes.  All pointers are borrowed device pointers (the caller keeps the memory
 * alive until the stream has run the kernel), the library allocates nothing on the device, every
 * launch is asynchronous on the given stream, and errors are negative status codes (no exceptions,
 * no abort).
 */
#ifndef TRITONBLAS_AMD_H
#define TRITONBLAS_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TB_ABI_VERSION 1

/* ---- status codes --------------------------------------------------------------------------- */
enum {
  TB_OK = 0,
  TB_ERR_NULL_POINTER = -1,
  TB_ERR_BAD_SHAPE = -2,        /* the reference's  assert "Incompatible Dimensions"  (matmul.py:81) */
  TB_ERR_BAD_DTYPE = -3,
  TB_ERR_BAD_LAYOUT = -4,       /* strides this kernel family cannot address                        */
  TB_ERR_BAD_TILE = -5,         /* (block_m, block_n, block_k) is not a built kernel variant        */
  TB_ERR_WORKSPACE = -6,        /* workspace missing or too small for the requested schedule        */
  TB_ERR_BAD_SCHEDULE = -7,     /* grid larger than what can be co-resident, bad group table, ...   */
  TB_ERR_LAUNCH = -8,           /* the HIP runtime refused the launch                               */
  TB_ERR_NO_DEVICE = -9,
  TB_ERR_BAD_ARGUMENT = -10
};

/* ---- element types -------------------------------------------------------------------------- */
enum {
  TB_F16 = 0,
  TB_BF16 = 1,
  TB_FP8_E4M3 = 2,  /* OCP e4m3fn                                                  */
  TB_FP4_E2M1 = 3,  /* two codes per byte, low nibble = even k (utils.py:585-587) */
  TB_F32 = 4,       /* operands (full fp32 products, 16x16x4 MFMA), output, bias, quantiser input */
  TB_I8 = 5,        /* operands (int32 sums, persistent_gemm.py:75); as output only with TB_I8 operands: fp32 epilogue
                       result truncated toward zero and saturated to [-128, 127]                    */
  TB_FP8_E5M2 = 6   /* OCP e5m2, operands of tb_gemm only (the type utils.py:46 lists next to e4m3); one operand may be
                       e4m3 and the other e5m2 (origami.py:98-112 takes a_dtype and b_dtype separately) -- the only
                       pair of different operand types tb_gemm accepts                               */
};
/* TB_FP8_E4M3 and TB_FP8_E5M2 are also accepted as the OUTPUT type of a GEMM with TB_FP8_E4M3 or TB_FP8_E5M2 operands:
 * the fp32 epilogue result is clamped to the format's largest finite value (+-448, +-57344; NaN stays NaN) and rounded
 * to nearest even (the reference's a8w8 oracle, tests/test_matmul_a8w8_lt.py:11-38). */

/* ---- schedules ------------------------------------------------------------------------------ */
enum {
  TB_SCHED_PERSISTENT = 0,    /* data parallel, resident grid loops over tiles (matmul.py:160-198)  */
  TB_SCHED_WORK_STEALING = 1, /* atomic tile queues per XCD x slot       (matmul.py:112-159)        */
  TB_SCHED_STREAMK = 2,       /* data parallel tiles + Stream-K tail     (matmul.py:202-366)        */
  TB_SCHED_STREAMK_WS = 3     /* the same with the data parallel tiles drawn from the work-stealing queues
                                 (matmul.py:279-323, kernels/streamk_gemm_work_stealing.py:9-418)   */
};

/* How work-stealing workgroups find tiles (kernels/persistent_gemm_work_stealing.py). */
enum tb_ws_mode {
  TB_WS_QUEUES = 0,        /* one queue per XCD x slot (:296-318); a workgroup whose queues ran dry
                              goes on to the other queues (this library's addition)                  */
  TB_WS_GLOBAL_ATOMIC = 1, /* GLOBAL_ATOMIC: one counter, entry i is tile chiplet_transform(i) (:292-295, :321) */
  TB_WS_HIERARCHICAL = 2   /* HIERARCHICAL: a queue of ws_local_tiles_per_xcd tiles per XCD, then one
                              shared pool of ws_global_tiles (:106-291; split: origami.py:288-311);
                              a workgroup that finds both empty looks into the other XCDs' queues, so
                              every tile is computed whatever the mask switches off (this library's
                              addition)                                                              */
};

/* ---- hardware descriptor (replaces origami.get_hardware_for_device, origami.py:166) --------- */
typedef struct tb_hw {
  int32_t n_cu;          /* compute units                                   */
  int32_t num_xcd;       /* accelerator complex dies (one L2 each)          */
  int32_t cu_per_xcd;
  int32_t lds_bytes;     /* LDS per CU                                      */
  int32_t l2_bytes;      /* L2 per XCD                                      */
  int32_t clock_khz;     /* peak engine clock                               */
  int32_t mem_clock_khz;
  int32_t wave_size;
  double hbm_gbps;       /* peak HBM bandwidth, GB/s                        */
  char arch[32];         /* "gfx950"                                        */
} tb_hw;

/* Fills *out for HIP device `device`; with device < 0 (or no GPU present and device == -1) fills
 * the MI355X defaults so that the analytical selector can run on a machine without a GPU. */
int tb_device_info(int device, tb_hw* out);

/* ---- analytical selector (replaces origami.select_config / select_workgroup_mapping and
 *      OrigamiMatmulSelector._compute_sk_grid / _select_ws_params, origami.py:232-286,349-416) --- */
typedef struct tb_problem {
  int64_t m, n, k;
  int32_t a_type, b_type, c_type;
  int32_t a_k_contiguous;   /* 1: A is (m,k) with unit k stride   */
  int32_t b_k_contiguous;   /* 1: B is stored (n,k) with unit k stride */
  int32_t streamk;          /* caller intends enable_streamk=True  */
  int32_t num_groups;       /* >0: grouped (MoE) problem, m = total rows */
} tb_problem;

typedef struct tb_selection {
  int32_t block_m, block_n, block_k;
  int32_t group_m;            /* GROUP_M swizzle height (origami.py:286)                  */
  int32_t num_xcds;           /* XCD remap modulus (selector.num_sms, origami.py:330)     */
  int32_t occupancy;          /* workgroups per CU the variant was sized for              */
  int32_t num_stages;
  int32_t sk_grid;            /* Stream-K grid (origami.py:349)                           */
  int32_t counters_per_xcd;   /* work-stealing slots per XCD (origami.py:266-284)         */
  int32_t lds_bytes;          /* LDS the chosen variant allocates                         */
  double est_compute_us, est_memory_us, est_total_us;
} tb_selection;

int tb_select(const tb_problem* problem, const tb_hw* hw, tb_selection* out);

/* Number of built tile variants for (a_type); fills up to `cap` (block_m, block_n, block_k) triples. */
int tb_list_tiles(int32_t a_type, int32_t* triples, int32_t cap);

/* ---- GEMM ----------------------------------------------------------------------------------- */
typedef struct tb_gemm_desc {
  uint32_t struct_bytes;      /* sizeof(tb_gemm_desc), checked                                       */
  int32_t a_type, b_type, c_type, bias_type;
  int64_t m, n, k;            /* logical sizes: A (m,k), B (k,n), C (m,n)                           */
  int64_t a_stride_m, a_stride_k;   /* element strides (torch's a.stride())                         */
  int64_t b_stride_k, b_stride_n;
  int64_t c_stride_m, c_stride_n;
  const void* a;
  const void* b;
  void* c;
  const float* a_scale;       /* per row of A (m), or NULL      (matmul_a8w8_lt, matmul.py:380)      */
  const float* b_scale;       /* per column of B (n), or NULL                                        */
  const void* bias;           /* per column (n), or NULL        (addmm, matmul.py:727)               */
  int64_t bias_stride;
  int32_t block_m, block_n, block_k;  /* tile variant, from tb_select; 0 = let the library select    */
  int32_t group_m, num_xcds;
  int32_t schedule;           /* TB_SCHED_*                                                         */
  int32_t grid;               /* workgroups to launch; 0 = default (what is co-resident).  A Stream-K
                                 grid beyond what is co-resident is replaced by the default          */
  int32_t counters_per_xcd;
  void* workspace;            /* tb_workspace_bytes() bytes, 256-byte aligned, zero-initialised once by
                                 the caller.  One workspace serves Stream-K and work-stealing launches in
                                 any order (their regions are disjoint, see tb_workspace_layout)          */
  size_t workspace_bytes;
  uint32_t epoch;             /* Stream-K: tags this launch's partial tiles.  Never 0 (a launch that needs
                                 the workspace is refused with TB_ERR_BAD_ARGUMENT), and never a value an
                                 earlier launch on this workspace used since it was last zeroed: count
                                 upwards (flags are not cleared between launches, a stale flag of an equal
                                 epoch would pass for published).  TB_EPOCH_ON_DEVICE instead of a number
                                 lets the workspace count for itself (control word 2, advanced by the last
                                 workgroup of every such launch): the form to use when launches are replayed
                                 from a captured graph, whose arguments cannot change.  Do not mix the two
                                 forms on one workspace without zeroing it in between                      */
  uint32_t spin_limit;        /* Stream-K: bound on flag polls per wait; 0 = default                 */
  /* work stealing only (config.py:23, persistent_gemm_work_stealing.py:70-81): */
  const int32_t* cu_mask;     /* device int32[cu_mask_len] or NULL; workgroup i leaves at once when
                                 cu_mask[i] == 0.  With grid == 0 the launch has cu_mask_len workgroups
                                 (the reference launches one per CU and masks by program id)          */
  int32_t cu_mask_len;
  int32_t ws_mode;            /* TB_WS_*                                                            */
  int32_t ws_local_tiles_per_xcd, ws_global_tiles;  /* TB_WS_HIERARCHICAL: both 0 = split by the
                                 reference's rule (tb_hierarchical_split) for the tile the launch
                                 runs; otherwise num_xcds * local + global must equal its tile count */
  int32_t column_split;       /* persistent schedule, tiles that do not fill a whole number of rounds of
                                 the resident grid: 0 = the library may run the columns that fill whole
                                 rounds with the given tile and the remaining columns as a second launch
                                 with the tile its model picks for them (when the model expects at least
                                 3 % from it; disjoint column ranges of C, same stream); -1 = one launch.
                                 No counterpart in the reference.                                       */
} tb_gemm_desc;

/* C = cast((A @ B) * a_scale[:,None] * b_scale[None,:] + bias[None,:]), fp32 accumulate.
 * Replaces persistent_matmul_lt / streamk_matmul_lt (matmul.py:69-366). */
int tb_gemm(const tb_gemm_desc* desc, void* stream);

/* Bytes of workspace tb_gemm needs for this descriptor (0 for the persistent schedule). */
size_t tb_workspace_bytes(const tb_gemm_desc* desc);

/* tb_gemm without a workspace from the caller and without any allocation: the queue counters, Stream-K
 * flags and partial tiles live in a buffer of TB_STATIC_WORKSPACE_BYTES that is part of the library's
 * device image (every GPU the library runs on holds it until the process ends).  desc->workspace,
 * workspace_bytes and epoch are ignored (the buffer counts its own launches, TB_EPOCH_ON_DEVICE); a launch that
 * needs more than TB_STATIC_WORKSPACE_BYTES is refused with TB_ERR_WORKSPACE.  No counterpart in the
 * reference: it is for callers that cannot allocate device memory where they launch -- code under HIP
 * graph capture, tight serving loops, harnesses that forbid it.  All calls on one GPU share the buffer:
 * calls that may overlap in time (different streams) race; calls on one stream do not. */
#define TB_STATIC_WORKSPACE_BYTES (16u << 20)
#define TB_EPOCH_ON_DEVICE 0xFFFFFFFFu
int tb_gemm_static_workspace(const tb_gemm_desc* desc, void* stream);

/* What a tb_gemm call with this descriptor would launch (nothing is launched): the tile, the kernel family
 * (waves per workgroup; four_wave: the hand-scheduled 256x256 kernel), the grid, how many tiles form the Stream-K
 * tail and in units of how many K steps their ranges are cut, whether the whole tiles come from the work-stealing
 * queues, whether the small-M streaming kernel runs instead of a tile kernel.  For tests and for callers that log
 * their launches; no counterpart in the reference (its launchers print the same facts when asked to be verbose). */
typedef struct tb_launch_info {
  int32_t block_m, block_n, block_k, waves, four_wave, mode, grid, total_tiles, sk_tiles, sk_unit, sk_ws, skinny;
} tb_launch_info;
int tb_gemm_launch_info(const tb_gemm_desc* desc, tb_launch_info* out);

/* Reads the status word of the current GPU's static workspace into *status (1: a Stream-K launch through
 * tb_gemm_static_workspace ran into spin_limit and stored NaN tiles) and, with clear != 0, sets it back to 0.
 * Waits for the device's earlier work; allocates nothing.  A caller-owned workspace carries the same word at
 * byte 0 (MatmulConfig.status() / check(), config.py of this package).  No counterpart in the reference. */
int tb_static_workspace_status(int* status, int clear);

/* Byte offsets of the regions of a workspace: [0, 256) control words -- word 0 is the status (set to 1
 * when a Stream-K wait ran into spin_limit: the tile concerned was then stored as NaN; cleared only by the
 * caller), word 1 counts workgroups that have finished (work stealing, and Stream-K with
 * TB_EPOCH_ON_DEVICE), word 2 is the workspace's own launch count for TB_EPOCH_ON_DEVICE; *counters_offset: work-stealing queue
 * counters, one per 256-byte line; *flags_offset: Stream-K flags (one word per workgroup), the partial
 * tiles follow at the next 256-byte boundary behind `grid` flags.  Replaces the separate buffers of
 * matmul_preamble (config.py:86-134). */
int tb_workspace_layout(size_t* counters_offset, size_t* flags_offset);

/* ---- MXFP4 GEMM (replaces matmul_fp4, matmul.py:519-625) ------------------------------------- */
typedef struct tb_gemm_fp4_desc {
  uint32_t struct_bytes;
  int32_t c_type;
  int64_t m, n, k;            /* k = unpacked element count, multiple of 32                          */
  const void* a;              /* (m, k/2) bytes, k-contiguous                                        */
  const void* b;              /* (n, k/2) bytes, k-contiguous                                        */
  void* c;
  int64_t a_stride_m, b_stride_n;     /* row strides in bytes                                        */
  int64_t c_stride_m, c_stride_n;
  const void* a_scales;       /* (m, k/32) E8M0 bytes                                                */
  const void* b_scales;       /* (n, k/32) E8M0 bytes                                                */
  int64_t a_scales_stride_m, a_scales_stride_k;
  int64_t b_scales_stride_n, b_scales_stride_k;
  int32_t block_m, block_n, block_k;  /* 0 = select                                                  */
  int32_t group_m, num_xcds;
} tb_gemm_fp4_desc;

int tb_gemm_fp4(const tb_gemm_fp4_desc* desc, void* stream);

/* ---- grouped (MoE) FP8 GEMM — no counterpart in the reference -------------------------------- */
typedef struct tb_grouped_gemm_desc {
  uint32_t struct_bytes;
  int32_t c_type;
  int64_t m_total, n, k;      /* rows over all experts, per-expert weight (n,k)                      */
  int32_t num_groups;
  const void* a;              /* (m_total, k) e4m3, rows sorted by expert, k-contiguous              */
  const void* w;              /* (num_groups, n, k) e4m3, k-contiguous                               */
  void* c;                    /* (m_total, n)                                                        */
  int64_t a_stride_m, w_stride_g, w_stride_n;
  int64_t c_stride_m, c_stride_n;
  const float* a_scale;       /* (m_total)                                                           */
  const float* w_scale;       /* (num_groups, n) contiguous                                          */
  const int32_t* group_offsets; /* device int32[num_groups+1], offsets[0]=0, offsets[g]=m_total     */
  int32_t block_m, block_n, block_k;
  int32_t group_m, num_xcds;
  int32_t small_rows;         /* > 0: an expert's last, partial row block of at most this many rows is
                                 left to a second launch with a short (32-row) tile instead of costing
                                 a whole tall tile per column block.  0: library default — threshold 64,
                                 and the kernels price both plans from the row counts on the device
                                 (rounds of tall tiles against rounds of short ones) and split only
                                 when that is cheaper; off when block_m is forced.  -1: one launch.
                                 The split needs k % 256 == 0 and a tall (>= 128-row) tile.            */
  int32_t streamk;            /* 1: the tiles that do not fill whole rounds of the grid are cut into K ranges
                                 (Stream-K, as kernels/streamk_gemm.py:160-384 does for one matrix) whenever the
                                 tile table -- known only on the device -- makes that cheaper than one more
                                 round; taken by the 256x256 four-wave kernel when k is a multiple of 512, ignored
                                 otherwise.  Needs the workspace below; results then differ from streamk = 0
                                 in the summation order of the cut tiles only.  0: whole tiles only.      */
  uint32_t epoch;             /* as tb_gemm_desc.epoch; TB_EPOCH_ON_DEVICE: the workspace counts       */
  uint32_t spin_limit;        /* as tb_gemm_desc.spin_limit                                           */
  void* workspace;            /* tb_grouped_workspace_bytes() bytes, 256-byte aligned, zeroed once       */
  size_t workspace_bytes;
} tb_grouped_gemm_desc;

int tb_grouped_gemm_fp8(const tb_grouped_gemm_desc* desc, void* stream);
/* Workspace a streamk = 1 call with this descriptor needs (0: none, the launch runs whole tiles only). */
size_t tb_grouped_workspace_bytes(const tb_grouped_gemm_desc* desc);
/* Host-side evaluation of the rule the grouped kernel applies on the device: of a table of total_tiles tiles
 * with k_units K units each (a unit = unit_steps K steps) on a grid of `grid` workgroups, how many tiles at
 * the end are cut into K ranges; fix_steps = what an extra piece of a tile costs its owner, in K steps.  For
 * tests; no counterpart in the reference. */
int tb_streamk_tail_tiles(int32_t total_tiles, int32_t grid, int32_t k_units, int32_t unit_steps, int32_t fix_steps);

/* ---- MXFP4 quantisation (replaces dynamic_mxfp4_quant, utils.py:743-789), optionally preceded
 *      by a 32-point blockwise Hadamard rotation along k (no counterpart in the reference) ------- */
typedef struct tb_quant_desc {
  uint32_t struct_bytes;
  int32_t x_type;             /* TB_BF16, TB_F16 or TB_F32                                           */
  int64_t m, n;               /* n multiple of 32                                                    */
  const void* x;
  int64_t x_stride_m;         /* elements; unit stride along n                                       */
  void* codes;                /* (m, n/2) bytes                                                      */
  int64_t codes_stride_m;
  void* scales;               /* (m, n/32) bytes                                                     */
  int64_t scales_stride_m;
  int32_t hadamard;           /* 1: rotate each block of 32 by H32/sqrt(32) first                    */
} tb_quant_desc;

int tb_hadamard_mxfp4_quant(const tb_quant_desc* desc, void* stream);

/* ---- tile order ------------------------------------------------------------------------------
 * Host-side evaluation of the kernels' tile id -> (row block, column block) map, for tests and tools.
 * With panel_n = 0 it is the reference's GROUP_M swizzle (kernels/stages/schedule.py:124-145); with
 * panel_n > 0 the tile list is cut into column panels of panel_n tiles that are each swept top to
 * bottom with that swizzle (no counterpart in the reference: a cache-residency choice of this library).
 * tb_default_panel gives the panel width tb_gemm uses for a launch grid. */
int tb_tile_coords(int32_t tile, int32_t tiles_m, int32_t tiles_n, int32_t group_m, int32_t panel_n, int32_t* pm, int32_t* pn);
int tb_default_panel(int32_t grid, int32_t chunk, int32_t group_m);

/* (tiles per XCD-local queue, tiles in the shared pool) for total_tiles tiles on hw_cus compute units
 * (the hardware count, not the active one) and num_xcds queues: hierarchical_split, origami.py:288-311;
 * the local share is capped at what divides evenly, so the two always add up to total_tiles. */
int tb_hierarchical_split(int64_t total_tiles, int32_t hw_cus, int32_t num_xcds, int32_t* local_tiles_per_xcd, int32_t* global_tiles);

/* Host-side evaluation of the work-stealing queues: queue `queue` of a launch over total_tiles tiles
 * (TB_WS_QUEUES: queue = xcd * counters_per_xcd + slot; TB_WS_GLOBAL_ATOMIC: queue 0;
 * TB_WS_HIERARCHICAL: queue = xcd, or num_xcds for the shared pool).  *count = entries of the queue,
 * *tile = tile id of entry idx (or -1 when idx >= *count). */
int tb_ws_queue_tile(int32_t ws_mode, int32_t queue, int32_t idx, int32_t total_tiles, int32_t num_xcds,
                     int32_t counters_per_xcd, int32_t local_tiles_per_xcd, int32_t* count, int32_t* tile);

/* ---- misc ----------------------------------------------------------------------------------- */
/* Tuning and test hooks.  Each has an environment variable that is read once, when the library first
 * plans a launch (TB_WAVES, TB_NO_MXLDS, TB_NO_CLINE, TB_NO_SKINNY, TB_SKINNY, TB_GRID, TB_PANEL,
 * TB_NO_COLUMN_SPLIT, TB_FORCE_COLUMN_SPLIT, TB_QUANT_DIV64); this call changes one afterwards, by its lower-case name
 * without the prefix ("waves", "no_skinny", ...; "panel" -1 = the library's choice).  Process-wide; not
 * meant for production callers.  No counterpart in the reference. */
int tb_debug_option(const char* name, int value);

const char* tb_status_string(int status);
int tb_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* TRITONBLAS_AMD_H */
