/*
 * hpspmm.h - C ABI of the gfx950 (MI355X) FP32 CSR SpMM library, libhpspmm.so.
 *
 *   C = A * B     A: sparse, CSR, int32 zero-based indices, FP32 values
 *                 B: dense  cols x k, FP32, row-major, leading dimension k
 *                 C: dense  rows x k, FP32, row-major, leading dimension k
 *                 alpha = 1, beta = 0 (C is overwritten), A not transposed.
 *
 * These are the operand conventions of the reference's SpMM entry points
 * (include/spmm/mm/spmm_kernel.h:17-21; descriptors at
 * spmm/mm/spmm_kernel.cu:82-108; indexing col*k + cid at :269).  Each entry
 * point below names the reference interface it stands in for.
 *
 * Conventions
 *   - Every pointer whose name starts with d_ is a DEVICE pointer owned by the
 *     caller; the library never frees or reallocates caller memory.
 *   - Sizes and counts are int64_t; index arrays are int32_t as in the
 *     reference's CSR container (include/spmm/mm/spmm_common.h:58-82), so
 *     rows, cols and nnz must each be <= INT32_MAX.  Byte offsets are computed
 *     in 64 bits (the reference's int byte counts overflow at 2^31 bytes,
 *     spmm/starml/operators/cuda/copy_kernel.cu:12,30).
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *     Launches are asynchronous; nothing synchronises with the host except
 *     hpspmm_plan_create (which reads back validation flags and statistics).
 *   - Every function returns HPSPMM_OK (0) or a positive hpspmm_status; after
 *     a failure hpspmm_last_error() gives a message for the calling thread.
 *     The reference has no error convention on this path (statuses are
 *     dropped, failed checks abort through loguru, loguru.h:1535); a status
 *     code replaces the abort.
 *   - A plan may be used from one stream at a time: it owns the scratch
 *     buffer that split rows are reduced through.
 */
#ifndef HPSPMM_H_
#define HPSPMM_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum hpspmm_status {
  HPSPMM_OK = 0,
  HPSPMM_ERR_INVALID_ARG = 1, /* null pointer, negative size, size > INT32_MAX, k <= 0 */
  HPSPMM_ERR_BAD_CSR = 2,     /* rowptr not monotone / rowptr[0] != 0 / rowptr[rows] != nnz / col out of range */
  HPSPMM_ERR_HIP = 3,         /* a HIP runtime call failed (message carries hipGetErrorString) */
  HPSPMM_ERR_NO_DEVICE = 4,   /* no usable GPU */
  HPSPMM_ERR_ALLOC = 5        /* device allocation for the plan failed */
} hpspmm_status;

/* hpspmm_plan_create flags */
#define HPSPMM_PLAN_DEFAULT 0u
#define HPSPMM_PLAN_NO_VALIDATE 1u    /* skip the device-side CSR check */
#define HPSPMM_PLAN_FORCE_ROWS 2u     /* always use the whole-row strategy */
#define HPSPMM_PLAN_FORCE_SEGMENTS 4u /* always use the nnz-segment kernel + carry fix-up */
#define HPSPMM_PLAN_NO_XCD_REMAP 8u   /* keep the hardware's round-robin workgroup->XCD order */
#define HPSPMM_PLAN_HUB_CACHE 16u     /* segments strategy: always keep the most referenced rows of B in a compact
                                         copy (default: only when they serve >= 25 % of the nonzeros) */
#define HPSPMM_PLAN_NO_HUB_CACHE 32u  /* never build the hub cache */
#define HPSPMM_PLAN_FORCE_ROUTED 64u  /* always use the routed strategy (hub columns pinned to one XCD each);
                                         bits 16..20 then give log2 of the total number of hub rows (0 = auto) */
#define HPSPMM_PLAN_NO_ROUTED 128u    /* never use the routed strategy */
/* bits 24..28, with FORCE_ROUTED: log2 of the shortest row that is routed (0 = default, 128) */
#define HPSPMM_PLAN_ROUTED_ROW_LOG2(log2_nnz) (((uint32_t)(log2_nnz) & 0x1Fu) << 24)
/* bits 29..31, with FORCE_ROUTED: number of phases every XCD cuts its slice of the columns into, 1..7 (0 = auto) */
#define HPSPMM_PLAN_ROUTED_PHASES(n) (((uint32_t)(n) & 0x7u) << 29)
/* bits 16..20: log2 of the number of cached rows, 4..24 (0 = default, 2^16) */
#define HPSPMM_PLAN_HUB_LOG2(log2_rows) (((uint32_t)(log2_rows) & 0x1Fu) << 16)
#define HPSPMM_PLAN_ALLOW_MOVED_CSR (1u << 21) /* hpspmm_csr_spmm accepts d_rowptr / d_col at other addresses than
                                         the plan was built from (the caller vouches that they hold the same
                                         structure); default: other addresses are HPSPMM_ERR_INVALID_ARG */
/* bits 8..11: log2 of the segment length to force (0 = choose automatically) */
#define HPSPMM_PLAN_SEGMENT_SHIFT(log2_len) (((uint32_t)(log2_len) & 0xFu) << 8)
#define HPSPMM_PLAN_CLUSTER 4096u     /* always look for clusters of rows that share columns and use the
                                         ordered strategy on the order found (default: from 2^22 nonzeros and
                                         12 MB of B up, when the matrix is not routed, and only if >= 15 % of the
                                         nonzeros stay inside clusters of <= 4096 rows and >= 15 % then read B
                                         from LDS).  A square A is taken as a graph on its rows, any other as the
                                         bipartite graph of its rows and columns.  The clustering is deterministic: two plans of one matrix
                                         order the rows alike and give the same bits of C */
#define HPSPMM_PLAN_NO_CLUSTER 8192u  /* never */
#define HPSPMM_PLAN_ROUTED_SORT_VALUES 32768u /* routed strategy: never cut the columns into consecutive ranges (which lets
                                         the kernel read the values in place); always spread them by popularity rank and
                                         hash and bring the values into the plan's order at the start of every SpMM */
#define HPSPMM_PLAN_NO_ROW_TILES 16384u /* rows strategy: walk the caller's CSR arrays instead of building row tiles */
#define HPSPMM_PLAN_FORCE_SWEEP (1u << 22) /* use the sweep strategy (all wavefronts walk the columns of B window by
                                         window, the row accumulators stay in LDS) whatever the size of the matrix
                                         (default: from 2^21 nonzeros and 5 MB of B up, where a cost model of the
                                         sweep is below the expected time of whole rows in stored order).  It needs
                                         at most 2^24 columns and less than 4 GB of B, otherwise the plan keeps to
                                         segments; rows whose columns are not in increasing order are laid out from
                                         a sorted copy made at plan time */
#define HPSPMM_PLAN_NO_SWEEP (1u << 23)    /* never use the sweep strategy */

/* strategy reported by hpspmm_plan_get_info */
#define HPSPMM_STRATEGY_ROWS 1
#define HPSPMM_STRATEGY_SEGMENTS 2
#define HPSPMM_STRATEGY_GENERIC_K 3 /* no longer reported: every k runs whole rows or segments on sub-waves */
#define HPSPMM_STRATEGY_ROUTED 4
#define HPSPMM_STRATEGY_ORDERED 5
#define HPSPMM_STRATEGY_SWEEP 6

typedef struct hpspmm_plan hpspmm_plan;

/*
 * Everything hpspmm_plan_create_ex can be told, one struct per call: nothing about a plan depends
 * on the environment or on other process-wide state (the reference's entry points have none either,
 * include/spmm/mm/spmm_kernel.h:17-21).  Zero in a field means "the library's default", so
 *     hpspmm_plan_options o = {0}; o.struct_size = sizeof o;
 * is hpspmm_plan_create with flags 0.  struct_size lets a library newer than its caller see where
 * the caller's struct ends (fields beyond are taken as zero).  The fields after d_row_order are
 * for measurements and tests: they override choices the plan otherwise makes from the matrix.
 */
typedef struct hpspmm_plan_options {
  uint32_t struct_size;       /* sizeof(hpspmm_plan_options) */
  uint32_t flags;             /* HPSPMM_PLAN_* bits; a size field below, when not 0, replaces the same
                                 size packed into the flag word */
  const int32_t *d_row_order; /* NULL, or the processing order of hpspmm_plan_create_ordered */
  int32_t segment_shift;      /* log2 of the segment length to force, 3..15 */
  int32_t hub_log2;           /* log2 of the rows of B in the hub cache / the routed compact buffer, 4..24 */
  int32_t routed_row_log2;    /* with FORCE_ROUTED: log2 of the shortest row that is routed */
  int32_t routed_phases;      /* with FORCE_ROUTED: phases by column subset, 1..7 */
  int32_t routed_tile_width;  /* routed strategy: 32 / 64 = work through B and C in column tiles of that
                                 width, one after the other on all XCDs (k a multiple of it); -1 = never */
  int32_t routed_split_launch; /* 1: hub phases and cold class as launches of their own (per-class timing) */
  int32_t routed_lds_rows;    /* column tiles of the routed strategy: rows of B a workgroup keeps in LDS (at most
                                 what fits; -1 = none) */
  int32_t xcd_dealing;        /* 0: probe how workgroups are dealt to the XCDs (once per device and process);
                                 1: take workgroup b to run on XCD b % 8; 2: take it not to */
  int32_t no_column_tiles;    /* 1: a k outside 32 / 64 / 128 never gets the sweep / routed / ordered
                                 layouts in column tiles */
  int32_t row_tiles_min_k;    /* row tiles serve a k outside the tuned set only from this k up */
  int32_t row_tiles_pad;      /* row tiles at such a k: 1 = never, 2 = whenever k is not a multiple of 32,
                                 read B through the padded copy */
  int32_t row_tiles_wide;     /* 1: 8 lanes per entry also at k <= 16 (instead of 4, or 1 at k <= 4) */
  int32_t row_tiles_round_robin; /* 1: deal the column tiles of a group of row tiles round robin over the XCDs */
  int32_t sweep_window_log2;  /* sweep strategy: log2 of the bytes of B per window */
  int32_t sweep_lead;         /* windows a wavefront may run ahead of the slowest of its CU */
  int32_t sweep_spin;         /* spin limit of its bounded wait; -1 = never wait */
  int32_t sweep_limit;        /* nonzeros per piece */
  int32_t sweep_no_priorities; /* 1: leave the wavefront priorities alone */
  int32_t cluster_sweeps;     /* label-propagation sweeps, at most (> 0 also keeps the search from ending after four sweeps where no clusters form) */
  int32_t report;             /* 1: plan-time reports on stderr */
  int32_t row_tiles_chunk_log2; /* row tiles at k = 32 / 64 / 128: deal 2^n consecutive groups of tiles to an XCD at a
                                 time instead of one (-1 = one; 0 = the library's choice, by the size) */
} hpspmm_plan_options;

typedef struct hpspmm_plan_info {
  int64_t rows, cols, nnz, k;
  int32_t strategy;        /* HPSPMM_STRATEGY_* */
  int32_t segment_length;  /* nonzeros per sub-wave segment (segments strategy), else 0 */
  int64_t num_segments;
  int64_t max_row_nnz;
  int64_t empty_rows;
  int64_t workspace_bytes; /* device memory owned by the plan */
  int32_t launches_per_spmm;
  int32_t column_tiles;    /* column tiles a row length other than 32 / 64 / 128 is served in by a tuned layout (else 1) */
  int64_t hub_rows;        /* rows of B kept in the hub cache (0 = none) */
  int64_t lds_served_nnz;  /* ordered strategy: nonzeros whose row of B comes from a workgroup's LDS copy */
  int64_t row_tiles;       /* rows strategy: 64-entry tiles of the plan's row-tile layout (0: the CSR arrays are walked) */
  double stored_order_miss_share; /* share of the gathers of rows of B that miss an L2 when the nonzeros are taken
                                     in stored order, as sampled for the choice of strategy (k = 32 / 64 / 128, from
                                     2^21 nonzeros, no forcing flag); -1 when it was not measured */
} hpspmm_plan_info;

/* Library version, major*10000 + minor*100 + patch. */
int hpspmm_version(void);

/*
 * What the library sees of the current device (hipDeviceProp figures, and whether
 * the probe of hpspmm_plan_create found workgroup b on XCD b % 8).  For reports:
 * the benchmark prices the L2 -> CU path with the clock given here.  No
 * counterpart in the reference.
 */
typedef struct hpspmm_device_info {
  int32_t device;
  int32_t compute_units;
  int32_t clock_khz;         /* engine clock */
  int32_t memory_clock_khz;
  int64_t l2_bytes;          /* as hipDeviceProp reports it (one XCD's) */
  int64_t lds_bytes_per_cu;
  int64_t global_bytes;
  int32_t xcd_dealing;       /* 1: workgroup b of a launch runs on XCD b % 8 */
  char arch[60];
} hpspmm_device_info;
int hpspmm_get_device_info(hpspmm_device_info *info_out);

/* Message of the last failure on the calling thread ("" if none). */
const char *hpspmm_last_error(void);

/*
 * Analyse the sparsity structure of A for a given k and build the device-side
 * work assignment.  The plan picks a strategy (reported by
 * hpspmm_plan_get_info): whole rows for small and medium matrices (below 2^24
 * nonzeros and nnz * k < 2^30, less when the rows are long) and for matrices
 * of any size whose stored order is local - rows that share columns with their
 * neighbours, which the plan measures on a sample of the column stream (the
 * rows cut into 8-nonzero slots and packed, by length class, into one 64-entry tile per
 * wavefront, so that a microsecond-scale SpMM is one launch with a two-step
 * dependent chain); fixed-length segments of nonzeros with a carry buffer;
 * for a large matrix of long rows whose B is small against the gather volume,
 * one workgroup per CU that keeps the accumulators of its rows in LDS while
 * all wavefronts walk the columns of B window by window at the same pace, so
 * that every L2 holds the stretch of B in use ("sweep"); segments inside
 * column slices pinned to one XCD each when a few columns take most of the
 * nonzeros ("routed"); or segments over a clustered row order with the reused
 * rows of B held in LDS when the matrix is a graph with communities
 * ("ordered").
 * k = 32, 64 and 128 are the tuned row lengths.  Any other k from 16 up is
 * served by the sweep, routed and ordered layouts one column tile of 128, 64
 * or 32 columns after the other (the reference tiles the columns the same way,
 * spmm/mm/spmm_kernel.cu:412-420: grid.y = ceil(k / 64)); a last tile narrower
 * than the layout leaves its surplus lanes idle.  When k is not a multiple of
 * 4 (41 classes, 47, 173 ...) the plan then keeps a copy of B with rows padded
 * to one - refreshed by one more launch at the start of every SpMM, part of
 * workspace_bytes - because 16-byte gathers from rows at 4-byte alignment cost
 * about twice; C is written in place.  All that is done when the matrix gets
 * one of those layouts (at least 2^22 nonzeros, or a forcing flag);
 * launches_per_spmm counts every tile's launches, column_tiles the tiles.
 * Otherwise whole rows run over the plan's row tiles in ceil(k / 32) column
 * tiles within one launch (column_tiles stays 1), B as it lies - 16-byte
 * gathers at 4-byte alignment when k is not a multiple of 4 - or, where that
 * pays (k > 32 and not a multiple of 8, 2^20 nonzeros and more, 40 for every
 * row of B), through such a copy with rows padded to a multiple of 32 floats;
 * k < 4 always through a copy with rows of 4 floats.  What remains -
 * matrices of 2^25 nonzeros and more whose rows are of even lengths, rows
 * beyond 2^18 nonzeros, very short rows at a k that is not a multiple of 32
 * on a large matrix - runs whole rows or segments with sub-waves of
 * ceil(k / 4) lanes rounded up to a power of two, rows of B and C read and
 * written at whatever alignment they have.
 * Replaces the host-side preprocessing the reference does before timing:
 * CSR->COO expansion (spmm/mm/spmm_common.cpp:185-235), the row re-ordering
 * (:237-296) and the choice of nnz_per_warp (spmm/mm/spmm_kernel.cu:749-751).
 * Synchronises `stream`.
 * Values are not read: the plan stays valid when d_val or B change, and must
 * be rebuilt when rowptr / col change - also when they are edited in place:
 * most strategies run from the plan's own copy of the structure and would go
 * on computing the old matrix.
 * The strategies that place work on particular XCDs (routed; the row-range
 * dealing of the others) are used only if a probe launch, once per device and
 * process, has seen workgroup b run on XCD b % 8, which is how the whole
 * (unpartitioned) device deals them; otherwise the plan keeps to segments,
 * rows and ordered without that placement (hpspmm_plan_options.xcd_dealing
 * replaces the probe by the caller's word).
 */
int hpspmm_plan_create(int64_t rows, int64_t cols, int64_t nnz, const int32_t *d_rowptr,
                       const int32_t *d_col, int64_t k, uint32_t flags, void *stream,
                       hpspmm_plan **plan_out);

/*
 * hpspmm_plan_create for a caller-chosen processing order of the rows:
 * d_row_order[i] = the row handled i-th (a permutation of 0..rows-1, device
 * memory, read only here).  Rows that share many columns should be neighbours
 * in it: every workgroup keeps the rows of B that its stretch of nonzeros uses
 * more than once in LDS.  C is written at the original row numbers, so the
 * result is that of hpspmm_plan_create up to summation order.  The role of the
 * row permutation that the reference reads from a .cugraph_reorder file for
 * HP-SpMM (spmm/mm/spmm_common.cpp:237-296: nonzeros emitted in that row
 * order, row indices kept).  k must be at least 16 for the order to be used.
 */
int hpspmm_plan_create_ordered(int64_t rows, int64_t cols, int64_t nnz, const int32_t *d_rowptr,
                               const int32_t *d_col, int64_t k, uint32_t flags,
                               const int32_t *d_row_order, void *stream, hpspmm_plan **plan_out);

/*
 * hpspmm_plan_create / hpspmm_plan_create_ordered with every option in one struct (see
 * hpspmm_plan_options; NULL = all defaults).  The two entry points above forward here.  A plan
 * keeps what it was told: hpspmm_csr_spmm reads nothing but the plan and its arguments.
 */
int hpspmm_plan_create_ex(int64_t rows, int64_t cols, int64_t nnz, const int32_t *d_rowptr,
                          const int32_t *d_col, int64_t k, const hpspmm_plan_options *options,
                          void *stream, hpspmm_plan **plan_out);

int hpspmm_plan_get_info(const hpspmm_plan *plan, hpspmm_plan_info *info_out);

/* Frees the plan's device memory.  NULL is accepted. */
int hpspmm_plan_destroy(hpspmm_plan *plan);

/*
 * Optional: declare that the nnz values at d_val will not change until the
 * next call of this function (or the destruction of the plan).  Strategies
 * that keep the nonzeros in an order of their own then bring the values into
 * that order once, here, instead of at the start of every SpMM; later
 * hpspmm_csr_spmm calls that pass this same d_val use the stored copy; a call
 * with any other pointer works as if nothing was bound and drops the binding.
 * d_val = NULL unbinds.  (Where a plan reads the values in place anyway - rows,
 * ordered, routed with column-range slices - binding changes nothing or, in
 * the last case, makes the plan keep a copy in its own order: device memory
 * for nnz floats is allocated here, not in hpspmm_csr_spmm.)
 * This is where the reference's HP-SpMM does the same work: its preprocessing
 * emits the values in its own processing order before the timed loop
 * (spmm/mm/spmm_common.cpp:269-277, test/test_all.cpp:38-40).  A caller that
 * overwrites the array in place must bind again (or unbind); otherwise SpMM
 * keeps using the values it copied.  Asynchronous on `stream`.
 */
int hpspmm_plan_bind_values(hpspmm_plan *plan, const float *d_val, void *stream);

/*
 * C = A * B with a plan.  One call = one SpMM = the body of one iteration of
 * the reference's launch loop in GESpMM (spmm/mm/spmm_kernel.cu:405-422) /
 * one cusparseSpMM call (spmm/mm/spmm_kernel.cu:129-141).  C need not be
 * zeroed beforehand; every element of C, empty rows included, is written.
 * The result is deterministic (no atomics).  The call only launches kernels (no
 * allocation, no memset, no host synchronisation), so it may be captured in a
 * HIP graph; a replay reads d_val and d_B as they are then.
 * d_rowptr and d_col must be the arrays the plan was built from: any other
 * address is HPSPMM_ERR_INVALID_ARG (the reference's launchers take whatever
 * they are given, spmm/mm/spmm_kernel.cu:389-426, and have no plan that could
 * go stale), unless the plan was created with HPSPMM_PLAN_ALLOW_MOVED_CSR.
 * All arrays may start at any multiple of 4 bytes; the kernels are tuned for
 * d_B and d_C at multiples of 16 bytes (what hipMalloc returns), other
 * addresses give the same result more slowly.
 */
int hpspmm_csr_spmm(hpspmm_plan *plan, const int32_t *d_rowptr, const int32_t *d_col,
                    const float *d_val, const float *d_B, float *d_C, void *stream);

/*
 * C = A * B without a plan: whole-row kernel, no preprocessing, no device
 * allocation.  Same contract as GESpMM's single launch
 * (spmm/mm/spmm_kernel.cu:406-421), for callers that cannot keep a plan.
 * As there, a row is served by one group of lanes however long it is, so the
 * longest row bounds the launch: on a matrix with hub rows a plan is several
 * times faster (R-MAT, 4.2 M rows, K = 128: 35 ms against 6 ms; 131 k rows:
 * 1.2 ms against 0.17 ms), on one without them 1.5 to 3 times.
 */
int hpspmm_csr_spmm_noplan(int64_t rows, int64_t cols, int64_t nnz, const int32_t *d_rowptr,
                           const int32_t *d_col, const float *d_val, const float *d_B, int64_t k,
                           float *d_C, void *stream);

/*
 * C = A * B like hpspmm_csr_spmm under the segments strategy, for callers that
 * cannot allocate device memory or keep a plan (code under HIP-graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): no hipMalloc, hipFree,
 * memset or host synchronisation - three kernel launches on `stream`.  It has
 * no counterpart in the reference.  The workspace a plan would own (row of
 * every nonzero, carry slots of split rows) is a 32 MiB array inside the
 * library's device image, one copy per GPU, kept until the process ends.
 * Limits: k in {32, 64, 128} and nnz <= 2^22 (HPSPMM_ERR_INVALID_ARG beyond).
 * Nothing in the array needs clearing between calls (every slot a call reads it
 * has written before), but all calls on one GPU share it: calls that overlap in
 * time on one GPU - two streams, two host threads - race.  The CSR arrays are
 * not validated.
 * The first call on a device looks up where that device holds the array, which
 * is not a thing to do on a capturing stream: call hpspmm_static_workspace_init
 * (or make one ordinary call) on the device beforehand.
 */
int hpspmm_csr_spmm_static(int64_t rows, int64_t cols, int64_t nnz, const int32_t *d_rowptr,
                           const int32_t *d_col, const float *d_val, const float *d_B, int64_t k,
                           float *d_C, void *stream);

/*
 * Looks up the static workspace of hpspmm_csr_spmm_static on the current
 * device (once per device; later calls return at once).  No allocation, no
 * launch.  It has no counterpart in the reference.
 */
int hpspmm_static_workspace_init(void);

/*
 * C += A * B for A in COO (row-index per nonzero), the contract of one launch
 * of LBSpMM (spmm/mm/spmm_kernel.cu:733-768: accumulates with atomics,
 * :463-476).  Entries of one row need not be contiguous, `nnz` may include
 * zero-valued padding entries (spmm/mm/spmm_common.cpp:220-226), and entries
 * may arrive in a permuted row order (spmm/mm/spmm_common.cpp:269-277).
 * The caller zeroes C first if it wants C = A * B.  Uses FP32 atomics, so the
 * summation order (not the set of terms) can differ between runs.
 */
int hpspmm_coo_spmm_accumulate(int64_t rows, int64_t cols, int64_t nnz, const int32_t *d_row,
                               const int32_t *d_col, const float *d_val, const float *d_B, int64_t k,
                               float *d_C, void *stream);

/* d_x[i] = value for i in [0, n): fill_matrix (spmm/mm/spmm_kernel.cu:23-34). */
int hpspmm_fill_f32(float *d_x, int64_t n, float value, void *stream);

/*
 * Time `iters` back-to-back hpspmm_csr_spmm launches on `stream` with HIP
 * events after `warmup` untimed ones and return the mean in milliseconds:
 * the measurement protocol of GESpMM / cusparseCSRSpMM
 * (include/spmm/utils/timer_cuda.h:3-40, spmm/mm/spmm_kernel.cu:128-145,
 * 404-424).  Synchronises `stream`.
 */
int hpspmm_csr_spmm_timed(hpspmm_plan *plan, const int32_t *d_rowptr, const int32_t *d_col,
                          const float *d_val, const float *d_B, float *d_C, void *stream,
                          int warmup, int iters, float *mean_ms_out);

/*
 * The same, for an SpMM of microseconds: when the `iters` launches take less
 * than min_total_ms together, a second region of as many launches as fill
 * min_total_ms at the rate just seen is timed and reported instead
 * (*iters_done_out = the launches of the region reported; may be NULL).  The
 * reference times 200 launches whatever they take
 * (include/spmm/utils/timer_cuda.h:3-4); 200 launches of 4 us are 0.8 ms,
 * within which clock ramps and launch jitter do not average out.
 */
int hpspmm_csr_spmm_timed_min(hpspmm_plan *plan, const int32_t *d_rowptr, const int32_t *d_col,
                              const float *d_val, const float *d_B, float *d_C, void *stream,
                              int warmup, int iters, float min_total_ms, float *mean_ms_out,
                              int64_t *iters_done_out);

/*
 * The same protocol with one more event after every kernel launch of an SpMM:
 * mean_ms_out[i] = mean duration of the i-th launch (i < *n_launches_out <=
 * max_launches), names_out[i] = its kernel's name (a string owned by the
 * library).  An SpMM of more launches than max_launches (or than the 32 the
 * library records) gets the time of those beyond as one last entry named
 * "(remaining launches)".  Every iteration ends with an event of its own that
 * the host waits for.  For reporting which launch of a multi-launch strategy
 * takes the time; the extra events keep launches from overlapping their
 * neighbours' start-up, so the sum is slightly above hpspmm_csr_spmm_timed's
 * mean.  The reference has no counterpart (its launchers are single kernels).
 */
int hpspmm_csr_spmm_timed_launches(hpspmm_plan *plan, const int32_t *d_rowptr, const int32_t *d_col,
                                   const float *d_val, const float *d_B, float *d_C, void *stream,
                                   int warmup, int iters, int max_launches, float *mean_ms_out,
                                   const char **names_out, int *n_launches_out);

#ifdef __cplusplus
}
#endif
#endif /* HPSPMM_H_ */
