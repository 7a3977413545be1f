/*
 * lapis_hip.h -- C ABI of the gfx950 (MI355X) kernel library behind
 * LAPIS-generated sparse CSR modules.
 *
 * Every entry point takes plain DEVICE pointers and sizes, launches on the
 * hipStream_t it is given (passed as void*, NULL = the null stream), returns a
 * status code and never synchronises unless its comment says so.  Index
 * buffers are int32 (posWidth = crdWidth = 32 of the reference's #sparse
 * encoding, benchmarks/spmv/spmv.mlir:1).
 *
 * Each declaration names the piece of the reference whose emitted Kokkos code
 * it replaces; paths are relative to the reference tree and
 * "emitter" = mlir/lib/Target/KokkosCpp/TranslateToKokkosCpp.cpp.
 */
#ifndef LAPIS_HIP_H
#define LAPIS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *lapis_hip_stream_t; /* a hipStream_t */

enum lapis_hip_status {
  LAPIS_HIP_OK = 0,
  LAPIS_HIP_ERR_INVALID_ARGUMENT = 1, /* null pointer with non-zero size, negative size, bad enum */
  LAPIS_HIP_ERR_RUNTIME = 2,          /* a HIP call or kernel launch failed */
  LAPIS_HIP_ERR_NOT_INITIALIZED = 3,  /* lapis_hip_init() has not been called */
  LAPIS_HIP_ERR_BAD_CSR = 4,          /* positions not monotone / coordinates out of range */
  LAPIS_HIP_ERR_UNSUPPORTED_DEVICE = 5, /* the current device is not gfx950 */
  LAPIS_HIP_ERR_PLAN_MISMATCH = 6,    /* plan was built for other sizes or buffers */
  LAPIS_HIP_ERR_NO_TILING = 7         /* the matrix has no room in the column-blocked tiling (too many columns,
                                         slices or row blocks): the plan keeps its CSR kernel */
};

/* ---- runtime ------------------------------------------------------------ */

/* Replaces `if(!Kokkos::is_initialized()) Kokkos::initialize();` of the emitted
 * lapis_initialize() (emitter :4284-4290).  Idempotent and reference counted;
 * checks that the current device is gfx950. */
int lapis_hip_init(void);
/* Replaces `Kokkos::finalize()` of the emitted lapis_finalize() (emitter :4352-4376). */
int lapis_hip_finalize(void);
/* Message of the last non-OK status returned on the calling thread, and the name of
 * a status code.  The reference has no status codes: its emitted code calls
 * Kokkos::abort (LAPISSupport.hpp:76,86; emitter :1294-1301); the generated-module
 * shim keeps that behaviour on top of these. */
const char *lapis_hip_last_error(void);
const char *lapis_hip_status_name(int status);
/* Replaces Kokkos::DefaultExecutionSpace().fence() (emitter :2680-2682). */
int lapis_hip_stream_synchronize(lapis_hip_stream_t stream);

/* ---- kernel timing -------------------------------------------------------------- */

/* Device-side duration of the dominant kernels (the SpMV main kernel of whichever
 * family runs, and the SpMM kernel): between start and stop every such launch
 * carries its own pair of HIP events, so the figure is the kernel's own run time
 * on its stream, not a host clock.  The reference times whole fenced calls with
 * Kokkos::Timer instead (benchmarks/spmv/main.cpp:52-62); these two calls exist
 * for the roofline report only.  `capacity` = launches to keep (later ones are
 * not timed).  stop synchronises the device and returns count / mean / min / max
 * in milliseconds (any output may be NULL). */
int lapis_hip_kernel_timing_start(int capacity);
int lapis_hip_kernel_timing_stop(int *count, double *mean_ms, double *min_ms, double *max_ms);
/* Median, in milliseconds, of the launches the last lapis_hip_kernel_timing_stop read (0 before the first). */
double lapis_hip_kernel_timing_median_ms(void);

/* Measurement only (`bench.py --calibrate-gather`): one launch in the shape of the
 * column-blocked SpMV kernels -- one workgroup of 512 threads per compute unit,
 * each thread per step streaming three 16-byte vectors from `stream_buf` (12 bytes
 * per gather, what crd + val of an fp64 non-zero take; NULL = no stream) and
 * gathering four doubles from the first `window_bytes` of `x`, with
 * `lanes_per_line` neighbouring lanes of a wave instruction in one 128-byte line
 * (0 = no gathers).  Returns the best of five timed launches in `elapsed_ms` and
 * what one launch did.  `sink` takes one double per compute unit.  The reference
 * has no counterpart; its table of measured SpMV times is
 * benchmarks/plots/spmv.csv.  Synchronises `stream`. */
int lapis_hip_calibrate_gather(const double *x, int64_t window_bytes, int lanes_per_line, const void *stream_buf,
                               int64_t stream_bytes, int64_t gathers, double *sink, double *elapsed_ms,
                               double *gathers_done, double *stream_bytes_done, lapis_hip_stream_t stream);

/* Measurement only (`bench.py --calibrate-gather`): the same two kinds of load in other
 * arrangements, to see whether any of them lets a compute unit overlap the stream with the
 * gathers.  A launch streams `stream_bytes` from `stream_buf` and does `gathers` gathers of
 * doubles from the first `window_bytes` of `x`, split evenly over the wavefronts that have
 * the role.  `cu_count` (16 * 256 ints) is needed for roles = 2 only.  Returns the best of
 * five timed launches and what one launch did; `cus_with_both_roles` = compute units that
 * ran one workgroup of each role (roles = 2), else -1.  No counterpart in the reference. */
typedef struct lapis_hip_calibrate_mode {
  int threads;           /* per workgroup, a multiple of 64 up to 1024 */
  int workgroups;        /* 0 = one per compute unit */
  int stream_in_flight;  /* 16-byte loads per lane and step: 0 (no stream), 3, 6 or 12 */
  int gathers_in_flight; /* gathers per lane and step: 0 (none), 2, 4 or 8 */
  int lanes_per_line;    /* neighbouring lanes of a gather instruction in one 128-byte line */
  int roles;             /* 0: every wavefront streams and gathers; 1: `producers` wavefronts of each
                            workgroup only stream, the others only gather; 2: by workgroup, in the
                            order in which workgroups arrive on a compute unit */
  int producers;
  int stream_behind;     /* 1: the stream loads of the next step are issued after this step's gathers */
  int stream_policy;     /* 0 plain, 1 nt, 2 sc0 sc1, 3 sc0 sc1 nt, 4 straight to LDS */
  int stream_in_l2;      /* 1: the stream wraps inside a window that stays in L2 */
  int scalar;            /* 1: the stream alone, read with 64-byte scalar loads; 2: as many helper
                            wavefronts as consumers touch the consumers' stream through the scalar
                            cache `scalar_ahead` steps ahead, one 4-byte load per `scalar_stride` bytes */
  int scalar_ahead;
  int scalar_stride;
} lapis_hip_calibrate_mode;
int lapis_hip_calibrate_mix(const lapis_hip_calibrate_mode *mode, const double *x, int64_t window_bytes,
                            const void *stream_buf, int64_t stream_buf_bytes, int64_t stream_bytes, int64_t gathers,
                            int *cu_count, double *sink, double *elapsed_ms, double *gathers_done,
                            double *stream_bytes_done, int *cus_with_both_roles, lapis_hip_stream_t stream);

/* ---- CSR plan: the team/vector loop-mapping decision ---------------------- */

/* Which kernel a plan launches for SpMV. */
enum lapis_hip_spmv_kernel {
  LAPIS_HIP_SPMV_AUTO = 0,
  /* `width` lanes per row (1,2,4,...,64), rows packed into wave64; the shape the
   * reference's TeamPolicy(league, team, vector) launch has (emitter :1976-2039). */
  LAPIS_HIP_SPMV_SUBWARP = 1,
  /* 64 consecutive rows per wavefront; their products are staged in LDS with
   * 128-bit coalesced loads and summed one row per lane in ascending order. */
  LAPIS_HIP_SPMV_ROWBLOCK = 2,
  /* equal non-zero count per wavefront whatever the row lengths (row split);
   * rows cut by a chunk boundary are completed by a small second kernel. */
  LAPIS_HIP_SPMV_NNZSPLIT = 3,
  /* column-blocked copy of the matrix, see lapis_hip_csr_plan_build_colblock */
  LAPIS_HIP_SPMV_COLBLOCK = 4
};

typedef struct lapis_hip_csr_stats {
  int64_t nrows, ncols, nnz;
  int64_t min_row_len, max_row_len, empty_rows;
  double mean_row_len, var_row_len;
  /* mean over chunks of 1024 consecutive non-zeros of (max column - min column):
   * how far the gathers of one wavefront wander over x; -1 if crd was not given */
  double mean_chunk_col_span;
  /* the reference's own decision for this matrix, for comparison:
   * hint = ceil((pos[n]-pos[0])/n) (KokkosLoopMapping.cpp:279-323) and
   * LAPIS::threadParallelVectorLength(hint) with vector_length_max = 64
   * (LAPISSupport.hpp:428-435) */
  int64_t reference_hint;
  int32_t reference_vector_length;
  /* what this plan launches */
  int32_t kernel;      /* enum lapis_hip_spmv_kernel, never AUTO */
  int32_t width;       /* lanes per row for SUBWARP, else 0 */
  int32_t chunk;       /* non-zeros per wavefront for NNZSPLIT (512, 1024 or 2048), else 0 */
  /* 1 if the column-blocked copy is expected to pay for this matrix (the gathers of a
   * 1024-non-zero chunk range over more of x than an XCD's L2 keeps, and the matrix has
   * at least 2^20 non-zeros); lapis_hip_csr_plan_analyze builds it when this is set
   * (plan creation cannot: it is not given the values) */
  int32_t colblock_recommended;
  /* enum lapis_hip_colblock_layout of the copy this plan holds, 0 if none */
  int32_t colblock_layout;
  /* fraction of the non-zeros with |column - row| <= 32, 64, 128, 256: how much of the
   * matrix sits in a band around the diagonal (what the LDS-staged SpMM kernel can
   * serve from its staged window of B); -1 if crd was not given */
  double near_diagonal_fraction[4];
} lapis_hip_csr_stats;

typedef struct lapis_hip_csr_plan lapis_hip_csr_plan;

/* Replaces estimateParallelism + the nestingLevel==2 branch of the loop-mapping
 * pass (KokkosLoopMapping.cpp:132-343, :888-921) and the per-launch
 * team_size_recommended query (emitter :2013-2033): reads the row-length
 * statistics of the matrix ONCE on the device, validates the structure
 * (monotone positions, pos[0]==0, pos[n]==nnz, coordinates inside [0,ncols) when
 * `crd` is non-NULL) and fixes the kernel.  `value_bytes` is 4 or 8.
 * Synchronises `stream`.  The plan keeps `pos` by address: it stays valid for as
 * long as that buffer holds the same positions. */
int lapis_hip_csr_plan_create(lapis_hip_csr_plan **plan, int64_t nrows, int64_t ncols, int64_t nnz,
                              const int32_t *pos, const int32_t *crd, int value_bytes,
                              lapis_hip_stream_t stream);
/* Second half of the loop-mapping decision, for callers that will run many SpMVs with
 * one matrix: given the values too, builds the column-blocked copy
 * (lapis_hip_csr_plan_build_colblock, AUTO layout) when the statistics recommend it, and
 * selects that kernel; otherwise leaves the plan as it is.  The copy costs about as
 * much as 40 SpMVs of the same matrix (one radix sort).  If the plan already holds a
 * copy made from `crd`, only its values are refreshed.  No counterpart in the reference
 * (its launch never looks at columns, KokkosLoopMapping.cpp:861-862).  Synchronises
 * `stream`. */
int lapis_hip_csr_plan_analyze(lapis_hip_csr_plan *plan, const int32_t *crd, const void *val, int value_bytes,
                               lapis_hip_stream_t stream);
/* Brings the values of the plan's column-blocked copy up to date with `val` (the
 * caller's CSR values, same order as at build time): one gather pass through the kept
 * sort permutation, no sort, no synchronisation.  The reference reads val on every
 * call (tests/Dialect/Kokkos/loop_mapping_2.mlir.gold:22); a copy cannot, so callers
 * that change values in place call this afterwards.  `val` may be a different buffer
 * than before: later SpMV calls must then pass this one.  A plan without a copy is left
 * alone (status OK). */
int lapis_hip_csr_plan_update_values(lapis_hip_csr_plan *plan, const void *val, int value_bytes,
                                     lapis_hip_stream_t stream);
/* 1 when `plan` was made for exactly this structure -- the same sizes, the same number of
 * non-zeros and the same position and coordinate buffers -- else 0 (also for a NULL plan).
 * For callers that keep a plan between calls: the SpMV entry points compare sizes and the
 * position buffer only (they take no nnz), which a second matrix of the same shape at the
 * same address would pass.  The reference has nothing to cache: its launch re-reads
 * pos[n] and pos[0] on the host every call (KokkosLoopMapping.cpp:290-322). */
int lapis_hip_csr_plan_matches(const lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, int64_t nnz,
                               const int32_t *pos, const int32_t *crd);
/* Name of the SpMV kernel a launch with `plan` runs ("spmv_subwarp_kernel", "spmv_rowblock_kernel",
 * "spmv_nnzsplit_kernel", "spmv_colblock_kernel", "spmv_colgroup_kernel", "spmv_colgroup_pc_kernel"; ""
 * for NULL): benchmark lines and profiles name the kernel they timed with it.  No counterpart in the
 * reference, whose kernel is fixed when the module is compiled (KokkosLoopMapping.cpp:888-921). */
const char *lapis_hip_csr_plan_kernel_name(const lapis_hip_csr_plan *plan);
/* lapis_hip_csr_plan_analyze for callers that need the same bits from every run: where the
 * copy pays it is built in the per-wavefront layout (LAPIS_HIP_COLBLOCK_WAVE, wave-private
 * row sums in a fixed order) instead of the faster workgroup layout, whose LDS atomics fix
 * no order.  The reference's Kokkos kernel is reproducible run to run
 * (tests/Dialect/Kokkos/loop_mapping_2.mlir.gold:14-35 fixes its order). */
int lapis_hip_csr_plan_analyze_reproducible(lapis_hip_csr_plan *plan, const int32_t *crd, const void *val,
                                            int value_bytes, lapis_hip_stream_t stream);
/* Waits for `stream` and reports whether a kernel of this plan gave up a wait between its
 * own wavefronts (the workgroup-blocked SpMV hands entries from streaming wavefronts to
 * gathering ones through LDS, and every such wait is bounded so that a launch always
 * ends): LAPIS_HIP_OK, or LAPIS_HIP_ERR_RUNTIME, in which case the last results computed
 * with the plan are not to be used.  No counterpart in the reference; for tests and for
 * callers that want the assurance. */
int lapis_hip_csr_plan_check(lapis_hip_csr_plan *plan, lapis_hip_stream_t stream);
/* Overrides the automatic choice (tuning and tests).  `width` is used by SUBWARP
 * (0 = the reference's rule); other kernels ignore it. */
int lapis_hip_csr_plan_set_kernel(lapis_hip_csr_plan *plan, int kernel, int width);
/* The statistics and the choice, including what the reference's rule would have
 * chosen (estimate of KokkosLoopMapping.cpp:279-323, vector length of
 * LAPISSupport.hpp:428-435). */
int lapis_hip_csr_plan_get_stats(const lapis_hip_csr_plan *plan, lapis_hip_csr_stats *stats);
/* Opt-in layouts for matrices whose x does not fit the 4 MB L2 of an XCD (wide,
 * uniformly random columns).  crd/val are copied once into an order in which a
 * block of consecutive rows walks its non-zeros slice by slice of x
 * (2^slice_log2_cols columns per slice, 0 = default), with the row sums of the block
 * in LDS; all blocks are resident and walk the slices together, so the chip gathers
 * from the same few slices at a time and they stay in L2.  Same 4+sizeof(T) bytes
 * per non-zero as CSR.
 *   WAVE : one wavefront per 1024 rows, entries of a tile in row order, the
 *          wavefronts paced by the clock (pace calibrated here, a few launches).
 *          Sums are added in a fixed order: results repeat bit for bit.  Needs
 *          ceil(log2(ncols)) <= 22.
 *   GROUP: one workgroup per up to 16384 rows, entries of a tile in COLUMN order,
 *          so neighbouring lanes gather from the same 128-byte lines (fewer requests
 *          to L2, which is what bounds these matrices).  Row sums are LDS atomics
 *          shared by the wavefronts of the group: the order of additions, and with it
 *          the last bits of y, can differ between runs.  Rows much longer than the
 *          rest (>= max(2048, 16 x mean) entries) are numbered apart and fill row
 *          blocks of their own; every block's entries are cut into equal work units,
 *          one workgroup each, so skewed matrices balance.  Blocks cut into several
 *          units, and the blocks of long rows, update y with hardware floating-point
 *          atomics: y must be ordinary (coarse-grained) device memory.  AUTO picks
 *          this layout.
 * The reference has no counterpart (its launch never looks at columns,
 * KokkosLoopMapping.cpp:861-862).  The copy holds the VALUES as they are now: after
 * changing val call lapis_hip_csr_plan_update_values (the sort permutation is kept,
 * 4 bytes per non-zero).  Selects the COLBLOCK kernel on success; SpMV calls with this
 * plan must pass the same crd and val buffers the copy was made from, anything else is
 * refused with LAPIS_HIP_ERR_PLAN_MISMATCH.  Synchronises `stream`. */
enum lapis_hip_colblock_layout {
  LAPIS_HIP_COLBLOCK_AUTO = 0,
  LAPIS_HIP_COLBLOCK_WAVE = 1,
  LAPIS_HIP_COLBLOCK_GROUP = 2
};
int lapis_hip_csr_plan_build_colblock(lapis_hip_csr_plan *plan, const int32_t *crd, const void *val,
                                      int value_bytes, int layout, int slice_log2_cols,
                                      lapis_hip_stream_t stream);
/* Frees the plan's device buffers; emitted code would call it where lapis_finalize()
 * frees the module's global views (emitter :4352-4376).  NULL is allowed. */
int lapis_hip_csr_plan_destroy(lapis_hip_csr_plan *plan);

/* ---- SpMV ------------------------------------------------------------------ */

/* y[i] = y[i] + sum_j val[j] * x[crd[j]],  j in [pos[i], pos[i+1]).
 * Replaces the TeamPolicy/ThreadVectorRange lambda the emitter prints for
 * tests/Dialect/Kokkos/loop_mapping_2.mlir.gold:12-37 (emitter :1966-2064 with
 * :1692-1845, :2127-2157, :1671-1690, :2073-2125).
 * `plan` may be NULL: the launch then follows the reference's rule, reading
 * pos[n] and pos[0] back to the host on every call as the emitted code does
 * (that read synchronises `stream`).  Calls sharing one plan must be ordered on
 * one stream (the plan owns the row-split workspace).  x and y must not alias. */
int lapis_hip_spmv_csr_f64_i32(lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols,
                               const int32_t *pos, const int32_t *crd, const double *val,
                               const double *x, double *y, lapis_hip_stream_t stream);
int lapis_hip_spmv_csr_f32_i32(lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols,
                               const int32_t *pos, const int32_t *crd, const float *val,
                               const float *x, float *y, lapis_hip_stream_t stream);

/* ---- SpMM ------------------------------------------------------------------ */

/* C[i,:] = C[i,:] + sum_kk val[kk] * B[crd[kk],:]; B is ncols-by-k with leading
 * dimension ldb, C is nrows-by-k with leading dimension ldc, both row-major.
 * Replaces the nest the sparsifier emits for CSR x dense linalg.matmul
 * (examples/spmm_dcsr_opdsl.py:73-110, examples/bspmm.py:22-50) under the
 * race-free parallelization strategies (Pipelines/Passes.h:41-56). */
int lapis_hip_spmm_csr_f32_i32(int64_t nrows, int64_t ncols, int64_t k, const int32_t *pos,
                               const int32_t *crd, const float *val, const float *B, int64_t ldb,
                               float *C, int64_t ldc, lapis_hip_stream_t stream);
int lapis_hip_spmm_csr_f64_i32(int64_t nrows, int64_t ncols, int64_t k, const int32_t *pos,
                               const int32_t *crd, const double *val, const double *B, int64_t ldb,
                               double *C, int64_t ldc, lapis_hip_stream_t stream);

/* The same product with the plan's statistics deciding the kernel.
 *   group per row: matrices with short, even rows (mean <= 256, longest <= 4 x mean)
 *     whose columns stay local (the B rows a stretch of 1024 non-zeros touches fit the
 *     L2s: stencils, meshes).  64/LPR rows per wavefront at a time, one group of lanes
 *     per row, no cross-lane reduction: 1.25x-5.8x faster than the kernel below there.
 *   wavefront per row: everything else, and `plan == NULL` (the entry points above).
 *   LDS-staged row block: a workgroup stages the rows of B of its block's diagonal
 *     window in LDS with coalesced 128-bit loads and serves the non-zeros inside the
 *     window from LDS.  Built and kept selectable (LAPIS_HIP_SPMM_KERNEL=lds) but never
 *     chosen: on MI355X it measured 1.6x-2.4x slower than group per row on the
 *     stencil and FEM matrices it is meant for.
 * The reference chooses between its loop mappings by strategy name
 * (Pipelines/Passes.h:41-56), never by looking at the columns. */
int lapis_hip_spmm_csr_f32_i32_plan(const lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, int64_t k,
                                    const int32_t *pos, const int32_t *crd, const float *val, const float *B,
                                    int64_t ldb, float *C, int64_t ldc, lapis_hip_stream_t stream);
int lapis_hip_spmm_csr_f64_i32_plan(const lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, int64_t k,
                                    const int32_t *pos, const int32_t *crd, const double *val, const double *B,
                                    int64_t ldb, double *C, int64_t ldc, lapis_hip_stream_t stream);

/* Name of the kernel the calling thread's last SpMM call launched ("spmm_wave_row_kernel",
 * "spmm_group_row_kernel", "spmm_rowblock_lds_kernel"; "" before the first call): benchmark lines name the
 * kernel they timed with it.  No counterpart in the reference, whose loop mapping is fixed when the module
 * is compiled (Pipelines/Passes.h:41-56). */
const char *lapis_hip_spmm_last_kernel(void);

/* Batched CSRV product of examples/bspmm.py:22-50 (out(n1,dh,nh) += A(n1,n2,nh) * V(n2,dh,nh)):
 * A is CSR over (n1, n2), each non-zero carries nh values (val has nnz*nh entries). */
int lapis_hip_bspmm_csrv_f32_i32(int64_t n1, int64_t n2, int64_t dh, int64_t nh, const int32_t *pos,
                                 const int32_t *crd, const float *val, const float *V, float *out,
                                 lapis_hip_stream_t stream);

/* ---- dense vector kernels of CG -------------------------------------------- */

/* *result = init + sum_i x[i]*y[i]; `result` is a DEVICE scalar (no host sync,
 * unlike the Kokkos::parallel_reduce into a host scalar it replaces: emitter
 * :1696-1705, :1790-1844; loop shape tests/Dialect/Kokkos/linalg_to_loops_0.mlir.gold:7-18).
 * Deterministic: fixed block partials summed in a fixed order. */
int lapis_hip_dot_f64(int64_t n, const double *x, const double *y, double init, double *result,
                      lapis_hip_stream_t stream);
int lapis_hip_dot_f32(int64_t n, const float *x, const float *y, float init, float *result,
                      lapis_hip_stream_t stream);
/* The dot product with its result on the HOST, the call returning when it is there: what
 * the reference's emitted code has, Kokkos::parallel_reduce into a host scalar followed by
 * the join with the initial value (TranslateToKokkosCpp.cpp:1696-1705,1838; 1671-1690).
 * For emitted code that needs the number at once; the device-scalar entries above are for
 * callers that can leave it on the device. */
int lapis_hip_dot_f64_host(int64_t n, const double *x, const double *y, double init, double *host_result,
                           lapis_hip_stream_t stream);
int lapis_hip_dot_f32_host(int64_t n, const float *x, const float *y, float init, float *host_result,
                           lapis_hip_stream_t stream);
/* dst = a*x + b*y and *result = init + sum dst[i]*z[i] in one pass over the vectors (z NULL:
 * dst . dst).  The pair the CG loop of examples/pcg_solve.py:80-82 runs back to back
 * (r = r - alpha*Ap, then r . r): fused it reads r and Ap once and writes r once, five
 * vector passes becoming three.  dst may be x or y.  With 16-byte-aligned buffers both
 * results have exactly the bits lapis_hip_axpby_* followed by lapis_hip_dot_* give.
 * `result` is a device scalar. */
int lapis_hip_axpby_dot_f64(int64_t n, double a, const double *x, double b, const double *y, double *dst,
                            const double *z, double init, double *result, lapis_hip_stream_t stream);
int lapis_hip_axpby_dot_f32(int64_t n, float a, const float *x, float b, const float *y, float *dst, const float *z,
                            float init, float *result, lapis_hip_stream_t stream);
/* lapis_hip_dot_f64 for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same kernels and the same result, bit for bit, as lapis_hip_dot_f64, but
 * the block partials live in a fixed 16 KB array inside the library's code object
 * (one copy per GPU, held until the process ends) instead of an allocated ring: the
 * call performs no hipMalloc / hipFree.  n above LAPIS_HIP_DOT_NOALLOC_MAX_N is
 * rejected with LAPIS_HIP_ERR_INVALID_ARGUMENT.  All calls on one GPU share the one
 * array: calls that overlap on one GPU (different streams or threads) race; order
 * them on one stream. */
#define LAPIS_HIP_DOT_NOALLOC_MAX_N (INT64_C(1) << 34)
int lapis_hip_dot_f64_noalloc(int64_t n, const double *x, const double *y, double init, double *result,
                              lapis_hip_stream_t stream);
/* dst[i] = a*x[i] + b*y[i] (examples/pcg_solve.py:30-38; RangePolicy parallel_for,
 * emitter :1710-1715).  dst may alias x or y. */
int lapis_hip_axpby_f64(int64_t n, double a, const double *x, double b, const double *y, double *dst,
                        lapis_hip_stream_t stream);
int lapis_hip_axpby_f32(int64_t n, float a, const float *x, float b, const float *y, float *dst,
                        lapis_hip_stream_t stream);
/* dst[i] = x[i]*y[i] (examples/pcg_solve.py:40-47). */
int lapis_hip_mult_f64(int64_t n, const double *x, const double *y, double *dst, lapis_hip_stream_t stream);
int lapis_hip_mult_f32(int64_t n, const float *x, const float *y, float *dst, lapis_hip_stream_t stream);
/* dst[i] = x[i]/y[i] (linalg.div of examples/hitting_times.py:120,146). */
int lapis_hip_div_f64(int64_t n, const double *x, const double *y, double *dst, lapis_hip_stream_t stream);
int lapis_hip_div_f32(int64_t n, const float *x, const float *y, float *dst, lapis_hip_stream_t stream);
/* dst[i] = v (linalg.fill, examples/pcg_solve.py:15-17). */
int lapis_hip_fill_f64(int64_t n, double v, double *dst, lapis_hip_stream_t stream);
int lapis_hip_fill_f32(int64_t n, float v, float *dst, lapis_hip_stream_t stream);
/* dst[i] = src[i] (linalg.copy, examples/pcg_solve.py:65-67). */
int lapis_hip_copy_f64(int64_t n, const double *src, double *dst, lapis_hip_stream_t stream);
int lapis_hip_copy_f32(int64_t n, const float *src, float *dst, lapis_hip_stream_t stream);
/* val[j] *= alpha in place (scale_csr, examples/hitting_times.py:51-71). */
int lapis_hip_scale_f64(int64_t n, double alpha, double *val, lapis_hip_stream_t stream);

/* ---- CG -------------------------------------------------------------------- */

/* The solver examples/pcg_solve.py:52-101 lowers to (host while-loop, emitter
 * :1512-1593): x0 = 0, Jacobi preconditioner `dinv` (NULL = unpreconditioned:
 * z = r, so the r.z and r.r products coincide and one iteration is
 * SpMV + 2 dots + 3 axpy), stop when relres <= tol or the iteration counter,
 * which starts at 1, equals maxiter.  All vectors are device buffers of length
 * n; `work` is 4*n doubles of device scratch or NULL (allocated and freed
 * inside).  Scalars stay on the device between kernels; the host looks at the
 * convergence flag every few iterations only.  `iters` and `relres` are HOST
 * outputs; the call synchronises `stream` before returning.
 * `plan` may be NULL (one is built and destroyed inside, with the column-blocked copy
 * when the matrix calls for it and maxiter >= 64 lets it pay back). */
int lapis_hip_pcg_f64_i32(lapis_hip_csr_plan *plan, int64_t n, const int32_t *pos, const int32_t *crd,
                          const double *val, const double *b, const double *dinv, double tol,
                          uint64_t maxiter, double *x, uint64_t *iters, double *relres, double *work,
                          lapis_hip_stream_t stream);

/* The solver variant of examples/hitting_times.py:97-149: the operator is the masked
 * normalized graph Laplacian plpt (:73-93), y = mask*(d*(mask*p) - A (mask*p)), and
 * the preconditioner is an elementwise division by d.  `work` is 5*n doubles or NULL. */
int lapis_hip_pcg_masked_f64_i32(lapis_hip_csr_plan *plan, int64_t n, const int32_t *pos, const int32_t *crd,
                                 const double *val, const double *b, const double *mask, const double *d,
                                 double tol, uint64_t maxiter, double *x, uint64_t *iters, double *relres,
                                 double *work, lapis_hip_stream_t stream);

/* func @mht of examples/hitting_times.py:153-179: scales val by alpha IN PLACE
 * (scale_csr, :51-71), then two masked CG solves for the first two hitting-time
 * moments.  A column-blocked copy in `plan` is refreshed after the scaling.
 * Synchronises `stream`. */
int lapis_hip_mht_f64_i32(lapis_hip_csr_plan *plan, int64_t n, int64_t nnz, const int32_t *pos,
                          const int32_t *crd, double *val, const double *mask, const double *d, double alpha,
                          double tol, uint64_t maxiter, double *mom1, double *mom2, lapis_hip_stream_t stream);
/* func @normalize_mom2 of examples/hitting_times.py:181-198: out = sqrt(mom2 - mom1*mom1). */
int lapis_hip_normalize_mom2_f64(int64_t n, const double *mom1, const double *mom2, double *out,
                                 lapis_hip_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LAPIS_HIP_H */
