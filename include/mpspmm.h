/*
 * mpspmm.h -- C ABI of the MI355X (gfx950) MergePath-SpMM library.
 *
 * The reference (cag-uconn/MergePath-SpMM) has no library interface: each
 * program is one translation unit whose main() parses a .csr file, builds the
 * schedule on the host and launches a kernel.  The entry points below are the
 * seams of those programs, one per step, so that a host program -- the C++
 * drivers shipped beside this library, or any FFI -- can replace the step it
 * names.  Each declaration cites the reference lines it stands in for.
 *
 * Conventions
 *   - Every function returns an int status: MPS_OK (0) or an mps_status
 *     value; HIP runtime failures return MPS_ERR_HIP + hipError_t.  Nothing
 *     throws and nothing calls exit().
 *   - "d_" arguments are device pointers, everything else is host memory.
 *   - The caller owns every buffer, including workspaces; the library
 *     allocates device memory only where a comment says so (plans).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     Calls are asynchronous with respect to the host; the caller
 *     synchronises.
 *   - Indices are 32-bit (as in the reference); n_rows + 1 + nnz must fit in
 *     an int.  The sparse matrix is square: column ids index the n_rows rows
 *     of the dense input (src/MergePathSpMM.cu:459-460).
 *   - Dense matrices are row-major, K columns, no padding.
 *   - fp16 data is IEEE binary16 passed as uint16_t bit patterns.
 *   - Y is overwritten (Y = A * X); results do not depend on what Y held and
 *     repeated calls give identical bits (merge-path and row-wise kernels).
 *   - d_X, d_Y and workspaces must be 16-byte aligned; index and value
 *     arrays need only their natural alignment.
 */
#ifndef MPSPMM_H
#define MPSPMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum mps_status {
    MPS_OK = 0,
    MPS_ERR_INVALID_ARG = 1,  /* null pointer, negative size, cost <= 0 ...      */
    MPS_ERR_UNSUPPORTED = 2,  /* sizes beyond 32-bit indexing, K out of range     */
    MPS_ERR_WORKSPACE = 3,    /* workspace missing or too small                   */
    MPS_ERR_ALIGNMENT = 4,    /* a device pointer is not 16-byte aligned          */
    MPS_ERR_IO = 5,           /* file cannot be opened / read / written           */
    MPS_ERR_FORMAT = 6,       /* malformed .csr text or generator spec            */
    MPS_ERR_TPW = 7,          /* threads_per_wave beyond what one wave can hold   */
    MPS_ERR_INVALID_CSR = 8,  /* device-side validation found a bad row_ptr/col   */
    MPS_ERR_UNSORTED = 9,     /* tiling needs column ids sorted within every row  */
    MPS_ERR_HIP = 1000        /* + hipError_t                                     */
} mps_status;

/* Human-readable text for a status value (static storage). */
const char *mps_status_string(int status);

/* Library version, "major.minor.patch". */
const char *mps_version(void);

/* ------------------------------------------------------------------------ */
/* Host side: sizes and schedule arithmetic                                  */
/* ------------------------------------------------------------------------ */

/* cost -> number of merge-path partitions.
 * Replaces src/MergePathSpMM.cu:138-139:
 *   P = (n_rows + 1 + nnz - 1) / cost;  if (P < 1024) P = 1024.
 * cost <= 0 is rejected (the reference divides by it). */
int mps_num_partitions(int n_rows, int nnz, int cost, int *P_out);

/* The cost this library uses when the caller names none (the reference has
 * no default; src/MergePathSpMM.cu:121 takes it from argv).  Measured on
 * MI355X: 32 merge items per partition, 64 from 2^25 items and 128 from 2^27
 * items on; and never fewer than about 512 items per wavefront, i.e. at least
 * 512 / partitions per wavefront for the given K and element size (32 at
 * K = 16 fp32, 128 at K = 64, 512 at K = 256: the carry-out records of a
 * wavefront are 8 K bytes, so wide rows want few of them); 1,024 items per
 * wavefront where the rows hold 32 nonzeros or more on average. */
int mps_default_cost(int n_rows, int nnz, int K, int elem_bytes, int *cost_out);

/* Merge items per partition, src/MergePathSpMM.cu:327-328:
 *   ceil((n_rows + 1 + nnz) / P). */
int mps_items_per_partition(int n_rows, int nnz, int P, int *ipt_out);

/* Largest threads_per_wave (partitions walked side by side by one 64-lane
 * wavefront) for feature width K and element size elem_bytes (4 = fp32,
 * 2 = fp16).  Stands in for WARP_SIZE / dimension at
 * src/MergePathSpMM.cu:224-228: a partition occupies K / (16 / elem_bytes)
 * lanes (one 16-byte load per lane), at least 4. */
int mps_max_threads_per_wave(int K, int elem_bytes, int *tpw_out);

/* ------------------------------------------------------------------------ */
/* Host side: .csr text files                                                */
/* ------------------------------------------------------------------------ */

/* Two-line comma-separated text: line 1 = row_ptr (n_rows + 1 integers),
 * line 2 = col_idx (nnz integers); every integer may be followed by ','.
 * Written by scripts/fetch_dataset.py:14-21 and scripts/npz_to_csr.py:21-28,
 * read by src/MergePathSpMM.cu:126-173.
 *
 * mps_csr_read_header: pass 1 of the reference reader (:131-137): n_rows is
 * the number of cells of line 1 minus one, nnz its last cell. */
int mps_csr_read_header(const char *path, int *n_rows_out, int *nnz_out);

/* Pass 2 (:147-173): fill row_ptr[n_rows + 1] and col_idx[nnz] (host memory,
 * sized from mps_csr_read_header).  MPS_ERR_FORMAT when a cell is not an
 * integer, line 2 does not hold exactly nnz cells, row_ptr is not
 * non-decreasing from 0, or a column id is outside [0, n_rows). */
int mps_csr_read(const char *path, int n_rows, int nnz, int *row_ptr, int *col_idx);

/* Writer with the byte layout of scripts/npz_to_csr.py:21-28 (each element
 * followed by ',', one '\n' between the lines, none at the end). */
int mps_csr_write(const char *path, int n_rows, const int *row_ptr, const int *col_idx);

/* ------------------------------------------------------------------------ */
/* Host side: seeded synthetic graphs and fills                              */
/* ------------------------------------------------------------------------ */

/* The reference ships no data (README.md:18-25 points at a download); these
 * generators make the benchmark graphs reproducibly from a spec string:
 *   "er:n=4096,deg=8"                          Erdos-Renyi G(n, deg/n), directed, no self-loops
 *   "chunglu:n=232965,nnz=114600000,gamma=2.1,dmax=20000[,sorted=1]"
 *                                              Chung-Lu, expected degrees ~ shifted power law
 *   "blockdiag:blocks=1178,min=100,max=600,deg=5"
 *                                              disjoint random-geometric blocks
 *   "rmat:scale=20,ef=16,a=0.57,b=0.19,c=0.19" R-MAT, duplicates removed
 *   "band:n=233000,deg=64,width=2000"          banded: Erdos-Renyi inside |row - column| <= width, no self-loops
 * Column ids are sorted and distinct within every row.  The result depends
 * only on (spec, seed), not on the number of host threads.
 * The graph is held by an opaque handle owned by the library. */
typedef struct mps_graph mps_graph;
int mps_graph_generate(const char *spec, uint64_t seed, mps_graph **graph_out);
int mps_graph_from_csr_file(const char *path, mps_graph **graph_out);
/* Edge list -> graph, what the reference's converter does with scipy
 * (scripts/npz_to_csr.py:14-20: coo_matrix((1, (src_li, dst_li))).tocsr(),
 * which sorts the column ids of every row and merges repeated edges).  The
 * matrix is square: n_rows = 1 + the largest id on either side (the kernels
 * index X and the degrees by column id, src/MergePathSpMM.cu:459-460). */
int mps_graph_from_edges(const int64_t *src, const int64_t *dst, int64_t n_edges, mps_graph **graph_out);
int mps_graph_dims(const mps_graph *g, int *n_rows_out, int *nnz_out, int *max_degree_out);
const int *mps_graph_row_ptr(const mps_graph *g); /* host, n_rows + 1 */
const int *mps_graph_col_idx(const mps_graph *g); /* host, nnz        */
void mps_graph_free(mps_graph *g);

/* out[i] = lo + (hi - lo) * u(seed, i), u uniform in [0, 1) with 24 random
 * bits; element i depends only on (seed, i).  Replaces the constant fill of
 * src/MergePathSpMM.cu:180-182. */
int mps_fill_uniform_f32(float *out, size_t n, uint64_t seed, float lo, float hi);
/* Same with 11 random bits so that every value is exact in binary16. */
int mps_fill_uniform_f16(uint16_t *out, size_t n, uint64_t seed, float lo, float hi);

/* ------------------------------------------------------------------------ */
/* Device side: validation                                                   */
/* ------------------------------------------------------------------------ */

/* Edge weights from degrees, on the device: the reference's implicit weight
 * written out as a value array, so that the SpMM entry points reproduce its
 * arithmetic on request.  Replaces the degree vector and the per-nonzero
 * product in the kernels, src/MergePathSpMM.cu:178,183-185 (degrees[i] =
 * row_ptr[i+1] - row_ptr[i]) and :450,459 (w = __fmaf_rn(float(deg_row),
 * float(deg_col), 0)); fp16: src/MergePathSpMM_fp16.cu:451,460 (both degrees
 * converted to half, multiplied in half: infinity beyond 65504).  The
 * reference's tail partials use a source weight of 1 (:468): a defect, not
 * reproduced.
 *   MPS_WEIGHT_DEGREE_PRODUCT  val[e] = deg(row of e) * deg(col_idx[e])
 *   MPS_WEIGHT_GCN             val[e] = 1 / sqrt(deg(row) * deg(col)), 0 where a degree is 0
 * The matrix must be square (column ids index row_ptr, as in the reference). */
#define MPS_WEIGHT_DEGREE_PRODUCT 0
#define MPS_WEIGHT_GCN 1
int mps_degree_values_f32(const int *d_row_ptr, const int *d_col_idx, int n_rows, int nnz, int mode, float *d_val,
                          void *stream);
int mps_degree_values_f16(const int *d_row_ptr, const int *d_col_idx, int n_rows, int nnz, int mode, void *d_val,
                          void *stream);

/* Checks on the device that row_ptr starts at 0, is non-decreasing, ends at
 * nnz, and that every column id lies in [0, n_cols).  Synchronises the
 * stream and allocates a 4-byte device flag for the duration of the call.
 * The reference performs no validation (src/MergePathSpMM.cu:147-173);
 * the SpMM entry points below trust their inputs just the same, so callers
 * holding untrusted data run this first. */
int mps_csr_validate(const int *d_row_ptr, const int *d_col_idx, int n_rows, int n_cols,
                     int nnz, void *stream);

/* ------------------------------------------------------------------------ */
/* Device side: merge-path partitioner                                       */
/* ------------------------------------------------------------------------ */

/* Path coordinates of the P + 1 partition boundaries.  Boundary i lies on
 * diagonal min(ipt * i, n_rows + 1 + nnz), ipt = mps_items_per_partition.
 * One thread per diagonal runs the binary search of MergePathSearch
 * (src/MergePathSpMM.cu:280-297) over row_ptr[0..n_rows] against the nonzero
 * index, with the diagonals of generate_mp_sched (:327-334); x counts
 * row_ptr entries consumed (current row = x - 1), y nonzeros consumed.
 * d_coord_x, d_coord_y: int[P + 1].  Bit-exact with the reference. */
int mps_partition(const int *d_row_ptr, int n_rows, int nnz, int P, int *d_coord_x,
                  int *d_coord_y, void *stream);

/* The same coordinates computed on the host (row_ptr, coord_x, coord_y are host
 * arrays), for callers without a GPU at hand and for checking the device
 * result: the host code of the reference, MergePathSearch and the diagonals of
 * generate_mp_sched (src/MergePathSpMM.cu:280-297, :327-334), on the host
 * thread pool.  Bit-exact with mps_partition. */
int mps_partition_host(const int *row_ptr, int n_rows, int nnz, int P, int *coord_x, int *coord_y);

/* The six per-partition arrays of generate_mp_sched
 * (src/MergePathSpMM.cu:300-385), including its zero-means-none encoding,
 * derived on the device from the coordinates of mps_partition.  Each output
 * is int[P].  Provided for parity with the reference schedule; the SpMM
 * kernels below consume the coordinates directly. */
int mps_schedule_legacy(const int *d_row_ptr, int n_rows, int nnz, int P,
                        const int *d_coord_x, const int *d_coord_y, int *d_feature_start,
                        int *d_feature_start_num, int *d_feature_end, int *d_feature_end_num,
                        int *d_start_row, int *d_end_row, void *stream);

/* ------------------------------------------------------------------------ */
/* Device side: merge-path SpMM                                              */
/* ------------------------------------------------------------------------ */

/* Bytes of device workspace mps_spmm_f32 / mps_spmm_f16 need for P
 * partitions, width K and threads_per_wave tpw (0 = as many as fit).  The
 * workspace holds one carry-out record per wavefront (the partial sums of
 * the rows that cross its boundaries); it needs no initialisation. */
int mps_spmm_workspace_bytes(int P, int K, int tpw, int elem_bytes, size_t *bytes_out);

/* Y = A * X with A in CSR (row_ptr, col_idx, val), fp32.
 * Replaces the launch loops and kernels spmm_merge_path / spmm_merge_path_64
 * (src/MergePathSpMM.cu:223-264, :388-574) with explicit edge values in place
 * of the degree product (:450,:459-460).
 *   P, d_coord_x, d_coord_y  partition count and coordinates from mps_partition
 *   tpw                      partitions per wavefront, 1..mps_max_threads_per_wave,
 *                            or 0 for the maximum (argv[4] of the reference CLI, :122)
 * Rows that lie inside one partition are stored once; rows that cross
 * partition or wavefront boundaries are completed from carry-out records by
 * a second small kernel -- no atomics, deterministic. */
int mps_spmm_f32(const int *d_row_ptr, const int *d_col_idx, const float *d_val,
                 const float *d_X, float *d_Y, int n_rows, int nnz, int K, int P,
                 const int *d_coord_x, const int *d_coord_y, int tpw, void *d_workspace,
                 size_t workspace_bytes, void *stream);

/* fp16 values and features, fp32 accumulation, fp16 result.
 * Replaces src/MergePathSpMM_fp16.cu:224-265, :389-575 (which accumulates in
 * half, :427-431,:460-461). */
int mps_spmm_f16(const int *d_row_ptr, const int *d_col_idx, const uint16_t *d_val,
                 const uint16_t *d_X, uint16_t *d_Y, int n_rows, int nnz, int K, int P,
                 const int *d_coord_x, const int *d_coord_y, int tpw, void *d_workspace,
                 size_t workspace_bytes, void *stream);

/* mps_spmm_f32 for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops, harnesses that forbid hipMalloc) and have
 * no workspace to hand over.  No counterpart in the reference.  The carry-out
 * records live in an array that is part of the library's device image (one
 * copy per GPU, MPS_STATIC_SCRATCH_MIB MiB, held until the process ends), so
 * the call allocates and frees nothing.  Same kernels, same bits as
 * mps_spmm_f32.  MPS_ERR_WORKSPACE when the records of P partitions do not
 * fit (mps_spmm_workspace_bytes(P, K, tpw, 4) > mps_static_scratch_bytes()):
 * at K = 16 that is beyond about 4 million partitions.  All calls on one GPU
 * share the array: calls that overlap there (different streams or threads)
 * race.  Nothing has to be cleared between calls: every record a call reads
 * it has written itself. */
#define MPS_STATIC_SCRATCH_MIB 32
int mps_static_scratch_bytes(size_t *bytes_out);
int mps_spmm_f32_static(const int *d_row_ptr, const int *d_col_idx, const float *d_val,
                        const float *d_X, float *d_Y, int n_rows, int nnz, int K, int P,
                        const int *d_coord_x, const int *d_coord_y, int tpw, void *stream);

/* The same two entry points with the kernels selectable, for per-kernel
 * timing: phases bit 0 = the main kernel, bit 1 = the carry-out fix-up. */
#define MPS_PHASE_MAIN 1u
#define MPS_PHASE_FIXUP 2u
#define MPS_PHASE_REDUCE 4u /* plans with column slabs only */
#define MPS_PHASE_PREPARE 8u /* row-block plans: the small kernel that gathers the hot columns' rows of X (a plan of one step and at most 256 blocks reads them in its main kernel instead) */
int mps_spmm_f32_phases(const int *d_row_ptr, const int *d_col_idx, const float *d_val,
                        const float *d_X, float *d_Y, int n_rows, int nnz, int K, int P,
                        const int *d_coord_x, const int *d_coord_y, int tpw,
                        void *d_workspace, size_t workspace_bytes, unsigned phases,
                        void *stream);
int mps_spmm_f16_phases(const int *d_row_ptr, const int *d_col_idx, const uint16_t *d_val,
                        const uint16_t *d_X, uint16_t *d_Y, int n_rows, int nnz, int K, int P,
                        const int *d_coord_x, const int *d_coord_y, int tpw,
                        void *d_workspace, size_t workspace_bytes, unsigned phases,
                        void *stream);

/* ------------------------------------------------------------------------ */
/* Device side: plans (per-matrix preprocessing of the merge-path SpMM)      */
/* ------------------------------------------------------------------------ */

/* A plan is this library's counterpart of the schedule that the reference
 * builds once per matrix before its repeat loop (generate_mp_sched and the
 * uploads that follow it, src/MergePathSpMM.cu:192-220): everything about the
 * sparse operand that does not change from launch to launch.  It is optional:
 * mps_partition + mps_spmm_f32 above work from the caller's CSR arrays alone.
 * A plan holds device memory that the library allocates (hipMalloc) at
 * creation and frees at destruction:
 *
 *   - Column-slab tiling (optional).  The dense-row gathers of the kernel are
 *     served by the 4 MiB L2 of the XCD a wavefront runs on; a feature matrix
 *     larger than that is bound by L2 misses.  The nonzeros are reordered
 *     slab-major: columns are cut into num_slabs slabs of slab_cols columns,
 *     "virtual row" v = s * n_rows + r holds the nonzeros of row r whose
 *     column lies in slab s, and the virtual rows are stored in order, so the
 *     running wavefronts gather from one ~3 MiB slab of X at a time.  The
 *     kernel then produces num_slabs fp32 partial rows per row, which a last
 *     kernel adds in slab order (deterministic).  Needs column ids sorted
 *     (non-decreasing) within every row; otherwise the plan is built untiled.
 *   - Hot columns (tiled plans, row pitch a power of two up to ~256 bytes).
 *     Inside every slab the hot_rows columns with the most nonzeros (as many
 *     rows of X as fit in the 160 KiB LDS of a CU beside the kernel's own
 *     buffers: 1,728 at K = 16 fp32) form a "hot" segment; the workgroups
 *     that process it copy those rows of X into LDS once and gather from
 *     there, the remaining columns of the slab form the "cold" segment,
 *     gathered through L2.  Segments are ordered hot first (virtual row
 *     v = seg * n_rows + r, 2 * num_slabs segments), each is partitioned on
 *     its own, and the plan runs two launches of the same kernel.  Used for
 *     fp32 when a row of X has at most 64 bytes (K = 16; wider rows are
 *     cheaper through L2), for fp16 at most 32 bytes (K = 16; at K = 32 the
 *     half-to-float conversions eat the gain), and when the gathers taken off the
 *     L2 path outweigh the second set of partial rows (on the 232,965-row
 *     power-law graph: from about 15 % of the nonzeros in hot columns);
 *     MPS_PLAN_FORCE_HOT lifts these limits.
 *   - The merge-path partition (mps_num_partitions, mps_partition) of the
 *     virtual rows for the given cost: one split of all of them, or, with hot
 *     columns, one split per segment (padded to whole workgroups).
 *   - The nonzeros "sliced" by that partition: the 16-nonzero windows that the
 *     partitions of one wavefront consume in the same round are stored side
 *     by side, so that a wavefront stages a round with one contiguous load.
 *   - The workspace (partial rows, carry-out records).
 *
 * Row-block plans (fp32, K = 16: a row of X is 64 bytes, half a cache line, so
 * every gather through L2 costs a full request for half its payload).  For
 * most matrices of this shape (see below) the plan is built differently:
 * rows are cut into contiguous blocks of about equal
 * nonzero count, one per 1,024-thread workgroup, whose output rows are summed
 * in LDS and written to Y once -- no partial rows, no carry-out records, one
 * kernel.  Columns are dealt to `steps` steps: the steps * table_rows columns
 * with the most nonzeros are gathered from a per-step LDS table of rows of X,
 * the others through L2, a contiguous range of column ids per step.  Inside a
 * (block, step) the nonzeros are cut into 16 runs of about equal length (one
 * per wavefront; a cut lies where the run before it fills its last rounds)
 * and a wavefront's hot and cold nonzeros are each dealt evenly to its 16
 * lane-groups.  Results are deterministic.  The layout is built with the passes
 * over the nonzeros on the device (row_ptr and the nonzero counts of the
 * columns go to the host for the decisions); with local tables, more than 64
 * steps, a cold stream that its packed form cannot hold, or
 * MPS_PLAN_HOST_BUILD, on the host from a copy of the CSR arrays.  Both ways
 * give the same plan.  mps_plan_create picks
 * this kind of plan by itself where it was measured to win: fp32, K = 16, X
 * below 192 MiB (3.1 M rows), except for matrices with many short rows and no
 * busy columns (fewer than 12 nonzeros per row on average, more than 2^18
 * rows), matrices whose columns stay near the diagonal but not within 8
 * tables' width of it (wide bands) and matrices with one row far longer than a
 * CU's share of the nonzeros, which keep the slab plans.  Bands of up to
 * 8 tables' width and block-diagonal matrices get local tables
 * (MPS_PLAN_LOCAL_TABLES): every block with tables of the consecutive
 * columns it uses most.  `steps` and the number of blocks follow from the size of X,
 * the nonzeros per block and the column histogram.  A caller that passes a
 * cost other than mps_default_cost's, a tpw other than 0 or the maximum, or
 * one of the tiling / hot-column flags is tuning a slab plan and gets one;
 * MPS_PLAN_NO_ROWBLOCK / MPS_PLAN_FORCE_ROWBLOCK override the choice.
 *
 * mps_tile_shape: the slab count and width mps_plan_create chooses for an X
 *   of n_rows x K elements (slab_bytes = 0: slabs of 3 or 6 MiB, whichever
 *   the library's cost model prefers: gathers get cheaper with smaller slabs,
 *   every slab adds one fp32 partial row per row); num_slabs == 1 means
 *   tiling does not pay (X fits in L2, or a row holds too few nonzeros per
 *   slab).  Where X exceeds 24 MiB and rows hold 16 nonzeros or more on
 *   average, mps_plan_create also looks at the matrix: it counts the nonzeros
 *   per column and, if they are concentrated in few columns (which then stay
 *   in L2 by themselves), may take slabs of 12 or 24 MiB instead.
 * mps_plan_create: d_val is fp32 (elem_bytes 4) or fp16 (2); cost and tpw as
 *   for mps_num_partitions / mps_spmm_f32.  Synchronises the stream.
 * mps_plan_set_values: the nonzero values changed, the pattern did not.
 * mps_plan_spmm_f32 / _f16: Y = A * X; same arithmetic (fp32 accumulation)
 *   and tolerance as mps_spmm_f32 / mps_spmm_f16, different summation order.
 *   Calls on one plan share its workspace: do not overlap them on different
 *   streams.
 * mps_plan_spmm_phases: the same with the kernels selectable, for timing
 *   (MPS_PHASE_PREPARE | MPS_PHASE_MAIN | MPS_PHASE_FIXUP | MPS_PHASE_REDUCE;
 *   a phase the plan's kind does not have launches nothing).
 * mps_plan_copy_array: copies one of the plan's device arrays to the host
 *   (bytes must equal its size), for inspection and tests.
 *
 * Degree weights (mps_plan_options.degree_weights, fp32 only): the reference
 * forms the weight of nonzero (r, c) from the degrees of r and c inside its
 * kernel instead of reading a value array (src/MergePathSpMM.cu:183-185, :450,
 * :459-460).  A plan with degree weights does the same without a value per
 * nonzero: it keeps one factor per node (the degree, or 1 / sqrt(degree)),
 * scales X by the column factor into a buffer of its own before the kernels
 * (MPS_PHASE_PREPARE), adds up rows of that buffer (the sliced arrays hold
 * column entries only) and multiplies every finished row by its row factor
 * where it is written.  Y = D A_pattern D X with the factors applied in that
 * order: within rounding of the product with mps_degree_values_f32's array
 * (row sums differ by a few ulp), half the sparse bytes per nonzero.
 * mps_plan_set_values returns MPS_ERR_UNSUPPORTED on such a plan; row-block
 * plans are not built for it. */
typedef struct mps_plan mps_plan;

#define MPS_PLAN_NO_TILING 1u    /* never tile                                  */
#define MPS_PLAN_FORCE_TILING 2u /* tile with slab_bytes slabs whatever the shape */
#define MPS_PLAN_NO_HOT 4u       /* never keep hot columns' rows of X in LDS     */
#define MPS_PLAN_FORCE_HOT 8u    /* hot columns even when they hold few nonzeros or rows of X are wider than 64 bytes (fp16: 32) */
#define MPS_PLAN_NO_ROWBLOCK 16u    /* never build a row-block plan (see below)  */
#define MPS_PLAN_FORCE_ROWBLOCK 32u /* row-block plan whatever the matrix looks like (fp32, K = 16 only) */
#define MPS_PLAN_LOCAL_TABLES 1024u  /* row-block plans: every block with tables of consecutive columns of its own, step t the
                                        table_rows columns from base[b] + t * table_rows (what the library builds by itself for
                                        matrices whose columns stay within 8 tables' width of the diagonal); with
                                        MPS_PLAN_FORCE_ROWBLOCK or mps_rowblock_layout_build */
#define MPS_PLAN_NO_SWEEP 2048u     /* never build a sweep plan (see below)       */
#define MPS_PLAN_FORCE_SWEEP 4096u  /* sweep plan whatever the matrix looks like (rows of X of whole dwords: any K in fp32, an even K in fp16;
                                       an X of 4 GiB or more: rows of whole 16 bytes) */
#define MPS_PLAN_HOST_BUILD 8192u   /* row-block and sweep plans: every pass over the nonzeros on the host, from a copy of the CSR
                                       arrays (the library makes these passes on the device where it can; both give the same plan) */
#define MPS_PLAN_NO_COLUMN_TILES 512u /* untiled plans with rows of X of 512 bytes and more: no passes over 128-byte column tiles */
#define MPS_PLAN_NO_RESIDENT 256u    /* untiled plans: no streaming hint on the gathers of unpopular columns (see below) */
#define MPS_PLAN_NO_ROW_MARKS 128u  /* plain column ids in the sliced array; the kernel follows row_ptr as on the caller's
                                       CSR arrays (what a matrix gets anyway whose column ids and row-end counts do not
                                       fit 32 bits together) */
#define MPS_PLAN_NO_SOURCES 64u     /* do not keep the original nonzero index of every slot: saves 4 bytes per
                                       nonzero of device memory; mps_plan_set_values then returns MPS_ERR_UNSUPPORTED */

typedef struct mps_plan_info {
    int n_rows, nnz, K, elem_bytes, cost, threads_per_wave;
    int num_slabs, slab_cols;      /* 1, n_rows when untiled                      */
    int num_partitions, num_waves; /* P and ceil(P / threads_per_wave)            */
    long long total_rounds;        /* sum over wavefronts of their 16-nonzero rounds */
    long long slice_slots;         /* nonzero slots incl. padding                 */
    size_t device_bytes;           /* device memory the plan holds                */
    int num_segments;              /* virtual-row segments: num_slabs, or 2 * num_slabs with hot columns */
    int hot_rows;                  /* rows of X per LDS table (0: no hot launch)  */
    int hot_waves;                 /* wavefronts of the hot launch                */
    long long hot_nnz;             /* nonzeros gathered from LDS                  */
    int hot_cost;                  /* merge items per partition of the hot segments (64 .. 256 by the amount of hot work, at least cost) */
    int mark_shift;                /* > 0: SLICE_COLS entries are column | row_ends << mark_shift */
    int hot_mark_shift;            /* the same for the entries of the hot wavefronts (column = LDS slot) */
    int hot_blocks;                /* workgroups of the hot launch: at most one per CU unless there are more hot segments than CUs */
    /* row-block plans (rowblock_steps > 0); the fields above that describe slabs, partitions and slices are then 0 / 1 */
    int rowblock_steps;            /* T: steps, one LDS table each                */
    int rowblock_table_rows;       /* H: rows of X per LDS table                  */
    int rowblock_blocks;           /* row blocks = workgroups                     */
    int rowblock_acc_rows;         /* rows of LDS accumulators per workgroup      */
    long long rowblock_hot_slots;  /* entries of the hot stream incl. padding     */
    long long rowblock_cold_slots; /* entries of the cold stream incl. padding    */
    /* resident columns (resident_cols > 0): SLICE_COLS entries are column | streamed << mark_shift | row_ends << (mark_shift + 1) */
    int resident_cols;             /* columns whose rows of X are gathered without the streaming hint */
    long long resident_nnz;        /* nonzeros in them                            */
    int rowblock_cold_index_bits;  /* row-block plans: > 0 when the cold stream is held in packed form (RB_COLD_PACKED): bits of a
                                      16-bit entry that hold the column, counted from the first column of the step's range */
    int rowblock_local_tables;     /* row-block plans: 1 when every block has a table of its own (RB_TABLE_BASE) */
    /* sweep plans (sweep_panels > 0); the fields about slabs, partitions, slices and row blocks are then 0 / 1 */
    int sweep_panels;              /* panels = workgroups per column tile          */
    int sweep_acc_rows;            /* accumulator rows per panel in LDS            */
    int sweep_lanes;               /* lanes per lane-group: 4 (rows of X of up to 64 bytes) or 8 (128-byte column tiles; the last one may be narrower) */
    int sweep_tiles;               /* column tiles per row of X                    */
    int sweep_col_bits;            /* an entry word is column | accumulator row << sweep_col_bits */
    int sweep_piece;               /* most entries of a row that one accumulator row takes */
    int sweep_together;            /* 1, or 2: entry q of a round's windows A and B are added up at the same time, no two
                                      entries of such a pair of instructions share an accumulator row */
    int sweep_split_rows;          /* rows cut into sub-rows that go to different panels */
    int sweep_partial_rows;        /* sub-rows of those rows                       */
    int sweep_listed_rows;         /* entries of SW_ROWS: n_rows - split rows + partial rows */
    long long sweep_rounds;        /* rounds of all wavefronts                     */
    long long sweep_slots;         /* entry slots incl. padding                    */
    int built_on_device;           /* row-block and sweep plans: 1 if the passes over the nonzeros ran on the device, 0 if
                                      on the host (the plan is the same either way); slab plans: always 1 */
} mps_plan_info;

/* Optional parameters of mps_plan_create_ex; zero means "the library chooses". */
typedef struct mps_plan_options {
    unsigned flags;          /* MPS_PLAN_*                                       */
    size_t slab_bytes;       /* column-slab size of a tiled plan                 */
    int rowblock_steps;      /* T of a row-block plan                            */
    int rowblock_table_rows; /* H of a row-block plan                            */
    int rowblock_block_rows; /* most rows per row block                          */
    int rowblock_blocks_per_round; /* row blocks are made in multiples of this (0: the number of CUs) */
    int degree_weights;      /* 0: values from d_val.  1: the weight of nonzero (r, c) is deg(r) * deg(c), 2: 1 / sqrt(deg(r) * deg(c))
                                (MPS_WEIGHT_DEGREE_PRODUCT + 1, MPS_WEIGHT_GCN + 1): d_val is not read, see "degree weights" below */
    size_t resident_bytes;   /* rows of X (of the busiest columns) that an untiled plan gathers without the streaming hint; set: whatever the size of X and the skew */
    int sweep_piece;         /* sweep plans: most entries of a row per accumulator row */
    int sweep_acc_rows;      /* sweep plans: most accumulator rows per panel (what fits in LDS if 0 or larger) */
    int sweep_panels_per_round; /* sweep plans: panels are made in multiples of this (0: the number of CUs) */
    int sweep_together;      /* sweep plans: 1 or 2 instructions added up at the same time (0: 2 for 64-byte rows of X, else 1) */
} mps_plan_options;

enum {
    MPS_PLAN_ARRAY_VROW_PTR = 0,   /* int[num_slabs * n_rows + 1]                 */
    MPS_PLAN_ARRAY_COORD_X = 1,    /* int[P + 1]                                  */
    MPS_PLAN_ARRAY_COORD_Y = 2,    /* int[P + 1]                                  */
    MPS_PLAN_ARRAY_WAVE_OFF = 3,   /* int[num_waves + 1]: first round of each wave */
    MPS_PLAN_ARRAY_SLICE_COLS = 4, /* int[slice_slots]                            */
    MPS_PLAN_ARRAY_SLICE_SRC = 5,  /* int[slice_slots]: original nonzero index, -1 = padding */
    MPS_PLAN_ARRAY_SLICE_VALS = 6, /* elem_bytes * slice_slots                    */
    MPS_PLAN_ARRAY_HOT_COLS = 7,   /* int[num_slabs * hot_rows]: column of each LDS slot, -1 = unused */
    /* row-block plans */
    MPS_PLAN_ARRAY_RB_BLOCK_ROW = 8,  /* int[blocks + 1]: first row of every block  */
    MPS_PLAN_ARRAY_RB_HOT_COLS = 9,   /* int[steps * table_rows]: column of each table slot, -1 = unused */
    MPS_PLAN_ARRAY_RB_META = 10,      /* int[blocks * steps * 16 * 4]: {hot entries, cold entries, first local row, 0} per wavefront */
    MPS_PLAN_ARRAY_RB_WAVE_BASE = 11, /* long long[blocks * 16 * 2]: first round of each wavefront's hot / cold stream */
    MPS_PLAN_ARRAY_RB_HOT = 12,       /* 8 bytes x hot slots: {index | rows_advanced << bits, value}; host layouts only (a device plan holds RB_HOT_PACKED) */
    MPS_PLAN_ARRAY_RB_COLD = 13,      /* 8 bytes x cold slots; a device plan holds it only when the packed form does not fit */
    MPS_PLAN_ARRAY_RB_HOT_SRC = 14,   /* int[hot slots]: original nonzero index, -1 = padding */
    MPS_PLAN_ARRAY_RB_COLD_SRC = 15,  /* int[cold slots]                            */
    MPS_PLAN_ARRAY_RB_HOT_PACKED = 16, /* 12 bytes x (hot slots / 2), what the device reads: per round and lane {value A, value B,
                                         half A | half B << 16}, half = table slot | piece << 11; the 5-bit pieces of a window's
                                         entries 0 and 1 are the low and the high half of its rows_advanced */
    MPS_PLAN_ARRAY_RB_COLD_PACKED = 17, /* 12 bytes x (cold slots / 2), if rowblock_cold_index_bits > 0: the same form; half =
                                         (column - first column of the step's range) | piece << index_bits, entry e of a window
                                         holds bits [e p, (e + 1) p) of its rows_advanced, p = 16 - index_bits */
    MPS_PLAN_ARRAY_RB_COLD_BEGIN = 18, /* int[steps + 1]: first column of every step's range of cold columns */
    MPS_PLAN_ARRAY_RB_TABLE_BASE = 19, /* int[blocks], plans with local tables: block b's table of step t holds the columns
                                         base[b] + t * table_rows .. base[b] + (t + 1) * table_rows - 1 (RB_HOT_COLS is all -1
                                         then, and RB_COLD_BEGIN is 0 for every step: a block's cold columns lie outside its tables) */
    /* sweep plans */
    MPS_PLAN_ARRAY_SW_PANEL_PTR = 20,   /* int[panels + 1]: a panel's listed rows are SW_ROWS[ptr[p] .. ptr[p + 1]) */
    MPS_PLAN_ARRAY_SW_ROWS = 21,        /* int[listed rows]: the row of Y a listed row is written to; n_rows + s: partial row s */
    MPS_PLAN_ARRAY_SW_PIECE_PTR = 22,   /* int[listed rows + panels]: per panel (from ptr[p] + p on) listed rows + 1 entries, the
                                           first accumulator row of every listed row and, last, the panel's count */
    MPS_PLAN_ARRAY_SW_WAVE_META = 23,   /* int[panels * 16 * 2]: {first round, rounds} of every wavefront */
    MPS_PLAN_ARRAY_SW_PANEL_ROUNDS = 24, /* int[panels]: most rounds of a wavefront of the panel */
    MPS_PLAN_ARRAY_SW_STREAM = 25,      /* 8 bytes x slots: per round, lane-group and lane of its quad {word A, value A, word B,
                                           value B}; word = column | LDS row of the accumulator row << sweep_col_bits, value fp32;
                                           lane q of a quad holds entry q of windows A and B; padding: value 0 */
    MPS_PLAN_ARRAY_SW_SRC = 26,         /* int[slots]: original nonzero index, -1 = padding */
    MPS_PLAN_ARRAY_SW_SPLIT_ROW = 27,   /* int[split rows] */
    MPS_PLAN_ARRAY_SW_SPLIT_PTR = 28    /* int[split rows + 1]: partial rows of every split row */
};

int mps_tile_shape(int n_rows, int nnz, int K, int elem_bytes, size_t slab_bytes, int *num_slabs_out,
                   int *slab_cols_out);
int mps_plan_create(const int *d_row_ptr, const int *d_col_idx, const void *d_val, int n_rows, int nnz,
                    int K, int elem_bytes, int cost, int tpw, unsigned flags, size_t slab_bytes,
                    void *stream, mps_plan **plan_out);
int mps_plan_create_ex(const int *d_row_ptr, const int *d_col_idx, const void *d_val, int n_rows, int nnz,
                       int K, int elem_bytes, int cost, int tpw, const mps_plan_options *options,
                       void *stream, mps_plan **plan_out);
void mps_plan_destroy(mps_plan *plan);
int mps_plan_get_info(const mps_plan *plan, mps_plan_info *info);
int mps_plan_set_values(mps_plan *plan, const void *d_val, void *stream);
int mps_plan_copy_array(const mps_plan *plan, int which, void *host_dst, size_t bytes);
int mps_plan_spmm_f32(const mps_plan *plan, const float *d_X, float *d_Y, void *stream);
int mps_plan_spmm_f16(const mps_plan *plan, const uint16_t *d_X, uint16_t *d_Y, void *stream);
int mps_plan_spmm_phases(const mps_plan *plan, const void *d_X, void *d_Y, unsigned phases, void *stream);

/* The layout of a row-block plan, built from host arrays without a GPU: what
 * mps_plan_create_ex uploads.  For inspection, tests and callers that prepare
 * plans offline.  options: rowblock_* fields as for mps_plan_create_ex
 * (rowblock_blocks_per_round 0 = 256).  mps_rowblock_layout_array hands out a
 * pointer into the layout (valid until it is freed) for MPS_PLAN_ARRAY_RB_*. */
typedef struct mps_rowblock_layout mps_rowblock_layout;
int mps_rowblock_layout_build(const int *row_ptr, const int *col_idx, const float *val, int n_rows, int nnz,
                              int K, const mps_plan_options *options, mps_rowblock_layout **layout_out);
int mps_rowblock_layout_info(const mps_rowblock_layout *layout, mps_plan_info *info);
int mps_rowblock_layout_array(const mps_rowblock_layout *layout, int which, const void **data_out,
                              size_t *bytes_out);
void mps_rowblock_layout_free(mps_rowblock_layout *layout);

/* The layout of a sweep plan, built from host arrays without a GPU: what
 * mps_plan_create_ex uploads.  val is fp32 whatever elem_bytes (2 or 4: the
 * type of X and Y, which decides the lane-group width and the accumulator
 * size).  options: sweep_* fields and MPS_PLAN_NO_SOURCES.
 * mps_sweep_layout_array hands out a pointer into the layout (valid until it
 * is freed) for MPS_PLAN_ARRAY_SW_*. */
typedef struct mps_sweep_layout mps_sweep_layout;
int mps_sweep_layout_build(const int *row_ptr, const int *col_idx, const float *val, int n_rows, int nnz, int K,
                           int elem_bytes, const mps_plan_options *options, mps_sweep_layout **layout_out);
int mps_sweep_layout_info(const mps_sweep_layout *layout, mps_plan_info *info);
int mps_sweep_layout_array(const mps_sweep_layout *layout, int which, const void **data_out, size_t *bytes_out);
void mps_sweep_layout_free(mps_sweep_layout *layout);

/* Parameter sweep for one matrix and K — what the reference leaves to the
 * user's hand (cost and partitions per warp are command-line arguments,
 * src/MergePathSpMM.cu:121-122, and its README reports the best of a sweep).
 * Builds a plan for each candidate (slab plans: costs 16 .. 256 with a full
 * wavefront, the default cost with half the partitions per wavefront, without
 * hot columns, without tiling, with slabs of 3, 6, 12 and 24 MiB where X holds
 * more than two of them and the library's cost model does not put them 50 %
 * behind the untiled plan; one row-block plan for fp32, K = 16 and an X below
 * 192 MiB), runs `repeats` timed products Y = A * X after two warm-ups
 * (HIP events on the stream) and reports the fastest.  d_Y is overwritten.
 * tried_out (optional) receives every candidate with its time;
 * *n_tried_io is its capacity on entry and the number of candidates on
 * return.  Allocates and frees one plan at a time; synchronises the stream. */
typedef struct mps_tune_result {
    int cost;             /* merge items per partition                       */
    int threads_per_wave; /* partitions per wavefront                        */
    unsigned flags;       /* MPS_PLAN_* flags of the candidate                */
    float ms;             /* average time of one product, all kernels         */
    unsigned long long slab_bytes; /* slab size of the candidate (0: the library's choice) */
} mps_tune_result;
int mps_plan_autotune(const int *d_row_ptr, const int *d_col_idx, const void *d_val, int n_rows, int nnz, int K,
                      int elem_bytes, const void *d_X, void *d_Y, int repeats, void *stream,
                      mps_tune_result *best_out, mps_tune_result *tried_out, int *n_tried_io);

/* ------------------------------------------------------------------------ */
/* Device side: comparison kernels                                           */
/* ------------------------------------------------------------------------ */

/* Row-wise split: wavefront w owns rows [int(step * w), int(step * (w + 1)))
 * with float step = (float)n_rows / num_waves, the arithmetic of
 * src/row_wise.cu:211-213; the last wavefront also takes any rows the float
 * rounding leaves over.  Replaces run_spmm_row_wise / spmm_row_wise
 * (src/row_wise.cu:172-240).  Any K; no workspace; plain stores. */
int mps_rowwise_spmm_f32(const int *d_row_ptr, const int *d_col_idx, const float *d_val,
                         const float *d_X, float *d_Y, int n_rows, int nnz, int K, int num_waves,
                         void *stream);

/* Row ranges of mps_rowwise_spmm_f32 (host arrays int[num_waves]). */
int mps_rowwise_bounds(int n_rows, int num_waves, int *row_start, int *row_end);

/* Nonzero splitting ("GNNAdvisor-opt"): every row is cut into groups of at
 * most part_size nonzeros.
 * mps_nzsplit_max_parts: upper bound for sizing (nnz / part_size + n_rows).
 * mps_nzsplit_build: replaces calculate_part_num + build_part
 *   (src/nz_splitting.cu:256-316) on the device: d_part_ptr[num_parts + 1]
 *   (first nonzero of each group, then nnz), d_part2node[num_parts];
 *   *num_parts_out is written on the host after the stream is synchronised.
 *   d_scratch: int[n_rows + 1 + 2048] device scratch. */
int mps_nzsplit_max_parts(int n_rows, int nnz, int part_size, int *max_parts_out);
int mps_nzsplit_build(const int *d_row_ptr, int n_rows, int part_size, int *d_part_ptr,
                      int *d_part2node, int max_parts, int *d_scratch, int *num_parts_out,
                      void *stream);
/* Replaces spmm_forward_cuda_kernel / _64 (src/nz_splitting.cu:212-240,
 * :318-445): one group per lane-group, column ids staged in LDS, every group
 * ends in fp32 atomic adds into Y, which this call zeroes first.  The order
 * of the atomic adds, and with it the last bits of Y, varies run to run. */
int mps_nzsplit_spmm_f32(const int *d_col_idx, const float *d_val, const float *d_X,
                         float *d_Y, int n_rows, int nnz, int K, const int *d_part_ptr,
                         const int *d_part2node, int num_parts, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MPSPMM_H */
