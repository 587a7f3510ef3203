/*
 * smat.h -- C ABI of the MI355X (gfx950) block-sparse SpMM library.
 *
 *     C (M x N) = A (M x K, 16x16 blocked CSR, fp16) * B (K x N, dense fp16),
 *     fp32 accumulation on the fp16 MFMA units.
 *
 * Everything here is `extern "C"`, takes plain pointers and sizes, and returns
 * an int status (SMAT_OK == 0).  A host compiled with g++ needs no HIP header:
 * device memory, streams and events are reachable through the thin wrappers at
 * the end of this file.  Citations name the file:line of the reference
 * (spcl/smat) interface that each entry point replaces.
 */
#ifndef SMAT_H
#define SMAT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SMAT_BS 16 /* block edge: MMA_M == MMA_K, src/cuda_hgemm/src/common/matrix.h:13-15 */

/* ---- status ------------------------------------------------------------- */
#define SMAT_OK 0
#define SMAT_ERR_INVALID (-1)     /* bad argument (shape not a multiple of 16/8, NULL, ...) */
#define SMAT_ERR_HIP (-2)         /* a HIP runtime call failed; see smat_last_error()       */
#define SMAT_ERR_NOMEM (-3)       /* host or device allocation failed                       */
#define SMAT_ERR_IO (-4)          /* file could not be opened / parsed                      */
#define SMAT_ERR_UNSUPPORTED (-5) /* valid request this build does not implement            */

/* Text of the most recent error on the calling thread ("" if none). */
const char *smat_last_error(void);
/* "smat-amd <version> gfx950" */
const char *smat_version(void);

/* ---- SpMM: the drop-in entry point --------------------------------------
 * Replaces `void mmaCBTKernel(half *bcsrValuesA, int *bcsrRowPtrA,
 * int *bcsrColIdxA, half *B, half *C, size_t M, size_t N, size_t K,
 * size_t nonzeroBlocks, int *blockInfo, int *relativeBlockIndexMapping)`
 * (src/cuda_hgemm/src/mma/mmaCBT.cu:83-88; shape HGEMM_FUNC_SPARSE2,
 * src/cuda_hgemm/src/main.cu:7) -- same positional arguments, same meaning:
 *
 *   vals     device, fp16, nnzb*256, block p at vals[p*256], row-major in block
 *   row_ptr  device, int32, M/16+1
 *   col_idx  device, int32, nnzb, ABSOLUTE first column of each block (matrix.h:455)
 *   B        device, fp16, column-major K x N: element (k,n) at B[n*K+k] (mmaCBT.cu:52)
 *   C        device, fp16, row-major M x N, OVERWRITTEN (mmaCBT.cu:36,72-79)
 *   M, K     multiples of 16 (mmio_highlevel.h:609-616); N a multiple of 8 (tester.h:40)
 *   block_info, rel_map   accepted for signature compatibility and ignored: the
 *            running block index equals the row_ptr/col_idx position
 *            (matrix.h:425-431 vs 441-463), so the dense maps carry nothing.
 *
 * On the null stream like the reference launch; returns a status where the reference returns void.
 *
 * Plan cache.  The reference's harness calls its launcher again and again with the same arguments
 * (common/tester.h:177-182,342-357).  The first call with a given (device, row_ptr, col_idx, M, K, nnzb, N)
 * copies row_ptr and col_idx to the host, makes a plan (as smat_plan_create with SMAT_KERNEL_AUTO does) and
 * keeps it; that call is synchronous and allocates device memory.  Later calls with the same key find the plan
 * and are asynchronous launches.  Up to 8 plans are kept, the one used longest ago makes room.
 *   - Another block pattern written into the SAME arrays: call smat_plan_cache_clear().  As a safety net a checksum
 *     of row_ptr / col_idx is taken on the device on every 64th call with a key (synchronous, a few microseconds)
 *     and the plan is rebuilt when it differs; the calls in between would have used the old pattern.
 *   - Block values are read by every launch, not cached: they may change between calls.  With
 *     SMAT_PLAN_CACHE=values in the environment the cached plans also look at the values
 *     (smat_plan_attach_values: compact and mixed kernels for blocks with few nonzero columns) and keep a copy,
 *     vals becomes part of the key, and the caller promises to call smat_plan_cache_clear() after changing values.
 *   - SMAT_PLAN_CACHE=0 switches the cache off: every call is a launch of the row-wise kernel over whole block
 *     rows, B read in place, nothing allocated (what smat_spmm_bcsr_f16_ex does without a plan).
 * Callers that must not allocate or synchronise use smat_spmm_bcsr_f16_static. */
int smat_spmm_bcsr_f16(const uint16_t *vals, const int32_t *row_ptr, const int32_t *col_idx,
                       const uint16_t *B, uint16_t *C, size_t M, size_t N, size_t K, size_t nnzb,
                       const int32_t *block_info, const int32_t *rel_map);
/* Drops every plan that smat_spmm_bcsr_f16 keeps (synchronous).  No counterpart in the reference. */
int smat_plan_cache_clear(void);

/* ---- SpMM with options / explicit stream / plan -------------------------- */
#define SMAT_B_COL_MAJOR 0 /* B[n*K + k]: the reference layout               */
#define SMAT_B_ROW_MAJOR 1 /* B[k*N + n].  The compact kernel reads rows of B and takes this layout in place
                            * (column-major B is first copied row-major into plan scratch on every launch).
                            * The row-wise and sweep kernels feed the MFMA 8 consecutive k of one column
                            * per lane: for them a row-major B is first transposed into the reference
                            * layout in plan scratch (one read and one write of B per launch), which needs
                            * a plan created with b_layout = SMAT_B_ROW_MAJOR and n_hint >= N; C has the
                            * same bits as for column-major B */
#define SMAT_C_F16 0       /* the reference output type                      */
#define SMAT_C_F32 1       /* keep the fp32 accumulators                     */

#define SMAT_KERNEL_AUTO 0
#define SMAT_KERNEL_ROWWISE 1 /* one wavefront per (block-row chunk, N panel), operands straight from L2;
                               * the plan decides whether B is first repacked slab-major into scratch   */
#define SMAT_KERNEL_SWEEP 2   /* workgroup sweeps K for a group of 64 block rows x 64 columns, B staged in LDS
                               * in chunks of 16 block columns; needs a plan made with col_idx_host, between 2
                               * and 2^23 - 1 blocks and K below 2^28.  SMAT_KERNEL_AUTO takes it when at least
                               * 5% of the blocks exist and (M/1024) x (N/64) workgroups fill the 256 CUs.
                               * It works from the plan's op list, NOT from the row_ptr / col_idx passed at
                               * launch: the plan must have been made from the same block pattern
                               * (smat_plan_check verifies that on request)                                 */
#define SMAT_KERNEL_ROWWISE_DIRECT 3 /* row-wise, B always read in place (plan or launch option)          */
#define SMAT_KERNEL_COMPACT 5  /* only the nonzero columns of the blocks are multiplied (needs
                               * smat_plan_attach_values); for blocks with few nonzero columns */
#define SMAT_KERNEL_MIXED 6    /* mixed dispatch inside one SpMM: block rows whose blocks are mostly full (at least
                               * 60% of their columns nonzero) go through a dense kernel (sweep or row-wise), the
                               * others through the compact kernel.  Where the block rows do not sort into two kinds
                               * but the blocks do (the classification of matrix.h:400-419), the split is per block:
                               * the plan's copy of the mostly full blocks goes through the sweep kernel and the
                               * compact kernel adds the columns of the other blocks to C.  Needs
                               * smat_plan_attach_values, which makes the split; SMAT_KERNEL_AUTO takes it when each
                               * kind holds at least a tenth of the blocks (and, per block, when its estimate of the
                               * run time beats the better single kernel) */
#define SMAT_KERNEL_ROWWISE_PACKED 4 /* row-wise, B always repacked (needs a plan created with this id) */

typedef struct smat_spmm_opts {
    int32_t b_layout; /* SMAT_B_COL_MAJOR | SMAT_B_ROW_MAJOR                */
    int32_t c_dtype;  /* SMAT_C_F16 | SMAT_C_F32                            */
    int32_t kernel;   /* SMAT_KERNEL_*                                      */
    int32_t reserved; /* must be 0                                          */
    void *stream;     /* hipStream_t, NULL = null stream                    */
} smat_spmm_opts;

/* A plan is the per-matrix work list (load balancing over block rows of skewed
 * length).  It plays the role the reference gives to the one-off host-side
 * BCSR build (SparseMatrix ctor, matrix.h:173): made once per matrix, outside
 * the timed loop (tester.h:342-358), reused by every launch. */
typedef struct smat_plan smat_plan;
/* Contract of a plan:
 *  - One launch in flight at a time.  Every launch with a plan writes plan-owned scratch (the repacked or
 *    transposed copy of B, the partial sums of split block rows): two launches of one plan that overlap
 *    (different streams, or one stream per thread) race and corrupt C without an error.  Launches on one
 *    stream are ordered and safe; for concurrent launches make one plan per stream.
 *  - A plan belongs to one block pattern.  The launch checks M, K and nnzb only; the sweep kernel takes the
 *    pattern from the plan, the compact kernel the pattern and the values (as attached).  A plan made from
 *    another matrix of the same size, or values changed without attaching them again, give a wrong C with
 *    SMAT_OK.  smat_plan_check compares the fingerprint of the host arrays the plan was made from. */

/* row_ptr_host: the HOST copy of the BCSR row pointer (M/16+1 entries).
 * col_idx_host: HOST copy of the BCSR column index (may be NULL unless
 *               opts->kernel requests SMAT_KERNEL_SWEEP; without it SMAT_KERNEL_AUTO
 *               never chooses that kernel).  The sweep kernel needs the columns of every
 *               block row strictly ascending, as csrToBcsr emits them (matrix.h:441-463):
 *               otherwise SMAT_KERNEL_SWEEP / SMAT_KERNEL_MIXED are refused with
 *               SMAT_ERR_INVALID and SMAT_KERNEL_AUTO stays with the row-wise kernel, which
 *               takes the blocks of a row in any order (as mmaCBT.cu:44-66 does).
 * n_hint: the N the plan will mostly be used with (panel width choice). */
int smat_plan_create(smat_plan **plan, const int32_t *row_ptr_host, const int32_t *col_idx_host,
                     size_t M, size_t K, size_t nnzb, size_t n_hint, const smat_spmm_opts *opts);
/* Optional: lets the plan look at the block values (DEVICE arrays of the matrix the plan was
 * made for; row_ptr_host must equal the array given to smat_plan_create, else SMAT_ERR_INVALID).  The plan lists the nonzero columns of every
 * block and keeps a COPY of them (32 bytes per nonzero column, in MFMA operand order), so that
 * SMAT_KERNEL_COMPACT multiplies only those and touches only the rows of B under them; with
 * SMAT_KERNEL_AUTO the plan switches to that kernel when fewer than 60% of the block columns
 * are nonzero.  The compact kernel works from the copy: attach again after the values change.
 * The new list is built before the old one is dropped; if the call fails the plan has no list and
 * SMAT_KERNEL_AUTO goes back to the sweep or row-wise kernel.  When the plan takes the compact kernel, the call also
 * times a few launches of it on zeros (temporary device buffers of K x n_hint and M x n_hint halves, freed before it
 * returns; skipped if they do not fit) to choose how the work is dealt to the GPU's eight XCDs: a choice that moves
 * no bit of any result.  Synchronous.  No counterpart in the reference, which multiplies every block as a dense
 * 16x16 (mmaCBT.cu:44-66). */
int smat_plan_attach_values(smat_plan *plan, const uint16_t *vals, const int32_t *row_ptr,
                            const int32_t *col_idx, const int32_t *row_ptr_host);
/* Staleness guard for the copy that smat_plan_attach_values keeps: *current = 1 when the block values in vals
 * (device) still have the checksum they had when they were attached (or when no kernel of the plan works from
 * a copy), 0 when they have changed and must be attached again.  One pass over vals at memory speed plus an
 * 8-byte copy back (synchronous): 3 us for 13 MB of values, 1.3 ms for the 5.7 GB of R-MAT scale 20.  Not
 * called by the SpMM itself.  No counterpart in the reference, which keeps no copy. */
int smat_plan_values_current(const smat_plan *plan, const uint16_t *vals, int *current);
int smat_plan_destroy(smat_plan *plan);
/* Opt-in check that `plan` was made from this block pattern: M, K, nnzb and a 64-bit FNV-1a hash of
 * row_ptr_host (and of col_idx_host if the plan was made with one; then it must be passed).  One pass over
 * the host arrays; SMAT_ERR_INVALID when they differ.  No counterpart in the reference. */
int smat_plan_check(const smat_plan *plan, const int32_t *row_ptr_host, const int32_t *col_idx_host,
                    size_t M, size_t K, size_t nnzb);
/* Fills info[0..11]: kernel id, row-wise work items, split block rows, chunk size,
 * workspace bytes, panel width, sweep stream entries, sweep (row group, K chunk) records,
 * bytes of the scratch copies of B (0 = B is read in place), nonzero block columns listed by
 * smat_plan_attach_values (0 = not attached), and for mixed dispatch the row-wise work items (-1: the
 * split is per block, not per block row) and the blocks that the dense kernel takes. */
int smat_plan_info(const smat_plan *plan, int64_t *info);

/* Same operands as smat_spmm_bcsr_f16; C is uint16_t* or float* per opts->c_dtype.
 * opts == NULL means defaults; plan == NULL means no work list (whole block
 * rows, one wavefront each).
 * Non-finite inputs: one MFMA covers two blocks.  The row-wise kernel multiplies an unpaired
 * block together with a block of zeros, the compact kernel pads a block row with zero columns
 * (0 x Inf = NaN where B holds Inf or NaN).  The sweep kernel multiplies an unpaired block together with
 * a neighbouring block of the SAME block row and 16 rows of zeros in place of B, and its filler ops multiply two
 * blocks of the block row they add to by zeros: an Inf or NaN in vals stays in its own block row of C (where a
 * block-by-block product, mmaCBT.cu:44-66, has an Inf or NaN as well).  Only a block that is alone in its block
 * row shares its MFMA with the block that follows it in vals (another row's), and a wavefront whose block rows all
 * have fewer than two blocks uses blocks 0 and 1 for its fillers: Inf or NaN in THOSE blocks can turn that row NaN.
 * Finite inputs give the same sums up to the fp32 summation order. */
int smat_spmm_bcsr_f16_ex(const uint16_t *vals, const int32_t *row_ptr, const int32_t *col_idx,
                          const uint16_t *B, void *C, size_t M, size_t N, size_t K, size_t nnzb,
                          const smat_spmm_opts *opts, const smat_plan *plan);

/* ---- SpMM that allocates nothing ------------------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Same operands and result type as
 * smat_spmm_bcsr_f16 plus the stream.  It runs what a SMAT_KERNEL_ROWWISE_PACKED plan runs for whole block
 * rows (B is first repacked slab-major, then the row-wise kernel), with the copy of B in a fixed array inside
 * the library instead of plan-owned memory: it calls no hipMalloc / hipFree.
 * Limit: K * N * 2 <= SMAT_STATIC_SCRATCH_BYTES, else SMAT_ERR_UNSUPPORTED.  Each GPU the library runs on holds
 * one such array until the process ends.  Every call on a GPU uses that GPU's array: calls that overlap on one
 * GPU (two streams, two threads) race; calls on one stream are ordered.  Nothing in the array has to survive
 * between calls (the repack rewrites every element it reads). */
#define SMAT_STATIC_SCRATCH_BYTES (64u << 20)
int smat_spmm_bcsr_f16_static(const uint16_t *vals, const int32_t *row_ptr, const int32_t *col_idx,
                              const uint16_t *B, uint16_t *C, size_t M, size_t N, size_t K, size_t nnzb,
                              void *stream);

/* ---- matrix load: Matrix Market -> CSR (host) ----------------------------
 * Replaces mmio_allinone (src/cuda_hgemm/src/common/mmio_highlevel.h:619-786):
 * M and K come back rounded up to multiples of 16, symmetric/hermitian files
 * are mirrored, entries keep file order inside a row, duplicates are kept,
 * values go double -> fp16.  Returns SMAT_OK or SMAT_ERR_IO; *ref_code receives
 * the reference's own code (-1 open, -2 banner, -4 size line; may be NULL).
 * Arrays are allocated by the library: release with smat_host_free. */
int smat_mtx_read(const char *path, size_t *M, size_t *K, size_t *nnz, int *is_symmetric,
                  int32_t **row_ptr, int32_t **col_idx, uint16_t **val, int *ref_code);
void smat_host_free(void *p);

/* ---- binary container (host) ----------------------------------------------
 * The reference keeps matrices as text only (.mtx read by mmio_allinone,
 * mmio_highlevel.h:619-786; .el for the reorder program, csr.cpp:153-290).  A
 * "SMATBIN1" file holds the same arrays in binary, optionally with the row and
 * column permutations of a reorder, behind a 64-byte header with a checksum.
 * kind: 1 = CSR (n = nnz, val = n halfs), 2 = BCSR (n = nonzero blocks,
 * row_ptr has M/16+1 entries, val = n*256 halfs).  perm_* may be NULL on write;
 * on read, pass NULL to skip them, and expect NULL back when the file has none.
 * Arrays returned by smat_bin_read are released with smat_host_free. */
#define SMAT_BIN_CSR 1
#define SMAT_BIN_BCSR 2
int smat_bin_write_csr(const char *path, size_t M, size_t K, const int32_t *row_ptr,
                       const int32_t *col_idx, const uint16_t *val, const int64_t *perm_rows,
                       const int64_t *perm_cols);
int smat_bin_write_bcsr(const char *path, size_t M, size_t K, size_t nnzb, const int32_t *b_row_ptr,
                        const int32_t *b_col_idx, const uint16_t *b_val, const int64_t *perm_rows,
                        const int64_t *perm_cols);
int smat_bin_read(const char *path, int *kind, size_t *M, size_t *K, size_t *n, int32_t **row_ptr,
                  int32_t **col_idx, uint16_t **val, int64_t **perm_rows, int64_t **perm_cols);
/* CSR -> Matrix Market "coordinate real general" (entries in storage order): the way back
 * to the reference's text format; smat_mtx_read of the result returns the same CSR. */
int smat_mtx_write(const char *path, size_t M, size_t K, const int32_t *row_ptr,
                   const int32_t *col_idx, const uint16_t *val);

/* ---- blocking: CSR -> 16x16 BCSR (host) -----------------------------------
 * Replaces SparseMatrix::csrToBcsr (src/cuda_hgemm/src/common/matrix.h:376-502)
 * and emits bit-identical row_ptr / col_idx / val without the two dense
 * (M/16)x(K/16) maps.  counts[0..2] = nonzero, "dense", "sparse" blocks as the
 * reference logs them (matrix.h:176, 2:4 heuristic matrix.h:400-419).
 * block_info / rel_map: pass non-NULL pointers only if the dense maps are
 * really wanted (they are (M/16)*(K/16) ints each); NULL skips them. */
int smat_csr_to_bcsr(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                     const uint16_t *val, int64_t *counts, int32_t **b_row_ptr,
                     int32_t **b_col_idx, uint16_t **b_val, int32_t **block_info,
                     int32_t **rel_map);

/* The same conversion on the GPU: row_ptr / col_idx / val are DEVICE arrays (nnz = row_ptr[M]
 * is passed by the caller), the three outputs are DEVICE arrays allocated by the library
 * (release with smat_free) and hold exactly what smat_csr_to_bcsr returns for the same input,
 * counts included.  row_ptr must be non-decreasing.  Synchronous. */
int smat_csr_to_bcsr_device(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                            const uint16_t *val, size_t nnz, int64_t *counts, int32_t **b_row_ptr,
                            int32_t **b_col_idx, uint16_t **b_val);

/* ---- reorder (host) --------------------------------------------------------
 * Row clustering that minimises the number of nonzero blocks: the reference's
 * `Matrix_Blocking -a 5 -F 1` path, BlockingEngine::GetGrouping
 * (preprocess/src/general/blocking.cpp:616-657) -> IterativeBlockingKeeper
 * (blocking.cpp:431-547) with JaccardDistanceGroup (blocking.cpp:904-975),
 * merge_rows (preprocess/src/general/utilities.cpp:145-173) and
 * get_fixed_size_grouping / get_permutation (utilities.cpp:8-54).
 *
 *   rows, row_ptr (int64, rows+1), col_idx (int64, sorted ascending in a row)
 *   col_block / row_block / tau : the -b / -B / -t flags (input.h:88-105)
 *   grouping  out, int64[rows]: block-row id of each row (the ".g" GROUPING line)
 *   perm      out, int64[rows]: perm[new_row] = old_row (CSR::reorder, csr.cpp:97-105)
 *   stats     out, int64[4]: comparison_counter, merge_counter,
 *             VBR_nzblocks_count, VBR_longest_row (utilities.cpp:217-224,
 *             blocking.cpp:562-614); may be NULL
 *
 * Matrices of 16,384 rows and more are scanned on several threads (the hardware's
 * count, at most 16; SMAT_REORDER_THREADS in the environment sets it, 1 = none):
 * the output does not depend on the number of threads.
 */
int smat_reorder_rows(int64_t rows, int64_t cols, const int64_t *row_ptr, const int64_t *col_idx,
                      int64_t col_block, int64_t row_block, float tau, int64_t *grouping,
                      int64_t *perm, int64_t *stats);

/* Row pass, then the same pass on the transpose of the row-permuted pattern
 * (what src/reorder.py:107-139,143-182 does through files), on a CSR with
 * int32 indices.  Trailing empty rows/columns keep their place, as they do not
 * exist in the reference's edge-list files (csr.cpp:262-263).
 * perm_rows[new]=old (M entries), perm_cols[new]=old (K entries). */
int smat_reorder_csr(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                     int64_t col_block, int64_t row_block, float tau, int do_cols,
                     int64_t *perm_rows, int64_t *perm_cols, int64_t *stats_rows,
                     int64_t *stats_cols);

/* Applies perm_rows / perm_cols (either may be NULL = identity) to a CSR with
 * values; columns inside a row come out ascending.  Output arrays are
 * allocated by the library (smat_host_free). */
int smat_permute_csr(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                     const uint16_t *val, const int64_t *perm_rows, const int64_t *perm_cols,
                     int32_t **out_row_ptr, int32_t **out_col_idx, uint16_t **out_val);

/* ---- thin device runtime wrappers (so hosts need no HIP headers) ----------
 * Stand in for the cudaMalloc / cudaMemcpy / cudaMemset / cudaDeviceSynchronize
 * calls of Matrix / SparseMatrix (matrix.h:30,40,78-101,158-199) and for
 * CudaTimer (src/cuda_hgemm/src/common/cuda_timer.h:7-45). */
int smat_device_count(int *n);
int smat_set_device(int dev);
int smat_device_name(int dev, char *buf, size_t len);
int smat_device_attr(int dev, int64_t *cus, int64_t *lds_bytes, int64_t *mem_bytes, int64_t *clock_khz);
int smat_malloc(void **dptr, size_t bytes);
int smat_free(void *dptr);
int smat_memcpy_h2d(void *dst, const void *src, size_t bytes);
int smat_memcpy_d2h(void *dst, const void *src, size_t bytes);
int smat_memcpy_d2d(void *dst, const void *src, size_t bytes);
int smat_memset(void *dptr, int byte, size_t bytes);
int smat_device_synchronize(void);
int smat_stream_create(void **stream);
int smat_stream_destroy(void *stream);
int smat_stream_synchronize(void *stream);
int smat_event_create(void **event);
int smat_event_destroy(void *event);
int smat_event_record(void *event, void *stream);
int smat_event_synchronize(void *event);
int smat_event_elapsed_ms(void *start, void *stop, float *ms);

/* Benchmark helper (no counterpart in the reference): the fp16 MFMA rate this device reaches on a kernel of
 * nothing but v_mfma_f32_16x16x32_f16 on registers, in TFLOP/s (best of seven timed passes, about 1 ms each).
 * The published peak assumes the maximum clock; this is what the card sustains. */
int smat_bench_mfma_peak(double *tflops);
/* Benchmark helper (no counterpart in the reference): the rate, in TFLOP/s of its MFMAs, of a kernel with the sweep
 * kernel's geometry and steady-state instruction mix on a static, regular schedule (8 wavefronts per CU; per op 4 LDS
 * reads of 1 KiB, one 1 KiB load of A, 5/8 of a 1 KiB global->LDS copy, 4 MFMAs), i.e. what the data flow delivers
 * without any bookkeeping.  variant 0: LDS reads and MFMAs only; 1: the full mix with the A operands inside 1 MiB
 * (resident in the L2); 2: the full mix with A spread over 13 MB like the headline matrix, the 8 workgroups of an
 * XCD slot reading the same blocks; 3 and 4: variants 1 and 2 with a workgroup barrier every 8 ops.  Best of four
 * timed passes of about a millisecond. */
int smat_bench_static_mix(int variant, double *tflops);

#ifdef __cplusplus
}
#endif
#endif /* SMAT_H */
