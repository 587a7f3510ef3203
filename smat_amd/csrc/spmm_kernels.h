// Internal interface between the C ABI (capi.hip) and the kernel launchers.
#pragma once
#include <hip/hip_runtime.h>

#include "sweep_format.h"
#include <mutex>
#include <utility>
#include <vector>
#include <stddef.h>
#include <stdint.h>

namespace smat {

// One unit of work for a wavefront: blocks [begin, end) of one block row.
struct WorkItem {
    int32_t block_row;
    int32_t begin;
    int32_t end;
    int32_t dst; // < 0: finished tile goes to C; >= 0: fp32 partial tile goes to this workspace slot
};

// A block row that was split over several work items: its partial tiles occupy
// workspace slots [slot_begin, slot_end), summed in that order.
struct SplitRow {
    int32_t block_row;
    int32_t slot_begin;
    int32_t slot_end;
    int32_t pad;
};

// How a launch over a work list deals its workgroups to the eight XCDs.  The dispatcher gives an XCD the workgroup
// ids that are equal modulo 8, whatever their work costs; the row-wise and the compact kernel lay the panel-major
// (panel, item) space (4 items per workgroup) out in runs of consecutive workgroups that the XCDs take in turn.
// One run per XCD keeps neighbouring block rows, which share rows of B, on one L2; short runs even out a list whose
// cost per item changes along it.
// choose_xcd_run: the longest run among {an eighth of the launch, 1024, 256, 64, 16, 4} that keeps the estimated load
// of the busiest XCD within 4 % of the mean (the best of them if none does); cost_prefix[i] = cost of the items
// before item i (n_items + 1 entries).
unsigned choose_xcd_run(const uint64_t *cost_prefix, uint64_t n_items, int n_panels);
struct XcdDeal {
    void set_costs(std::vector<uint64_t> &&prefix); // of another list: forgets the choices made for the old one
    // the choice for a launch of n_items x n_panels (kept once made); an eighth of the launch if the costs are not
    // those of a list of n_items
    unsigned run(size_t n_items, int n_panels) const;
private:
    std::vector<uint64_t> cost_prefix_;
    mutable std::mutex mutex_;
    mutable std::vector<std::pair<int, unsigned>> known_;
};

struct SpmmArgs {
    const uint16_t *vals;
    const int32_t *row_ptr;
    const int32_t *col_idx;
    const uint16_t *B;
    void *C;
    size_t M, N, K, nnzb;
    bool c_f32;
    int panel_tiles;       // 0 = choose from N; else 1, 2, 4, 8 or 16 n-tiles of 16 per wavefront
    const WorkItem *items; // device; nullptr = one item per block row
    int n_items;
    const SplitRow *split_rows; // device
    int n_split_rows;
    float *workspace; // device, n_slots * 16 * N floats
    uint16_t *b_packed; // device scratch of K * N halves, or nullptr: read the column-major B directly
    int max_item_blocks; // blocks of the longest work item, 0 = not known (no plan): lets short rows take the short-row kernel
    const XcdDeal *deal; // how to deal the items to the XCDs; nullptr = an eighth of the launch each
};

// Stream format and geometry of the sweep kernel: sweep_format.h (shared with the host-side plan builder).

struct SweepArgs {
    const uint16_t *vals;
    const uint16_t *B;
    void *C;
    size_t M, N, K, nnzb;
    bool c_f32;
    const int32_t *rg_chunk_ptr; // device, n_rg + 1: range of the row group in chunk_ids
    const int32_t *chunk_ids;    // device: the K chunks in which the row group has blocks, ascending (+ SWEEP_CHUNK_PAD entries)
    const int32_t *op_ptr;       // device, n_rg * SWEEP_WAVES + 1: range of (row group, wavefront) in ops
    const SweepOp *ops;          // device, op streams (sweep_format.h)
    const int32_t *row_map;      // device, n_rg * SWEEP_G: block row of (row group, wavefront, local row), -1 = none
    int n_rg;
};

// Sums the fp32 partial tiles of split block rows (workspace[(slot*16 + i)*N + n]) in slot order.
hipError_t launch_reduce(const float *workspace, const SplitRow *split_rows, int n_split_rows, void *C, size_t N,
                         bool c_f32, hipStream_t st);

// ---- compacted-column kernel (spmm_compact.hip) ----
// For matrices whose blocks hold only a few nonzero columns: the nonzero columns of a block
// row are listed once (from the zero pattern of the values) and multiplied 32 at a time.
struct CompactPlan {
    int32_t *d_cols = nullptr;   // row of B (absolute column of A) of every listed column; block rows padded to 32
    uint16_t *d_acol = nullptr;  // the 16 values of every listed column, in MFMA operand order (32 bytes per column)
    WorkItem *d_items = nullptr; // begin/end index the padded list
    SplitRow *d_split = nullptr;
    float *d_workspace = nullptr; // n_slots * 16 * n_cap floats
    int n_items = 0, n_split_rows = 0, n_slots = 0;
    int64_t n_cols = 0;           // nonzero block columns listed (without padding)
    int64_t n_cols_all = 0;       // nonzero block columns of the whole matrix
    uint64_t values_checksum = 0; // of the block values the lists were made from
    XcdDeal deal;                 // cost of an item: its steps of 32 columns, and two more
    // Measured once, when the values are attached (compact_tune): the run length of the deal to the XCDs for
    // launches of tuned_n columns; 0 = not measured, the estimate from the costs decides.
    size_t tuned_n = 0;
    unsigned tuned_run = 0;
};
// vals / row_ptr / col_idx: device BCSR arrays; row_ptr_host: host copy of row_ptr.
// dense_rows != NULL and dense_share > 0: block rows with at least that share of nonzero columns get no list and no
// work item (a dense kernel multiplies them); *dense_rows receives one flag per block row.
// skip_blocks_host != NULL: one flag per block; flagged blocks get no listed columns (another kernel multiplies them).
// block_cols != NULL: receives the number of nonzero columns of every block.
hipError_t compact_build(const uint16_t *vals, const int32_t *row_ptr, const int32_t *col_idx,
                         const int32_t *row_ptr_host, size_t mb, size_t nnzb, size_t n_cap, double dense_share,
                         std::vector<uint8_t> *dense_rows, CompactPlan **out, const uint8_t *skip_blocks_host = nullptr,
                         std::vector<uint8_t> *block_cols = nullptr);
// out[j * 256 ..] = block ids_host[j] of vals (device to device, synchronous).
hipError_t copy_blocks(const uint16_t *vals, const int32_t *ids_host, size_t n, uint16_t *out);
void compact_destroy(CompactPlan *p);
// Order-independent checksum of nnzb * 256 block values on the device (synchronous, one pass over vals).
hipError_t values_checksum(const uint16_t *vals, size_t nnzb, uint64_t *out);
struct CompactArgs {
    const uint16_t *B; // column-major, or row-major with b_row_major
    bool b_row_major;  // B is already B[k*N + n]: no copy is made
    uint16_t *Bt;      // scratch, K * (N rounded up to 256) halves: the copy of B in panels of rows made at the start of the launch
    void *C;
    size_t M, N, K;
    bool c_f32;
    unsigned xcd_run = 0; // 0 = the plan's choice
    const CompactPlan *plan;
    bool accumulate = false; // C += A B instead of C = A B (plans without split rows only)
};
hipError_t launch_compact(const CompactArgs &a, hipStream_t st);
// Times launches of M x N x K with a few run lengths of the deal to the XCDs (the estimate's choice, an eighth of the
// launch, a half and a quarter of that) on zeros in temporary buffers and keeps the fastest for launches of N columns
// (tuned_n, tuned_run).  The deal decides where an item runs, not what it computes: the results do not depend on
// it.  Synchronous, default stream; a plan too large for the temporary buffers, or whose single launch takes
// longer than 20 ms, keeps the estimate's choice.
hipError_t compact_tune(CompactPlan &p, uint16_t *Bt, size_t M, size_t N, size_t K, bool b_row_major, bool accumulate);
hipError_t launch_b_to_col_major(const uint16_t *B_row_major, uint16_t *out, size_t N, size_t K, hipStream_t st);

int rowwise_panel_tiles(size_t N, int requested, size_t n_items);
hipError_t launch_sweep(const SweepArgs &a, hipStream_t st);
hipError_t launch_rowwise(const SpmmArgs &a, hipStream_t st);

} // namespace smat
