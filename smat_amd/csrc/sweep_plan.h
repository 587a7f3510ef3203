// Host-side work list of the sweep kernel (see spmm_sweep.hip): per row group of 64 block rows the
// K chunks it touches, per (row group, wavefront) a stream of ops.  Plain C++: built and checked
// without a GPU.
#pragma once
#include <stddef.h>
#include <stdint.h>

#include <vector>

#include "sweep_format.h"

namespace smat {

typedef SweepOp SweepOpHost; // sweep_format.h

struct SweepPlanHost {
    std::vector<int32_t> rg_chunk_ptr; // n_rg + 1
    std::vector<int32_t> chunk_ids;    // K chunk of every (row group, listed chunk), + SWEEP_CHUNK_PAD entries
    std::vector<int32_t> op_ptr;       // n_rg * 8 + 1
    std::vector<int32_t> row_map;      // n_rg * 64: block row of (row group, wavefront, local row), -1 = none
    std::vector<SweepOpHost> ops;      // streams (ops, ends) + SWEEP_OP_PAD entries
    size_t n_pairs = 0, n_singles = 0, n_fillers = 0;
};

// row_ptr / col_idx: host BCSR (col_idx = absolute first column of each block, validated by the caller);
// at least two blocks.  rows != NULL: only these n_rows block rows (ascending) are multiplied and stored, packed
// 64 to a row group; the others belong to another kernel.  The rows go to the row groups in list order, or, where
// that leaves one group with over 1.08 x the blocks of an average one, by their block count (row_map says where).
void build_sweep_plan(const int32_t *row_ptr, const int32_t *col_idx, size_t mb, size_t kb, SweepPlanHost &out,
                      const int32_t *rows = nullptr, size_t n_rows = 0);

} // namespace smat
