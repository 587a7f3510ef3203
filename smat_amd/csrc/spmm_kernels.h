// Internal interface between the C ABI (capi.hip) and the kernel launchers.
#pragma once
#include <hip/hip_runtime.h>
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

struct SpmmArgs {
    const uint16_t *vals;
    const int32_t *row_ptr;
    const int32_t *col_idx;
    const uint16_t *B;
    void *C;
    size_t M, N, K, nnzb;
    bool c_f32;
    int panel_tiles;       // 0 = choose from N; else 1, 2, 4 or 8 n-tiles of 16 per wavefront
    const WorkItem *items; // device; nullptr = one item per block row
    int n_items;
    const SplitRow *split_rows; // device
    int n_split_rows;
    float *workspace; // device, n_slots * 16 * N floats
};

int rowwise_panel_tiles(size_t N, int requested);
hipError_t launch_rowwise(const SpmmArgs &a, hipStream_t st);

} // namespace smat
