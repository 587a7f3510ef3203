// Builds the op streams of the sweep kernel.  Layout of an op: spmm_kernels.h (SweepOp).
#include "sweep_plan.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "../../include/smat.h"

namespace smat {

namespace {
// mirrors spmm_kernels.h (that header needs the HIP runtime; this file is compiled by g++)
constexpr uint32_t OP_ZERO_HI = 1u << 0, OP_ZERO_LO = 1u << 1, OP_BOUNDARY = 1u << 2;
constexpr int G = 64, RW = 8, WAVES = 8, S = 16, STAGES = 4, MIN_OPS = 2, OP_PAD = 384;
constexpr uint32_t ROW_CODE = 40; // bytes of code per block row in the kernel's MFMA dispatch

// LDS byte offset of the 16 rows of B under a block: chunk position in the row group's list, block column in the chunk
uint32_t lds_offset(int32_t chunk_pos, int32_t slab)
{
    const uint32_t slot = (uint32_t)(chunk_pos % STAGES) * S + (uint32_t)slab;
    return (slot >> 3) * 16384u + (slot & 7u) * 32u;
}
} // namespace

void build_sweep_plan(const int32_t *row_ptr, const int32_t *col_idx, size_t mb, size_t kb, SweepPlanHost &out)
{
    const size_t n_rg = (mb + G - 1) / G;
    const size_t n_kchunks = (kb + S - 1) / S;
    const int32_t nnzb = row_ptr[mb];
    out = SweepPlanHost();
    out.rg_chunk_ptr.assign(n_rg + 1, 0);
    out.op_ptr.reserve(n_rg * WAVES + 1);
    std::vector<int32_t> local(n_kchunks, -1); // K chunk -> position in the row group's chunk list
    struct Ranked { int rank; int row; SweepOpHost op; };
    std::vector<std::vector<Ranked>> by_chunk;
    for (size_t rg = 0; rg < n_rg; rg++) {
        const size_t r_begin = rg * G, r_end = std::min(mb, (rg + 1) * G);
        // the chunks this row group touches, ascending
        const size_t first_chunk = out.chunk_ids.size();
        for (int32_t q = row_ptr[r_begin]; q < row_ptr[r_end]; q++) local[(size_t)(col_idx[q] / 16) / S] = 0;
        for (size_t c = 0; c < n_kchunks; c++)
            if (local[c] == 0) {
                local[c] = (int32_t)(out.chunk_ids.size() - first_chunk);
                out.chunk_ids.push_back((int32_t)c);
            }
        const size_t n_chunks = out.chunk_ids.size() - first_chunk;
        out.rg_chunk_ptr[rg + 1] = (int32_t)out.chunk_ids.size();
        for (int w = 0; w < WAVES; w++) {
            out.op_ptr.push_back((int32_t)out.ops.size());
            by_chunk.assign(n_chunks, {});
            for (int r = 0; r < RW; r++) {
                const size_t br = r_begin + (size_t)w * RW + r;
                if (br >= r_end) break;
                int32_t q = row_ptr[br];
                const int32_t q_end = row_ptr[br + 1];
                while (q < q_end) {
                    const int32_t bc0 = col_idx[q] / 16;
                    const int32_t cl0 = local[(size_t)bc0 / S];
                    const uint32_t off0 = lds_offset(cl0, bc0 % S);
                    SweepOpHost op{0, 0, 0, 0};
                    int32_t exec = cl0;
                    bool pair = false;
                    if (q + 1 < q_end) {
                        const int32_t bc1 = col_idx[q + 1] / 16;
                        const int32_t cl1 = local[(size_t)bc1 / S];
                        if (cl1 - cl0 <= 1) { // same chunk or the next listed one: both stages are resident
                            op.w0 = (uint32_t)q * 512u;
                            op.w1 = off0;
                            op.w2 = lds_offset(cl1, bc1 % S) - off0;
                            op.w3 = (uint32_t)r * ROW_CODE << 23;
                            exec = cl1;
                            pair = true;
                        }
                    }
                    if (!pair) {
                        if (q + 1 < nnzb) { // blocks (q, q + 1), the second multiplied by zeros
                            op.w0 = (uint32_t)q * 512u;
                            op.w3 = OP_ZERO_HI | ((uint32_t)r * ROW_CODE << 23);
                        } else { // last block of the matrix: blocks (q - 1, q), the first multiplied by zeros
                            op.w0 = (uint32_t)(q - 1) * 512u;
                            op.w3 = OP_ZERO_LO | ((uint32_t)r * ROW_CODE << 23);
                        }
                        op.w1 = off0; // both halves read the rows of B under this block
                        op.w2 = 0;
                    }
                    (pair ? out.n_pairs : out.n_singles)++;
                    // rank = how many ops of this block row the chunk already holds: ops of one block
                    // row (same accumulators) end up spread over the chunk
                    int rank = 0;
                    for (const Ranked &x : by_chunk[(size_t)exec]) rank += x.row == r;
                    by_chunk[(size_t)exec].push_back(Ranked{rank, r, op});
                    q += pair ? 2 : 1;
                }
            }
            for (size_t c = 0; c < n_chunks; c++) {
                std::vector<Ranked> &list = by_chunk[c];
                std::stable_sort(list.begin(), list.end(), [](const Ranked &a, const Ranked &b) {
                    if (a.rank != b.rank) return a.rank < b.rank;
                    return a.row < b.row;
                });
                while (list.size() < (size_t)MIN_OPS) { // filler: blocks 0 and 1 times zeros, first slab of this chunk
                    const uint32_t off = lds_offset((int32_t)c, 0);
                    list.push_back(Ranked{0, 0, SweepOpHost{0, off, 0, OP_ZERO_HI | OP_ZERO_LO}});
                    out.n_fillers++;
                }
                if (c > 0) list[0].op.w3 |= OP_BOUNDARY;
                for (const Ranked &x : list) out.ops.push_back(x.op);
            }
        }
        for (size_t c = first_chunk; c < out.chunk_ids.size(); c++) local[(size_t)out.chunk_ids[c]] = -1;
    }
    out.op_ptr.push_back((int32_t)out.ops.size());
    // what the kernel reads ahead of the last op: fetched, never executed
    out.ops.resize(out.ops.size() + OP_PAD, SweepOpHost{0, 0, 0, OP_ZERO_HI | OP_ZERO_LO});
}

} // namespace smat

// Test hook (not part of smat.h): builds the work list on the host and hands it out.  Arrays are
// allocated with malloc; release each with smat_host_free.  counts[0..5] = row groups, listed
// chunks, ops (with fillers, without padding), pairs, singles, fillers.
extern "C" int smat_internal_sweep_plan(const int32_t *row_ptr, const int32_t *col_idx, size_t M, size_t K,
                                         int32_t **rg_chunk_ptr, int32_t **chunk_ids, int32_t **op_ptr,
                                         uint32_t **ops, int64_t *counts)
{
    if (!row_ptr || !col_idx || !rg_chunk_ptr || !chunk_ids || !op_ptr || !ops || !counts) return SMAT_ERR_INVALID;
    if (M == 0 || M % 16 || K % 16 || row_ptr[M / 16] < 2) return SMAT_ERR_INVALID;
    smat::SweepPlanHost p;
    try {
        smat::build_sweep_plan(row_ptr, col_idx, M / 16, K / 16, p);
    } catch (...) {
        return SMAT_ERR_NOMEM;
    }
    auto dup = [](const void *src, size_t bytes) -> void * {
        void *d = malloc(bytes ? bytes : 1);
        if (d && bytes) memcpy(d, src, bytes);
        return d;
    };
    *rg_chunk_ptr = (int32_t *)dup(p.rg_chunk_ptr.data(), p.rg_chunk_ptr.size() * 4);
    *chunk_ids = (int32_t *)dup(p.chunk_ids.data(), p.chunk_ids.size() * 4);
    *op_ptr = (int32_t *)dup(p.op_ptr.data(), p.op_ptr.size() * 4);
    *ops = (uint32_t *)dup(p.ops.data(), p.ops.size() * 16);
    if (!*rg_chunk_ptr || !*chunk_ids || !*op_ptr || !*ops) return SMAT_ERR_NOMEM;
    counts[0] = (int64_t)p.rg_chunk_ptr.size() - 1;
    counts[1] = (int64_t)p.chunk_ids.size();
    counts[2] = (int64_t)p.ops.size() - 384;
    counts[3] = (int64_t)p.n_pairs;
    counts[4] = (int64_t)p.n_singles;
    counts[5] = (int64_t)p.n_fillers;
    return SMAT_OK;
}
