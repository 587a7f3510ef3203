// CSR -> 16x16 blocked CSR on the host.
//
// Produces exactly the arrays of SparseMatrix::csrToBcsr
// (src/cuda_hgemm/src/common/matrix.h:376-502): row_ptr per block row, col_idx =
// ABSOLUTE first column of each nonzero block, ascending inside a block row
// (matrix.h:441-463), values row-major inside a block with the later duplicate
// winning (matrix.h:470-487), and the three block counters of the log line
// (matrix.h:176) including the "three adjacent columns ending at c%4 in {2,3}"
// test that promotes a block from "sparse" to "dense" (matrix.h:400-419).
//
// The reference walks two dense (M/16)x(K/16) int maps (blockInfo,
// relativeBlockIndexMapping).  Blocks are numbered in the same row-major order
// in which row_ptr/col_idx are emitted, so the map value of a nonzero block
// always equals its position in col_idx; this implementation therefore keeps
// one K/16-entry scratch row per block row and never forms the dense maps
// unless the caller asks for them.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/smat.h"
#include "errors.h"

using namespace smat;

static int smat_csr_to_bcsr_impl(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                                 const uint16_t *val, int64_t *counts, int32_t **b_row_ptr,
                                 int32_t **b_col_idx, uint16_t **b_val, int32_t **block_info,
                                 int32_t **rel_map)
{
    if (!row_ptr || !b_row_ptr || !b_col_idx || !b_val)
        return set_error(SMAT_ERR_INVALID, "NULL argument");
    if (M == 0 || K == 0 || M % 16 || K % 16)
        return set_error(SMAT_ERR_INVALID, "M (%zu) and K (%zu) must be positive multiples of 16", M, K);
    const int64_t nnz = row_ptr[M];
    if (nnz && (!col_idx || !val)) return set_error(SMAT_ERR_INVALID, "col_idx/val must not be NULL");
    const size_t mb = M / 16, kb = K / 16;

    // pass A: per block row, discover blocks and classify them in entry order
    std::vector<int32_t> slot(kb, -1);     // block column -> index into `touched`
    std::vector<int32_t> touched;          // block columns seen in this block row
    std::vector<int8_t> state;             // 1 = "sparse", 2 = "dense" (reference naming)
    std::vector<int32_t> rp(mb + 1, 0);
    std::vector<int32_t> cols;             // absolute columns, all block rows
    std::vector<int8_t> states;            // classification aligned with cols
    int64_t dense = 0;
    for (size_t br = 0; br < mb; br++) {
        touched.clear();
        state.clear();
        for (size_t row = br * 16; row < br * 16 + 16; row++) {
            if (row_ptr[row + 1] < row_ptr[row]) return set_error(SMAT_ERR_INVALID, "row_ptr must be non-decreasing");
            for (int64_t j = row_ptr[row]; j < row_ptr[row + 1]; j++) {
                const int32_t col = col_idx[j];
                if (col < 0 || (size_t)col >= K)
                    return set_error(SMAT_ERR_INVALID, "column %d of row %zu is outside 0..%zu", col, row, K - 1);
                const int32_t bc = col / 16;
                if (slot[bc] < 0) {
                    slot[bc] = (int32_t)touched.size();
                    touched.push_back(bc);
                    state.push_back(1);
                } else if (state[slot[bc]] == 1) {
                    const int r = col % 4;
                    if ((r == 2 || r == 3) && j >= (int64_t)row_ptr[row] + 2 && col_idx[j - 1] == col - 1 &&
                        col_idx[j - 2] == col - 2)
                        state[slot[bc]] = 2;
                }
            }
        }
        std::vector<int32_t> order(touched.begin(), touched.end());
        std::sort(order.begin(), order.end());
        for (int32_t bc : order) {
            cols.push_back(bc * 16);
            states.push_back(state[slot[bc]]);
            dense += state[slot[bc]] == 2;
        }
        for (int32_t bc : touched) slot[bc] = -1;
        if (cols.size() > 0x7fffffffu) return set_error(SMAT_ERR_INVALID, "more than 2^31-1 nonzero blocks");
        rp[br + 1] = (int32_t)cols.size();
    }
    const size_t nnzb = cols.size();

    int32_t *orp = (int32_t *)malloc(sizeof(int32_t) * (mb + 1));
    int32_t *oci = (int32_t *)malloc(sizeof(int32_t) * std::max<size_t>(nnzb, 1));
    uint16_t *ov = (uint16_t *)calloc(std::max<size_t>(nnzb, 1) * 256, sizeof(uint16_t));
    if (!orp || !oci || !ov) {
        free(orp); free(oci); free(ov);
        return set_error(SMAT_ERR_NOMEM, "out of host memory for %zu blocks", nnzb);
    }
    memcpy(orp, rp.data(), sizeof(int32_t) * (mb + 1));
    if (nnzb) memcpy(oci, cols.data(), sizeof(int32_t) * nnzb);

    // pass B: scatter values; position of block (br, bc) = rp[br] + rank of bc
    for (size_t br = 0; br < mb; br++) {
        for (int32_t p = rp[br]; p < rp[br + 1]; p++) slot[cols[p] / 16] = p;
        for (size_t row = br * 16; row < br * 16 + 16; row++)
            for (int64_t j = row_ptr[row]; j < row_ptr[row + 1]; j++) {
                const int32_t col = col_idx[j];
                ov[(size_t)slot[col / 16] * 256 + (row % 16) * 16 + col % 16] = val[j];
            }
        for (int32_t p = rp[br]; p < rp[br + 1]; p++) slot[cols[p] / 16] = -1;
    }

    if (block_info || rel_map) {
        const size_t cells = mb * kb;
        int32_t *info = block_info ? (int32_t *)calloc(std::max<size_t>(cells, 1), sizeof(int32_t)) : nullptr;
        int32_t *rel = rel_map ? (int32_t *)malloc(sizeof(int32_t) * std::max<size_t>(cells, 1)) : nullptr;
        if ((block_info && !info) || (rel_map && !rel)) {
            free(info); free(rel); free(orp); free(oci); free(ov);
            return set_error(SMAT_ERR_NOMEM, "out of host memory for the dense %zu x %zu block maps", mb, kb);
        }
        if (rel) for (size_t i = 0; i < cells; i++) rel[i] = -1;
        for (size_t br = 0; br < mb; br++)
            for (int32_t p = rp[br]; p < rp[br + 1]; p++) {
                const size_t cell = br * kb + (size_t)cols[p] / 16;
                if (info) info[cell] = states[p];
                if (rel) rel[cell] = p;
            }
        if (block_info) *block_info = info;
        if (rel_map) *rel_map = rel;
    }
    if (counts) {
        counts[0] = (int64_t)nnzb;
        counts[1] = dense;
        counts[2] = (int64_t)nnzb - dense;
    }
    *b_row_ptr = orp; *b_col_idx = oci; *b_val = ov;
    return SMAT_OK;
}

extern "C" int smat_csr_to_bcsr(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                                 const uint16_t *val, int64_t *counts, int32_t **b_row_ptr,
                                 int32_t **b_col_idx, uint16_t **b_val, int32_t **block_info,
                                 int32_t **rel_map)
{
    return smat::guarded("smat_csr_to_bcsr", [&] { return smat_csr_to_bcsr_impl(M, K, row_ptr, col_idx, val, counts, b_row_ptr, b_col_idx, b_val, block_info, rel_map); });
}
