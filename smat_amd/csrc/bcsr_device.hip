// CSR -> 16x16 blocked CSR on the GPU: same arrays, bit for bit, as the host
// smat_csr_to_bcsr (and therefore as SparseMatrix::csrToBcsr,
// src/cuda_hgemm/src/common/matrix.h:376-502), without the host pass over the matrix.
//
//   1. key(entry) = block_row * Kb + block_col for every stored entry (entry-parallel, the row
//      of an entry is found by bisection of row_ptr);
//   2. radix sort of the keys, then unique: the sorted distinct keys ARE the blocks in the
//      row-major block order in which the reference numbers them (matrix.h:425-431), so
//      col_idx = (key % Kb) * 16 and row_ptr[br] = lower_bound(keys, br * Kb);
//   3. values: one thread per CSR row walks its entries in storage order and writes
//      b_val[block * 256 + (row % 16) * 16 + col % 16]; a later duplicate of the same (row, col)
//      overwrites the earlier one exactly as the serial loop does (matrix.h:470-487).  Rows
//      longer than LONG_ROW entries are handled by a whole wavefront, 64 entries per step, the
//      steps separated by a wait for the stores of the step before;
//   4. the "dense"/"sparse" counters of the reference's log line (matrix.h:176, 400-419): a
//      block is "dense" when some entry (r, c) with c % 4 in {2, 3} directly follows entries
//      (r, c-1) and (r, c-2) in storage order.  Such a triple lies in one block and its last
//      entry is never the first entry of the block, so the test is independent per entry.
#include <hip/hip_runtime.h>
#include <hipcub/hipcub.hpp>
#include <stdint.h>

#include "../../include/smat.h"
#include "devmem.h"
#include "errors.h"

using namespace smat;

namespace {

constexpr int LONG_ROW = 512;

__device__ __forceinline__ int64_t row_of_entry(const int32_t *__restrict__ row_ptr, int64_t M, int64_t i)
{
    // largest r with row_ptr[r] <= i
    int64_t lo = 0, hi = M;
    while (hi - lo > 1) {
        const int64_t mid = (lo + hi) >> 1;
        if (row_ptr[mid] <= i) lo = mid; else hi = mid;
    }
    return lo;
}

__global__ void make_keys_kernel(const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col_idx,
                                 int64_t M, int64_t K, int64_t nnz, uint64_t *__restrict__ keys,
                                 int32_t *__restrict__ bad)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    const int32_t col = col_idx[i];
    if (col < 0 || col >= K) { *bad = 1; keys[i] = 0; return; }
    const int64_t row = row_of_entry(row_ptr, M, i);
    keys[i] = (uint64_t)(row >> 4) * (uint64_t)(K >> 4) + (uint64_t)(col >> 4);
}

__global__ void block_index_kernel(const uint64_t *__restrict__ ukeys, int64_t nnzb, int64_t mb, int64_t kb,
                                   int32_t *__restrict__ b_row_ptr, int32_t *__restrict__ b_col_idx)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < nnzb) b_col_idx[t] = (int32_t)(ukeys[t] % (uint64_t)kb) * 16;
    if (t <= mb) {
        const uint64_t want = (uint64_t)t * (uint64_t)kb;
        int64_t lo = 0, hi = nnzb; // first p with ukeys[p] >= want
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (ukeys[mid] < want) lo = mid + 1; else hi = mid;
        }
        b_row_ptr[t] = (int32_t)lo;
    }
}

// position of block column `bc` inside block row [lo, hi) of b_col_idx (it is always present)
__device__ __forceinline__ int32_t find_block(const int32_t *__restrict__ b_col_idx, int32_t lo, int32_t hi, int32_t col16)
{
    while (hi - lo > 1) {
        const int32_t mid = (lo + hi) >> 1;
        if (b_col_idx[mid] <= col16) lo = mid; else hi = mid;
    }
    return lo;
}

__device__ __forceinline__ bool promotes(const int32_t *__restrict__ col_idx, int64_t j, int64_t row_start, int32_t col)
{
    const int r = col & 3;
    return (r == 2 || r == 3) && j >= row_start + 2 && col_idx[j - 1] == col - 1 && col_idx[j - 2] == col - 2;
}

// one thread per CSR row of at most LONG_ROW entries
__global__ void scatter_rows_kernel(const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col_idx,
                                    const uint16_t *__restrict__ val, int64_t M,
                                    const int32_t *__restrict__ b_row_ptr, const int32_t *__restrict__ b_col_idx,
                                    uint16_t *__restrict__ b_val, uint8_t *__restrict__ dense_flag)
{
    const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= M) return;
    const int64_t begin = row_ptr[row], end = row_ptr[row + 1];
    if (end - begin > LONG_ROW) return;
    const int32_t lo = b_row_ptr[row >> 4], hi = b_row_ptr[(row >> 4) + 1];
    int32_t last_c16 = -1, p = 0;
    for (int64_t j = begin; j < end; j++) {
        const int32_t col = col_idx[j];
        const int32_t c16 = col & ~15;
        if (c16 != last_c16) { p = find_block(b_col_idx, lo, hi, c16); last_c16 = c16; }
        b_val[(int64_t)p * 256 + (row & 15) * 16 + (col & 15)] = val[j];
        if (promotes(col_idx, j, begin, col)) dense_flag[p] = 1;
    }
}

// one wavefront per CSR row with more than LONG_ROW entries
__global__ __launch_bounds__(256) void scatter_long_rows_kernel(
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col_idx, const uint16_t *__restrict__ val,
    int64_t M, const int32_t *__restrict__ b_row_ptr, const int32_t *__restrict__ b_col_idx,
    uint16_t *__restrict__ b_val, uint8_t *__restrict__ dense_flag)
{
    const int64_t row = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (row >= M) return;
    const int64_t begin = row_ptr[row], end = row_ptr[row + 1];
    if (end - begin <= LONG_ROW) return; // wave-uniform
    const int32_t lo = b_row_ptr[row >> 4], hi = b_row_ptr[(row >> 4) + 1];
    for (int64_t base = begin; base < end; base += 64) {
        const int64_t j = base + lane;
        const bool live = j < end;
        const int32_t col = live ? col_idx[j] : -1;
        // a later entry of this step with the same column wins: drop this one
        bool shadowed = false;
        for (int d = 1; d < 64; d++) {
            const int32_t other = __shfl_down(col, d);
            if (lane + d < 64 && other == col) shadowed = true;
        }
        if (live) {
            const int32_t p = find_block(b_col_idx, lo, hi, col & ~15);
            if (!shadowed) b_val[(int64_t)p * 256 + (row & 15) * 16 + (col & 15)] = val[j];
            if (promotes(col_idx, j, begin, col)) dense_flag[p] = 1;
        }
        // stores of this step are complete before the next step may overwrite them
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    }
}

__global__ void count_flags_kernel(const uint8_t *__restrict__ flags, int64_t n, int32_t *__restrict__ total)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int mine = i < n ? flags[i] : 0;
    const unsigned long long ballot = __ballot(mine != 0);
    if ((threadIdx.x & 63) == 0 && ballot) atomicAdd(total, __popcll(ballot));
}

struct Scratch {
    void *p = nullptr;
    ~Scratch() { if (p) (void)dev_free(p); }
    hipError_t alloc(size_t bytes) { return dev_malloc(&p, bytes ? bytes : 16); }
};

} // namespace

static int smat_csr_to_bcsr_device_impl(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                                        const uint16_t *val, size_t nnz, int64_t *counts,
                                        int32_t **b_row_ptr, int32_t **b_col_idx, uint16_t **b_val)
{
    if (!row_ptr || !b_row_ptr || !b_col_idx || !b_val)
        return set_error(SMAT_ERR_INVALID, "NULL argument");
    if (M == 0 || K == 0 || M % 16 || K % 16)
        return set_error(SMAT_ERR_INVALID, "M (%zu) and K (%zu) must be positive multiples of 16", M, K);
    if (nnz && (!col_idx || !val)) return set_error(SMAT_ERR_INVALID, "col_idx/val must not be NULL");
    if (nnz > 0x7fffffffu) return set_error(SMAT_ERR_INVALID, "more than 2^31-1 entries");
    const size_t mb = M / 16, kb = K / 16;
    *b_row_ptr = nullptr; *b_col_idx = nullptr; *b_val = nullptr;

#define SMAT_TRY(call)                                                                             \
    do {                                                                                           \
        hipError_t e_ = (call);                                                                    \
        if (e_ != hipSuccess) return set_error(SMAT_ERR_HIP, "%s: %s", #call, hipGetErrorString(e_)); \
    } while (0)

    Scratch keys, sorted, ukeys, n_unique, bad, tmp, flags;
    SMAT_TRY(keys.alloc(nnz * 8));
    SMAT_TRY(sorted.alloc(nnz * 8));
    SMAT_TRY(ukeys.alloc(nnz * 8));
    SMAT_TRY(n_unique.alloc(8));
    SMAT_TRY(bad.alloc(4));
    SMAT_TRY(hipMemset(bad.p, 0, 4));
    SMAT_TRY(hipMemset(n_unique.p, 0, 8));

    int64_t nnzb = 0;
    if (nnz) {
        const unsigned blocks = (unsigned)((nnz + 255) / 256);
        hipLaunchKernelGGL(make_keys_kernel, dim3(blocks), dim3(256), 0, 0, row_ptr, col_idx, (int64_t)M,
                           (int64_t)K, (int64_t)nnz, (uint64_t *)keys.p, (int32_t *)bad.p);
        SMAT_TRY(hipGetLastError());
        int end_bit = 1;
        while (end_bit < 64 && ((uint64_t)mb * kb) >> end_bit) end_bit++;
        size_t tmp_bytes = 0;
        SMAT_TRY(hipcub::DeviceRadixSort::SortKeys(nullptr, tmp_bytes, (uint64_t *)keys.p, (uint64_t *)sorted.p,
                                                   (int)nnz, 0, end_bit));
        size_t tmp2 = 0;
        SMAT_TRY(hipcub::DeviceSelect::Unique(nullptr, tmp2, (uint64_t *)sorted.p, (uint64_t *)ukeys.p,
                                              (int *)n_unique.p, (int)nnz));
        SMAT_TRY(tmp.alloc(std::max(tmp_bytes, tmp2)));
        SMAT_TRY(hipcub::DeviceRadixSort::SortKeys(tmp.p, tmp_bytes, (uint64_t *)keys.p, (uint64_t *)sorted.p,
                                                   (int)nnz, 0, end_bit));
        SMAT_TRY(hipcub::DeviceSelect::Unique(tmp.p, tmp2, (uint64_t *)sorted.p, (uint64_t *)ukeys.p,
                                              (int *)n_unique.p, (int)nnz));
        int32_t h_unique = 0, h_bad = 0;
        SMAT_TRY(hipMemcpy(&h_unique, n_unique.p, 4, hipMemcpyDeviceToHost));
        SMAT_TRY(hipMemcpy(&h_bad, bad.p, 4, hipMemcpyDeviceToHost));
        if (h_bad) return set_error(SMAT_ERR_INVALID, "a column index is outside 0..%zu", K - 1);
        nnzb = h_unique;
    }

    int32_t *orp = nullptr, *oci = nullptr;
    uint16_t *ov = nullptr;
    hipError_t e = dev_malloc(&orp, (mb + 1) * sizeof(int32_t));
    if (e == hipSuccess) e = dev_malloc(&oci, std::max<size_t>(nnzb, 1) * sizeof(int32_t));
    if (e == hipSuccess) e = dev_malloc(&ov, std::max<size_t>(nnzb, 1) * 512);
    if (e == hipSuccess) e = hipMemset(ov, 0, std::max<size_t>(nnzb, 1) * 512);
    if (e == hipSuccess) e = flags.alloc(std::max<size_t>(nnzb, 1));
    if (e == hipSuccess) e = hipMemset(flags.p, 0, std::max<size_t>(nnzb, 1));
    int64_t dense = 0;
    if (e == hipSuccess) {
        const int64_t threads = std::max<int64_t>(nnzb, (int64_t)mb + 1);
        hipLaunchKernelGGL(block_index_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, 0,
                           (const uint64_t *)ukeys.p, nnzb, (int64_t)mb, (int64_t)kb, orp, oci);
        e = hipGetLastError();
    }
    if (e == hipSuccess && nnz) {
        hipLaunchKernelGGL(scatter_rows_kernel, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, 0, row_ptr,
                           col_idx, val, (int64_t)M, orp, oci, ov, (uint8_t *)flags.p);
        e = hipGetLastError();
        if (e == hipSuccess) {
            hipLaunchKernelGGL(scatter_long_rows_kernel, dim3((unsigned)((M * 64 + 255) / 256)), dim3(256), 0, 0,
                               row_ptr, col_idx, val, (int64_t)M, orp, oci, ov, (uint8_t *)flags.p);
            e = hipGetLastError();
        }
        if (e == hipSuccess && counts && nnzb) {
            Scratch sum;
            e = sum.alloc(4);
            if (e == hipSuccess) e = hipMemset(sum.p, 0, 4);
            if (e == hipSuccess) {
                hipLaunchKernelGGL(count_flags_kernel, dim3((unsigned)((nnzb + 255) / 256)), dim3(256), 0, 0,
                                   (const uint8_t *)flags.p, nnzb, (int32_t *)sum.p);
                e = hipGetLastError();
            }
            int32_t h = 0;
            if (e == hipSuccess) e = hipMemcpy(&h, sum.p, 4, hipMemcpyDeviceToHost);
            dense = h;
        }
    }
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        if (orp) (void)dev_free(orp);
        if (oci) (void)dev_free(oci);
        if (ov) (void)dev_free(ov);
        return set_error(SMAT_ERR_HIP, "device blocking failed: %s", hipGetErrorString(e));
    }
    if (counts) {
        counts[0] = nnzb;
        counts[1] = dense;
        counts[2] = nnzb - dense;
    }
    *b_row_ptr = orp; *b_col_idx = oci; *b_val = ov;
    return SMAT_OK;
#undef SMAT_TRY
}

extern "C" int smat_csr_to_bcsr_device(size_t M, size_t K, const int32_t *row_ptr, const int32_t *col_idx,
                                        const uint16_t *val, size_t nnz, int64_t *counts,
                                        int32_t **b_row_ptr, int32_t **b_col_idx, uint16_t **b_val)
{
    return smat::guarded("smat_csr_to_bcsr_device", [&] { return smat_csr_to_bcsr_device_impl(M, K, row_ptr, col_idx, val, nnz, counts, b_row_ptr, b_col_idx, b_val); });
}
