// SpMM for block matrices whose 16x16 blocks hold only a few nonzero COLUMNS (random sparse
// matrices blocked without much clustering: about one nonzero per block).  The dense kernels
// gather 16 rows of B for every block; here only the rows of B that meet a nonzero column of A
// are touched, and 32 such columns of one block row are multiplied per MFMA step.
//
// Same product as the reference kernel (src/cuda_hgemm/src/mma/mmaCBT.cu:13-88): an all-zero
// column of a block contributes nothing to C, so leaving it out changes no result (with finite B).
//
//  * compact_build (once per matrix, from the block values):
//      colmask_kernel   16-bit mask of the nonzero columns of every block (two blocks per
//                       wavefront step, OR over the 16 rows with cross-lane shuffles);
//      exclusive scan   of the popcounts; the per-block-row totals go to the host, which pads
//                       every block row to a multiple of 32 columns (zero columns) and cuts the
//                       list into work items (whole block rows, long ones in chunks whose fp32
//                       partial tiles are summed afterwards);
//      gather_kernel    writes, for every nonzero column, its row of B (absolute column index)
//                       and a COPY of its 16 values in MFMA operand order:
//                       acol[((step*4 + g)*16 + m)*8 + j] = A[m][column 32*step + 8*g + j],
//                       so that the A operand of a step is one coalesced 16-byte load per lane.
//    The SpMM then does not read the block values any more: they must be attached again when
//    they change.
//  * transpose_b_kernel: column-major B (B[n*K + k]) -> Bt at the start of every launch, so that
//    the row of B under a nonzero column is contiguous.  Bt holds the panels of 64*TQ columns one
//    after the other, each a row-major K x 64*TQ matrix: the pass over a panel gathers from one
//    contiguous K * 128*TQ bytes.
//  * spmm_compact_kernel<TQ>: one wavefront per (work item, panel of 64*TQ columns).  A step takes
//    32 columns = K of one v_mfma_f32_16x16x32_f16.  The product is formed as
//    C^T = B^T * A^T like in the other kernels:
//      A operand   lane (m = lane % 16, g = lane / 16): one 16-byte load from acol;
//      B operand   lane (i = lane % 16, g) needs, for each of its 8 entries (listed columns 8g .. 8g+7 of the
//                  step), the columns of C its tiles own.  Every gather is 16 bytes per lane: a CU keeps a
//                  limited number of vector memory instructions (and of cache lines) in flight, so an
//                  instruction should bring as much as it can (8-byte gathers: 12 % slower on every config).
//                  TQ = 2: 8 columns 8i .. 8i+7 of the 128-column panel per entry (16 lanes read 256
//                  contiguous bytes); one v_perm_b32 per word merges the t-th halves of two consecutive
//                  entries into the operand word of n-tile t, so tile t of the group owns columns 8i + t.
//                  TQ = 1 (rows of 128 bytes): lanes i < 8 gather the even entries of the group, lanes
//                  i >= 8 the odd ones, 8 columns 8 (i & 7) .. + 7 each (4 instructions, not 8); lane i and
//                  lane i ^ 8 then trade halves (one DPP row rotation per word), so that each has 4 columns
//                  of all 8 entries: tile t owns columns 8 (i & 7) + 4 (i >> 3) + t.
//                  The index list keeps, inside every group of 8, the even entries first and then the odd
//                  ones, so the four indices such a lane needs are 16 contiguous bytes; one load instruction
//                  fetches them for 8 steps at a time (lane i16 & 7 = step) and DPP row broadcasts hand them round.
//      result      TQ = 2: lane (m, g) holds 32 consecutive columns of C row m;
//                  TQ = 1: after one v_permlane32_swap per value, 16 consecutive columns.
#include <hip/hip_runtime.h>
#include <hipcub/hipcub.hpp>
#include <stdint.h>

#include <algorithm>
#include <type_traits>
#include <vector>

#include "devmem.h"
#include "spmm_kernels.h"

namespace smat {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

int g_force_run = 0;
int g_tune = 1; // test hook: 0 = attaching values measures nothing, the estimate decides the deal
int g_last_run = 0; // test hook: the run length of the latest launch
int g_force_tq = 0; // test hook: 1 or 2 = panels of 64 or 128 columns whatever the sizes say, 0 = the launcher decides

constexpr int LIST_PAD = 640; // entries readable past the end of the list (the index loads of the 64-column panel run up to 16 steps ahead)

// ---- census of nonzero block columns ----

__global__ __launch_bounds__(256) void colmask_kernel(const uint16_t *__restrict__ vals, long nnzb,
                                                      uint16_t *__restrict__ mask, int32_t *__restrict__ count)
{
    const int lane = threadIdx.x & 63;
    const long wave = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const long n_waves = ((long)gridDim.x * blockDim.x) >> 6;
    for (long pb = wave * 2; pb < nnzb; pb += n_waves * 2) {
        const long blk = pb + (lane >> 5);
        // lane % 32 = row * 2 + half: 8 values of one row
        u32x4 w = {0u, 0u, 0u, 0u};
        if (blk < nnzb) w = *reinterpret_cast<const u32x4 *>(vals + blk * 256 + (lane & 31) * 8);
        w &= 0x7fff7fffu; // -0.0 is a zero
#pragma unroll
        for (int d = 2; d <= 16; d <<= 1) { // OR over the 16 rows (lane bits 1..4)
            w[0] |= __shfl_xor(w[0], d);
            w[1] |= __shfl_xor(w[1], d);
            w[2] |= __shfl_xor(w[2], d);
            w[3] |= __shfl_xor(w[3], d);
        }
        uint32_t bits = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (w[q] & 0xffffu) bits |= 1u << (2 * q);
            if (w[q] >> 16) bits |= 1u << (2 * q + 1);
        }
        const uint32_t other = __shfl_xor(bits, 1); // the other half of the row
        if ((lane & 31) == 0 && blk < nnzb) {
            const uint32_t m = bits | (other << 8);
            mask[blk] = (uint16_t)m;
            count[blk] = __popc(m);
        }
    }
}

// Order-independent 64-bit checksum of the block values: sum over all dwords of value * (2 * index + 1).
__global__ __launch_bounds__(256) void values_checksum_kernel(const uint32_t *__restrict__ vals, long n_dwords,
                                                              unsigned long long *__restrict__ out)
{
    unsigned long long sum = 0;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n_dwords; i += (long)gridDim.x * blockDim.x)
        sum += (unsigned long long)vals[i] * (2ull * (unsigned long long)i + 1ull);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d);
    if ((threadIdx.x & 63) == 0) atomicAdd(out, sum);
}

// One thread per block: its nonzero columns go to positions padded_start[br] + (offset[p] -
// offset[row_ptr[br]]) .. of the padded list.
__global__ void gather_kernel(const uint16_t *__restrict__ vals, const uint16_t *__restrict__ mask,
                              const int32_t *__restrict__ offset, const int32_t *__restrict__ row_ptr,
                              const int32_t *__restrict__ col_idx, const int32_t *__restrict__ padded_start,
                              long mb, long nnzb, int32_t *__restrict__ cols, uint16_t *__restrict__ acol)
{
    const long p = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= nnzb) return;
    uint32_t m = mask[p];
    if (!m) return;
    long lo = 0, hi = mb; // block row of p: largest br with row_ptr[br] <= p
    while (hi - lo > 1) {
        const long mid = (lo + hi) >> 1;
        if (row_ptr[mid] <= p) lo = mid; else hi = mid;
    }
    if (padded_start[lo] < 0) return; // a block row that another kernel multiplies
    long o = (long)padded_start[lo] + (offset[p] - offset[row_ptr[lo]]);
    const int32_t c0 = col_idx[p];
    const uint16_t *blk = vals + p * 256;
    while (m) {
        const int k = __ffs(m) - 1;
        m &= m - 1;
        // inside its group of 8 the even entries come first, then the odd ones: the lanes of the product kernel that
        // gather the even (odd) entries of a group read their four indices with one 16-byte load
        cols[(o & ~7L) + ((o & 1) << 2) + ((o & 7) >> 1)] = c0 + k;
        uint16_t *dst = acol + ((o >> 3) * 16) * 8 + (o & 7); // (step*4 + g) = o / 8
#pragma unroll
        for (int r = 0; r < 16; r++) dst[r * 8] = blk[r * 16 + k];
        o++;
    }
}

// raw[br] = first (unpadded) list position of block row br; raw[mb] = total
__global__ void row_offsets_kernel(const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ offset,
                                   const int32_t *__restrict__ count, long mb, long nnzb, int32_t *__restrict__ raw)
{
    const long br = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (br > mb) return;
    const long p = row_ptr[br];
    raw[br] = p < nnzb ? offset[p] : (nnzb ? offset[nnzb - 1] + count[nnzb - 1] : 0);
}

// Blocks that another kernel multiplies (per-block split of a mixed plan): no listed columns.
__global__ void drop_blocks_kernel(const uint8_t *__restrict__ skip, long nnzb, uint16_t *__restrict__ mask, int32_t *__restrict__ count)
{
    const long p = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (p < nnzb && skip[p]) {
        mask[p] = 0;
        count[p] = 0;
    }
}

// out[j] = block ids[j] of vals (512 bytes each; 32 lanes x 16 bytes per block).
__global__ __launch_bounds__(256) void copy_blocks_kernel(const uint16_t *__restrict__ vals, const int32_t *__restrict__ ids, long n,
                                                          uint16_t *__restrict__ out)
{
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long j = t >> 5;
    if (j >= n) return;
    const int piece = (int)(t & 31);
    reinterpret_cast<u32x4 *>(out + j * 256)[piece] = reinterpret_cast<const u32x4 *>(vals + (long)ids[j] * 256)[piece];
}

// ---- B: column-major -> row-major ----
// 64 n x 64 k tile through LDS.  A thread reads 16 bytes (8 k) of two neighbouring columns, pairs
// the values of equal k into dwords and writes them to the transposed tile; then every thread
// reads 8 n of one k back (two 8-byte LDS reads) and stores 16 bytes.
// The output is split into panels of `panel` columns, each a K x panel row-major matrix of leading
// dimension ld, one panel after the other (panel >= N and ld = N: plain row-major K x N).
__global__ __launch_bounds__(256) void transpose_b_kernel(const uint16_t *__restrict__ B, uint16_t *__restrict__ Bt,
                                                          int N, long K, int panel, long ld)
{
    constexpr int LD = 68; // halfs per LDS row (k): 8-byte aligned rows, dword writes spread over the banks
    __shared__ __align__(16) uint16_t tile[64 * LD];
    const int t = threadIdx.x;
    const long k0 = (long)blockIdx.x * 64;
    const int n0 = blockIdx.y * 64;
    {
        const int np = t >> 3, seg = t & 7; // columns 2np, 2np+1; k = 8seg .. 8seg+7
        u32x4 v0 = {0u, 0u, 0u, 0u}, v1 = {0u, 0u, 0u, 0u};
        if (k0 + seg * 8 < K) {
            if (n0 + 2 * np < N) v0 = *reinterpret_cast<const u32x4 *>(B + (long)(n0 + 2 * np) * K + k0 + seg * 8);
            if (n0 + 2 * np + 1 < N) v1 = *reinterpret_cast<const u32x4 *>(B + (long)(n0 + 2 * np + 1) * K + k0 + seg * 8);
        }
#pragma unroll
        for (int w = 0; w < 4; w++) {
            uint32_t *row = reinterpret_cast<uint32_t *>(tile + (seg * 8 + 2 * w) * LD + 2 * np);
            row[0] = __builtin_amdgcn_perm(v1[w], v0[w], 0x05040100u);      // k = 8seg + 2w
            row[LD / 2] = __builtin_amdgcn_perm(v1[w], v0[w], 0x07060302u); // k = 8seg + 2w + 1
        }
    }
    __syncthreads();
    const int a = t >> 3, seg = t & 7;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        const int k = a + 32 * half;
        if (k0 + k < K && n0 + seg * 8 < N) {
            const uint2 lo = *reinterpret_cast<const uint2 *>(tile + k * LD + seg * 8);
            const uint2 hi = *reinterpret_cast<const uint2 *>(tile + k * LD + seg * 8 + 4);
            uint16_t *out = Bt + (long)(n0 / panel) * K * panel + (k0 + k) * ld + n0 % panel + seg * 8;
            *reinterpret_cast<u32x4 *>(out) = (u32x4){lo.x, lo.y, hi.x, hi.y};
        }
    }
}

// ---- the product ----

// C_ACC: the result is added to what C holds (the per-block split of a mixed plan: a dense kernel has written the
// part of the blocks it multiplies); work items that go through the workspace are not made for such plans.
template <int TQ, bool C_F32, bool C_ACC>
__global__ __launch_bounds__(256) void spmm_compact_kernel(
    const uint16_t *__restrict__ acol, const int32_t *__restrict__ cols, const uint16_t *__restrict__ Bt,
    void *__restrict__ Cout, float *__restrict__ workspace, const WorkItem *__restrict__ items, int n_items, int N,
    int n_panels, long panel_stride, long row_stride, unsigned xcd_run)
{
    constexpr int PANEL = 64 * TQ;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Panel-major order of the (panel, item) space.  An XCD gets the workgroup ids that are equal modulo 8, whatever
    // their work costs; here the XCDs take runs of xcd_run consecutive workgroups of that order in turn (gridDim.x is a
    // multiple of 8 * xcd_run).  One run per XCD keeps neighbouring block rows, which share rows of B, on one L2;
    // short runs even out a list whose cost per item changes along it (R-MAT: 60 to 70 % of the steps are in the first
    // quarter of the items, and the launch took as long as the XCD that got them).
    const long total = (long)n_items * n_panels;
    const unsigned slot = blockIdx.x >> 3;
    const unsigned run = __builtin_amdgcn_readfirstlane(slot / xcd_run);
    const long wg = ((long)run * 8 + (blockIdx.x & 7)) * xcd_run + (slot - run * xcd_run);
    const long w = wg * 4 + wave;
    if (w >= total) return;
    const int panel = (int)(w / n_items);
    const int it = (int)(w - (long)panel * n_items);
    const WorkItem wi = items[it];
    const int br = __builtin_amdgcn_readfirstlane(wi.block_row);
    const int e0 = __builtin_amdgcn_readfirstlane(wi.begin);
    const int e1 = __builtin_amdgcn_readfirstlane(wi.end);
    const int dst = __builtin_amdgcn_readfirstlane(wi.dst);

    const int i16 = lane & 15, g = lane >> 4;
    const int n0 = panel * PANEL;
    // Row `col` of this panel of B starts at Bp + col * row_stride (B in place: panel_stride = PANEL,
    // row_stride = N; the transposed copy: panels one after the other, row_stride = PANEL).
    const uint16_t *Bp = Bt + (long)panel * panel_stride;
    // Every gather is 16 bytes per lane: what a CU can keep in flight is a number of vector memory instructions
    // and of cache lines, so an instruction should bring as much as it can.
    //   WIDE (TQ = 2): a lane takes 8 columns of the 128-column panel, for each of its 8 entries.
    //   PAIRED (TQ = 1, rows of 128 bytes): lanes i16 < 8 take the even entries, lanes i16 >= 8 the odd ones, 8
    //   columns each (4 instructions instead of 8); the two lanes then trade halves, so that each has 4 columns of
    //   all 8 entries again.
    constexpr bool WIDE = TQ % 2 == 0, PAIRED = TQ == 1;
    static_assert(TQ == 1 || TQ == 2, "panels of 64 or 128 columns");
    constexpr int NG = WIDE ? TQ / 2 : 1; // groups of 128 columns (WIDE)
    const bool odd_entries = (i16 & 8) != 0; // PAIRED
    int boff[NG]; // element offset of this lane's 8 columns inside the panel row (its column 0 when out of range)
#pragma unroll
    for (int q = 0; q < NG; q++) {
        const int n = WIDE ? 128 * q + 8 * i16 : 8 * (i16 & 7);
        boff[q] = n0 + n < N ? n : 0; // N % 8 == 0: all of the lane's columns or none
    }

    f32x4 acc[TQ][4];
#pragma unroll
    for (int q = 0; q < TQ; q++)
#pragma unroll
        for (int t = 0; t < 4; t++) acc[q][t] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // Software pipeline over steps of 32 columns (items start and end on multiples of 32): the
    // column indices of step s+2, then the operands of step s+1 (whose indices arrived a step
    // ago) are requested before the MFMAs of step s.  Loads past the end of the item read the
    // next item's data or the padding behind the arrays: always valid addresses, never used.
    struct Entries { u32x4 r[PAIRED ? 1 : 2]; }; // the indices of a group of 8: entries 0, 2, 4, 6, then 1, 3, 5, 7
    struct Operands { u32x4 aw; u32x4 L[NG][PAIRED ? 4 : 8]; };
    auto load_entries = [&](int e, Entries &x) {
        const u32x4 *lp = reinterpret_cast<const u32x4 *>(cols + e + 8 * g); // the 128-column panel; the other has its own loop
        x.r[0] = lp[0];
        if constexpr (!PAIRED) x.r[1] = lp[1];
    };
    auto load_operands = [&](int e, const Entries &x, Operands &o) {
        o.aw = *reinterpret_cast<const u32x4 *>(acol + ((long)(e >> 3) + g) * 128 + i16 * 8);
        if constexpr (PAIRED) {
#pragma unroll
            for (int j = 0; j < 4; j++)
                o.L[0][j] = *reinterpret_cast<const u32x4 *>(Bp + (long)x.r[0][j] * row_stride + boff[0]); // entry 2j or 2j + 1
        } else {
#pragma unroll
            for (int q = 0; q < NG; q++)
#pragma unroll
                for (int j = 0; j < 8; j++)
                    o.L[q][j] = *reinterpret_cast<const u32x4 *>(Bp + (long)x.r[j & 1][j >> 1] * row_stride + boff[q]);
        }
    };
    auto multiply = [&](const Operands &o) {
        const f16x8 av = __builtin_bit_cast(f16x8, o.aw);
        if constexpr (WIDE) {
#pragma unroll
            for (int q = 0; q < NG; q++)
#pragma unroll
                for (int t = 0; t < 8; t++) { // tile t of the group takes the t-th of the lane's eight columns
                    u32x4 b;
#pragma unroll
                    for (int p = 0; p < 4; p++)
                        b[p] = __builtin_amdgcn_perm(o.L[q][2 * p + 1][t >> 1], o.L[q][2 * p][t >> 1], (t & 1) ? 0x07060302u : 0x05040100u);
                    acc[2 * q + (t >> 2)][t & 3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, b), av, acc[2 * q + (t >> 2)][t & 3], 0, 0, 0);
                }
        } else {
            // Lane i16 < 8 holds columns 8 i16 .. + 7 of the even entries, lane i16 + 8 the same columns of the odd
            // entries.  Each sends the half the other needs (row rotation by 8 lanes) and ends up with 4 columns of
            // both entries of every pair: columns 8 (i16 & 7) + 4 (i16 >> 3) + t, t = tile.
            u32x4 b[4];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const u32x4 x = o.L[0][p];
                const uint32_t s0 = odd_entries ? x[0] : x[2], s1 = odd_entries ? x[1] : x[3];
                const uint32_t k0 = odd_entries ? x[2] : x[0], k1 = odd_entries ? x[3] : x[1];
                const uint32_t r0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)s0, 0x128, 0xf, 0xf, false); // row_ror:8
                const uint32_t r1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)s1, 0x128, 0xf, 0xf, false);
                const uint32_t ev0 = odd_entries ? r0 : k0, ev1 = odd_entries ? r1 : k1; // entry 2p
                const uint32_t od0 = odd_entries ? k0 : r0, od1 = odd_entries ? k1 : r1; // entry 2p + 1
                b[0][p] = __builtin_amdgcn_perm(od0, ev0, 0x05040100u);
                b[1][p] = __builtin_amdgcn_perm(od0, ev0, 0x07060302u);
                b[2][p] = __builtin_amdgcn_perm(od1, ev1, 0x05040100u);
                b[3][p] = __builtin_amdgcn_perm(od1, ev1, 0x07060302u);
            }
#pragma unroll
            for (int t = 0; t < 4; t++)
                acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, b[t]), av, acc[0][t], 0, 0, 0);
        }
    };
    if constexpr (PAIRED) {
        // The index loads of 8 steps in one instruction (an instruction that brings 128 bytes costs the vector memory
        // path as much as one that brings 1 KiB): lane (i16, g) asks for the four indices that its kind of lane (group g,
        // even or odd entries) needs at step i16 & 7 of a block of 8 steps; at step k of the block every lane takes them
        // from the lane that holds step k, with one DPP row broadcast per half of the 16-lane row and word.  Blocks are
        // asked for one block ahead; what lies past the end of the item is the next item's list or the padding.
        if (e0 < e1) {
            auto load_block = [&](int e, u32x4 &x) {
                x = *reinterpret_cast<const u32x4 *>(cols + e + 32 * (i16 & 7) + 8 * g + (odd_entries ? 4 : 0));
            };
            auto indices = [&](const u32x4 &x, auto kc, Entries &out) {
                constexpr int K = decltype(kc)::value;
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    int r = __builtin_amdgcn_update_dpp(0, (int)x[w], 0x150 + K, 0xf, 0x3, false); // row_newbcast:K     -> lanes 0-7 of the row
                    r = __builtin_amdgcn_update_dpp(r, (int)x[w], 0x150 + 8 + K, 0xf, 0xc, false); // row_newbcast:8 + K -> lanes 8-15
                    out.r[0][w] = (uint32_t)r;
                }
            };
            u32x4 blk_a, blk_b;
            Entries ent;
            Operands op_a, op_b;
            load_block(e0, blk_a);
            load_block(e0 + 256, blk_b);
            indices(blk_a, std::integral_constant<int, 0>{}, ent);
            load_operands(e0, ent, op_a);
            int e = e0;
            while (true) {
#define SMAT_TWO_STEPS(KA, KB, BLK_B)                                                                  \
                indices(blk_a, std::integral_constant<int, KA>{}, ent);                                \
                load_operands(e + 32, ent, op_b);                                                      \
                multiply(op_a);                                                                        \
                e += 32;                                                                               \
                if (e >= e1) break;                                                                    \
                indices(BLK_B, std::integral_constant<int, KB>{}, ent);                                \
                load_operands(e + 32, ent, op_a);                                                      \
                multiply(op_b);                                                                        \
                e += 32;                                                                               \
                if (e >= e1) break;
                SMAT_TWO_STEPS(1, 2, blk_a)
                SMAT_TWO_STEPS(3, 4, blk_a)
                SMAT_TWO_STEPS(5, 6, blk_a)
                SMAT_TWO_STEPS(7, 0, blk_b)
#undef SMAT_TWO_STEPS
                blk_a = blk_b;
                load_block(e + 256, blk_b);
            }
        }
    } else if (e0 < e1) {
        Entries ent_a, ent_b;
        Operands op_a, op_b;
        load_entries(e0, ent_a);
        load_entries(e0 + 32, ent_b);
        load_operands(e0, ent_a, op_a);
        int e = e0;
        while (true) {
            load_entries(e + 64, ent_a);
            load_operands(e + 32, ent_b, op_b);
            multiply(op_a);
            e += 32;
            if (e >= e1) break;
            load_entries(e + 64, ent_b);
            load_operands(e + 32, ent_a, op_a);
            multiply(op_b);
            e += 32;
            if (e >= e1) break;
        }
    }

    const long m = (long)br * 16 + i16;
    if constexpr (WIDE) {
        // tile t8 = 4 * (q & 1) + t of group q / 2: acc[q][t][r] = C[br*16 + i16][n0 + 128 (q/2) + 32g + 8r + t8]
#pragma unroll
        for (int q2 = 0; q2 < NG; q2++) {
            const int c0 = n0 + 128 * q2 + 32 * g;
            float o[32];
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int t = 0; t < 8; t++) o[8 * r + t] = acc[2 * q2 + (t >> 2)][t & 3][r];
            if (dst >= 0 || C_F32) {
                float *row = dst >= 0 ? workspace + ((long)dst * 16 + i16) * (long)N
                                      : reinterpret_cast<float *>(Cout) + m * (long)N;
#pragma unroll
                for (int h = 0; h < 8; h++)
                    if (c0 + 4 * h < N) {
                        f32x4 v = {o[4 * h], o[4 * h + 1], o[4 * h + 2], o[4 * h + 3]};
                        if (C_ACC && dst < 0) v += *reinterpret_cast<const f32x4 *>(row + c0 + 4 * h);
                        *reinterpret_cast<f32x4 *>(row + c0 + 4 * h) = v;
                    }
            } else {
                uint16_t *row = reinterpret_cast<uint16_t *>(Cout) + m * (long)N;
#pragma unroll
                for (int h = 0; h < 4; h++) {
                    if (c0 + 8 * h >= N) continue;
                    f16x8 v;
                    if (C_ACC) {
                        const f16x8 old = *reinterpret_cast<const f16x8 *>(row + c0 + 8 * h);
#pragma unroll
                        for (int j = 0; j < 8; j++) v[j] = (_Float16)(o[8 * h + j] + (float)old[j]);
                    } else {
#pragma unroll
                        for (int j = 0; j < 8; j++) v[j] = (_Float16)o[8 * h + j];
                    }
                    *reinterpret_cast<f16x8 *>(row + c0 + 8 * h) = v;
                }
            }
        }
    } else {
        // acc[0][t][r] = C[br*16 + i16][n0 + cb + t] with cb = 32 g + 8 r (g < 2) or 32 (g - 2) + 8 r + 4 (g >= 2): lane
        // (i16, g) and lane (i16, g + 2) hold the two halves of the same 8-column groups.  One swap per value between
        // the halves of the wavefront (the lower lanes hand over r = 2, 3 and get r = 0, 1) leaves every lane with 16
        // consecutive columns, starting at 32 (g & 1) + 16 (g >> 1).
        float o[16];
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
            for (int rr = 0; rr < 2; rr++) {
                const float lo = acc[0][t][rr], hi = acc[0][t][rr + 2]; // scalars first: a bit cast of a vector element reads element 0
                const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
                o[8 * rr + t] = __uint_as_float((uint32_t)sw[0]);
                o[8 * rr + 4 + t] = __uint_as_float((uint32_t)sw[1]);
            }
        const int c0 = n0 + 32 * (g & 1) + 16 * (g >> 1);
        if (dst >= 0 || C_F32) {
            float *row = dst >= 0 ? workspace + ((long)dst * 16 + i16) * (long)N
                                  : reinterpret_cast<float *>(Cout) + m * (long)N;
#pragma unroll
            for (int h = 0; h < 4; h++)
                if (c0 + 4 * h < N) {
                    f32x4 v = {o[4 * h], o[4 * h + 1], o[4 * h + 2], o[4 * h + 3]};
                    if (C_ACC && dst < 0) v += *reinterpret_cast<const f32x4 *>(row + c0 + 4 * h);
                    *reinterpret_cast<f32x4 *>(row + c0 + 4 * h) = v;
                }
        } else {
            uint16_t *row = reinterpret_cast<uint16_t *>(Cout) + m * (long)N;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                if (c0 + 8 * h >= N) continue;
                f16x8 v;
                if (C_ACC) {
                    const f16x8 old = *reinterpret_cast<const f16x8 *>(row + c0 + 8 * h);
#pragma unroll
                    for (int j = 0; j < 8; j++) v[j] = (_Float16)(o[8 * h + j] + (float)old[j]);
                } else {
#pragma unroll
                    for (int j = 0; j < 8; j++) v[j] = (_Float16)o[8 * h + j];
                }
                *reinterpret_cast<f16x8 *>(row + c0 + 8 * h) = v;
            }
        }
    }
}

template <int TQ>
hipError_t launch_compact_tq(const CompactArgs &a, hipStream_t st)
{
    const CompactPlan &p = *a.plan;
    constexpr int PANEL = 64 * TQ;
    const int n_panels = (int)((a.N + PANEL - 1) / PANEL);
    long panel_stride = PANEL, row_stride = (long)a.N;
    if (!a.b_row_major) {
        dim3 grid((unsigned)((a.K + 63) / 64), (unsigned)((a.N + 63) / 64));
        hipLaunchKernelGGL(transpose_b_kernel, grid, dim3(256), 0, st, a.B, a.Bt, (int)a.N, (long)a.K, PANEL, (long)PANEL);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        panel_stride = (long)a.K * PANEL;
        row_stride = PANEL;
    }
    const long total = (long)p.n_items * n_panels;
    long wgs = (total + 3) / 4;
    if (wgs == 0) return hipSuccess;
    long xcd_run = p.deal.run((size_t)p.n_items, n_panels);
    if (p.tuned_run > 0 && p.tuned_n == a.N) xcd_run = p.tuned_run;
    if (a.xcd_run > 0) xcd_run = a.xcd_run;
    if (g_force_run > 0) xcd_run = g_force_run;
    xcd_run = std::min<long>((wgs + 7) / 8, xcd_run);
    g_last_run = (int)xcd_run;
    wgs = (wgs + 8 * xcd_run - 1) / (8 * xcd_run) * (8 * xcd_run);
    if (wgs > 0x7fffffffL) return hipErrorInvalidValue;
    if (a.accumulate && p.n_split_rows > 0) return hipErrorInvalidValue; // partial tiles through the workspace overwrite C
#define SMAT_LAUNCH_COMPACT(F32, ACC)                                                                                           \
    hipLaunchKernelGGL((spmm_compact_kernel<TQ, F32, ACC>), dim3((unsigned)wgs), dim3(256), 0, st, p.d_acol, p.d_cols, a.Bt, a.C, \
                       p.d_workspace, p.d_items, p.n_items, (int)a.N, n_panels, panel_stride, row_stride, (unsigned)xcd_run)
    if (a.c_f32) {
        if (a.accumulate) SMAT_LAUNCH_COMPACT(true, true); else SMAT_LAUNCH_COMPACT(true, false);
    } else {
        if (a.accumulate) SMAT_LAUNCH_COMPACT(false, true); else SMAT_LAUNCH_COMPACT(false, false);
    }
#undef SMAT_LAUNCH_COMPACT
    return hipGetLastError();
}

struct Scratch {
    void *p = nullptr;
    ~Scratch() { if (p) (void)dev_free(p); }
    hipError_t alloc(size_t bytes) { return dev_malloc(&p, bytes ? bytes : 16); }
};

} // namespace

// Row-major B (B[k*N + n]) -> column-major out[n*K + k]: the same tile transposition with the roles of the
// two dimensions swapped (N % 8 == 0 and K % 16 == 0 keep every 16-byte access aligned).
hipError_t launch_b_to_col_major(const uint16_t *B_row_major, uint16_t *out, size_t N, size_t K, hipStream_t st)
{
    dim3 grid((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64));
    hipLaunchKernelGGL(transpose_b_kernel, grid, dim3(256), 0, st, B_row_major, out, (int)K, (long)N, 0x7fffffff, (long)K);
    return hipGetLastError();
}

// The panel width of a launch, in units of 64 columns.
static int compact_panel_width(const CompactPlan &p, size_t N, size_t K)
{
    const long items = p.n_items;
    int tq = 1;
    if (N >= 128 && items * (long)(N / 128) >= 2048 && p.n_cols >= (int64_t)items * 384) tq = 2;
    if (g_force_tq == 1 || g_force_tq == 2) tq = g_force_tq;
    while (tq > 1 && K * (size_t)(64 * tq) * sizeof(uint16_t) > ((size_t)128 << 20)) tq >>= 1;
    return tq;
}

hipError_t launch_compact(const CompactArgs &a_in, hipStream_t st)
{
    CompactArgs a = a_in;
    hipError_t e = hipSuccess;
    if (a.b_row_major) a.Bt = const_cast<uint16_t *>(a.B); // read in place, never written
    // Panels of 128 columns read the A operand and the indices half as often as panels of 64; those of 64 give twice
    // the wavefronts.  Measured (N = 256 .. 4096): 128 wins where the items are long (dense blocks, 25 steps per
    // block row: 218 against 244 us), 64 where they are short (one nonzero per block, 4 to 8 steps: 21.7 against
    // 22.5 us, 94 against 97 us); panels of 256 columns never won.  The panels are swept one after the other, so the
    // rows of B that the gathers hit at random come from one panel at a time: a panel is kept under half of the
    // 256 MiB memory-side cache (the lists of A and the rows of C stream through it too).  On a 2^20-row B at
    // N = 128 the panel of 64 columns (128 MiB) takes 0.74 x the time of the panel of 128.
    const int tq = compact_panel_width(*a.plan, a.N, a.K);
    if (tq == 2) e = launch_compact_tq<2>(a, st);
    else e = launch_compact_tq<1>(a, st);
    if (e != hipSuccess) return e;
    if (a.plan->n_split_rows > 0)
        e = launch_reduce(a.plan->d_workspace, a.plan->d_split, a.plan->n_split_rows, a.C, a.N, a.c_f32, st);
    return e;
}

hipError_t compact_tune(CompactPlan &p, uint16_t *Bt, size_t M, size_t N, size_t K, bool b_row_major, bool accumulate)
{
    p.tuned_n = 0;
    p.tuned_run = 0;
    if (!g_tune || p.n_items == 0 || N == 0 || !Bt) return hipSuccess;
    Scratch B, C;
    if (B.alloc(K * N * sizeof(uint16_t)) != hipSuccess || C.alloc(M * N * sizeof(uint16_t)) != hipSuccess) {
        (void)hipGetLastError(); // no room for the trial: not an error of the plan
        return hipSuccess;
    }
    hipError_t e = hipMemset(B.p, 0, K * N * sizeof(uint16_t));
    if (e == hipSuccess) e = hipMemset(C.p, 0, M * N * sizeof(uint16_t));
    hipEvent_t t0 = nullptr, t1 = nullptr;
    if (e == hipSuccess) e = hipEventCreate(&t0);
    if (e == hipSuccess) e = hipEventCreate(&t1);
    CompactArgs a{};
    a.B = static_cast<const uint16_t *>(B.p); a.b_row_major = b_row_major; a.Bt = Bt; a.C = C.p;
    a.M = M; a.N = N; a.K = K; a.c_f32 = false; a.plan = &p; a.accumulate = accumulate;
    auto time_of = [&](unsigned run, int launches, float *ms) {
        a.xcd_run = run;
        hipError_t r = launch_compact(a, nullptr); // warm-up
        if (r == hipSuccess) r = hipEventRecord(t0, nullptr);
        for (int i = 0; i < launches && r == hipSuccess; i++) r = launch_compact(a, nullptr);
        if (r == hipSuccess) r = hipEventRecord(t1, nullptr);
        if (r == hipSuccess) r = hipEventSynchronize(t1);
        if (r == hipSuccess) r = hipEventElapsedTime(ms, t0, t1);
        *ms /= (float)launches;
        return r;
    };
    // the run length of an untuned launch, as launch_compact_tq computes it for this N
    const int tq = compact_panel_width(p, N, K);
    const int n_panels = (int)((N + 64 * tq - 1) / (64 * tq));
    const long wgs = ((long)p.n_items * n_panels + 3) / 4;
    const unsigned eighth = (unsigned)std::max<long>((wgs + 7) / 8, 1);
    const unsigned base = std::min(eighth, p.deal.run((size_t)p.n_items, n_panels));
    float t_base = 0.f;
    if (e == hipSuccess) e = time_of(base, 1, &t_base);
    if (e == hipSuccess && t_base <= 20.f) {
        std::vector<unsigned> runs{base};
        if (base * 4 >= eighth) // a list that the estimate finds even: the longer runs are worth a try
            for (unsigned r : {eighth, eighth / 2, eighth / 4})
                if (r >= 4 && std::find(runs.begin(), runs.end(), r) == runs.end()) runs.push_back(r);
        const int launches = t_base < 0.2f ? 20 : t_base < 2.f ? 6 : 3;
        unsigned best_run = base;
        float best = 0.f;
        for (size_t i = 0; i < runs.size() && e == hipSuccess; i++) {
            float ms = 0.f;
            e = time_of(runs[i], launches, &ms);
            if (i == 0) best = ms * 0.97f; // another run length has to be 3 % faster than the estimate's choice
            else if (ms < best) best = ms, best_run = runs[i];
        }
        if (e == hipSuccess) p.tuned_n = N, p.tuned_run = best_run;
    }
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    return e;
}

hipError_t values_checksum(const uint16_t *vals, size_t nnzb, uint64_t *out)
{
    *out = 0;
    if (!nnzb) return hipSuccess;
    unsigned long long *d = nullptr;
    hipError_t e = dev_malloc(&d, sizeof(unsigned long long));
    if (e != hipSuccess) return e;
    e = hipMemset(d, 0, sizeof(unsigned long long));
    if (e == hipSuccess) {
        const long n_dwords = (long)nnzb * 128;
        const unsigned blocks = (unsigned)std::min<long>((n_dwords + 255) / 256, 256L * 16);
        hipLaunchKernelGGL(values_checksum_kernel, dim3(blocks), dim3(256), 0, 0, reinterpret_cast<const uint32_t *>(vals), n_dwords, d);
        e = hipGetLastError();
    }
    unsigned long long h = 0;
    if (e == hipSuccess) e = hipMemcpy(&h, d, sizeof h, hipMemcpyDeviceToHost);
    (void)dev_free(d);
    *out = h;
    return e;
}

void compact_destroy(CompactPlan *p)
{
    if (!p) return;
    if (p->d_cols) (void)dev_free(p->d_cols);
    if (p->d_acol) (void)dev_free(p->d_acol);
    if (p->d_items) (void)dev_free(p->d_items);
    if (p->d_split) (void)dev_free(p->d_split);
    if (p->d_workspace) (void)dev_free(p->d_workspace);
    delete p;
}

hipError_t copy_blocks(const uint16_t *vals, const int32_t *ids_host, size_t n, uint16_t *out)
{
    if (!n) return hipSuccess;
    Scratch ids;
    hipError_t e = ids.alloc(n * sizeof(int32_t));
    if (e == hipSuccess) e = hipMemcpy(ids.p, ids_host, n * sizeof(int32_t), hipMemcpyHostToDevice);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(copy_blocks_kernel, dim3((unsigned)((n * 32 + 255) / 256)), dim3(256), 0, 0, vals, (const int32_t *)ids.p, (long)n, out);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipDeviceSynchronize(); // ids goes out of scope
    return e;
}

hipError_t compact_build(const uint16_t *vals, const int32_t *row_ptr, const int32_t *col_idx,
                         const int32_t *row_ptr_host, size_t mb, size_t nnzb, size_t n_cap, double dense_share,
                         std::vector<uint8_t> *dense_rows, CompactPlan **out, const uint8_t *skip_blocks_host,
                         std::vector<uint8_t> *block_cols)
{
    *out = nullptr;
    CompactPlan *p = new (std::nothrow) CompactPlan();
    if (!p) return hipErrorOutOfMemory;
    hipError_t e = hipSuccess;
    Scratch mask, count, offset, tmp, cc;
#define SMAT_STEP(call)                                                                            \
    do {                                                                                           \
        if (e == hipSuccess) e = (call);                                                           \
    } while (0)
    SMAT_STEP(mask.alloc(nnzb * 2));
    SMAT_STEP(count.alloc(nnzb * 4));
    SMAT_STEP(offset.alloc(nnzb * 4));
    SMAT_STEP(cc.alloc((mb + 1) * 4));
    int64_t n_cols = 0;
    std::vector<int32_t> raw(mb + 1, 0), padded(mb + 1, 0);
    if (e == hipSuccess && nnzb) {
        const long waves = std::min<long>((long)(nnzb + 1) / 2, 256L * 32);
        hipLaunchKernelGGL(colmask_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, 0, vals, (long)nnzb,
                           (uint16_t *)mask.p, (int32_t *)count.p);
        e = hipGetLastError();
        if (block_cols) { // nonzero columns of every block, for the caller's choice of a split
            std::vector<int32_t> cnt(nnzb);
            SMAT_STEP(hipMemcpy(cnt.data(), count.p, nnzb * 4, hipMemcpyDeviceToHost));
            block_cols->resize(nnzb);
            for (size_t i = 0; i < nnzb; i++) (*block_cols)[i] = (uint8_t)cnt[i];
        }
        if (skip_blocks_host && e == hipSuccess) {
            Scratch skip;
            SMAT_STEP(skip.alloc(nnzb));
            SMAT_STEP(hipMemcpy(skip.p, skip_blocks_host, nnzb, hipMemcpyHostToDevice));
            if (e == hipSuccess) {
                hipLaunchKernelGGL(drop_blocks_kernel, dim3((unsigned)((nnzb + 255) / 256)), dim3(256), 0, 0, (const uint8_t *)skip.p,
                                   (long)nnzb, (uint16_t *)mask.p, (int32_t *)count.p);
                e = hipGetLastError();
            }
            SMAT_STEP(hipDeviceSynchronize()); // skip goes out of scope
        }
        size_t bytes = 0;
        SMAT_STEP(hipcub::DeviceScan::ExclusiveSum(nullptr, bytes, (int32_t *)count.p, (int32_t *)offset.p, (int)nnzb));
        SMAT_STEP(tmp.alloc(bytes));
        SMAT_STEP(hipcub::DeviceScan::ExclusiveSum(tmp.p, bytes, (int32_t *)count.p, (int32_t *)offset.p, (int)nnzb));
        if (e == hipSuccess) {
            hipLaunchKernelGGL(row_offsets_kernel, dim3((unsigned)((mb + 1 + 255) / 256)), dim3(256), 0, 0, row_ptr,
                               (const int32_t *)offset.p, (const int32_t *)count.p, (long)mb, (long)nnzb, (int32_t *)cc.p);
            e = hipGetLastError();
        }
        SMAT_STEP(hipMemcpy(raw.data(), cc.p, (mb + 1) * 4, hipMemcpyDeviceToHost));
        n_cols = raw[mb];
    }
    // Block rows whose blocks are mostly full (at least dense_share of their 16 x blocks columns are nonzero) are
    // left to a dense kernel when the caller asks for the split: they get no list and no work item here.
    std::vector<uint8_t> dense(mb, 0);
    p->n_cols_all = n_cols;
    if (dense_rows && dense_share > 0.0)
        for (size_t i = 0; i < mb; i++) {
            const int64_t blocks = row_ptr_host[i + 1] - row_ptr_host[i];
            if (blocks > 0 && (double)(raw[i + 1] - raw[i]) >= dense_share * 16.0 * (double)blocks) {
                dense[i] = 1;
                n_cols -= raw[i + 1] - raw[i];
            }
        }
    p->n_cols = n_cols;
    // every block row is padded to a multiple of 32 columns (one MFMA step); padding = zero columns
    int64_t total = 0;
    std::vector<int32_t> padded_dev(mb + 1, 0); // what the gather kernel sees: -1 for rows without a list
    for (size_t i = 0; i < mb; i++) {
        padded[i] = (int32_t)total;
        padded_dev[i] = dense[i] ? -1 : (int32_t)total;
        if (!dense[i]) total += ((int64_t)(raw[i + 1] - raw[i]) + 31) / 32 * 32;
        if (total > 0x7fffff00) e = hipErrorInvalidValue;
    }
    padded[mb] = (int32_t)total;
    padded_dev[mb] = (int32_t)total;
    const size_t cap = (size_t)total + LIST_PAD;
    SMAT_STEP(dev_malloc(&p->d_cols, cap * sizeof(int32_t)));
    SMAT_STEP(hipMemset(p->d_cols, 0, cap * sizeof(int32_t))); // padding: row 0 of B
    SMAT_STEP(dev_malloc(&p->d_acol, cap * 16 * sizeof(uint16_t)));
    SMAT_STEP(hipMemset(p->d_acol, 0, cap * 16 * sizeof(uint16_t)));
    if (e == hipSuccess && nnzb) {
        SMAT_STEP(hipMemcpy(cc.p, padded_dev.data(), (mb + 1) * 4, hipMemcpyHostToDevice));
        if (e == hipSuccess) {
            hipLaunchKernelGGL(gather_kernel, dim3((unsigned)((nnzb + 255) / 256)), dim3(256), 0, 0, vals,
                               (const uint16_t *)mask.p, (const int32_t *)offset.p, row_ptr, col_idx,
                               (const int32_t *)cc.p, (long)mb, (long)nnzb, p->d_cols, p->d_acol);
            e = hipGetLastError();
        }
    }
    // work items: whole block rows; rows much longer than the average in chunks of 32-column steps
    const std::vector<int32_t> &cc_host = padded;
    size_t nonempty = 0;
    for (size_t i = 0; i < mb; i++) nonempty += cc_host[i + 1] > cc_host[i];
    const double avg = nonempty ? (double)total / (double)nonempty : 0.0;
    long chunk = (long)(4.0 * avg + 0.5);
    chunk = std::max(chunk, 512L);
    chunk = (chunk + 31) / 32 * 32;
    std::vector<WorkItem> items;
    std::vector<SplitRow> split;
    int slot = 0;
    for (size_t i = 0; i < mb; i++) {
        const long len = cc_host[i + 1] - cc_host[i];
        if (len <= chunk || dense[i]) continue;
        SplitRow sr{(int32_t)i, slot, slot, 0};
        for (long b = cc_host[i]; b < cc_host[i + 1]; b += chunk)
            items.push_back(WorkItem{(int32_t)i, (int32_t)b, (int32_t)std::min<long>(b + chunk, cc_host[i + 1]), slot++});
        sr.slot_end = slot;
        split.push_back(sr);
    }
    for (size_t i = 0; i < mb; i++) {
        const long len = cc_host[i + 1] - cc_host[i];
        if (len > chunk || dense[i]) continue;
        items.push_back(WorkItem{(int32_t)i, cc_host[i], cc_host[i + 1], -1});
    }
    if (dense_rows) *dense_rows = dense;
    // what an item costs, for the deal of the items to the XCDs: its steps, and two more for fetching the item, the
    // first indices and the stores of its tile
    std::vector<uint64_t> cost_prefix(items.size() + 1, 0);
    for (size_t i = 0; i < items.size(); i++)
        cost_prefix[i + 1] = cost_prefix[i] + (uint64_t)((items[i].end - items[i].begin + 31) / 32) + 2;
    p->deal.set_costs(std::move(cost_prefix));
    p->n_items = (int)items.size();
    p->n_split_rows = (int)split.size();
    p->n_slots = slot;
    SMAT_STEP(dev_malloc(&p->d_items, std::max<size_t>(items.size(), 1) * sizeof(WorkItem)));
    if (!items.empty()) SMAT_STEP(hipMemcpy(p->d_items, items.data(), items.size() * sizeof(WorkItem), hipMemcpyHostToDevice));
    if (!split.empty()) {
        SMAT_STEP(dev_malloc(&p->d_split, split.size() * sizeof(SplitRow)));
        SMAT_STEP(hipMemcpy(p->d_split, split.data(), split.size() * sizeof(SplitRow), hipMemcpyHostToDevice));
        SMAT_STEP(dev_malloc(&p->d_workspace, (size_t)slot * 16 * n_cap * sizeof(float)));
    }
    SMAT_STEP(values_checksum(vals, nnzb, &p->values_checksum));
    SMAT_STEP(hipDeviceSynchronize());
#undef SMAT_STEP
    if (e != hipSuccess) {
        compact_destroy(p);
        return e;
    }
    *out = p;
    return hipSuccess;
}

} // namespace smat

// Test hook (not part of smat.h): 1 or 2 = the compact kernel works on panels of 64 or 128 columns whatever the sizes
// say (each width has its own way of gathering the rows of B), 0 = the launcher decides (the default).
extern "C" void smat_internal_compact_panel(int tq) { smat::g_force_tq = tq; }
// Test hooks for the deal of the compact kernel's workgroups to the XCDs: a run length that every launch uses
// (0 = chosen per plan and number of panels), the run length of the latest launch, and the choice itself for a list
// of item costs (host only).
extern "C" void smat_internal_compact_run(int run) { smat::g_force_run = run; }
extern "C" int smat_internal_compact_last_run(void) { return smat::g_last_run; }
extern "C" void smat_internal_compact_tune(int on) { smat::g_tune = on; }
extern "C" unsigned smat_internal_choose_xcd_run(const uint64_t *cost_prefix, uint64_t n_items, int n_panels)
{
    return smat::choose_xcd_run(cost_prefix, n_items, n_panels);
}
