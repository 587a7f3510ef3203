// Block-sparse SpMM kernels for gfx950 (MI355X): C = A_bcsr(16x16, fp16) * B(fp16),
// fp32 accumulation on v_mfma_f32_16x16x32_f16.
//
// Replaces the reference's live kernel mmaCBTKernelSparse and its launcher
// (src/cuda_hgemm/src/mma/mmaCBT.cu:13-88).  Same operands and semantics
// (absolute col_idx, column-major B, row-major C overwritten), different
// machine mapping:
//
//  * The product is formed transposed, C^T = B^T * A^T, so that a lane ends up
//    owning runs of consecutive C columns of one C row (wide stores) and both
//    MFMA operands are 16-byte, k-contiguous loads: B^T rows are the columns of
//    the column-major B, A^T columns are the rows of a row-major 16x16 block.
//  * One MFMA consumes two nonzero blocks of the same block row (K = 32 = 2x16):
//    lanes 0-31 feed block p, lanes 32-63 feed block p+1; a pair of blocks is one
//    contiguous, fully coalesced 1 KiB load.
//  * Work is a list of (block row, block range) items; block rows longer than
//    the chunk size are split and their fp32 partial tiles are summed in a fixed
//    order by a second kernel, so results do not depend on scheduling.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "spmm_kernels.h"

#define SMAT_ORDER_FENCE()                      \
    do {                                        \
        asm volatile("" ::: "memory");          \
        __builtin_amdgcn_sched_barrier(0);      \
    } while (0)

namespace smat {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f16x8 load_f16x8(const uint16_t *p)
{
    return *reinterpret_cast<const f16x8 *>(p);
}

__device__ __forceinline__ f16x8 zero_f16x8()
{
    f16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    return z;
}

// Column of C owned by MFMA output row i (0..15) of n-tile t inside a wave's
// panel.  Tiles are taken in groups of TG = min(TN, 4); inside a group the
// assignment interleaves tiles so that the 4*TG values a lane holds for one C
// row are consecutive columns.
template <int TN>
__device__ __forceinline__ int ncol_of(int t, int i)
{
    constexpr int TG = TN < 4 ? TN : 4;
    return 16 * TG * (t / TG) + 4 * TG * (i >> 2) + 4 * (t % TG) + (i & 3);
}

// One wavefront per work item x N panel.  blockDim = 256 (4 wavefronts).
//   items == nullptr : item w is the whole block row w (no work list)
//   items != nullptr : items[w] = {block row, first block, end block, dst}
//                      dst < 0  -> write the finished tile to C
//                      dst >= 0 -> write the fp32 partial tile to workspace slot dst
// Item index runs fastest inside a panel, so the four wavefronts of a workgroup
// and neighbouring workgroups share one B panel (K x 16*TN) in L2.  Workgroup
// ids are dealt round-robin to the 8 XCDs by the dispatcher; the remap below
// gives the XCDs runs of xcd_run consecutive workgroups of the (panel-major) item
// space in turn: an eighth of the launch each, so that an XCD's private L2 holds few
// distinct B panels, or shorter runs where the items' cost changes along the list
// (gridDim.x is a multiple of 8 * xcd_run).
// amdgpu_waves_per_eu(1, 4): at most 4 wavefronts per SIMD are asked for, which leaves the
// compiler 128 registers; with the default target of 8 it squeezes the kernel into 64 and
// gets there by loading each operand right before its MFMA, one memory latency apiece.
//
// PACKED: B is the slab-major copy made by pack_b_kernel, Bp[(bc/16 * N + n) * 16 + k % 16]:
// the 16 x 16 operand of one (block column, n-tile) is 512 contiguous bytes and a
// wavefront load touches 8 full cache lines instead of 32 quarter-used ones.
template <int TN, bool C_F32, bool PACKED>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 4))) void spmm_rowwise_kernel(
    const uint16_t *__restrict__ vals, const int32_t *__restrict__ row_ptr,
    const int32_t *__restrict__ col_idx, const uint16_t *__restrict__ B, void *__restrict__ Cout,
    float *__restrict__ workspace, const WorkItem *__restrict__ items, int n_items, int N, long K,
    int n_panels, unsigned xcd_run)
{
    constexpr int TG = TN < 4 ? TN : 4;
    constexpr int PANEL = 16 * TN;
    const int lane = threadIdx.x & 63;
    // wavefront-uniform values are forced into scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    const long total = (long)n_items * n_panels;
    const unsigned slot = blockIdx.x >> 3;
    const unsigned run = __builtin_amdgcn_readfirstlane(slot / xcd_run);
    const long wg = ((long)run * 8 + (blockIdx.x & 7)) * xcd_run + (slot - run * xcd_run);
    const long w = wg * 4 + wave;
    if (w >= total) return;
    const int panel = (int)(w / n_items);
    const int it = (int)(w - (long)panel * n_items);

    int br, p0, p1, dst;
    if (items) {
        WorkItem wi = items[it];
        br = wi.block_row; p0 = wi.begin; p1 = wi.end; dst = wi.dst;
    } else {
        br = it; p0 = row_ptr[it]; p1 = row_ptr[it + 1]; dst = -1;
    }
    br = __builtin_amdgcn_readfirstlane(br);
    p0 = __builtin_amdgcn_readfirstlane(p0);
    p1 = __builtin_amdgcn_readfirstlane(p1);
    dst = __builtin_amdgcn_readfirstlane(dst);

    const int i16 = lane & 15; // A row m / B^T row (n within tile)
    const int g = lane >> 4;   // k group 0..3
    const int sel = g >> 1;    // which block of the pair
    const int kh = g & 1;      // which half (8 k) of the block
    const int n0 = panel * PANEL;

    f32x4 acc[TN];
    long boff[TN];
#pragma unroll
    for (int t = 0; t < TN; t++) {
        acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
        // columns past N read column 0 instead: what they produce is never stored
        const int n = n0 + ncol_of<TN>(t, i16);
        boff[t] = PACKED ? (long)(n < N ? n : 0) * 16 + kh * 8 : (long)(n < N ? n : 0) * K + kh * 8;
    }
    const uint16_t *abase = vals + i16 * 16 + kh * 8;
    const f16x8 zero8 = zero_f16x8();

    // Every load below is unconditional (indices are clamped instead of branching): loads
    // inside branches cannot be counted by the compiler's vmcnt bookkeeping, which then
    // waits for everything in flight and serialises load and MFMA phases.
    // Two register sets: the operands of pair j+1 are in flight while pair j is multiplied.
    for (int pb = p0; pb < p1; pb += 64) {
        const int cnt = (p1 - pb) < 64 ? (p1 - pb) : 64;
        const int npair = (cnt + 1) >> 1;
        // one coalesced load of up to 64 column indices, then lane broadcasts
        const int myc = col_idx[pb + (lane < cnt ? lane : cnt - 1)];

        auto issue = [&](int j, f16x8 &a, f16x8 (&b)[TN]) {
            const int jj = j < npair ? j : npair - 1; // past the end: reload the last pair (unused)
            const int second = (2 * jj + 1 < cnt) ? 2 * jj + 1 : 2 * jj; // a single block pairs with itself
            const int c0 = __builtin_amdgcn_readlane(myc, 2 * jj);
            const int c1 = __builtin_amdgcn_readlane(myc, second);
            const int bc = sel ? c1 : c0;
            const long pp = (long)pb + (sel ? second : 2 * jj);
            a = load_f16x8(abase + pp * 256);
            // column-major: + first column of the block; packed: + slab of the block column
            const long boffs = PACKED ? (long)bc * N : (long)bc;
#pragma unroll
            for (int t = 0; t < TN; t++) b[t] = load_f16x8(B + boff[t] + boffs);
        };
        auto multiply = [&](int j, f16x8 a, const f16x8 (&b)[TN]) {
            if (2 * j + 1 >= cnt) a = sel ? zero8 : a; // single block: the upper K half contributes nothing
#pragma unroll
            for (int t = 0; t < TN; t++)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[t], a, acc[t], 0, 0, 0);
        };

        // The main loop multiplies two pairs per trip with no branch around either of them:
        // a multiply inside a branch drags its loads into the branch with it (they sink to
        // their only use) and the prefetch distance collapses.  The fences pin the issue
        // order against the scheduler.
        f16x8 a0, a1, b0[TN], b1[TN];
        issue(0, a0, b0);
        SMAT_ORDER_FENCE();
        int j = 0;
        for (; j + 2 <= npair; j += 2) {
            issue(j + 1, a1, b1);
            SMAT_ORDER_FENCE();
            multiply(j, a0, b0);
            SMAT_ORDER_FENCE();
            issue(j + 2, a0, b0); // past the end this reloads the last pair, unused
            SMAT_ORDER_FENCE();
            multiply(j + 1, a1, b1);
            SMAT_ORDER_FENCE();
        }
        if (j < npair) multiply(j, a0, b0); // odd number of pairs: the last one is already in set 0
    }

    // Epilogue.  acc[t][r] = C[br*16 + i16][n0 + ncol_of(t, 4*g + r)].
    const long m = (long)br * 16 + i16;
#pragma unroll
    for (int u = 0; u < TN / TG; u++) {
        const int nbase = n0 + 16 * TG * u + 4 * TG * g; // first of 4*TG consecutive columns
        if (dst >= 0) {
            // fp32 partial tile: slot-major, then the same row-major M x N addressing
            float *wrow = workspace + ((long)dst * 16 + i16) * (long)N;
#pragma unroll
            for (int tt = 0; tt < TG; tt++) {
                int n = nbase + 4 * tt;
                if (n < N) *reinterpret_cast<f32x4 *>(wrow + n) = acc[u * TG + tt];
            }
        } else if (C_F32) {
            float *crow = reinterpret_cast<float *>(Cout) + m * (long)N;
#pragma unroll
            for (int tt = 0; tt < TG; tt++) {
                int n = nbase + 4 * tt;
                if (n < N) *reinterpret_cast<f32x4 *>(crow + n) = acc[u * TG + tt];
            }
        } else {
            uint16_t *crow = reinterpret_cast<uint16_t *>(Cout) + m * (long)N;
            if constexpr (TG == 1) {
                f32x4 v = acc[u];
                f16x4 h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
                if (nbase < N) *reinterpret_cast<f16x4 *>(crow + nbase) = h;
            } else {
#pragma unroll
                for (int tt = 0; tt < TG; tt += 2) {
                    f32x4 v0 = acc[u * TG + tt], v1 = acc[u * TG + tt + 1];
                    f16x8 h = {(_Float16)v0[0], (_Float16)v0[1], (_Float16)v0[2], (_Float16)v0[3],
                               (_Float16)v1[0], (_Float16)v1[1], (_Float16)v1[2], (_Float16)v1[3]};
                    int n = nbase + 4 * tt;
                    if (n < N) *reinterpret_cast<f16x8 *>(crow + n) = h;
                }
            }
        }
    }
}

// Small problems with short block rows (a band matrix: 9 blocks per row, 256 rows): the kernel above keeps the
// operands of two block pairs in flight, so a row of five pairs costs four memory latencies one after the other
// and the launch is over before the chip is busy.  Here a wavefront asks for the operands of all its pairs
// (at most NP) at once: work item -> column indices -> operands, three latencies, then NP x TN MFMAs (pairs past
// the end of the row multiply zeros).  Whole block rows only (dst < 0), B in place.
template <int TN, bool C_F32, int NP>
__global__ __launch_bounds__(256) void spmm_rowwise_short_kernel(
    const uint16_t *__restrict__ vals, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col_idx,
    const uint16_t *__restrict__ B, void *__restrict__ Cout, const WorkItem *__restrict__ items, int n_items, int N,
    long K, int n_panels)
{
    static_assert(TN == 2 || TN == 4, "panels of 32 or 64 columns");
    constexpr int PANEL = 16 * TN;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const long w = (long)blockIdx.x * 4 + wave;
    if (w >= (long)n_items * n_panels) return;
    const int panel = (int)(w / n_items);
    const int it = (int)(w - (long)panel * n_items);
    int br, p0, p1;
    if (items) {
        const WorkItem wi = items[it];
        br = wi.block_row; p0 = wi.begin; p1 = wi.end;
    } else {
        br = it; p0 = row_ptr[it]; p1 = row_ptr[it + 1];
    }
    br = __builtin_amdgcn_readfirstlane(br);
    p0 = __builtin_amdgcn_readfirstlane(p0);
    p1 = __builtin_amdgcn_readfirstlane(p1);
    const int cnt = p1 - p0; // <= 2 * NP: the launcher has checked the work list
    const int npair = (cnt + 1) >> 1;

    const int i16 = lane & 15, g = lane >> 4, sel = g >> 1, kh = g & 1;
    const int n0 = panel * PANEL;
    f32x4 acc[TN];
#pragma unroll
    for (int t = 0; t < TN; t++) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (cnt > 0) { // uniform over the wavefront
        long boff[TN];
#pragma unroll
        for (int t = 0; t < TN; t++) {
            const int n = n0 + ncol_of<TN>(t, i16);
            boff[t] = (long)(n < N ? n : 0) * K + kh * 8; // columns past N read column 0: never stored
        }
        const uint16_t *abase = vals + i16 * 16 + kh * 8;
        const f16x8 zero8 = zero_f16x8();
        const int myc = col_idx[p0 + (lane < cnt ? lane : cnt - 1)];
        f16x8 a[NP], b[NP][TN];
#pragma unroll
        for (int j = 0; j < NP; j++) {
            const int jj = j < npair ? j : npair - 1; // past the end: the last pair again, multiplied by zeros below
            const int second = (2 * jj + 1 < cnt) ? 2 * jj + 1 : 2 * jj; // a single block pairs with itself
            const int c0 = __builtin_amdgcn_readlane(myc, 2 * jj);
            const int c1 = __builtin_amdgcn_readlane(myc, second);
            const long pp = (long)p0 + (sel ? second : 2 * jj);
            a[j] = load_f16x8(abase + pp * 256);
            const long bc = sel ? c1 : c0;
#pragma unroll
            for (int t = 0; t < TN; t++) b[j][t] = load_f16x8(B + boff[t] + bc);
        }
        SMAT_ORDER_FENCE();
#pragma unroll
        for (int j = 0; j < NP; j++) {
            f16x8 aj = a[j];
            if (j >= npair) aj = zero8;
            else if (2 * j + 1 >= cnt) aj = sel ? zero8 : aj; // single block: the upper K half contributes nothing
#pragma unroll
            for (int t = 0; t < TN; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[j][t], aj, acc[t], 0, 0, 0);
        }
    }
    // acc[t][r] = C[br*16 + i16][n0 + ncol_of(t, 4*g + r)]: 4*TN consecutive columns per lane, as in the kernel above
    const long m = (long)br * 16 + i16;
    const int nbase = n0 + 4 * TN * g;
    if (C_F32) {
        float *crow = reinterpret_cast<float *>(Cout) + m * (long)N;
#pragma unroll
        for (int t = 0; t < TN; t++)
            if (nbase + 4 * t < N) *reinterpret_cast<f32x4 *>(crow + nbase + 4 * t) = acc[t];
    } else {
        uint16_t *crow = reinterpret_cast<uint16_t *>(Cout) + m * (long)N;
#pragma unroll
        for (int t = 0; t < TN; t += 2) {
            const f32x4 v0 = acc[t], v1 = acc[t + 1];
            const f16x8 h = {(_Float16)v0[0], (_Float16)v0[1], (_Float16)v0[2], (_Float16)v0[3],
                             (_Float16)v1[0], (_Float16)v1[1], (_Float16)v1[2], (_Float16)v1[3]};
            if (nbase + 4 * t < N) *reinterpret_cast<f16x8 *>(crow + nbase + 4 * t) = h;
        }
    }
}

// Sums the fp32 partial tiles of every split block row in slot order and writes
// the finished rows to C.  One thread per 4 consecutive columns of one row.
template <bool C_F32>
__global__ __launch_bounds__(256) void spmm_reduce_kernel(const float *__restrict__ workspace,
                                                         const SplitRow *__restrict__ rows,
                                                         int n_rows, void *__restrict__ Cout, int N)
{
    const int quads = N >> 2; // N % 8 == 0
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long per_row = (long)16 * quads;
    if (tid >= per_row * n_rows) return;
    const int r = (int)(tid / per_row);
    const long rem = tid - (long)r * per_row;
    const int i = (int)(rem / quads);
    const int q = (int)(rem - (long)i * quads);
    const SplitRow sr = rows[r];
    // Four running sums, slot k into sum k % 4 (a fixed order: the result does not depend on the launch): the loads of
    // four slots are under way at a time instead of one, which is what a block row of many slots waits for.
    const float *base = workspace + (long)i * (long)N + 4 * q;
    const long slot_stride = 16L * (long)N;
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0, s2 = s0, s3 = s0;
    int slot = sr.slot_begin;
    for (; slot + 4 <= sr.slot_end; slot += 4) {
        const f32x4 v0 = *reinterpret_cast<const f32x4 *>(base + (long)slot * slot_stride);
        const f32x4 v1 = *reinterpret_cast<const f32x4 *>(base + (long)(slot + 1) * slot_stride);
        const f32x4 v2 = *reinterpret_cast<const f32x4 *>(base + (long)(slot + 2) * slot_stride);
        const f32x4 v3 = *reinterpret_cast<const f32x4 *>(base + (long)(slot + 3) * slot_stride);
        s0 += v0; s1 += v1; s2 += v2; s3 += v3;
    }
    if (slot < sr.slot_end) s0 += *reinterpret_cast<const f32x4 *>(base + (long)slot * slot_stride);
    if (slot + 1 < sr.slot_end) s1 += *reinterpret_cast<const f32x4 *>(base + (long)(slot + 1) * slot_stride);
    if (slot + 2 < sr.slot_end) s2 += *reinterpret_cast<const f32x4 *>(base + (long)(slot + 2) * slot_stride);
    const f32x4 s = (s0 + s1) + (s2 + s3);
    const long m = (long)sr.block_row * 16 + i;
    if (C_F32) {
        *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(Cout) + m * (long)N + 4 * q) = s;
    } else {
        f16x4 h = {(_Float16)s[0], (_Float16)s[1], (_Float16)s[2], (_Float16)s[3]};
        *reinterpret_cast<f16x4 *>(reinterpret_cast<uint16_t *>(Cout) + m * (long)N + 4 * q) = h;
    }
}

// Column-major B (B[n*K + k]) -> slab-major Bp[(k/16 * N + n) * 16 + k % 16].
// One workgroup moves a tile of 64 n x 64 k through LDS: reads are 128-byte runs along k,
// writes are 2 KiB runs (64 n x 32 B) per block column.
__global__ __launch_bounds__(256) void pack_b_kernel(const uint16_t *__restrict__ B,
                                                     uint16_t *__restrict__ Bp, int N, long K)
{
    __shared__ __align__(16) unsigned char tile[8192];
    const int t = threadIdx.x;
    const long k0 = (long)blockIdx.x * 64;
    const int n0 = blockIdx.y * 64;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int idx = i * 256 + t;
        const int nl = idx >> 3, seg = idx & 7; // seg: 8 k (16 bytes) along k
        f16x8 v = zero_f16x8();
        if (n0 + nl < N && k0 + seg * 8 < K) v = load_f16x8(B + (long)(n0 + nl) * K + k0 + seg * 8);
        *reinterpret_cast<f16x8 *>(tile + ((seg >> 1) * 64 + nl) * 32 + (seg & 1) * 16) = v;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int idx = i * 256 + t;
        const int bcl = idx >> 7, nl = (idx & 127) >> 1, half = idx & 1;
        if (n0 + nl < N && k0 + bcl * 16 < K)
            *reinterpret_cast<f16x8 *>(Bp + ((k0 / 16 + bcl) * N + n0 + nl) * 16 + half * 8) =
                *reinterpret_cast<const f16x8 *>(tile + (size_t)idx * 16);
    }
}

template <int TN>
static hipError_t launch_rowwise_tn(const SpmmArgs &a, hipStream_t st)
{
    const int panel = 16 * TN;
    const int n_panels = (int)((a.N + panel - 1) / panel);
    const long total = (long)a.n_items * n_panels;
    long wgs = (total + 3) / 4;
    if (wgs == 0) return hipSuccess;
    const long xcd_run = a.deal && a.items ? (long)a.deal->run((size_t)a.n_items, n_panels) : (wgs + 7) / 8;
    wgs = (wgs + 8 * xcd_run - 1) / (8 * xcd_run) * (8 * xcd_run);
    if (wgs > 0x7fffffffL) return hipErrorInvalidValue;
    dim3 grid((unsigned)wgs), block(256);
#define SMAT_LAUNCH_ROWWISE(F32, PK)                                                              \
    hipLaunchKernelGGL((spmm_rowwise_kernel<TN, F32, PK>), grid, block, 0, st, a.vals, a.row_ptr, \
                       a.col_idx, a.b_packed ? a.b_packed : a.B, a.C, a.workspace, a.items,       \
                       a.n_items, (int)a.N, (long)a.K, n_panels, (unsigned)xcd_run)
    if (a.b_packed) {
        if (a.c_f32) SMAT_LAUNCH_ROWWISE(true, true);
        else SMAT_LAUNCH_ROWWISE(false, true);
    } else {
        if (a.c_f32) SMAT_LAUNCH_ROWWISE(true, false);
        else SMAT_LAUNCH_ROWWISE(false, false);
    }
#undef SMAT_LAUNCH_ROWWISE
    return hipGetLastError();
}

unsigned choose_xcd_run(const uint64_t *P, uint64_t n, int n_panels)
{
    const uint64_t total = n * (uint64_t)n_panels;
    const uint64_t wgs = (total + 3) / 4;
    const uint64_t eighth = std::max<uint64_t>((wgs + 7) / 8, 1);
    if (n == 0 || P[n] == 0) return (unsigned)eighth;
    auto cost_before = [&](uint64_t wg) { // of the workgroups before wg in the panel-major item space
        const uint64_t w = std::min(wg * 4, total);
        return (w / n) * P[n] + P[w % n];
    };
    uint64_t best_run = eighth;
    double best = 1e30;
    for (uint64_t run : {eighth, (uint64_t)1024, (uint64_t)256, (uint64_t)64, (uint64_t)16, (uint64_t)4}) {
        if (run > eighth || (run == eighth && best < 1e30)) continue;
        if (wgs / run > ((uint64_t)1 << 26)) break; // a launch this large is not walked run by run on the host
        uint64_t load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (uint64_t first = 0, x = 0; first < wgs; first += run, x = (x + 1) & 7)
            load[x] += cost_before(first + run) - cost_before(first);
        const uint64_t busiest = *std::max_element(load, load + 8);
        const double ratio = (double)busiest * 8.0 / (double)std::max<uint64_t>(cost_before(wgs), 1);
        if (ratio < best) best = ratio, best_run = run;
        if (ratio <= 1.04) break;
    }
    return (unsigned)best_run;
}

void XcdDeal::set_costs(std::vector<uint64_t> &&prefix)
{
    std::lock_guard<std::mutex> lock(mutex_);
    cost_prefix_ = std::move(prefix);
    known_.clear();
}

unsigned XcdDeal::run(size_t n_items, int n_panels) const
{
    const uint64_t n = n_items;
    std::lock_guard<std::mutex> lock(mutex_);
    if (n == 0 || cost_prefix_.size() != n + 1) // no costs for this list: an eighth of the launch each
        return (unsigned)std::max<uint64_t>(((n * (uint64_t)n_panels + 3) / 4 + 7) / 8, 1);
    for (const auto &k : known_)
        if (k.first == n_panels) return k.second;
    const unsigned r = choose_xcd_run(cost_prefix_.data(), n, n_panels);
    known_.emplace_back(n_panels, r);
    return r;
}

int rowwise_panel_tiles(size_t N, int requested, size_t n_items)
{
    if (requested == 1 || requested == 2 || requested == 4 || requested == 8 || requested == 16) return requested;
    if (N >= 1024) return 16; // 256 columns per wavefront: every A block is read once per 256 columns of C
    if (N >= 512) return 8;
    // Below that, 64-column panels: measured faster than 128-column ones even where the work
    // list alone fills the chip (R-MAT scale 20, N = 128: 13.8 ms against 18.2 ms), more
    // wavefronts in flight outweighing the second pass over A.
    (void)n_items;
    if (N >= 64) return 4;
    if (N >= 32) return 2;
    return 1;
}

// The short-row kernel: rows of at most 2 * SHORT_NP blocks, no split rows, B in place, few wavefronts.
constexpr int SHORT_NP = 5;
constexpr long SHORT_MAX_WAVES = 8192;

template <int TN>
static hipError_t launch_rowwise_short(const SpmmArgs &a, hipStream_t st)
{
    const int n_panels = (int)((a.N + 16 * TN - 1) / (16 * TN));
    const long total = (long)a.n_items * n_panels;
    if (total == 0) return hipSuccess;
    dim3 grid((unsigned)((total + 3) / 4)), block(256);
    if (a.c_f32)
        hipLaunchKernelGGL((spmm_rowwise_short_kernel<TN, true, SHORT_NP>), grid, block, 0, st, a.vals, a.row_ptr, a.col_idx,
                           a.B, a.C, a.items, a.n_items, (int)a.N, (long)a.K, n_panels);
    else
        hipLaunchKernelGGL((spmm_rowwise_short_kernel<TN, false, SHORT_NP>), grid, block, 0, st, a.vals, a.row_ptr, a.col_idx,
                           a.B, a.C, a.items, a.n_items, (int)a.N, (long)a.K, n_panels);
    return hipGetLastError();
}

hipError_t launch_rowwise(const SpmmArgs &a, hipStream_t st)
{
    hipError_t e;
    if (!a.b_packed && a.n_split_rows == 0 && a.max_item_blocks > 0 && a.max_item_blocks <= 2 * SHORT_NP && a.N >= 32 &&
        (long)a.n_items * (long)((a.N + 31) / 32) <= SHORT_MAX_WAVES) {
        // 32-column panels while that still leaves the chip short of wavefronts, else 64
        const bool narrow = (long)a.n_items * (long)((a.N + 63) / 64) < 2048;
        return narrow ? launch_rowwise_short<2>(a, st) : launch_rowwise_short<4>(a, st);
    }
    if (a.b_packed) {
        dim3 grid((unsigned)((a.K + 63) / 64), (unsigned)((a.N + 63) / 64));
        hipLaunchKernelGGL(pack_b_kernel, grid, dim3(256), 0, st, a.B, a.b_packed, (int)a.N, (long)a.K);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    switch (rowwise_panel_tiles(a.N, a.panel_tiles, (size_t)a.n_items)) {
    case 16: e = launch_rowwise_tn<16>(a, st); break;
    case 8: e = launch_rowwise_tn<8>(a, st); break;
    case 4: e = launch_rowwise_tn<4>(a, st); break;
    case 2: e = launch_rowwise_tn<2>(a, st); break;
    default: e = launch_rowwise_tn<1>(a, st); break;
    }
    if (e != hipSuccess) return e;
    if (a.n_split_rows > 0) e = launch_reduce(a.workspace, a.split_rows, a.n_split_rows, a.C, a.N, a.c_f32, st);
    return e;
}

hipError_t launch_reduce(const float *workspace, const SplitRow *split_rows, int n_split_rows, void *C, size_t N,
                         bool c_f32, hipStream_t st)
{
    const long threads = (long)n_split_rows * 16 * (long)(N / 4);
    const long blocks = (threads + 255) / 256;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    if (c_f32)
        hipLaunchKernelGGL((spmm_reduce_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, st, workspace,
                           split_rows, n_split_rows, C, (int)N);
    else
        hipLaunchKernelGGL((spmm_reduce_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, st, workspace,
                           split_rows, n_split_rows, C, (int)N);
    return hipGetLastError();
}

} // namespace smat
