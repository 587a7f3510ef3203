// "Sweep" SpMM kernel for block matrices that are dense enough (a few percent of
// the 16x16 blocks present) and wide N: one workgroup owns a group of 32 block
// rows x 128 columns of C and sweeps over K in chunks of 16 block columns.
//
//  * The B panel of a chunk (256 k x 128 n, 64 KiB) is staged once per workgroup
//    in LDS and shared by all block rows of the group; global reads of it are
//    256-byte contiguous runs of the column-major B (B[n*K + k]), i.e. fully
//    used cache lines, instead of the 32-byte gathers a per-block read costs.
//  * LDS holds a chunk as [8-slab group][n][16 slots of 16 B]; a slot is 8
//    consecutive k of one n.  The slot index is XOR-ed with a 4-bit function of
//    n chosen so that the 16 lanes of one ds_read_b128 phase (which read 16
//    different n, same logical slot) hit 16 different 16-byte bank groups, and
//    the 16 lanes that fill one n write 256 contiguous bytes: no bank conflicts
//    on either side.
//  * Each wavefront owns 4 block rows (128 fp32 accumulator registers) and runs
//    a host-built table of MFMA ops with a fixed number of slots per block row
//    (so the accumulator registers of every slot are known at compile time):
//    pairs of blocks of one block row inside the chunk feed one
//    v_mfma_f32_16x16x32_f16 (K = 32 = 2 blocks).  A chunk whose ops do not fit
//    the table continues in a following record that reuses the resident B stage.
//    A operands are 512-byte coalesced global reads straight into MFMA layout.
//  * Software pipeline over chunks, everything for chunk c+1 is issued before the
//    MFMA work of chunk c starts and is only waited for after it: the A operands of
//    chunk c+1 (into a second set of registers) and the B panel of chunk c+1 (global
//    -> LDS asynchronously with global_load_lds_dwordx4, no staging registers, into
//    the other LDS stage).  The op table of chunk c+2 is requested right after the
//    MFMA work of chunk c, into the registers of the table just used.  The loop is
//    unrolled by two so that the two register sets swap roles without copies.  The
//    MFMA loop itself touches only registers and LDS.  One barrier per chunk.
//  * Vector memory instructions are the scarce resource of the load phase: the load
//    path of a CU takes about one 64-lane instruction (up to 1 KiB) per 16 clocks and
//    the issuing wavefront stalls meanwhile.  So the op tables are read with scalar
//    loads (64 bytes per record and wavefront), empty table slots load no A, and the
//    B copies move 16 bytes per lane from a scalar base plus a 32-bit lane offset.
//
// Same operand semantics as the reference launcher
// (src/cuda_hgemm/src/mma/mmaCBT.cu:83-88).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.h"

namespace smat {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int TN = SWEEP_TN, RW = SWEEP_RW, W = SWEEP_WAVES, S = SWEEP_S;
constexpr int NT = 16 * TN;                 // 128 columns per panel
constexpr int THREADS = 64 * W;             // 512
constexpr int OCTS = S / 8;                 // 8-slab groups per chunk
constexpr int ROW_BYTES = 256;              // 8 slabs x 16 k x 2 B per n
constexpr int STAGE_BYTES = OCTS * NT * ROW_BYTES; // 65536
constexpr int FILL_ITERS = STAGE_BYTES / 16 / THREADS; // 16-byte slots per thread per chunk: 8

// LDS slot swizzle: physical slot = logical slot ^ ((n & 3) | ((n >> 2) & 12)), n = column in the panel.

// Issues the asynchronous global -> LDS copies of one chunk of the B panel into
// `stage`.  One wave instruction moves 64 x 16 B = 1 KiB: four n-rows of 256 B.
// LDS destination = wave-uniform base + lane * 16 (hardware addressing of
// global_load_lds_dwordx4); the global source is per lane, so the XOR swizzle is
// applied on the source side.  Columns beyond N are skipped (their LDS rows only
// feed C columns that are never stored) and k is clamped into the matrix (slabs
// past K are referenced by no op).
__device__ __forceinline__ void fill_issue(unsigned char *stage, const uint16_t *__restrict__ B,
                                           int chunk, int n0, int N, long K, int wave, int lane)
{
    // Instruction `it` of wavefront `wave` covers rows (it*W + wave)*4 .. +3 of the
    // stage, i.e. slab group o = it/4 and n = (it%4)*32 + wave*4 + lane/16.
    static_assert(W == 8 && NT == 128 && FILL_ITERS == 8, "fill mapping assumes 8 waves x 128 columns");
    const int q = lane >> 4, ps = lane & 15;
    // swizzle_of_n(n) = q | bit4(n) << 2 | bit5(n) << 3 with bit4(n) = wave/4, bit5(n) = it & 1
    const int ls0 = ps ^ (q | (((wave >> 2) & 1) << 2));
    // Source address = wave-uniform base (column block of the instruction) + 32-bit lane
    // offset: the launcher checks that B is smaller than 4 GiB.
    const uint32_t kmax = (uint32_t)K - 8u;
    const uint32_t col_off = (uint32_t)(n0 + wave * 4 + q) * (uint32_t)K; // in elements
    const uint32_t k0 = (uint32_t)chunk * (S * 16);
#pragma unroll
    for (int it = 0; it < FILL_ITERS; it++) {
        const int nrow = n0 + (it & 3) * 32 + wave * 4; // first of 4 columns, wave-uniform
        if (nrow >= N) continue;                          // N % 8 == 0: all four or none
        const uint32_t ls = (uint32_t)(ls0 ^ ((it & 1) << 3));
        uint32_t k = k0 + (it >> 2) * 128 + ls * 8;
        k = k < kmax ? k : kmax; // slabs past K are never referenced; keep the read in bounds
        const uint32_t voff = (col_off + k) * 2u;
        const uint16_t *sbase = B + (long)((it & 3) * 32) * K;
        // Issued from inline assembly on purpose: the compiler orders every later LDS
        // read after a global->LDS copy it knows about (it cannot tell the two stages
        // apart) and would wait for the copy before the MFMA work of the current
        // chunk.  The copies are waited for explicitly (vmcnt(0)) before the barrier.
        const uint32_t dst = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)(
            stage + (size_t)(it * W + wave) * 1024);
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(voff), "s"(sbase), "s"(dst)
                     : "memory", "m0");
    }
}

} // namespace

typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));

// The op table of (record, wavefront): 8 slots of {w0, w1}.  Read through the constant
// address space with a wave-uniform address: one scalar load, no vector memory
// instruction and no v_readlane to get at a slot.
__device__ __forceinline__ u32x16 load_op_table(const SweepOp *__restrict__ ops, int record, int wave)
{
    static_assert(SWEEP_CAP * sizeof(SweepOp) == sizeof(u32x16), "one table = 16 dwords");
    typedef const __attribute__((address_space(4))) u32x16 *table_ptr;
    return *(table_ptr)(uintptr_t)(ops + ((long)record * W + wave) * SWEEP_CAP);
}

// LDS byte offset (without the per-lane XOR) of a slab of the staged chunk
__device__ __forceinline__ uint32_t slab_offset(uint32_t slab)
{
    return (slab >> 3) * (uint32_t)(NT * 256) + (slab & 7u) * 32u;
}

template <bool C_F32>
__global__ __launch_bounds__(THREADS) void spmm_sweep_kernel(
    const uint16_t *__restrict__ vals, const uint16_t *__restrict__ B, void *__restrict__ Cout,
    const int32_t *__restrict__ rg_chunk_ptr, const int32_t *__restrict__ chunk_ids,
    const SweepOp *__restrict__ ops, int Mb, int N, long K, int n_rg, int n_panels)
{
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr int CAP = SWEEP_CAP;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // panel-major work order, row group fastest; each XCD gets a contiguous eighth
    const int total = n_rg * n_panels;
    const int per_xcd = gridDim.x >> 3;
    const int wg = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (wg >= total) return;
    const int panel = wg / n_rg;
    const int rg = wg - panel * n_rg;
    const int n0 = panel * NT;

    const int i16 = lane & 15, g = lane >> 4, sel = g >> 1, kh = g & 1;
    // column (within the panel) of MFMA row i16 in tile 0; tile t adds 64*(t/4) + 4*(t%4).
    // The swizzle value of every such column equals i16.
    const int n_lane = 16 * (i16 >> 2) + (i16 & 3);
    const int rd_base = n_lane * ROW_BYTES;
    const uint32_t lane_xor = (uint32_t)((kh ^ i16) << 4); // ((2*slab | kh) ^ i16) << 4 == (slab * 32) ^ lane_xor

    f32x4 acc[RW][TN];
#pragma unroll
    for (int r = 0; r < RW; r++)
#pragma unroll
        for (int t = 0; t < TN; t++) acc[r][t] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int c_begin = rg_chunk_ptr[rg], c_end = rg_chunk_ptr[rg + 1];
    const uint32_t a_lane_bytes = (uint32_t)(i16 * 16 + kh * 8) * 2u; // this lane's 16 bytes inside a block
    const f16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // A operands of one chunk: slot k <- the two blocks of op k (lanes 0-31: first block,
    // 32-63: second).  Empty slots load nothing: a vector memory instruction costs the
    // load path of the CU 16 clocks whatever it fetches.  The missing second block of a
    // single re-reads the first (zeroed at use).
    auto load_a = [&](f16x8 (&dst)[CAP], const u32x16 &tab) {
        constexpr int CAPR = CAP / RW;
#pragma unroll
        for (int r = 0; r < RW; r++) {
#pragma unroll
            for (int j = 0; j < CAPR; j++) {
                const int k = r * CAPR + j;
                const uint32_t w0 = tab[2 * k], w1 = tab[2 * k + 1];
                if (w0 == SWEEP_EMPTY_SLOT) break; // the slots of a block row fill up in order
                const uint32_t b1 = (w0 & 0xFFFFFFu) * 512u; // nnzb < 2^23 is checked by the plan
                const uint32_t p2 = w1 & 0xFFFFFFu;
                const uint32_t b2 = p2 == SWEEP_NO_BLOCK ? b1 : p2 * 512u;
                const uint32_t off = (sel ? b2 : b1) + a_lane_bytes;
                dst[k] = *reinterpret_cast<const f16x8 *>(reinterpret_cast<const char *>(vals) + off);
            }
        }
    };

    // Two sets of op-table registers and of A operand registers; consecutive records use
    // them in swapped roles (the loop below is unrolled by two), so nothing is copied.
    u32x16 tab0, tab1;
#pragma unroll
    for (int k = 0; k < 16; k++) { tab0[k] = SWEEP_EMPTY_SLOT; tab1[k] = SWEEP_EMPTY_SLOT; }
    f16x8 a0[CAP], a1[CAP];
#pragma unroll
    for (int k = 0; k < CAP; k++) { a0[k] = zero8; a1[k] = zero8; }

    int stage = 0;
    const int last = c_end - 1;
    if (c_begin < c_end) {
        tab0 = load_op_table(ops, c_begin, wave);
        tab1 = load_op_table(ops, c_begin + 1 < last ? c_begin + 1 : last, wave);
        fill_issue(lds, B, chunk_ids[c_begin] & ~SWEEP_CONT_FLAG, n0, N, K, wave, lane);
        load_a(a0, tab0);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0): the copies of this wavefront have landed
    __syncthreads();

    // One record: tab_c / a_c hold the op table and A operands of record ci, tab_n the table of
    // record ci + 1, whose A operands go to a_n.
    auto record = [&](int ci, u32x16 &tab_c, const u32x16 &tab_n, f16x8 (&a_c)[CAP], f16x8 (&a_n)[CAP]) {
        // ---- everything record ci+1 needs ----
        bool next_is_new = false;
        if (ci + 1 < c_end) {
            load_a(a_n, tab_n);
            // A record that continues the chunk of the previous record (its ops did not
            // fit one table) has bit 30 set: no B copy, the LDS stage stays.
            const int next_chunk = chunk_ids[ci + 1];
            next_is_new = !(next_chunk & SWEEP_CONT_FLAG);
            if (next_is_new)
                fill_issue(lds + (stage ^ 1) * STAGE_BYTES, B, next_chunk, n0, N, K, wave, lane);
        }
        // ---- MFMA work of record ci: registers and LDS only ----
        const unsigned char *cur = lds + stage * STAGE_BYTES + rd_base;
#pragma unroll
        for (int r = 0; r < RW; r++) {
            // table slot k belongs to block row k / CAPR of this wavefront: the accumulator
            // registers of every slot are fixed at compile time
            constexpr int CAPR = CAP / RW;
#pragma unroll
            for (int j = 0; j < CAPR; j++) {
                const int k = r * CAPR + j;
                const uint32_t w0 = tab_c[2 * k], w1 = tab_c[2 * k + 1];
                if (w0 == SWEEP_EMPTY_SLOT) break; // the slots of a block row fill up in order
                const uint32_t soff = sel ? slab_offset(w1 >> 24) : slab_offset(w0 >> 24);
                const unsigned char *bp = cur + (soff ^ lane_xor);
                f16x8 av = a_c[k];
                if ((w1 & 0xFFFFFFu) == SWEEP_NO_BLOCK) // single: no second block
                    av = sel ? zero8 : av;
#pragma unroll
                for (int u = 0; u < TN / 4; u++) {
                    f16x8 b[4];
#pragma unroll
                    for (int tt = 0; tt < 4; tt++)
                        b[tt] = *reinterpret_cast<const f16x8 *>(bp + (64 * u + 4 * tt) * ROW_BYTES);
#pragma unroll
                    for (int tt = 0; tt < 4; tt++)
                        acc[r][u * 4 + tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            b[tt], av, acc[r][u * 4 + tt], 0, 0, 0);
                }
                // order of the 8 LDS reads and 8 MFMAs of this op: four reads ahead, then one
                // MFMA per further read, so an MFMA never waits on the read issued just before it
                __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
            }
        }
        // the table of record ci+2 replaces the one just used (a scalar load: it returns
        // while this wavefront waits for the copies and at the barrier)
        if (ci + 2 <= last) tab_c = load_op_table(ops, ci + 2, wave);
        __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0): next record's B and A have landed
        __syncthreads();
        if (next_is_new) stage ^= 1;
    };
    for (int ci = c_begin; ci < c_end; ci += 2) {
        record(ci, tab0, tab1, a0, a1);
        if (ci + 1 < c_end) record(ci + 1, tab1, tab0, a1, a0);
    }
    // Epilogue: acc[r][t][e] = C[(rg*G + wave*RW + r)*16 + i16][n0 + 64*(t/4) + 16*g + 4*(t%4) + e]
#pragma unroll
    for (int r = 0; r < RW; r++) {
        const int br = rg * SWEEP_G + wave * RW + r;
        if (br >= Mb) continue;
        const long m = (long)br * 16 + i16;
#pragma unroll
        for (int u = 0; u < TN / 4; u++) {
            const int nbase = n0 + 64 * u + 16 * g;
            if (C_F32) {
                float *crow = reinterpret_cast<float *>(Cout) + m * (long)N;
#pragma unroll
                for (int tt = 0; tt < 4; tt++)
                    if (nbase + 4 * tt < N)
                        *reinterpret_cast<f32x4 *>(crow + nbase + 4 * tt) = acc[r][u * 4 + tt];
            } else {
                uint16_t *crow = reinterpret_cast<uint16_t *>(Cout) + m * (long)N;
#pragma unroll
                for (int tt = 0; tt < 4; tt += 2) {
                    const f32x4 v0 = acc[r][u * 4 + tt], v1 = acc[r][u * 4 + tt + 1];
                    f16x8 h = {(_Float16)v0[0], (_Float16)v0[1], (_Float16)v0[2], (_Float16)v0[3],
                               (_Float16)v1[0], (_Float16)v1[1], (_Float16)v1[2], (_Float16)v1[3]};
                    if (nbase + 4 * tt < N) *reinterpret_cast<f16x8 *>(crow + nbase + 4 * tt) = h;
                }
            }
        }
    }
}

hipError_t launch_sweep(const SweepArgs &a, hipStream_t st)
{
    static bool attr_set[2] = {false, false};
    const int lds_bytes = 2 * STAGE_BYTES;
    const int which = a.c_f32 ? 1 : 0;
    if (!attr_set[which]) {
        hipError_t e = a.c_f32
            ? hipFuncSetAttribute(reinterpret_cast<const void *>(&spmm_sweep_kernel<true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes)
            : hipFuncSetAttribute(reinterpret_cast<const void *>(&spmm_sweep_kernel<false>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess) return e;
        attr_set[which] = true;
    }
    const int n_panels = (int)((a.N + NT - 1) / NT);
    long wgs = (long)a.n_rg * n_panels;
    wgs = (wgs + 7) / 8 * 8;
    if (wgs == 0) return hipSuccess;
    if (wgs > 0x7fffffffL) return hipErrorInvalidValue;
    dim3 grid((unsigned)wgs), block(THREADS);
    if (a.c_f32)
        hipLaunchKernelGGL((spmm_sweep_kernel<true>), grid, block, lds_bytes, st, a.vals, a.B, a.C,
                           a.rg_chunk_ptr, a.chunk_ids, a.ops, (int)(a.M / 16), (int)a.N, (long)a.K,
                           a.n_rg, n_panels);
    else
        hipLaunchKernelGGL((spmm_sweep_kernel<false>), grid, block, lds_bytes, st, a.vals, a.B, a.C,
                           a.rg_chunk_ptr, a.chunk_ids, a.ops, (int)(a.M / 16), (int)a.N, (long)a.K,
                           a.n_rg, n_panels);
    return hipGetLastError();
}

} // namespace smat

