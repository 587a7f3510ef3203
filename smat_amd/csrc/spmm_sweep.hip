// "Sweep" SpMM kernel for block matrices that are dense enough (a few percent of the 16x16 blocks
// present) and wide N.  One workgroup (8 wavefronts) owns 64 block rows x 64 columns of C and sweeps
// over K in chunks of 16 block columns.
//
//  * B.  The panel of a chunk (256 k x 64 n, 32 KiB) is copied global -> LDS asynchronously
//    (global_load_lds_dwordx4, no staging registers) into a ring of four stages and is shared by the
//    64 block rows.  Global reads are 256-byte contiguous runs of the column-major B (B[n*K + k]).
//    A stage is [8-slab group][n][16 slots of 16 B]; a slot is 8 consecutive k of one n.  The slot
//    index is XOR-ed with a 4-bit function of n so that the 16 lanes of one ds_read_b128 phase
//    (16 different n, same logical slot) hit 16 different 16-byte bank groups and the 16 lanes that
//    fill one n write 256 contiguous bytes: no bank conflicts on either side.
//  * Work.  A wavefront owns 8 block rows x 64 columns (128 fp32 accumulator registers) and runs a
//    host-built stream of ops.  One op = two blocks of one block row = one K = 32 step of
//    v_mfma_f32_16x16x32_f16 per 16 columns (4 MFMAs).  The two blocks may sit in the same chunk or
//    in two consecutive chunks (the ring keeps the previous stage), so few blocks stay unpaired; an
//    unpaired block multiplies zeros in the upper K half.
//  * Pipeline.  The op stream of a wavefront is one flat loop over the whole K sweep, unrolled by
//    six: the B operands of an op are read from LDS two ops ahead (three register sets), its A
//    operand (two neighbouring 512-byte blocks, one load straight into MFMA layout) comes from global
//    memory four ops ahead (ring of six), its descriptor (16 bytes, offsets ready to use) is read
//    six ops ahead from a window of the op stream that is itself copied into LDS 64 ops at a time.
//    LDS reads are ordinary loads (the compiler counts them); everything that goes through the
//    vector memory path (A loads, copies) is issued from inline assembly with explicit s_waitcnt
//    vmcnt, because only the kernel knows which copies an A load does not have to wait for: vector
//    memory instructions complete in order, and the number of younger ones is known at every wait.
//  * Accumulators live in a[0:127] and are touched by inline assembly only: the block row of an op
//    is a run-time value, and the choice between register sets is a branch between MFMA groups.
//  * Synchronisation.  One barrier per chunk.  Entering chunk c: the copies of chunk c+1 (issued one
//    chunk earlier) have landed, barrier, then the copies of chunk c+2 are issued into the stage
//    that held chunk c-2.  Reads may therefore run ahead into chunk c+1 across the barrier.  The
//    plan gives every wavefront at least two ops per chunk (zero-valued filler ops where a
//    wavefront has fewer), so an op two ahead is never further than the next chunk and every
//    wavefront passes every barrier.
//
// Same operand semantics as the reference launcher (src/cuda_hgemm/src/mma/mmaCBT.cu:83-88).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "spmm_kernels.h"

namespace smat {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int TN = SWEEP_TN, RW = SWEEP_RW, W = SWEEP_WAVES, S = SWEEP_S, NS = SWEEP_STAGES;
constexpr int NT = 16 * TN;                           // 64 columns per panel
constexpr int THREADS = 64 * W;                       // 512
constexpr int ROW_BYTES = 256;                        // 8 slabs x 16 k x 2 B per n
constexpr int STAGE_BYTES = (S / 8) * NT * ROW_BYTES; // 32768
constexpr int COPIES = STAGE_BYTES / 1024 / W;        // copy instructions per wavefront and chunk: 4
constexpr int PB = 2;                                 // B operands are read PB ops ahead (PB + 1 register sets)
constexpr int DA = 6;                                 // A operand ring (register sets)
constexpr int AHEAD = 4;                              // A operands are loaded AHEAD ops ahead (< DA)
constexpr int DQ = 6;                                 // op descriptors are read from LDS DQ ops ahead (ring of DQ scalar pairs)
constexpr int UNROLL = 6;                             // multiple of PB + 1, DA and DQ
constexpr int WIN_SLOTS = 3;                          // descriptor windows (64 ops, 1 KiB) resident per wavefront
constexpr int WINDOW_BYTES = W * WIN_SLOTS * 1024;    // 24 KiB
static_assert(TN == 4 && RW == 8 && W == 8 && S == 16 && NS == 4 && COPIES == 4, "geometry the code below assumes");
static_assert(UNROLL % (PB + 1) == 0 && UNROLL % DA == 0 && UNROLL % DQ == 0 && AHEAD < DA && AHEAD < DQ && PB < DQ,
              "register sets are addressed by the unroll position");

__device__ __forceinline__ void zero_accumulators()
{
#define Z4(b) "v_accvgpr_write_b32 a" #b ", 0\n\t"
#define Z16(b0, b1, b2, b3, b4, b5, b6, b7, b8, b9, b10, b11, b12, b13, b14, b15) \
    Z4(b0) Z4(b1) Z4(b2) Z4(b3) Z4(b4) Z4(b5) Z4(b6) Z4(b7) Z4(b8) Z4(b9) Z4(b10) Z4(b11) Z4(b12) Z4(b13) Z4(b14) Z4(b15)
    asm volatile(Z16(0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15) Z16(16, 17, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28, 29, 30, 31)
                 Z16(32, 33, 34, 35, 36, 37, 38, 39, 40, 41, 42, 43, 44, 45, 46, 47) Z16(48, 49, 50, 51, 52, 53, 54, 55, 56, 57, 58, 59, 60, 61, 62, 63)
                 :
                 :
                 : "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15", "a16", "a17", "a18", "a19",
                   "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31", "a32", "a33", "a34", "a35", "a36", "a37",
                   "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47", "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55",
                   "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63");
    asm volatile(Z16(64, 65, 66, 67, 68, 69, 70, 71, 72, 73, 74, 75, 76, 77, 78, 79) Z16(80, 81, 82, 83, 84, 85, 86, 87, 88, 89, 90, 91, 92, 93, 94, 95)
                 Z16(96, 97, 98, 99, 100, 101, 102, 103, 104, 105, 106, 107, 108, 109, 110, 111)
                 Z16(112, 113, 114, 115, 116, 117, 118, 119, 120, 121, 122, 123, 124, 125, 126, 127)
                 :
                 :
                 : "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79", "a80", "a81",
                   "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", "a96", "a97", "a98", "a99",
                   "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", "a110", "a111", "a112", "a113", "a114",
                   "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127");
#undef Z16
#undef Z4
}

// The four MFMAs of one op on block row R of the wavefront: a[16R + 4t .. + 3] += b[t] x a.
template <int R>
__device__ __forceinline__ void mfma_row(const f16x8 (&b)[TN], const f16x8 &a)
{
    asm volatile("s_nop 1\n\t"
                 "v_mfma_f32_16x16x32_f16 a[%5:%6], %0, %4, a[%5:%6]\n\t"
                 "v_mfma_f32_16x16x32_f16 a[%7:%8], %1, %4, a[%7:%8]\n\t"
                 "v_mfma_f32_16x16x32_f16 a[%9:%10], %2, %4, a[%9:%10]\n\t"
                 "v_mfma_f32_16x16x32_f16 a[%11:%12], %3, %4, a[%11:%12]"
                 :
                 : "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3]), "v"(a), "n"(16 * R), "n"(16 * R + 3), "n"(16 * R + 4), "n"(16 * R + 7),
                   "n"(16 * R + 8), "n"(16 * R + 11), "n"(16 * R + 12), "n"(16 * R + 15));
}

// Reads accumulator tile (R, T) after the last MFMA has retired.
template <int R, int T>
__device__ __forceinline__ f32x4 read_acc()
{
    f32x4 v;
    asm volatile("v_accvgpr_read_b32 %0, a[%4]\n\tv_accvgpr_read_b32 %1, a[%5]\n\tv_accvgpr_read_b32 %2, a[%6]\n\tv_accvgpr_read_b32 %3, a[%7]"
                 : "=v"(v[0]), "=v"(v[1]), "=v"(v[2]), "=v"(v[3])
                 : "n"(16 * R + 4 * T), "n"(16 * R + 4 * T + 1), "n"(16 * R + 4 * T + 2), "n"(16 * R + 4 * T + 3));
    return v;
}

} // namespace

template <bool C_F32>
__global__ __launch_bounds__(THREADS) void spmm_sweep_kernel(
    const uint16_t *__restrict__ vals, const uint16_t *__restrict__ B, void *__restrict__ Cout,
    const int32_t *__restrict__ rg_chunk_ptr, const int32_t *__restrict__ chunk_ids,
    const int32_t *__restrict__ op_ptr, const SweepOp *__restrict__ ops, int Mb, int N, long K, int n_rg, int n_panels,
    uint32_t vals_bytes)
{
    extern __shared__ __align__(16) unsigned char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // Tile order: blocks of 4 row groups; inside a block panel-major, row group fastest.  Each XCD
    // (workgroup id modulo 8) takes a contiguous eighth, so the 32 workgroups it runs at a time are
    // 4 row groups x 8 panels: every A block is wanted by 8 of them, every B chunk by 4.
    const int total = n_rg * n_panels;
    const int per_xcd = gridDim.x >> 3;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= total) return;
    constexpr int RGB = 4;
    const int n_blk = (n_rg + RGB - 1) / RGB;
    int gb = tile / (RGB * n_panels);
    gb = gb < n_blk - 1 ? gb : n_blk - 1;
    const int rem = tile - gb * RGB * n_panels;
    const int rgs_here = n_rg - gb * RGB < RGB ? n_rg - gb * RGB : RGB;
    const int panel = rem / rgs_here;
    const int rg = gb * RGB + rem - panel * rgs_here;
    const int n0 = panel * NT;

    const int i16 = lane & 15, g = lane >> 4, sel = g >> 1, kh = g & 1;
    const uint32_t lbase = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)lds;
    // column (within the panel) of MFMA row i16 in n-tile 0 is 16*(i16>>2) + (i16&3); n-tile t adds 4*t.
    // The swizzle value of every such column equals i16.
    const uint32_t rd_lane = (uint32_t)(16 * (i16 >> 2) + (i16 & 3)) * ROW_BYTES; // byte offset in a stage
    const uint32_t lane_xor = (uint32_t)((kh ^ i16) << 4); // ((2*slab | kh) ^ i16) << 4 == (slab * 32) ^ lane_xor
    const uint32_t a_lane_bytes = (uint32_t)(i16 * 16 + kh * 8) * 2u; // this lane's 16 bytes inside a block

    // The 8 x 4 accumulator tiles (4 registers each) live in a[0:127], tile (r, t) in a[16r + 4t .. + 3], and are
    // touched only by the assembly below: which block row an op adds to is known at run time only, and a
    // run-time choice between register sets is a branch between otherwise identical MFMA groups.
    zero_accumulators();

    // vals as a raw buffer: base, no stride, nnzb * 512 bytes, 32-bit untyped data
    i32x4 vals_rsrc;
    vals_rsrc[0] = (int)(uint32_t)(uintptr_t)vals;
    vals_rsrc[1] = (int)(uint32_t)((uintptr_t)vals >> 32) & 0xffff;
    vals_rsrc[2] = (int)vals_bytes;
    vals_rsrc[3] = 0x00020000;

    const int c_begin = rg_chunk_ptr[rg], n_chunks = rg_chunk_ptr[rg + 1] - c_begin;
    const int op_begin = op_ptr[rg * W + wave];
    const int n_ops = op_ptr[rg * W + wave + 1] - op_begin;

    if (n_chunks > 0) { // uniform over the workgroup: every wavefront has the chunk list of its row group
        // Vector memory instructions complete in order.  `age` counts the ops (= A loads) since the last chunk
        // boundary, `burst` the copy instructions issued at that boundary: together they give the immediate of
        // every vmcnt wait.
        int age = 0, burst = 0;
        auto lds_copy = [&](uint32_t voff, const void *sbase, uint32_t dst) { // 64 lanes x 16 B -> LDS dst + lane * 16
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :
                         : "v"(voff), "s"(sbase), "s"(dst)
                         : "memory");
            burst++;
        };

        // ---- B panel copies: this wavefront fills rows ((wave & 3) * 4 + it) * 4 .. + 3 of slab group wave / 4 ----
        // lane -> (row q = lane / 16, physical slot ps = lane % 16); logical slot = ps ^ swizzle(n),
        // swizzle(n) = (n & 3) | ((n >> 2) & 12) = q | (wave & 3) << 2 for these rows.
        const int q = lane >> 4;
        const uint32_t ls = (uint32_t)((lane & 15) ^ (q | ((wave & 3) << 2)));
        const uint32_t k_lane = (uint32_t)(wave >> 2) * 128u + ls * 8u; // k inside the chunk
        const uint32_t col_lane = (uint32_t)q * (uint32_t)K;            // elements; the launcher checks K < 2^28
        const uint32_t kmax = (uint32_t)K - 8u;
        auto issue_copies = [&](int cl) {
            const uint32_t k0 = (uint32_t)chunk_ids[c_begin + cl] * (uint32_t)(S * 16);
            uint32_t k = k0 + k_lane;
            k = k < kmax ? k : kmax; // slabs past K are referenced by no op; keep the read inside the matrix
            const uint32_t voff = (col_lane + k) * 2u;
            const uint32_t dst0 = lbase + (uint32_t)(cl % NS) * STAGE_BYTES + (uint32_t)(wave * COPIES) * 1024u;
#pragma unroll
            for (int it = 0; it < COPIES; it++) {
                const int row4 = ((wave & 3) * 4 + it) * 4; // first of four columns, wave-uniform
                if (n0 + row4 >= N) continue;               // N % 8 == 0: all four columns or none
                lds_copy(voff, B + (long)(n0 + row4) * K, dst0 + (uint32_t)it * 1024u);
            }
        };

        // ---- op descriptors: windows of 64 ops (1 KiB, one copy instruction) in three LDS slots per wavefront ----
        const SweepOp *op_base = ops + op_begin; // the plan pads the array: reads past n_ops stay inside it
        const uint32_t win_base = (uint32_t)(NS * STAGE_BYTES) + (uint32_t)wave * (WIN_SLOTS * 1024u); // byte offset in LDS
        int win_next = 0; // first window not requested yet
        auto copy_window = [&]() {
            lds_copy((uint32_t)lane * 16u, op_base + (long)win_next * 64, lbase + win_base + (uint32_t)(win_next % WIN_SLOTS) * 1024u);
            win_next++;
        };
        // plain LDS read, same address in every lane; made scalar where it is used, several ops later
        auto read_desc = [&](int x) {
            return *reinterpret_cast<const uint4 *>(lds + win_base + (uint32_t)((x >> 6) % WIN_SLOTS) * 1024u + (uint32_t)(x & 63) * 16u);
        };

        // ---- operand registers ----
        f16x8 bq[PB + 1][TN];
        f16x8 aq[DA];
        uint4 dq[DQ];      // descriptors of ops i .. i + DQ - 1 (slot = op % DQ), one copy per lane
        uint32_t fq[PB + 1]; // flags and block row (word 1) of the ops whose B operands are under way
        const f16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
        // A operand: one buffer load of the 1 KiB pair, lanes 32-63 take the second block.  Where a block does not
        // belong to the op its lanes get an offset past the end of the buffer, for which the load returns zeros:
        // between the load and the MFMAs nothing touches the operand registers.
        const uint32_t a_voff = (uint32_t)sel * 512u + a_lane_bytes;
        const uint32_t a_voff_zero_hi = sel ? 0x80000000u : a_voff;
        const uint32_t a_voff_zero_lo = sel ? a_voff : 0x80000000u;
        const uint32_t a_voff_zero = 0x80000000u;

        // reads the B operands of an op: lanes 0-31 from the slab of its first block, 32-63 of the second
        auto issue_b = [&](f16x8(&b)[TN], uint32_t w1, uint32_t w2) {
            const uint32_t off0 = w1 & SWEEP_LDS_MASK, off1 = w2;
            const unsigned char *p = lds + rd_lane + ((sel ? off1 : off0) ^ lane_xor);
#pragma unroll
            for (int tt = 0; tt < TN; tt++) b[tt] = *reinterpret_cast<const f16x8 *>(p + tt * 4 * ROW_BYTES);
        };
        // loads the A operand of an op: its two blocks are neighbours in vals, 1 KiB in MFMA operand order
        auto issue_a = [&](f16x8 &a, uint32_t w0, uint32_t w1) {
            const uint32_t z = w1 & (SWEEP_OP_ZERO_HI | SWEEP_OP_ZERO_LO);
            if (z == 0)
                asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(a) : "v"(a_voff), "s"(vals_rsrc), "s"(w0));
            else if (z == SWEEP_OP_ZERO_HI)
                asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(a) : "v"(a_voff_zero_hi), "s"(vals_rsrc), "s"(w0));
            else if (z == SWEEP_OP_ZERO_LO)
                asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(a) : "v"(a_voff_zero_lo), "s"(vals_rsrc), "s"(w0));
            else
                asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(a) : "v"(a_voff_zero), "s"(vals_rsrc), "s"(w0));
        };

        // ---- prologue: chunks 0 and 1 resident, descriptors of the first 192 ops, first operands under way ----
        issue_copies(0);
        if (n_chunks > 1) issue_copies(1);
        copy_window();
        copy_window();
        copy_window();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
#pragma unroll
        for (int d = 0; d < DQ; d++) dq[d] = read_desc(d);
#pragma unroll
        for (int d = 0; d < AHEAD; d++)
            issue_a(aq[d], __builtin_amdgcn_readfirstlane(dq[d].x), __builtin_amdgcn_readfirstlane(dq[d].y));
        burst = 0;
        if (n_chunks > 2) issue_copies(2); // after the first A loads, like the copies of a boundary
#pragma unroll
        for (int d = AHEAD; d < DA; d++) aq[d] = zero8;
#pragma unroll
        for (int d = 0; d < PB; d++) {
            fq[d] = __builtin_amdgcn_readfirstlane(dq[d].y);
            issue_b(bq[d], fq[d], __builtin_amdgcn_readfirstlane(dq[d].z));
        }
        fq[PB] = 0;
#pragma unroll
        for (int tt = 0; tt < TN; tt++) bq[PB][tt] = zero8;

        int cur = 0; // chunk (index into the row group's chunk list) the executed ops belong to
        int i = 0;   // op executed next

        // One op.  J = i % UNROLL selects the register sets.
        auto step = [&](auto jc) {
            constexpr int J = decltype(jc)::value;
            const uint32_t w1 = fq[J % (PB + 1)];
            if (w1 & SWEEP_OP_BOUNDARY) {
                // entering chunk cur: the copies of chunk cur + 1 (issued when chunk cur - 1 was entered, `age` A
                // loads ago) have landed; after the barrier every wavefront is done with chunk cur - 1, and the
                // stage of chunk cur - 2 takes the copies of chunk cur + 2
                cur++;
                if (age <= AHEAD) { // else an A load issued after them has been waited for
                    if (age == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
                    else if (age == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
                    else if (age == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                }
                asm volatile("s_barrier" ::: "memory");
                burst = 0;
                age = 0;
                if (cur + 2 < n_chunks) issue_copies(cur + 2);
                // descriptor windows: those up to two ahead of the current op are requested here; a chunk holds
                // at most 72 ops of a wavefront, so a window is requested at least 50 ops before its first read
                // and the windows requested at the last boundary cover the read-ahead past the last op
                while ((i >> 6) + 2 >= win_next) copy_window();
            }
            // Operands of later ops.  Unconditional: past the end of the stream the descriptors are the plan's
            // padding (block 0, first slab), whose operands are fetched and never used.  A condition here would
            // make the compiler wait for every LDS read before the MFMAs (it has to assume the path on which
            // the younger reads were not issued).
            {
                const uint4 &db = dq[(J + PB) % DQ];
                fq[(J + PB) % (PB + 1)] = __builtin_amdgcn_readfirstlane(db.y);
                issue_b(bq[(J + PB) % (PB + 1)], fq[(J + PB) % (PB + 1)], __builtin_amdgcn_readfirstlane(db.z));
                const uint4 &da = dq[(J + AHEAD) % DQ];
                issue_a(aq[(J + AHEAD) % DA], __builtin_amdgcn_readfirstlane(da.x), __builtin_amdgcn_readfirstlane(da.y));
                dq[J % DQ] = read_desc(i + DQ); // replaces the descriptor of op i, whose word 1 is in w1
            }
            __builtin_amdgcn_sched_barrier(0);
            // the A operand of op i: AHEAD younger A loads, and the copies of the last boundary if that young
            // (the waits carry no operands: an operand tied to the wait lets the compiler copy the register
            // before it; the operand registers go from the load straight to the MFMAs)
            if (age < AHEAD) {
                if (burst == COPIES) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
                else if (burst == COPIES + 1) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
                else if (burst == COPIES + 2) asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); // fewer copies (last panel, last chunks): waits for them too
            } else {
                asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            }
            static_assert(AHEAD == 4 && COPIES == 4, "immediates above");
            age++;
            const f16x8 &av = aq[J % DA];
            f16x8(&bc)[TN] = bq[J % (PB + 1)];
            switch (w1 >> 28) {
            case 0: mfma_row<0>(bc, av); break;
            case 1: mfma_row<1>(bc, av); break;
            case 2: mfma_row<2>(bc, av); break;
            case 3: mfma_row<3>(bc, av); break;
            case 4: mfma_row<4>(bc, av); break;
            case 5: mfma_row<5>(bc, av); break;
            case 6: mfma_row<6>(bc, av); break;
            default: mfma_row<7>(bc, av); break;
            }
        };
        while (i < n_ops) {
            step(std::integral_constant<int, 0>{}); if (++i >= n_ops) break;
            step(std::integral_constant<int, 1>{}); if (++i >= n_ops) break;
            step(std::integral_constant<int, 2>{}); if (++i >= n_ops) break;
            step(std::integral_constant<int, 3>{}); if (++i >= n_ops) break;
            step(std::integral_constant<int, 4>{}); if (++i >= n_ops) break;
            step(std::integral_constant<int, 5>{}); ++i;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); // the last MFMAs retire before their results are read

    // Epilogue: tile (r, t), element e = C[(rg*64 + wave*8 + r)*16 + i16][n0 + 16*g + 4*t + e]
    auto store_row = [&](auto rc) {
        constexpr int R = decltype(rc)::value;
        const int br = rg * SWEEP_G + wave * RW + R;
        if (br >= Mb) return;
        const long m = (long)br * 16 + i16;
        const int nbase = n0 + 16 * g;
        const f32x4 v0 = read_acc<R, 0>(), v1 = read_acc<R, 1>(), v2 = read_acc<R, 2>(), v3 = read_acc<R, 3>();
        if (C_F32) {
            float *crow = reinterpret_cast<float *>(Cout) + m * (long)N + nbase;
            if (nbase < N) { *reinterpret_cast<f32x4 *>(crow) = v0; *reinterpret_cast<f32x4 *>(crow + 4) = v1; }
            if (nbase + 8 < N) { *reinterpret_cast<f32x4 *>(crow + 8) = v2; *reinterpret_cast<f32x4 *>(crow + 12) = v3; }
        } else {
            uint16_t *crow = reinterpret_cast<uint16_t *>(Cout) + m * (long)N + nbase;
            const f16x8 h0 = {(_Float16)v0[0], (_Float16)v0[1], (_Float16)v0[2], (_Float16)v0[3],
                              (_Float16)v1[0], (_Float16)v1[1], (_Float16)v1[2], (_Float16)v1[3]};
            const f16x8 h1 = {(_Float16)v2[0], (_Float16)v2[1], (_Float16)v2[2], (_Float16)v2[3],
                              (_Float16)v3[0], (_Float16)v3[1], (_Float16)v3[2], (_Float16)v3[3]};
            if (nbase < N) *reinterpret_cast<f16x8 *>(crow) = h0;
            if (nbase + 8 < N) *reinterpret_cast<f16x8 *>(crow + 8) = h1;
        }
    };
    store_row(std::integral_constant<int, 0>{}); store_row(std::integral_constant<int, 1>{});
    store_row(std::integral_constant<int, 2>{}); store_row(std::integral_constant<int, 3>{});
    store_row(std::integral_constant<int, 4>{}); store_row(std::integral_constant<int, 5>{});
    store_row(std::integral_constant<int, 6>{}); store_row(std::integral_constant<int, 7>{});
}

hipError_t launch_sweep(const SweepArgs &a, hipStream_t st)
{
    const int lds_bytes = NS * STAGE_BYTES + WINDOW_BYTES;
    // dynamic LDS above 64 KiB has to be allowed once per kernel and device; the call is cheap and idempotent
    hipError_t e = a.c_f32
        ? hipFuncSetAttribute(reinterpret_cast<const void *>(&spmm_sweep_kernel<true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes)
        : hipFuncSetAttribute(reinterpret_cast<const void *>(&spmm_sweep_kernel<false>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return e;
    if (a.K >= ((size_t)1 << 28)) return hipErrorInvalidValue; // copy offsets: (3 * K + k) * 2 in 32 bits
    const int n_panels = (int)((a.N + NT - 1) / NT);
    long wgs = (long)a.n_rg * n_panels;
    wgs = (wgs + 7) / 8 * 8;
    if (wgs == 0) return hipSuccess;
    if (wgs > 0x7fffffffL) return hipErrorInvalidValue;
    dim3 grid((unsigned)wgs), block(THREADS);
    if (a.c_f32)
        hipLaunchKernelGGL((spmm_sweep_kernel<true>), grid, block, lds_bytes, st, a.vals, a.B, a.C,
                           a.rg_chunk_ptr, a.chunk_ids, a.op_ptr, a.ops, (int)(a.M / 16), (int)a.N, (long)a.K,
                           a.n_rg, n_panels, (uint32_t)(a.nnzb * 512));
    else
        hipLaunchKernelGGL((spmm_sweep_kernel<false>), grid, block, lds_bytes, st, a.vals, a.B, a.C,
                           a.rg_chunk_ptr, a.chunk_ids, a.op_ptr, a.ops, (int)(a.M / 16), (int)a.N, (long)a.K,
                           a.n_rg, n_panels, (uint32_t)(a.nnzb * 512));
    return hipGetLastError();
}

} // namespace smat
