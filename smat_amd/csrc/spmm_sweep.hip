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
//  * Work.  A wavefront owns 8 of the 64 block rows (the plan picks which, so that the wavefronts have
//    about the same work in every chunk) x 64 columns, 128 fp32 accumulator registers, and runs a
//    host-built stream of ops.  One op = two blocks of one block row = one K = 32 step of
//    v_mfma_f32_16x16x32_f16 per 16 columns (4 MFMAs).  The two blocks may sit up to two
//    listed chunks apart (three chunks are resident while the middle one is swept), so few blocks stay unpaired.
//  * Interpreter.  The stream of a wavefront is threaded code (gen_sweep_loop.py, sweep_format.h): every 16-byte
//    entry carries the offset of the code block that executes it, a block ends in a jump to the block of the
//    next entry.  Blocks are specialised for the stream position modulo 8 (register sets), the block row
//    (accumulators) and the s_waitcnt the op needs, so an op costs its 4 MFMAs, 4 LDS reads, one A load, the
//    address arithmetic of the reads, two waits and the jump: 18 instructions.  Entries come in through scalar
//    loads, two at a time, seven positions ahead.
//  * Pipeline.  The B operands of an op are read from LDS one position ahead (two register sets), its A
//    operand (two neighbouring 512-byte blocks, one load straight into MFMA layout) comes from global memory
//    four positions ahead (ring of eight).  Vector memory operations complete in order, so the number of
//    younger ones at every wait is known when the plan is built: 4, or 8 when a chunk boundary issued its copies in
//    between.  A half of an MFMA that must not contribute (unpaired block) reads a 16 KiB region of zeros.
//  * Accumulators live in a[0:127] and are touched by inline assembly only.
//  * Synchronisation.  One barrier per chunk, in the boundary code that the first op of the chunk runs through
//    before its own block (it is no stream position: no descriptor, no operand load is spent on it).  Boundary of
//    chunk c: the wavefront's own copies of chunk c+1 (issued one boundary earlier) have landed, barrier, then the
//    copies of chunk c+2 go into the stage that held chunk c-2.  The plan gives every wavefront at least four ops
//    per chunk (filler ops that multiply zeros where it has fewer), so boundaries are at least four positions
//    apart and every wavefront passes every barrier.
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
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int TN = SWEEP_TN, RW = SWEEP_RW, W = SWEEP_WAVES, S = SWEEP_S, NS = SWEEP_STAGES;
constexpr int NT = 16 * TN;                           // 64 columns per panel
constexpr int THREADS = 64 * W;                       // 512
constexpr int ROW_BYTES = 256;                        // 8 slabs x 16 k x 2 B per n
constexpr int STAGE_BYTES = (S / 8) * NT * ROW_BYTES; // 32768
constexpr int COPIES = STAGE_BYTES / 1024 / W;        // copy instructions per wavefront and chunk: 4
constexpr int ZERO_BYTES = 16384;                     // the region of zeros behind the stages
static_assert(TN == 4 && RW == 8 && W == 8 && S == 16 && NS == 4 && COPIES == SWEEP_COPIES && STAGE_BYTES == (int)SWEEP_STAGE_BYTES,
              "geometry the code below assumes");

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
    const int32_t *__restrict__ op_ptr, const SweepOp *__restrict__ ops, const int32_t *__restrict__ row_map, int N, long K, int n_rg, int n_panels,
    uint32_t vals_bytes, int n_vb)
{
    extern __shared__ __align__(16) unsigned char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // Tile order: blocks of 4 row groups; inside a block panel-major, row group fastest.  Each XCD
    // (workgroup id modulo 8) takes a contiguous eighth, so the 32 workgroups it runs at a time are
    // 4 row groups x 8 panels: every A block is wanted by 8 of them, every B chunk by 4.
    // A workgroup takes the tiles vb = blockIdx.x, blockIdx.x + gridDim.x, ... of the virtual grid n_vb.
    const int total = n_rg * n_panels;
    const int per_xcd = n_vb >> 3;
    constexpr int RGB = 4;
    const int n_blk = (n_rg + RGB - 1) / RGB;
    bool zeros_written = false;
  for (int vb = blockIdx.x; vb < n_vb; vb += gridDim.x) {
    const int tile = (vb & 7) * per_xcd + (vb >> 3);
    if (tile >= total) continue;
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
    // the block rows this wavefront stores at the end (the plan spreads the rows of the group over the wavefronts):
    // asked for here in two loads, so that the epilogue does not wait for eight of them one after the other
    const i32x4 *my_rows = reinterpret_cast<const i32x4 *>(row_map + (rg * W + wave) * RW);
    const i32x4 rows_lo = my_rows[0], rows_hi = my_rows[1];
    static_assert(RW == 8, "two 16-byte loads hold the block rows of a wavefront");

    if (n_chunks > 0) { // uniform over the workgroup: every wavefront has the chunk list of its row group
        auto lds_copy = [&](uint32_t voff, const void *sbase, uint32_t dst) { // 64 lanes x 16 B -> LDS dst + lane * 16
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :
                         : "v"(voff), "s"(sbase), "s"(dst)
                         : "memory");
        };
        // ---- B panel copies: this wavefront fills rows ((wave & 3) * 4 + it) * 4 .. + 3 of slab group wave / 4 ----
        // lane -> (row q = lane / 16, physical slot ps = lane % 16); logical slot = ps ^ swizzle(n),
        // swizzle(n) = (n & 3) | ((n >> 2) & 12) = q | (wave & 3) << 2 for these rows.
        const int q = lane >> 4;
        const uint32_t ls = (uint32_t)((lane & 15) ^ (q | ((wave & 3) << 2)));
        const uint32_t k_lane = (uint32_t)(wave >> 2) * 128u + ls * 8u;  // k inside the chunk
        const uint32_t col_bytes = (uint32_t)q * (uint32_t)K * 2u;       // the launcher checks K < 2^28
        const uint32_t copy_off = col_bytes + k_lane * 2u;               // byte offset of this lane's 16 bytes for chunk id 0
        const uint32_t copy_lim = col_bytes + ((uint32_t)K - 8u) * 2u;   // slabs past K are referenced by no op: the read stays inside the matrix
        const uint32_t dst_wave = lbase + (uint32_t)(wave * COPIES) * 1024u;
        // the four copy instructions of a chunk: scalar base = first of their four columns of B.  Columns past N
        // (last panel, N % 8 == 0) are replaced by the last four: what lands in their rows is never stored, and
        // every wavefront issues the same number of copies (the plan counts them).
        const int col0 = n0 + (wave & 3) * 16;
        auto col_base = [&](int c) { return B + (long)(c + 4 <= N ? c : N - 4) * K; };
        const uint16_t *sb0 = col_base(col0), *sb1 = col_base(col0 + 4), *sb2 = col_base(col0 + 8), *sb3 = col_base(col0 + 12);
        const int32_t *chunk_ptr = chunk_ids + c_begin;
        auto issue_copies = [&](int cl) { // chunk cl of the row group's list into stage cl % NS
            uint32_t voff = (uint32_t)chunk_ptr[cl] * (uint32_t)(S * 16 * 2) + copy_off;
            voff = voff < copy_lim ? voff : copy_lim;
            const uint32_t dst0 = dst_wave + (uint32_t)(cl % NS) * STAGE_BYTES;
            lds_copy(voff, sb0, dst0);
            lds_copy(voff, sb1, dst0 + 1024u);
            lds_copy(voff, sb2, dst0 + 2048u);
            lds_copy(voff, sb3, dst0 + 3072u);
        };
        // ---- entry: chunks 0, 1, 2 on their way, the region of zeros written ----
        if (zeros_written) __syncthreads(); // a later tile of this workgroup: everybody has left the stages of the tile before
        issue_copies(0);
        if (n_chunks > 1) issue_copies(1);
        if (n_chunks > 2) issue_copies(2);
        if (!zeros_written) {
            i32x4 *zero = reinterpret_cast<i32x4 *>(lds + NS * STAGE_BYTES);
            zero[tid] = i32x4{0, 0, 0, 0};
            zero[tid + THREADS] = i32x4{0, 0, 0, 0};
            static_assert(ZERO_BYTES == 2 * THREADS * 16, "two 16-byte stores per lane fill the region of zeros");
            zeros_written = true;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

        // ---- the interpreter: see gen_sweep_loop.py ----
        const uint32_t rd_addr = lbase + (uint32_t)(16 * (i16 >> 2) + (i16 & 3)) * ROW_BYTES; // LDS address of this lane's column in stage 0
        const uint32_t a_voff = (uint32_t)sel * 512u + a_lane_bytes; // lanes 32-63 take the second block of the pair
        const uint32_t sel01 = (uint32_t)sel;
        const uint32_t n_chunks_u = __builtin_amdgcn_readfirstlane((uint32_t)n_chunks);
        const SweepOp *op_base = ops + op_begin;
        const uint32_t op_lo = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)op_base);
        const uint32_t op_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uintptr_t)op_base >> 32));
        const uint32_t chunk_lo = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)chunk_ptr);
        const uint32_t chunk_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uintptr_t)chunk_ptr >> 32));
#include "spmm_sweep_loop.inc"
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); // the last MFMAs retire before their results are read

    // Epilogue: tile (r, t), element e = C[(rg*64 + wave*8 + r)*16 + i16][n0 + 16*g + 4*t + e]
    auto store_row = [&](auto rc) {
        constexpr int R = decltype(rc)::value;
        const int br = R < 4 ? rows_lo[R & 3] : rows_hi[R & 3];
        if (br < 0) return;
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
            // h0 / h1 are columns 16g .. 16g+7 / 16g+8 .. 16g+15 of this lane's row.  Stored as they are, one store
            // instruction would write four 16-byte pieces with 16-byte holes into every 128-byte row.  Two lane
            // swaps (rows of 16 lanes, then halves of the wavefront) regroup them so that the first store writes
            // bytes 0 .. 63 of each row and the second bytes 64 .. 127, 16 bytes per lane at 16 * g.
            (void)crow;
            const u32x4 x = __builtin_bit_cast(u32x4, h0), y = __builtin_bit_cast(u32x4, h1);
            u32x4 d1, d2;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const auto r = __builtin_amdgcn_permlane16_swap(x[w], y[w], false, false); // {X0 Y0 X2 Y2}, {X1 Y1 X3 Y3} by lane row
                const auto q = __builtin_amdgcn_permlane32_swap(r[0], r[1], false, false); // {X0 Y0 X1 Y1}, {X2 Y2 X3 Y3}
                d1[w] = q[0];
                d2[w] = q[1];
            }
            uint16_t *row0 = reinterpret_cast<uint16_t *>(Cout) + m * (long)N + n0 + 8 * g;
            if (n0 + 8 * g < N) *reinterpret_cast<u32x4 *>(row0) = d1;
            if (n0 + 32 + 8 * g < N) *reinterpret_cast<u32x4 *>(row0 + 32) = d2;
        }
    };
    store_row(std::integral_constant<int, 0>{}); store_row(std::integral_constant<int, 1>{});
    store_row(std::integral_constant<int, 2>{}); store_row(std::integral_constant<int, 3>{});
    store_row(std::integral_constant<int, 4>{}); store_row(std::integral_constant<int, 5>{});
    store_row(std::integral_constant<int, 6>{}); store_row(std::integral_constant<int, 7>{});
  }
}

hipError_t launch_sweep(const SweepArgs &a, hipStream_t st)
{
    const int lds_bytes = NS * STAGE_BYTES + ZERO_BYTES;
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
    // One workgroup per CU at a time (144 KiB of LDS, 512 threads x 256 registers): with more tiles than CUs a
    // workgroup keeps its CU and takes its tiles one after the other, which saves the dispatch of the later
    // ones and lets the stores of a tile drain while the next one fetches its first chunks.
    long launched = wgs;
    {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus >= 8) {
            const long resident = cus / 8 * 8; // workgroup ids are dealt round-robin to the 8 XCDs: keep a multiple of 8
            if (launched > resident) launched = resident;
        }
    }
    dim3 grid((unsigned)launched), block(THREADS);
    if (a.c_f32)
        hipLaunchKernelGGL((spmm_sweep_kernel<true>), grid, block, lds_bytes, st, a.vals, a.B, a.C,
                           a.rg_chunk_ptr, a.chunk_ids, a.op_ptr, a.ops, a.row_map, (int)a.N, (long)a.K,
                           a.n_rg, n_panels, (uint32_t)(a.nnzb * 512), (int)wgs);
    else
        hipLaunchKernelGGL((spmm_sweep_kernel<false>), grid, block, lds_bytes, st, a.vals, a.B, a.C,
                           a.rg_chunk_ptr, a.chunk_ids, a.op_ptr, a.ops, a.row_map, (int)a.N, (long)a.K,
                           a.n_rg, n_panels, (uint32_t)(a.nnzb * 512), (int)wgs);
    return hipGetLastError();
}

} // namespace smat
