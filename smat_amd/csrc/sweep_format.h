// Stream format of the sweep kernel (spmm_sweep.hip), shared by the kernel, its generated interpreter
// (gen_sweep_loop.py) and the host-side plan builder (sweep_plan.cpp).  No HIP types.
#pragma once
#include <stdint.h>

namespace smat {

// Geometry (fixed at compile time).
constexpr int SWEEP_TN = 4;      // n-tiles of 16 per workgroup panel -> 64 columns
constexpr int SWEEP_RW = 8;      // block rows per wavefront
constexpr int SWEEP_WAVES = 8;   // wavefronts per workgroup
constexpr int SWEEP_G = SWEEP_RW * SWEEP_WAVES; // 64 block rows per workgroup
constexpr int SWEEP_S = 16;      // block columns (slabs) per K chunk
constexpr int SWEEP_STAGES = 4;  // chunks resident in LDS
constexpr int SWEEP_AHEAD = 4; // an A operand is loaded this many stream positions before its op
constexpr int SWEEP_LDS_AHEAD = 1; // the B operands of an op are read from LDS this many stream positions before it
constexpr int SWEEP_COPIES = 4;  // copy instructions per wavefront and chunk
constexpr int SWEEP_MIN_OPS = SWEEP_AHEAD; // ops per wavefront and chunk: two chunk boundaries are at least AHEAD positions apart (at most one of them between the load of an A operand and its use), and a boundary finds the copies of the boundary before it older than the A loads of the MIN_OPS positions since
constexpr int SWEEP_OP_PAD = 16;   // descriptors after the end of the last stream (loaded ahead, never executed)
constexpr int SWEEP_CHUNK_PAD = 4; // chunk ids after the last list (loaded ahead, never used)

// One stream entry (16 bytes).  The stream of a (row group, wavefront) is
//     ops of chunk 0, ops of chunk 1, ..., ops of the last chunk, end
// where "chunk" counts positions in the row group's chunk list.  Position i in the stream decides the register
// sets its code uses (i % 8).
//   w0  op: byte offset in vals of the first of two neighbouring blocks (q * 512); both are loaded.  End: 0.
//   w1  LDS byte offset of the 16 rows of B that the first block is multiplied with (lanes 0-31)
//   w2  the same for the second block (lanes 32-63), minus w1 (signed)
//   w3  byte offset, from the first code block, of the code that executes the entry:
//         op      ((i % 8 * 8 + local block row) * 2 + v) * SWEEP_BLOCK_BYTES,  v = 1 when the copies of a chunk
//                 boundary were issued after the load of this op's A operand (the op that opens the chunk and the
//                 AHEAD - 1 positions behind it)
//         first op of every chunk but the first:  SWEEP_TRAMP_BASE + (the op's block index) * SWEEP_TRAMP_BYTES: a
//                 trampoline that runs the chunk boundary code (own copies landed, barrier, next copies) and then
//                 the op's block.  A chunk boundary is no stream position: no operand load is spent on it
//         end     SWEEP_END_OFF
// An op is two blocks of one block row (K = 32 of one MFMA per 16 columns) in the chunk the op is listed under or
// the one before.  LDS offset of a block = sweep_lds_offset(chunk position, block column in the chunk); a half
// that must not contribute (unpaired block, filler op, end) points at SWEEP_ZERO_OFF, 16 KiB of zeros.
struct SweepOp {
    uint32_t w0, w1, w2, w3;
};
constexpr uint32_t SWEEP_STAGE_BYTES = 32768;
constexpr uint32_t SWEEP_ZERO_OFF = SWEEP_STAGES * SWEEP_STAGE_BYTES; // 131072
constexpr uint32_t SWEEP_BLOCK_BYTES = 128;
constexpr uint32_t SWEEP_N_BLOCKS = 8 * 8 * 2;                                       // stream position % 8 x block row x v
constexpr uint32_t SWEEP_TRAMP_BASE = SWEEP_N_BLOCKS * SWEEP_BLOCK_BYTES;            // 16384
constexpr uint32_t SWEEP_TRAMP_BYTES = 8;
constexpr uint32_t SWEEP_MARK_OFF = SWEEP_TRAMP_BASE + SWEEP_N_BLOCKS * SWEEP_TRAMP_BYTES; // 17408: the chunk boundary code
constexpr uint32_t SWEEP_MARK_BYTES = 512;
constexpr uint32_t SWEEP_END_OFF = SWEEP_MARK_OFF + SWEEP_MARK_BYTES;               // 17920

inline uint32_t sweep_lds_offset(int32_t chunk_pos, int32_t slab)
{
    const uint32_t slot = (uint32_t)(chunk_pos % SWEEP_STAGES) * SWEEP_S + (uint32_t)slab;
    return (slot >> 3) * 16384u + (slot & 7u) * 32u;
}
inline uint32_t sweep_op_code(int pos, int row, int v) { return (uint32_t)(((pos % 8) * 8 + row) * 2 + v) * SWEEP_BLOCK_BYTES; }
// the same op as the first of its chunk: through the chunk boundary code
inline uint32_t sweep_boundary_op_code(int pos, int row, int v) { return SWEEP_TRAMP_BASE + (uint32_t)(((pos % 8) * 8 + row) * 2 + v) * SWEEP_TRAMP_BYTES; }

} // namespace smat
