#!/usr/bin/env python3
"""Writes spmm_sweep_loop.inc: the op interpreter of the sweep kernel as one inline-assembly statement.

The stream of one wavefront (see spmm_sweep.hip for the scheme) is threaded code: every 16-byte
descriptor ends in the byte offset of the code block that executes it, and every block ends in a jump
to the block of the next descriptor.  A block is specialised for

    J  the position of the op in the stream modulo 8 (which register sets it uses),
    r  the block row of the wavefront the op adds to (which accumulators),
    v  whether the copies of a chunk boundary were issued between the load of its A operand and now (which s_waitcnt vmcnt),

so the run-time choices cost no instruction besides the jump.  It is written by hand because a
wavefront issues in order: every instruction next to its MFMAs adds to its run time.  Blocks have a
fixed size (the host computes their offsets; .org fails the build if one outgrows its slot).
Run after changing:

    python3 gen_sweep_loop.py > spmm_sweep_loop.inc

Stream position i, J = i % 8.  Block of op i (AHEAD = 4):
    even position: LDS reads of the B operands of op i + 1 (into set (J + 1) % 2), then a wait until only those
    four are left: LDS reads return in order, so the reads of op i are in registers.  Scalar loads share the
    counter and return in any order; with one of them under way the same wait holds for the reads of op i
    (it then also waits for the first read of op i + 1 or for the scalar load, whichever comes first)
    odd position: wait for everything (the reads of op i, and the descriptors that the odd position before it
    asked for), scalar load of the descriptors of ops i + 7 and i + 8 (32 bytes), LDS reads of op i + 1
    load of the A operand of op i + AHEAD (into slot (J + AHEAD) % 8)
    wait for the A operand of op i, 4 MFMAs, jump to op i + 1
    The set that the reads of op i + 1 land in is the one the MFMAs of op i - 1 took their operands from a few
    instructions earlier: an MFMA reads its A and B sources when it starts, LDS data arrives 64 clocks later
    at the earliest.
Chunk boundary (before the first op of every chunk but the first): the descriptor of that op names a trampoline
instead of its block; the trampoline notes the block's offset and branches to the boundary code: own copies of
the next chunk have landed, barrier, copies of the chunk after next, then on to the op's block.  The boundary is
no stream position: no operand load and no descriptor slot is spent on it.

Registers (fixed, all listed as clobbers):
    v40-v71    B operands, two sets of 4 tiles x 4 registers
    v72-v103   A operands, ring of eight
    v104-v106  temporaries
    s40-s71    descriptor ring, op i in slot i % 8: w0 w1 w2 w3
    s72-s86    state: descriptor pointer, code base, chunk counter, next chunk id, chunk list pointer,
               temporaries, jump target, the block a chunk boundary continues with
    a0-a127    accumulators (block row r, tile t in a[16r + 4t .. + 3])
"""

import sys

if len(sys.argv) > 1:
    sys.exit("gen_sweep_loop.py takes no arguments: it writes the one loop the library ships")

AHEAD = 4                                # SWEEP_AHEAD: A operands are loaded this many stream positions ahead (ring of eight)
BSETS, ARING = 2, 8                      # B operands are read from LDS one position ahead (two register sets)

RING = 8
BLOCK_BYTES = 128                        # SWEEP_BLOCK_BYTES
N_BLOCKS = 8 * 8 * 2                     # SWEEP_N_BLOCKS: stream position % 8 x block row x v
TRAMP_BASE = N_BLOCKS * BLOCK_BYTES      # SWEEP_TRAMP_BASE: after the op blocks
TRAMP_BYTES = 8                          # SWEEP_TRAMP_BYTES
MARK_OFF = TRAMP_BASE + N_BLOCKS * TRAMP_BYTES   # SWEEP_MARK_OFF
MARK_BYTES = 512                         # SWEEP_MARK_BYTES
END_OFF = MARK_OFF + MARK_BYTES          # SWEEP_END_OFF
COPIES = 4
MIN_OPS = AHEAD            # SWEEP_MIN_OPS
VM_MARK = MIN_OPS          # a boundary's copies of one boundary ago are older than the A loads of the MIN_OPS positions since

S_RING0 = 40
DESC_AHEAD = 7   # an odd position loads the descriptors of ops i + DESC_AHEAD and the one after
S_DP, S_BASE, S_CUR, S_NEXTK, S_CP, S_T0, S_T1, S_JMP = 72, 74, 76, 77, 78, 80, 81, 84
S_RET = 86
S_LAST = 86
V_B0 = 40
V_A0 = V_B0 + 16 * BSETS
V_T0 = V_A0 + 4 * ARING
V_T1, V_COPY = V_T0 + 1, V_T0 + 2


def ring(slot, word):
    return f"s{S_RING0 + 4 * (slot % RING) + word}"


def bset(s, t):
    b = V_B0 + 16 * (s % BSETS) + 4 * t
    return f"v[{b}:{b + 3}]"


def aslot(d):
    b = V_A0 + 4 * (d % ARING)
    return f"v[{b}:{b + 3}]"


out = []


def emit(line=""):
    out.append(line)


def label(name):
    emit(f"{name}_%=:")


def b_reads(dst_set, desc_slot):
    """B operands of the op in ring slot desc_slot: lanes 0-31 at w1, lanes 32-63 at w1 + w2."""
    emit(f"v_mul_i32_i24 v{V_T0}, {ring(desc_slot, 2)}, %[sel01]")
    emit(f"v_add_u32 v{V_T0}, {ring(desc_slot, 1)}, v{V_T0}")
    emit(f"v_xad_u32 v{V_T1}, v{V_T0}, %[lane_xor], %[rd_lane]")
    for t in range(4):
        off = f" offset:{1024 * t}" if t else ""
        emit(f"ds_read_b128 {bset(dst_set, t)}, v{V_T1}{off}")


def a_load(slot):
    emit(f"buffer_load_dwordx4 {aslot(slot)}, %[a_voff], %[rsrc], {ring(slot, 0)} offen")


def top_wait(J):
    """B operands of op i are in registers.  An even position asks for the reads of op i + 1 first and waits until
    only they are left; an odd position waits for everything (reads of op i, descriptors asked for two positions
    ago), asks for two descriptors and then for the reads of op i + 1."""
    if J % 2 == 0:
        b_reads(J + 1, J + 1)
        emit("s_waitcnt lgkmcnt(4)")
        return
    emit("s_waitcnt lgkmcnt(0)")
    s0 = S_RING0 + 4 * ((J + DESC_AHEAD) % RING)
    emit(f"s_load_dwordx8 s[{s0}:{s0 + 7}], s[{S_DP}:{S_DP + 1}], 0x0")
    emit(f"s_add_u32 s{S_DP}, s{S_DP}, 32")
    emit(f"s_addc_u32 s{S_DP + 1}, s{S_DP + 1}, 0")
    b_reads(J + 1, J + 1)


def jump(desc_slot):
    emit(f"s_add_u32 s{S_JMP}, s{S_BASE}, {ring(desc_slot, 3)}")
    emit(f"s_addc_u32 s{S_JMP + 1}, s{S_BASE + 1}, 0")
    emit(f"s_setpc_b64 s[{S_JMP}:{S_JMP + 1}]")


def op_block(J, r, v):
    k = (J * 8 + r) * 2 + v
    label(f"Lb{k}")
    top_wait(J)
    a_load(J + AHEAD)
    emit(f"s_waitcnt vmcnt({AHEAD + COPIES * v})")
    for t in range(4):
        acc = f"a[{16 * r + 4 * t}:{16 * r + 4 * t + 3}]"
        emit(f"v_mfma_f32_16x16x32_f16 {acc}, {bset(J, t)}, {aslot(J)}, {acc}")
    jump(J + 1)
    emit(f".org Lb0_%= + {(k + 1) * BLOCK_BYTES}")


def trampoline(k):
    label(f"Lt{k}")
    emit(f"s_movk_i32 s{S_RET}, {k * BLOCK_BYTES}")
    emit("s_branch Lmark_%=")
    emit(f".org Lb0_%= + {TRAMP_BASE + (k + 1) * TRAMP_BYTES}")


def boundary_code():
    label("Lmark")
    emit(f"s_waitcnt vmcnt({VM_MARK})")               # own copies of the chunk after the one being entered (issued one boundary ago) have landed
    emit("s_barrier")
    emit(f"s_add_u32 s{S_CUR}, s{S_CUR}, 1")          # chunk (position in the row group's list) being entered
    emit(f"s_add_u32 s{S_T0}, s{S_CUR}, 2")
    emit(f"s_cmp_ge_u32 s{S_T0}, %[n_chunks]")
    emit("s_cbranch_scc1 Lmn_%=")
    # copies of chunk cur + 2 into stage (cur + 2) % 4: rows of B from k = 256 * id (the id was loaded by the previous boundary)
    emit(f"s_lshl_b32 s{S_T1}, s{S_NEXTK}, 9")
    emit(f"v_add_u32 v{V_COPY}, s{S_T1}, %[copy_off]")
    emit(f"v_min_u32 v{V_COPY}, v{V_COPY}, %[copy_lim]")
    emit(f"s_and_b32 s{S_T0}, s{S_T0}, 3")
    emit(f"s_lshl_b32 s{S_T0}, s{S_T0}, 15")
    emit(f"s_add_u32 s{S_T0}, s{S_T0}, %[dst_wave]")
    for it in range(COPIES):
        emit(f"s_add_u32 m0, s{S_T0}, {1024 * it}")
        emit("s_nop 0")
        emit(f"global_load_lds_dwordx4 v{V_COPY}, %[sb{it}]")
    label("Lmn")
    emit(f"s_load_dword s{S_NEXTK}, s[{S_CP}:{S_CP + 1}], 0x0")   # id of chunk cur + 3, for the next boundary
    emit(f"s_add_u32 s{S_CP}, s{S_CP}, 4")
    emit(f"s_addc_u32 s{S_CP + 1}, s{S_CP + 1}, 0")
    emit(f"s_add_u32 s{S_JMP}, s{S_BASE}, s{S_RET}")             # on to the block of the op that opens the chunk
    emit(f"s_addc_u32 s{S_JMP + 1}, s{S_BASE + 1}, 0")
    emit(f"s_setpc_b64 s[{S_JMP}:{S_JMP + 1}]")
    emit(f".org Lb0_%= + {MARK_OFF + MARK_BYTES}")


# ---- entry: descriptors of ops 0..5, A operands of ops 0..AHEAD-1, B operands of ops 0 and 1 ----
emit(f"s_mov_b32 s{S_DP}, %[op_lo]")
emit(f"s_mov_b32 s{S_DP + 1}, %[op_hi]")
emit(f"s_load_dwordx16 s[{S_RING0}:{S_RING0 + 15}], s[{S_DP}:{S_DP + 1}], 0x0")
emit(f"s_load_dwordx16 s[{S_RING0 + 16}:{S_RING0 + 31}], s[{S_DP}:{S_DP + 1}], 0x40")
emit(f"s_add_u32 s{S_DP}, s{S_DP}, 128")
emit(f"s_addc_u32 s{S_DP + 1}, s{S_DP + 1}, 0")
emit(f"s_mov_b32 s{S_CP}, %[chunk_lo]")
emit(f"s_mov_b32 s{S_CP + 1}, %[chunk_hi]")
emit(f"s_load_dword s{S_NEXTK}, s[{S_CP}:{S_CP + 1}], 0xc")      # id of chunk 3, for the first marker
emit(f"s_add_u32 s{S_CP}, s{S_CP}, 16")
emit(f"s_addc_u32 s{S_CP + 1}, s{S_CP + 1}, 0")
emit(f"s_mov_b32 s{S_CUR}, 0")
emit("s_waitcnt lgkmcnt(0)")
for k in range(AHEAD):
    a_load(k)
emit(f"s_waitcnt vmcnt({AHEAD})")                     # the copies of chunks 0, 1, 2 (issued before these loads) have landed
emit("s_barrier")
b_reads(0, 0)
emit(f"s_getpc_b64 s[{S_BASE}:{S_BASE + 1}]")
label("Lpc")
emit(f"s_add_u32 s{S_BASE}, s{S_BASE}, Lb0_%=-Lpc_%=")
emit(f"s_addc_u32 s{S_BASE + 1}, s{S_BASE + 1}, 0")
jump(0)
emit(".p2align 7")
for J in range(8):
    for r in range(8):
        for v in range(2):
            op_block(J, r, v)
for k in range(N_BLOCKS):
    trampoline(k)
boundary_code()
label("Lend")                                         # offset END_OFF: the descriptor after the last op jumps here
emit("s_waitcnt vmcnt(0) lgkmcnt(0)")

clob = ([f'"v{i}"' for i in range(V_B0, V_COPY + 1)] + [f'"s{i}"' for i in range(S_RING0, S_LAST + 2)] +
        [f'"a{i}"' for i in range(128)] + ['"vcc"', '"scc"', '"memory"'])
print("// generated by gen_sweep_loop.py; do not edit")
print(f"static_assert(SWEEP_AHEAD == {AHEAD} && SWEEP_MIN_OPS == {MIN_OPS} && SWEEP_BLOCK_BYTES == {BLOCK_BYTES} && SWEEP_TRAMP_BASE == {TRAMP_BASE} && "
      f"SWEEP_TRAMP_BYTES == {TRAMP_BYTES} && SWEEP_MARK_OFF == {MARK_OFF} && SWEEP_END_OFF == {END_OFF}, \"regenerate spmm_sweep_loop.inc\");")
print("asm volatile(")
for line in out:
    end = "\\n" if line.endswith(":") else "\\n\\t"
    print(f'    "{line}{end}"')
print("    :")
print('    : [sel01] "v"(sel01), [lane_xor] "v"(lane_xor), [rd_lane] "v"(rd_addr), [a_voff] "v"(a_voff), [rsrc] "s"(vals_rsrc),')
print('      [copy_off] "v"(copy_off), [copy_lim] "v"(copy_lim), [dst_wave] "s"(dst_wave), [n_chunks] "s"(n_chunks_u),')
print('      [sb0] "s"(sb0), [sb1] "s"(sb1), [sb2] "s"(sb2), [sb3] "s"(sb3),')
print('      [op_lo] "s"(op_lo), [op_hi] "s"(op_hi), [chunk_lo] "s"(chunk_lo), [chunk_hi] "s"(chunk_hi)')
print("    : " + ", ".join(clob) + ");")
