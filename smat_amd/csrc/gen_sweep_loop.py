#!/usr/bin/env python3
"""Writes spmm_sweep_loop.inc: the main loop of the sweep kernel as one inline-assembly statement.

The loop runs the op stream of one wavefront (see spmm_sweep.hip for the scheme).  It is written by
hand because every instruction a wavefront issues besides its MFMAs adds to its run time (a
wavefront issues in order), and the compiler's code for the run-time choices in the loop (which
accumulators, which wait) costs several times the instructions needed.  This script only unrolls
the six positions of the register rings and numbers the registers; run it after changing it:

    python3 gen_sweep_loop.py > spmm_sweep_loop.inc

Registers (fixed, all listed as clobbers):
    (with the default ring of six)
    v40-v87    B operands, three sets of 4 tiles x 4 registers (op i uses set i % 3)
    v88-v111   A operands, ring of six (op i uses slot i % 6)
    v112-v119  two descriptors being read from LDS
    v120-v126  temporaries; v124-v126 = A offsets with the upper / lower / both halves out of range
    s40..      loop state, s52-s75 descriptor ring (op i in slot i % 6: w0 w1 w2 w3)
    a0-a127    accumulators (block row r, tile t in a[16r + 4t .. + 3])
"""

import argparse

ap = argparse.ArgumentParser()
ap.add_argument("--unroll", type=int, default=6, help="ring positions: A ring slots = descriptor ring slots; multiple of 6")
ap.add_argument("--ahead", type=int, default=4, help="A operands are loaded this many ops ahead (< unroll)")
ap.add_argument("--ablate", default="", help="timing experiments only, wrong results: any of a,copy,barrier,mfma,bread")
args = ap.parse_args()
UNROLL = args.unroll
AHEAD = args.ahead
PB = 2         # B operands are read PB ops ahead
DQ = UNROLL    # descriptor ring slots; a descriptor is read DQ + 1 ops ahead and made scalar two ops later
ABL = set(x for x in args.ablate.split(",") if x)
assert UNROLL % (PB + 1) == 0 and UNROLL % 2 == 0 and PB < AHEAD < UNROLL

S_I, S_AGE, S_BURST, S_CUR, S_WINNEXT, S_DP, S_T0, S_T1, S_T2, S_T3, S_T4, S_T5 = range(40, 52)
RING0 = 52     # s[52 + 4*slot + word]
assert RING0 + 4 * UNROLL <= 100
V_TOP = 128
V_T0, V_T1, V_T2, V_COPY, V_AZH, V_AZL, V_AZB = range(V_TOP - 8, V_TOP - 1)
V_DESC = V_TOP - 16  # two buffers of four registers
V_A0 = V_DESC - 4 * UNROLL
V_B0 = V_A0 - 16 * (PB + 1)
V_FIRST = V_B0


def ring(slot, word):
    return f"s{RING0 + 4 * (slot % UNROLL) + word}"


def bset(s, t):
    b = V_B0 + 16 * (s % (PB + 1)) + 4 * t
    return f"v[{b}:{b + 3}]"


def aslot(d):
    b = V_A0 + 4 * (d % UNROLL)
    return f"v[{b}:{b + 3}]"


out = []


def emit(line=""):
    out.append(line)


def label(name):
    emit(f"{name}_%=:")


def a_load(dst_slot, desc_slot, tag):
    """A operand of the op whose descriptor sits in ring slot desc_slot."""
    if "a" in ABL:
        return
    emit(f"s_and_b32 s{S_T0}, {ring(desc_slot, 3)}, 3")          # which halves are zeros: SCC = any
    emit(f"s_cbranch_scc1 Lazero_{tag}_%=")
    emit(f"buffer_load_dwordx4 {aslot(dst_slot)}, %[a_voff], %[rsrc], {ring(desc_slot, 0)} offen")
    label(f"Ladone_{tag}")


def a_load_slow(dst_slot, desc_slot, tag):
    if "a" in ABL:
        return
    label(f"Lazero_{tag}")
    emit(f"s_cmp_eq_u32 s{S_T0}, 1")
    emit(f"s_cbranch_scc1 Lazh_{tag}_%=")
    emit(f"s_cmp_eq_u32 s{S_T0}, 2")
    emit(f"s_cbranch_scc1 Lazl_{tag}_%=")
    emit(f"buffer_load_dwordx4 {aslot(dst_slot)}, v{V_AZB}, %[rsrc], {ring(desc_slot, 0)} offen")
    emit(f"s_branch Ladone_{tag}_%=")
    label(f"Lazh_{tag}")
    emit(f"buffer_load_dwordx4 {aslot(dst_slot)}, v{V_AZH}, %[rsrc], {ring(desc_slot, 0)} offen")
    emit(f"s_branch Ladone_{tag}_%=")
    label(f"Lazl_{tag}")
    emit(f"buffer_load_dwordx4 {aslot(dst_slot)}, v{V_AZL}, %[rsrc], {ring(desc_slot, 0)} offen")
    emit(f"s_branch Ladone_{tag}_%=")


def b_reads(dst_set, desc_slot):
    """B operands of the op in ring slot desc_slot: lanes 0-31 at w1, lanes 32-63 at w1 + w2."""
    emit(f"v_mul_i32_i24 v{V_T1}, {ring(desc_slot, 2)}, %[sel01]")
    emit(f"v_add_u32 v{V_T1}, {ring(desc_slot, 1)}, v{V_T1}")
    emit(f"v_xad_u32 v{V_T2}, v{V_T1}, %[lane_xor], %[rd_lane]")
    for t in range(4):
        off = f" offset:{1024 * t}" if t else ""
        if "bread" in ABL:
            emit("s_nop 0")
            continue
        emit(f"ds_read_b128 {bset(dst_set, t)}, v{V_T2}{off}")


def desc_read(buf):
    b = V_DESC + 4 * (buf % 2)
    emit(f"s_add_u32 s{S_DP}, s{S_DP}, 16")
    emit(f"s_and_b32 s{S_DP}, s{S_DP}, 0xfff")
    emit(f"s_add_u32 s{S_T0}, s{S_DP}, %[win_lds]")
    emit(f"v_mov_b32 v{V_T0}, s{S_T0}")
    emit(f"ds_read_b128 v[{b}:{b + 3}], v{V_T0}")


def desc_scalar(slot, buf):
    b = V_DESC + 4 * (buf % 2)
    for w in range(4):
        emit(f"v_readfirstlane_b32 {ring(slot, w)}, v{b + w}")


def mfma_dispatch(J):
    w3 = ring(J, 3)
    if "jump" in ABL:                                            # always block row 0, no jump
        emit("s_nop 1")
        for t in range(4):
            acc = f"a[{4 * t}:{4 * t + 3}]"
            emit(f"v_mfma_f32_16x16x32_f16 {acc}, {bset(J, t)}, {aslot(J)}, {acc}")
        return
    emit(f"s_lshr_b32 s{S_T0}, {w3}, 23")                        # block row * 40
    emit("s_getpc_b64 vcc")
    label(f"Lpc_{J}")
    emit(f"s_add_u32 s{S_T0}, s{S_T0}, Lrow0_{J}_%=-Lpc_{J}_%=")
    emit(f"s_add_u32 vcc_lo, vcc_lo, s{S_T0}")
    emit("s_addc_u32 vcc_hi, vcc_hi, 0")
    emit("s_setpc_b64 vcc")
    for r in range(8):                                           # 40 bytes each: s_nop, 4 x 8, s_branch
        label(f"Lrow{r}_{J}")
        emit("s_nop 1")
        for t in range(4):
            acc = f"a[{16 * r + 4 * t}:{16 * r + 4 * t + 3}]"
            if "mfma" in ABL:
                emit("v_nop")
                emit("v_nop")
                continue
            emit(f"v_mfma_f32_16x16x32_f16 {acc}, {bset(J, t)}, {aslot(J)}, {acc}")
        if r < 7:
            emit(f"s_branch Lmdone_{J}_%=")
    label(f"Lmdone_{J}")


def boundary(J):
    """First op of a chunk: wait for the copies of the next chunk, barrier, issue the copies of the one after."""
    label(f"Lbound_{J}")
    emit(f"s_add_u32 s{S_CUR}, s{S_CUR}, 1")
    # the copies were issued `age` A loads ago; beyond AHEAD one of those loads has been waited for already
    emit(f"s_cmp_gt_u32 s{S_AGE}, {AHEAD}")
    emit(f"s_cbranch_scc1 Lbw_{J}_%=")
    ages = list(range(2, AHEAD + 1))
    for a in ages:
        emit(f"s_cmp_eq_u32 s{S_AGE}, {a}")
        emit(f"s_cbranch_scc1 Lbw{a}_{J}_%=")
    emit("s_waitcnt vmcnt(0)")
    emit(f"s_branch Lbw_{J}_%=")
    for a in ages:
        label(f"Lbw{a}_{J}")
        emit(f"s_waitcnt vmcnt({a})")
        if a != ages[-1]:
            emit(f"s_branch Lbw_{J}_%=")
    label(f"Lbw_{J}")
    if "barrier" not in ABL:
        emit("s_barrier")
    emit(f"s_mov_b32 s{S_BURST}, 0")
    emit(f"s_mov_b32 s{S_AGE}, 0")
    # copies of chunk cur + 2 into stage (cur + 2) % 4
    emit(f"s_add_u32 s{S_T0}, s{S_CUR}, 2")
    emit(f"s_cmp_ge_u32 s{S_T0}, %[n_chunks]")
    emit(f"s_cbranch_scc1 Lnocopy_{J}_%=")
    emit(f"s_lshl_b32 s{S_T1}, s{S_T0}, 2")
    emit(f"s_load_dword s{S_T2}, %[chunk_ptr], s{S_T1}")
    emit(f"s_and_b32 s{S_T1}, s{S_T0}, 3")
    emit(f"s_lshl_b32 s{S_T1}, s{S_T1}, 15")
    emit(f"s_add_u32 s{S_T1}, s{S_T1}, %[dst_wave]")
    emit("s_waitcnt lgkmcnt(0)")
    emit(f"s_lshl_b32 s{S_T2}, s{S_T2}, 8")                      # first k of the chunk
    emit(f"v_add_u32 v{V_T0}, s{S_T2}, %[k_lane]")
    emit(f"v_min_u32 v{V_T0}, %[kmax], v{V_T0}")
    emit(f"v_lshl_add_u32 v{V_COPY}, v{V_T0}, 1, %[col_bytes]")
    for it in range(4):
        emit(f"s_bitcmp1_b32 %[copy_mask], {it}")
        emit(f"s_cbranch_scc0 Lskip{it}_{J}_%=")
        emit(f"s_mov_b32 m0, s{S_T1}")
        emit("s_nop 0")
        if "copy" not in ABL:
            emit(f"global_load_lds_dwordx4 v{V_COPY}, %[sb{it}]")
            emit(f"s_add_u32 s{S_BURST}, s{S_BURST}, 1")
        label(f"Lskip{it}_{J}")
        if it < 3:
            emit(f"s_add_u32 s{S_T1}, s{S_T1}, 1024")
    label(f"Lnocopy_{J}")
    # descriptor windows up to two ahead of the current op
    label(f"Lwin_{J}")
    emit(f"s_lshr_b32 s{S_T0}, s{S_I}, 6")
    emit(f"s_add_u32 s{S_T0}, s{S_T0}, 2")
    emit(f"s_cmp_lt_u32 s{S_T0}, s{S_WINNEXT}")
    emit(f"s_cbranch_scc1 Lwdone_{J}_%=")
    emit(f"s_lshl_b32 s{S_T1}, s{S_WINNEXT}, 10")
    emit(f"s_add_u32 s{S_T2}, %[op_lo], s{S_T1}")
    emit(f"s_addc_u32 s{S_T3}, %[op_hi], 0")
    emit(f"s_and_b32 s{S_T1}, s{S_WINNEXT}, 3")
    emit(f"s_lshl_b32 s{S_T1}, s{S_T1}, 10")
    emit(f"s_add_u32 s{S_T1}, s{S_T1}, %[win_lds]")
    emit(f"s_mov_b32 m0, s{S_T1}")
    emit("s_nop 0")
    emit(f"global_load_lds_dwordx4 %[lane16], s[{S_T2}:{S_T3}]")
    emit(f"s_add_u32 s{S_BURST}, s{S_BURST}, 1")
    emit(f"s_add_u32 s{S_WINNEXT}, s{S_WINNEXT}, 1")
    emit(f"s_branch Lwin_{J}_%=")
    label(f"Lwdone_{J}")
    emit(f"s_branch Lbdone_{J}_%=")


def vm_slow(J):
    """A wait while the copies of the last boundary are younger than the A operand needed."""
    label(f"Lvmslow_{J}")
    for b in (4, 5, 6):
        emit(f"s_cmp_eq_u32 s{S_BURST}, {b}")
        emit(f"s_cbranch_scc1 Lvm{b}_{J}_%=")
    emit(f"s_waitcnt vmcnt({AHEAD})")                            # fewer copies than usual: waits for them too
    emit(f"s_branch Lvmdone_{J}_%=")
    for b in (4, 5, 6):
        label(f"Lvm{b}_{J}")
        emit(f"s_waitcnt vmcnt({AHEAD + b})")
        emit(f"s_branch Lvmdone_{J}_%=")


def step(J):
    label(f"Lstep_{J}")
    emit(f"s_bitcmp1_b32 {ring(J, 3)}, 2")                       # first op of a chunk?
    emit(f"s_cbranch_scc1 Lbound_{J}_%=")
    label(f"Lbdone_{J}")
    # LDS returns in order: per step one descriptor read, then four B reads.  What the step before the
    # previous one issued is needed now (B operands of this op, descriptor of op i + DQ - 1); the five reads
    # of the previous step may still be under way.
    if "lgkm" not in ABL:
        emit("s_waitcnt lgkmcnt(5)")
    if "desc" not in ABL:
        desc_scalar(J + DQ - 1, J)                               # read two steps ago into buffer J % 2
        desc_read(J)                                             # op i + DQ + 1
    b_reads(J + PB, J + PB)
    a_load(J + AHEAD, J + AHEAD, f"s{J}")
    emit(f"s_cmp_lt_u32 s{S_AGE}, {AHEAD}")
    emit(f"s_cbranch_scc1 Lvmslow_{J}_%=")
    if "vm" not in ABL:
        emit(f"s_waitcnt vmcnt({AHEAD})")
    label(f"Lvmdone_{J}")
    emit(f"s_add_u32 s{S_AGE}, s{S_AGE}, 1")
    mfma_dispatch(J)
    emit(f"s_add_u32 s{S_I}, s{S_I}, 1")
    emit(f"s_cmp_ge_u32 s{S_I}, %[n_ops]")
    emit("s_cbranch_scc1 Lexit_%=")
    if J == UNROLL - 1:
        emit("s_branch Lstep_0_%=")


# ---- prologue: chunks 0, 1 and three descriptor windows are resident, all wavefronts are past the barrier ----
emit(f"s_mov_b32 s{S_I}, 0")
emit(f"s_mov_b32 s{S_AGE}, 0")
emit(f"s_mov_b32 s{S_BURST}, 0")
emit(f"s_mov_b32 s{S_CUR}, 0")
emit(f"s_mov_b32 s{S_WINNEXT}, 3")
# A offsets whose upper / lower / both halves are out of range (the load returns zeros there)
emit("v_cmp_ne_u32 vcc, 0, %[sel01]")
emit(f"v_mov_b32 v{V_AZB}, 0x80000000")
emit(f"v_cndmask_b32 v{V_AZH}, %[a_voff], v{V_AZB}, vcc")
emit(f"v_cndmask_b32 v{V_AZL}, v{V_AZB}, %[a_voff], vcc")
# descriptors of ops 0 .. DQ - 2 into the ring
for x in range(DQ - 1):
    emit(f"s_add_u32 s{S_T0}, %[win_lds], {16 * x}")
    emit(f"v_mov_b32 v{V_T0}, s{S_T0}")
    emit(f"ds_read_b128 v[{V_DESC}:{V_DESC + 3}], v{V_T0}")
    emit("s_waitcnt lgkmcnt(0)")
    desc_scalar(x, 0)
for x in range(AHEAD):
    a_load(x, x, f"p{x}")
# copies of chunk 2, after the first A loads like the copies of a boundary
emit("s_cmp_lt_u32 %[n_chunks], 3")
emit("s_cbranch_scc1 Lpnocopy_%=")
emit(f"s_load_dword s{S_T2}, %[chunk_ptr], 8")
emit(f"s_add_u32 s{S_T1}, %[dst_wave], {2 * 32768}")
emit("s_waitcnt lgkmcnt(0)")
emit(f"s_lshl_b32 s{S_T2}, s{S_T2}, 8")
emit(f"v_add_u32 v{V_T0}, s{S_T2}, %[k_lane]")
emit(f"v_min_u32 v{V_T0}, %[kmax], v{V_T0}")
emit(f"v_lshl_add_u32 v{V_COPY}, v{V_T0}, 1, %[col_bytes]")
for it in range(4):
    emit(f"s_bitcmp1_b32 %[copy_mask], {it}")
    emit(f"s_cbranch_scc0 Lpskip{it}_%=")
    emit(f"s_mov_b32 m0, s{S_T1}")
    emit("s_nop 0")
    if "copy" not in ABL:
        emit(f"global_load_lds_dwordx4 v{V_COPY}, %[sb{it}]")
        emit(f"s_add_u32 s{S_BURST}, s{S_BURST}, 1")
    label(f"Lpskip{it}")
    if it < 3:
        emit(f"s_add_u32 s{S_T1}, s{S_T1}, 1024")
label("Lpnocopy")
# LDS reads in flight when step 0 starts, oldest first, as in the steady state: descriptor of op DQ - 1 (buffer 0,
# made scalar in step 0), B of op 0, descriptor of op DQ (buffer 1, made scalar in step 1), B of op 1
emit(f"s_mov_b32 s{S_DP}, {16 * (DQ - 2)}")
desc_read(0)
b_reads(0, 0)
desc_read(1)
b_reads(1, 1)
emit("s_branch Lstep_0_%=")

for J in range(UNROLL):
    step(J)
for J in range(UNROLL):
    boundary(J)
    vm_slow(J)
    a_load_slow(J + AHEAD, J + AHEAD, f"s{J}")
for x in range(AHEAD):
    a_load_slow(x, x, f"p{x}")
label("Lexit")
emit("s_waitcnt vmcnt(0) lgkmcnt(0)")

clobber_v = [f"v{r}" for r in range(V_FIRST, V_TOP)]
clobber_s = [f"s{r}" for r in range(40, RING0 + 4 * UNROLL)]
print("// Generated by gen_sweep_loop.py -- do not edit.")
print("asm volatile(")
for line in out:
    end = "\\n" if line.endswith(":") else "\\n\\t"
    print(f'    "{line}{end}"')
print("    :")
print('    : [rsrc] "s"(vals_rsrc), [a_voff] "v"(a_voff), [sel01] "v"(sel01), [lane_xor] "v"(lane_xor), [rd_lane] "v"(rd_addr),')
print('      [win_lds] "s"(win_lds), [n_ops] "s"(n_ops_u), [n_chunks] "s"(n_chunks_u), [chunk_ptr] "s"(chunk_ptr), [dst_wave] "s"(dst_wave),')
print('      [k_lane] "v"(k_lane), [kmax] "s"(kmax), [col_bytes] "v"(col_bytes), [copy_mask] "s"(copy_mask), [sb0] "s"(sb0), [sb1] "s"(sb1),')
print('      [sb2] "s"(sb2), [sb3] "s"(sb3), [op_lo] "s"(op_lo), [op_hi] "s"(op_hi), [lane16] "v"(lane16)')
print("    : " + ", ".join(f'"{c}"' for c in clobber_v + clobber_s) + ', "vcc", "scc", "memory");')
