"""Work list of the sweep kernel, checked on the CPU: the streams are replayed in numpy with the kernel's
own rules and the replay has to give A x B.

What the replay pins: every block is multiplied exactly once, with the rows of B under its block column,
into its own block row; the LDS stage an op reads holds the chunk it needs at that moment; the code offset
of every entry names the block of its stream position, block row and wait class; the wait class and the
marker's wait are right for the order in which the kernel issues vector memory operations."""
import ctypes as C

import numpy as np
import pytest

from smat_amd import generators as gen
from smat_amd._lib import lib

G, RW, WAVES, S, STAGES = 64, 8, 8, 16, 4
_params = (C.c_int32 * 4)()
lib.smat_internal_sweep_params(_params)
AHEAD, PB, MIN_OPS, COPIES = (int(x) for x in _params)  # A read-ahead, LDS read-ahead (positions), ops per chunk, copies per marker
assert (AHEAD, PB) == (4, 1) and MIN_OPS == AHEAD
ZERO_OFF = 131072
BLOCK_BYTES, N_BLOCKS, TRAMP_BYTES = 128, 128, 8
TRAMP_BASE = N_BLOCKS * BLOCK_BYTES         # first ops of a chunk go through a trampoline: chunk boundary code, then the op's block
MARK_OFF = TRAMP_BASE + N_BLOCKS * TRAMP_BYTES
END_OFF = MARK_OFF + 512
LDS_MASK = 0x1C0E0
PAD, CHUNK_PAD = 16, 4


def sweep_plan(row_ptr, col_idx, M, K, rows=None):
    """rows: the ascending block rows the plan is made for (what mixed dispatch hands to the sweep kernel); None = all."""
    fn = lib.smat_internal_sweep_plan
    fn.restype = C.c_int
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t] + [C.POINTER(C.c_void_p)] * 5 + [C.POINTER(C.c_int64)]
    row_ptr = np.ascontiguousarray(row_ptr, np.int32)
    col_idx = np.ascontiguousarray(col_idx, np.int32)
    rows_arr = None if rows is None else np.ascontiguousarray(rows, np.int32)
    out = [C.c_void_p() for _ in range(5)]
    counts = (C.c_int64 * 6)()
    rc = fn(row_ptr.ctypes.data, col_idx.ctypes.data, M, K, None if rows is None else rows_arr.ctypes.data,
            0 if rows is None else rows_arr.size, *[C.byref(o) for o in out], counts)
    assert rc == 0
    n_rg, n_chunks, n_ops = counts[0], counts[1], counts[2]

    def take(ptr, n, dtype):
        a = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), shape=(n,)).copy()
        lib.smat_host_free(ptr)
        return a
    plan = {
        "rg_chunk_ptr": take(out[0], n_rg + 1, np.int32), "chunk_ids": take(out[1], n_chunks + CHUNK_PAD, np.int32),
        "op_ptr": take(out[2], n_rg * WAVES + 1, np.int32), "ops": take(out[3], (n_ops + PAD) * 4, np.uint32).reshape(-1, 4),
        "row_map": take(out[4], n_rg * G, np.int32),
        "pairs": counts[3], "singles": counts[4], "fillers": counts[5], "n_entries": n_ops,
    }
    # sum over (row group, chunk period) of the op count of the busiest wavefront
    total = 0
    for rg in range(n_rg):
        n_periods = plan["rg_chunk_ptr"][rg + 1] - plan["rg_chunk_ptr"][rg]
        load = np.zeros((WAVES, max(n_periods, 1)), int)
        for w in range(WAVES):
            w3 = plan["ops"][plan["op_ptr"][rg * WAVES + w]:plan["op_ptr"][rg * WAVES + w + 1], 3]
            opens = (w3 >= TRAMP_BASE) & (w3 < MARK_OFF)
            period = np.cumsum(opens)
            is_op = w3 < MARK_OFF
            np.add.at(load[w], period[is_op], 1)
        total += int(load.max(0).sum())
    plan["period_max_sum"] = total
    return plan


def slot_of(off):
    """LDS offset -> (stage, block column inside the chunk)"""
    assert off & ~LDS_MASK == 0
    slot = (off >> 14) * 8 + ((off >> 5) & 7)
    return slot // S, slot % S


def replay(plan, A, Bd, rows=None):
    """Runs the streams on dense numpy operands. A: dict from gen (BCSR), Bd: K x N float64.  rows: the block rows
    the plan was made for (None = all): only their blocks may be used, 64 of them to a row group in this order."""
    M, K, rp, ci = A["M"], A["K"], A["b_row_ptr"], A["b_col_idx"]
    blocks = A["b_val"].view(np.float16).astype(np.float64).reshape(-1, 16, 16)
    nnzb = ci.size
    Cd = np.zeros((M, Bd.shape[1]))
    used = np.zeros(nnzb, int)
    block_row = np.repeat(np.arange(M // 16), np.diff(rp))
    n_rg = plan["rg_chunk_ptr"].size - 1
    n_real = n_fill = 0
    subset = np.arange(M // 16) if rows is None else np.asarray(rows)
    row_len = np.diff(rp)
    group_of = {}  # block row -> its row group
    for rg in range(n_rg):
        got = plan["row_map"][rg * G:(rg + 1) * G]
        for b in got[got >= 0]:
            assert int(b) not in group_of
            group_of[int(b)] = rg
    for rg in range(n_rg):
        chunks = plan["chunk_ids"][plan["rg_chunk_ptr"][rg]:plan["rg_chunk_ptr"][rg + 1]]
        assert np.all(np.diff(chunks) > 0)
        for w in range(WAVES):
            ops = plan["ops"][plan["op_ptr"][rg * WAVES + w]:plan["op_ptr"][rg * WAVES + w + 1]]
            if chunks.size == 0:
                assert ops.shape[0] == 0
                continue
            # vector memory operations in issue order: the entry code loads the A operands of positions 0..AHEAD-1 after
            # the copies of chunks 0..2; position i loads the operand of i + AHEAD, an op that opens a chunk issues the
            # copies of the chunk boundary first
            seq = AHEAD
            a_issue = {k: k + 1 for k in range(AHEAD)}
            copy_seq = {0: 0, 1: 0, 2: 0}
            cur, in_chunk, ended = 0, 0, False
            period = []  # chunk period of every stream position
            for i, (w0, w1, w2, w3) in enumerate(tuple(int(x) for x in e) for e in ops):
                assert not ended, "entries after the end of a stream"
                if w3 == END_OFF:
                    assert (w0, w1, w2) == (0, ZERO_OFF, 0)
                    ended = True
                    continue
                assert w3 < MARK_OFF, "an entry names code that is no op block and no trampoline"
                if w3 >= TRAMP_BASE:  # chunk boundary in front of this op: own copies landed, barrier, next copies
                    assert (w3 - TRAMP_BASE) % TRAMP_BYTES == 0
                    k = (w3 - TRAMP_BASE) // TRAMP_BYTES
                    assert in_chunk >= MIN_OPS, "fewer ops in a chunk than the read-ahead needs"
                    cur, in_chunk = cur + 1, 0
                    # the boundary waits until at most MIN_OPS operations are under way: its copies of the next chunk
                    # (issued by the boundary before it, or by the entry code) are older than that
                    if cur + 1 < chunks.size:
                        assert seq - copy_seq[cur + 1] >= MIN_OPS
                    if cur + 2 < chunks.size:
                        seq += COPIES
                        copy_seq[cur + 2] = seq
                    opened = True
                else:
                    assert w3 % BLOCK_BYTES == 0
                    k = w3 // BLOCK_BYTES
                    opened = False
                # what the LDS reads issued for this position could see: they were issued one position earlier
                period.append(cur)
                seq += 1
                a_issue[i + AHEAD] = seq
                in_chunk += 1
                pos, r, v = k // 16, (k // 2) % 8, k % 2
                assert pos == i % 8, "code block of another stream position"
                assert seq - a_issue[i] == AHEAD + COPIES * v, "wait class does not match the operations issued since the A load"
                q = w0 // 512
                assert w0 % 512 == 0 and 0 <= q and q + 1 < nnzb
                br = int(plan["row_map"][(rg * WAVES + w) * RW + r])
                off_lo, off_hi = w1, (w1 + int(np.int32(np.uint32(w2)))) & 0xFFFFFFFF
                if off_lo == ZERO_OFF and off_hi == ZERO_OFF:
                    n_fill += 1
                    # a filler adds two blocks times zeros to block row br: they are that row's own blocks, unless
                    # no row of this wavefront has two (then blocks 0 and 1, which the kernel can always load)
                    mine = plan["row_map"][(rg * WAVES + w) * RW:(rg * WAVES + w + 1) * RW]
                    if any(b >= 0 and row_len[b] >= 2 for b in mine):
                        assert br >= 0 and block_row[q] == br and block_row[q + 1] == br
                    else:
                        assert q == 0
                    continue
                n_real += 1
                assert group_of.get(br) == rg
                # both loaded blocks belong to the op's block row, also when one of them multiplies zeros: only a
                # block that is alone in its row travels with another row's block
                if row_len[br] >= 2:
                    assert block_row[q] == br and block_row[q + 1] == br
                for half, off in enumerate((off_lo, off_hi)):
                    if off == ZERO_OFF:
                        continue
                    stage, slab = slot_of(off)
                    # while chunk cur is swept the stages hold chunks cur - 1, cur and cur + 1 (the fourth is being filled)
                    held = [p for p in (cur + 1, cur, cur - 1) if 0 <= p < chunks.size and p % STAGES == stage]
                    assert held, "op reads the stage that is being overwritten"
                    # its LDS reads were issued one position earlier (for the op that opens a chunk: in front of the
                    # barrier, in the period before): that period sees the chunks up to its next one
                    assert held[0] <= period[max(i - PB, 0)] + 1
                    blk = q + half
                    k0 = int(chunks[held[0]]) * S * 16 + slab * 16
                    assert ci[blk] == k0 and block_row[blk] == br
                    used[blk] += 1
                    Cd[br * 16:br * 16 + 16] += blocks[blk] @ Bd[k0:k0 + 16]
            assert ended and cur == chunks.size - 1 and in_chunk >= MIN_OPS
    in_subset = np.isin(block_row, subset)
    assert np.all(used[in_subset] == 1) and not used[~in_subset].any(), "a block is multiplied zero or several times, or is not the plan's"
    assert n_fill == plan["fillers"] and n_real == plan["pairs"] + plan["singles"]
    mapped = plan["row_map"][plan["row_map"] >= 0]
    assert np.array_equal(np.sort(mapped), np.sort(subset)), "row_map is not a partition of the plan's block rows"
    # Row group rg holds the rows subset[64 rg : 64 rg + 64] (the slots that are left say -1) - unless that grouping
    # leaves one group with more than 1.08 x the blocks of an average one: then the rows are dealt out by their block
    # count, heaviest first to the lightest group with room, and every group keeps its size
    groups = [plan["row_map"][rg * G:(rg + 1) * G] for rg in range(n_rg)]
    groups = [g[g >= 0] for g in groups]
    in_order = [row_len[subset[rg * G:(rg + 1) * G]].sum() for rg in range(n_rg)]
    skewed = n_rg > 1 and max(in_order) * subset.size > 1.08 * sum(in_order) * G
    plan["dealt"] = bool(skewed)
    for rg in range(n_rg):
        assert groups[rg].size == subset[rg * G:(rg + 1) * G].size
        if not skewed:
            assert np.array_equal(np.sort(groups[rg]), np.sort(subset[rg * G:(rg + 1) * G]))
    if skewed:
        dealt = np.array([row_len[g].sum() for g in groups])
        full = [rg for rg in range(n_rg) if groups[rg].size == G]
        # no full group is heavier than the lightest full group by more than one row (what dealing heaviest-first gives)
        assert dealt[full].max() - dealt[full].min() <= row_len[subset].max()
        assert dealt.max() <= max(in_order)
    # read-ahead: the entries after the last stream exist and are harmless
    tail = plan["ops"][plan["n_entries"]:]
    assert tail.shape[0] == PAD and np.all(tail == np.array([0, ZERO_OFF, 0, END_OFF], np.uint32))
    return Cd


def dense_of(A):
    M, K, rp, ci = A["M"], A["K"], A["b_row_ptr"], A["b_col_idx"]
    D = np.zeros((M, K))
    blocks = A["b_val"].view(np.float16).astype(np.float64).reshape(-1, 16, 16)
    rows = np.repeat(np.arange(M // 16), np.diff(rp))
    for b, (r, c) in enumerate(zip(rows, ci)):
        D[r * 16:r * 16 + 16, c:c + 16] = blocks[b]
    return D


def random_mask_matrix(mb, kb, density, seed, empty_rows=(), long_rows=()):
    rng = np.random.default_rng(seed)
    mask = rng.random((mb, kb)) < density
    for r in empty_rows:
        mask[r] = False
    for r in long_rows:
        mask[r] = True
    if mask.sum() < 2:
        mask[0, :2] = True
    rp = np.concatenate([[0], np.cumsum(mask.sum(1))]).astype(np.int32)
    ci = (np.nonzero(mask)[1] * 16).astype(np.int32)
    val = gen.f16_bits(rng.normal(size=ci.size * 256))
    return {"M": mb * 16, "K": kb * 16, "b_row_ptr": rp, "b_col_idx": ci, "b_val": val, "nnzb": ci.size}


@pytest.mark.parametrize("mb,kb,density,seed", [(64, 64, 0.10, 1), (70, 40, 0.30, 2), (130, 100, 0.05, 3), (8, 200, 0.5, 4),
                                                 (64, 16, 1.0, 5), (200, 33, 0.02, 6), (3, 3, 1.0, 7), (64, 48, 0.01, 8)])
def test_replay_gives_a_times_b(mb, kb, density, seed):
    A = random_mask_matrix(mb, kb, density, seed, empty_rows=(1,) if mb > 2 else (), long_rows=(2,) if mb > 3 else ())
    plan = sweep_plan(A["b_row_ptr"], A["b_col_idx"], A["M"], A["K"])
    rng = np.random.default_rng(seed + 100)
    Bd = rng.normal(size=(A["K"], 8))
    Cd = replay(plan, A, Bd)
    assert np.allclose(Cd, dense_of(A) @ Bd, rtol=1e-12, atol=1e-12)
    assert plan["pairs"] * 2 + plan["singles"] == A["nnzb"]


@pytest.mark.parametrize("mb,kb,density,seed,pick", [(200, 64, 0.10, 11, "odd"), (150, 40, 0.3, 12, "random"), (300, 33, 0.05, 13, "blocks_of_3"),
                                                      (70, 48, 0.2, 14, "one")])
def test_replay_of_a_row_subset(mb, kb, density, seed, pick):
    """The plan of mixed dispatch: only some block rows (interleaved with rows that another kernel takes), packed 64
    to a row group.  Exactly their blocks are used, once each; an unpaired block never travels with a block of a
    row outside the subset unless it is alone in its row; the last row group is partly empty."""
    A = random_mask_matrix(mb, kb, density, seed, empty_rows=(1, 5), long_rows=(7,))
    rng = np.random.default_rng(seed)
    if pick == "odd":
        rows = np.arange(1, mb, 2)
    elif pick == "random":
        rows = np.sort(rng.choice(mb, size=mb // 3, replace=False))
    elif pick == "blocks_of_3":
        rows = np.array([r for r in range(mb) if (r // 3) % 2 == 0])
    else:
        rows = np.array([7])
    assert rows.size % G != 0  # the last row group has unused slots
    plan = sweep_plan(A["b_row_ptr"], A["b_col_idx"], A["M"], A["K"], rows=rows)
    Bd = rng.normal(size=(A["K"], 8))
    Cd = replay(plan, A, Bd, rows=rows)
    D = dense_of(A)
    keep = np.zeros(A["M"], bool)
    for r in rows:
        keep[r * 16:r * 16 + 16] = True
    D[~keep] = 0
    assert np.allclose(Cd, D @ Bd, rtol=1e-12, atol=1e-12)
    row_blocks = np.diff(A["b_row_ptr"])[rows].sum()
    assert plan["pairs"] * 2 + plan["singles"] == row_blocks


def test_single_last_block_is_listed_as_second_half():
    """An unpaired block at the very end of vals must not make the kernel read past the array."""
    mask = np.zeros((2, 40), bool)
    mask[0, [0, 1]] = True
    mask[1, [39]] = True  # last block of the matrix, alone in its row
    rp = np.concatenate([[0], np.cumsum(mask.sum(1))]).astype(np.int32)
    ci = (np.nonzero(mask)[1] * 16).astype(np.int32)
    A = {"M": 32, "K": 640, "b_row_ptr": rp, "b_col_idx": ci, "b_val": gen.f16_bits(np.ones(ci.size * 256)), "nnzb": ci.size}
    plan = sweep_plan(rp, ci, 32, 640)
    real = plan["ops"][:plan["n_entries"]]
    lo_zero = real[(real[:, 1] == ZERO_OFF) & (real[:, 2] != 0) & (real[:, 3] < MARK_OFF)]  # first half reads zeros, second half a stage
    assert lo_zero.shape[0] == 1 and lo_zero[0, 0] == (ci.size - 2) * 512
    Cd = replay(plan, A, np.ones((640, 8)))
    assert np.allclose(Cd, dense_of(A) @ np.ones((640, 8)))


def test_headline_matrix_pairs_nearly_everything():
    A = gen.block_pruned(8192, 0.10, 0.02)
    plan = sweep_plan(A["b_row_ptr"], A["b_col_idx"], A["M"], A["K"])
    assert plan["pairs"] * 2 + plan["singles"] == A["nnzb"]
    # blocks paired inside a chunk or across two consecutive chunks: few stay single, few fillers
    assert plan["singles"] < 0.12 * A["nnzb"] and plan["fillers"] < 0.01 * (plan["pairs"] + plan["singles"])
    # ops run a period early or late where their chunks are resident, and the rows are dealt to the wavefronts for
    # the cheapest caps: the busiest wavefront of a period has hardly more ops than the average one (1.23 x with
    # every op in its nominal period)
    assert plan["period_max_sum"] * WAVES < 1.045 * (plan["pairs"] + plan["singles"] + plan["fillers"])
    per_wave = np.diff(plan["op_ptr"])
    assert per_wave.min() >= 4 * 32 + 1 and per_wave.max() <= 72 * 32


def test_unevenly_pruned_rows_are_dealt_to_even_row_groups():
    """A workgroup multiplies one row group under several panels, so a launch takes as long as its heaviest row group.
    Block rows whose density falls from 18 % to 2 % would give the first of four groups 1.6 x the average; the plan
    deals the rows out instead, and the streams still multiply every block once into its own rows of C."""
    A = gen.block_pruned_skewed(4096, 0.18, 0.02)
    lens = np.diff(A["b_row_ptr"])
    in_order = lens.reshape(-1, G).sum(1)
    assert in_order.max() > 1.5 * in_order.mean()
    plan = sweep_plan(A["b_row_ptr"], A["b_col_idx"], A["M"], A["K"])
    Bd = np.random.default_rng(3).normal(size=(A["K"], 4))
    Cd = replay(plan, A, Bd)
    assert plan["dealt"]
    assert np.allclose(Cd, dense_of(A) @ Bd, rtol=1e-12, atol=1e-12)
    dealt = np.array([lens[g[g >= 0]].sum() for g in plan["row_map"].reshape(-1, G)])
    assert dealt.max() < 1.01 * dealt.mean()
    # the busiest wavefront of a period still has hardly more ops than the average one
    assert plan["period_max_sum"] * WAVES < 1.06 * (plan["pairs"] + plan["singles"] + plan["fillers"])


def test_evenly_pruned_rows_stay_in_order():
    A = gen.block_pruned(8192, 0.10, 0.02)
    plan = sweep_plan(A["b_row_ptr"], A["b_col_idx"], A["M"], A["K"])
    for rg, g in enumerate(plan["row_map"].reshape(-1, G)):
        assert np.array_equal(np.sort(g), np.arange(rg * G, (rg + 1) * G))


def test_committed_interpreter_loop_is_what_the_generator_writes():
    """spmm_sweep_loop.inc is generated code kept in the repository: it has to be the output of the generator
    next to it, and the generator takes no switches (the build makes the same comparison)."""
    import os
    import subprocess
    import sys
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "smat_amd", "csrc")
    run = subprocess.run([sys.executable, os.path.join(csrc, "gen_sweep_loop.py")], capture_output=True, text=True, check=True)
    with open(os.path.join(csrc, "spmm_sweep_loop.inc")) as f:
        committed = f.read()
    assert run.stdout == committed
    assert committed.splitlines()[0] == "// generated by gen_sweep_loop.py; do not edit"
    bad = subprocess.run([sys.executable, os.path.join(csrc, "gen_sweep_loop.py"), "--ablate", "mfma"], capture_output=True, text=True)
    assert bad.returncode != 0 and bad.stdout == ""
