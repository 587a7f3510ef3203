"""GPU parity tests: the HIP SpMM, called through the C ABI, against the CPU oracle.

Bar: max_j |C[i][j] - ref[i][j]| / ||ref[i][:]||_2 <= 1e-3 for the fp16 output
(the tolerance the port's acceptance criterion states), and <= 2e-6 for the
fp32-output variant (only the summation order differs from the oracle)."""
import numpy as np
import pytest

from smat_amd import generators as gen

pytestmark = pytest.mark.gpu

TOL_F16 = 1e-3
TOL_F32 = 2e-6


def to_dev(torch, arr, device):
    a = np.ascontiguousarray(arr)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(device)
    return torch.from_numpy(a).to(device)


def gpu_spmm(smat, cuda, A, B_bits, N, plan=False, c_f32=False, drop_in=False, poison=True, kernel=0):
    """A: dict with M, K, b_row_ptr, b_col_idx, b_val. Returns C as numpy (uint16 bits or float32)."""
    import torch
    M, K, nnzb = A["M"], A["K"], int(A["b_col_idx"].shape[0])
    vals = to_dev(torch, A["b_val"] if nnzb else np.zeros(8, np.uint16), cuda)
    rp = to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda)
    ci = to_dev(torch, A["b_col_idx"].astype(np.int32) if nnzb else np.zeros(1, np.int32), cuda)
    B = to_dev(torch, B_bits, cuda)
    if c_f32:
        C = torch.full((M, N), float("nan") if poison else 0.0, dtype=torch.float32, device=cuda)
    else:
        C = torch.full((M, N), 0x7E00 if poison else 0, dtype=torch.int16, device=cuda)  # fp16 NaN pattern
    p = None
    if plan:
        p = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=kernel)
    torch.cuda.synchronize()
    if drop_in:  # fresh tensors may sit where another test's matrix of the same size sat: no plan from before
        smat.lib.smat_plan_cache_clear()
    smat.spmm(vals, rp, ci, B, C, M, N, K, nnzb, plan=p, c_f32=c_f32, drop_in=drop_in, kernel=kernel)
    torch.cuda.synchronize()
    out = C.cpu().numpy()
    if p is not None:
        p.close()
    return out if c_f32 else out.view(np.uint16)


def rel_err_f32(c, ref):
    nrm = np.sqrt((ref.astype(np.float64) ** 2).sum(axis=1))
    nrm[nrm == 0] = 1.0
    d = np.abs(c.astype(np.float64) - ref.astype(np.float64)).max(axis=1)
    return float((d / nrm).max())


def oracle_ref(oracle, A, B_bits, N):
    return oracle.spmm_bcsr(A["M"], N, A["K"], A["b_row_ptr"], A["b_col_idx"], A["b_val"], B_bits, threads=8)


def test_single_identity_block_gathers_b_rows(smat, cuda, oracle):
    # A = one 16x16 identity block at block column 2 of a 16 x 64 matrix: C = B[32:48, :]
    eye = np.eye(16, dtype=np.float16).view(np.uint16).ravel()
    A = {"M": 16, "K": 64, "b_row_ptr": np.array([0, 1], np.int32), "b_col_idx": np.array([32], np.int32),
         "b_val": eye}
    for N in (8, 16, 24, 64, 136):
        B = gen.dense_b(64, N, seed=7, dist="uniform")
        C = gpu_spmm(smat, cuda, A, B, N)
        expect = B.reshape(N, 64).T[32:48, :]  # column-major B: element (k, n) at [n*K + k]
        assert np.array_equal(C, expect), f"N={N}"


def test_asymmetric_block_pins_operand_orientation(smat, cuda, oracle):
    # one block with a single nonzero at (row 3, col 11): C[3, :] = 2 * B[16*1 + 11, :], all else 0
    blk = np.zeros((16, 16), dtype=np.float16)
    blk[3, 11] = 2.0
    A = {"M": 32, "K": 48, "b_row_ptr": np.array([0, 0, 1], np.int32), "b_col_idx": np.array([16], np.int32),
         "b_val": blk.view(np.uint16).ravel()}
    N = 40
    B = gen.dense_b(48, N, seed=9, dist="uniform")
    C = gpu_spmm(smat, cuda, A, B, N).view(np.float16).astype(np.float32)
    Bm = B.view(np.float16).reshape(N, 48).T.astype(np.float32)
    expect = np.zeros((32, N), dtype=np.float32)
    expect[16 + 3, :] = 2.0 * Bm[16 + 11, :]
    assert np.array_equal(C, expect)


@pytest.mark.parametrize("N", [8, 16, 24, 32, 40, 64, 72, 128, 136, 256, 520, 1032])
def test_random_bcsr_all_panel_widths(smat, cuda, oracle, N):
    A = gen.random_bcsr(9, 13, 0.35, seed=100 + N)
    B = gen.dense_b(A["K"], N, seed=200 + N, dist="normal")
    ref = oracle_ref(oracle, A, B, N)
    C = gpu_spmm(smat, cuda, A, B, N)
    err = oracle.compare(C, ref)[0]
    assert err <= TOL_F16, (N, err)
    C32 = gpu_spmm(smat, cuda, A, B, N, c_f32=True)
    assert rel_err_f32(C32, ref) <= TOL_F32
    # the fp16 output is exactly the rounded fp32 output
    assert np.array_equal(C32.astype(np.float16).view(np.uint16), C)


@pytest.mark.parametrize("mb,kb,density,N,n_hint", [
    (40, 128, 0.30, 256, 256),
    (24, 160, 0.25, 264, 264),    # N not a multiple of the 64-column repack tile
    (33, 130, 0.20, 200, 512),    # plan built for a wider N than the launch uses
    (64, 256, 0.10, 1032, 1032),  # several N panels, ragged last one
])
def test_repacked_b_rowwise_is_bit_identical_to_direct(smat, cuda, oracle, mb, kb, density, N, n_hint):
    """The slab-major scratch copy of B changes addresses only: same products, same order."""
    import torch
    A = gen.random_bcsr(mb, kb, density, seed=mb * 7 + kb)
    B = gen.dense_b(A["K"], N, seed=N + 3, dist="normal")
    M, K, nnzb = A["M"], A["K"], int(A["b_col_idx"].shape[0])
    vals, Bd = to_dev(torch, A["b_val"], cuda), to_dev(torch, B, cuda)
    rp, ci = to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda), to_dev(torch, A["b_col_idx"].astype(np.int32), cuda)
    out = {}
    for kernel in (4, 3):  # always repacked, never repacked
        p = smat.Plan(A["b_row_ptr"], M, K, nnzb, n_hint, col_idx_host=A["b_col_idx"], kernel=kernel)
        assert (p.info()["b_pack_bytes"] > 0) == (kernel == 4)
        for c_f32 in (False, True):
            C = torch.full((M, N), float("nan"), dtype=torch.float32, device=cuda) if c_f32 else \
                torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
            smat.spmm(vals, rp, ci, Bd, C, M, N, K, nnzb, plan=p, c_f32=c_f32, kernel=kernel)
            torch.cuda.synchronize()
            out[kernel, c_f32] = C.cpu().numpy()
        p.close()
    assert np.array_equal(out[4, False], out[3, False])
    assert np.array_equal(out[4, True].view(np.uint32), out[3, True].view(np.uint32))
    ref = oracle_ref(oracle, A, B, N)
    assert oracle.compare(out[4, False].view(np.uint16), ref)[0] <= TOL_F16
    assert rel_err_f32(out[4, True], ref) <= TOL_F32
    assert not np.array_equal(B, 0)  # B itself is left untouched by the repack
    assert np.array_equal(Bd.cpu().numpy().view(np.uint16), B)


def test_drop_in_entry_matches_options_entry(smat, cuda, oracle):
    A = gen.random_bcsr(20, 20, 0.2, seed=5)
    N = 96
    B = gen.dense_b(A["K"], N, seed=6)
    c1 = gpu_spmm(smat, cuda, A, B, N, drop_in=True)
    c2 = gpu_spmm(smat, cuda, A, B, N, drop_in=False)
    assert np.array_equal(c1, c2)
    assert oracle.compare(c1, oracle_ref(oracle, A, B, N))[0] <= TOL_F16


def cache_stats(smat):
    import ctypes as C
    out = (C.c_int64 * 4)()
    smat.lib.smat_internal_plan_cache_stats(out)
    return {"built": out[0], "hits": out[1], "rebuilt": out[2], "entries": out[3]}


def test_drop_in_entry_point_keeps_a_plan_per_matrix(smat, cuda, oracle, monkeypatch):
    """smat_spmm_bcsr_f16 (the reference's positional signature, no plan argument) makes a plan on its first call
    with a matrix and reuses it: two matrices in turn, each result bit for bit what an explicit plan gives; a
    pattern rewritten in place is caught by the checksum (or by smat_plan_cache_clear); SMAT_PLAN_CACHE=0 goes back
    to plain launches."""
    import ctypes as C
    import torch
    lib = smat.lib
    lib.smat_plan_cache_clear()
    lib.smat_internal_plan_cache_check_every(C.c_uint64(0))

    def setup(A, N, seed):
        B = gen.dense_b(A["K"], N, seed=seed, dist="normal")
        t = {"A": A, "N": N, "B": B, "vals": to_dev(torch, A["b_val"], cuda), "rp": to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda),
             "ci": to_dev(torch, A["b_col_idx"].astype(np.int32), cuda), "Bd": to_dev(torch, B, cuda)}
        t["C"] = torch.full((A["M"], N), 0x7E00, dtype=torch.int16, device=cuda)
        return t

    def drop_in(t):
        A = t["A"]
        t["C"].fill_(0x7E00)
        smat.spmm(t["vals"], t["rp"], t["ci"], t["Bd"], t["C"], A["M"], t["N"], A["K"], A["nnzb"], drop_in=True)
        torch.cuda.synchronize()
        return t["C"].cpu().numpy().view(np.uint16)

    def planned(t):
        A = t["A"]
        p = smat.Plan(A["b_row_ptr"], A["M"], A["K"], A["nnzb"], t["N"], col_idx_host=A["b_col_idx"])
        kernel = p.info()["kernel"]
        Cp = torch.full((A["M"], t["N"]), 0x7E00, dtype=torch.int16, device=cuda)
        smat.spmm(t["vals"], t["rp"], t["ci"], t["Bd"], Cp, A["M"], t["N"], A["K"], A["nnzb"], plan=p)
        torch.cuda.synchronize()
        p.close()
        return Cp.cpu().numpy().view(np.uint16), kernel

    one = setup(gen.random_bcsr(512, 64, 0.2, seed=31), 2048, 41)   # the plan's choice is the sweep kernel
    two = setup(gen.random_bcsr(96, 80, 0.2, seed=32), 264, 42)     # row-wise
    want1, k1 = planned(one)
    want2, k2 = planned(two)
    assert (k1, k2) == (SWEEP, 1)
    s0 = cache_stats(smat)
    for t, want in ((one, want1), (two, want2), (one, want1), (two, want2), (two, want2)):
        assert np.array_equal(drop_in(t), want)
    s1 = cache_stats(smat)
    assert s1["built"] - s0["built"] == 2 and s1["hits"] - s0["hits"] == 3 and s1["entries"] == 2
    assert oracle.compare(want1, oracle_ref(oracle, one["A"], one["B"], one["N"]))[0] <= TOL_F16
    # block values are read by every launch: new values in the same array, same plan, new result
    one["vals"].copy_(to_dev(torch, gen.random_bcsr(512, 64, 0.2, seed=31)["b_val"][::-1].copy(), cuda))
    A1b = dict(one["A"], b_val=one["A"]["b_val"][::-1].copy())
    assert oracle.compare(drop_in(one), oracle_ref(oracle, A1b, one["B"], one["N"]))[0] <= TOL_F16
    assert cache_stats(smat)["built"] == s1["built"]
    # another block pattern written into the same arrays (same number of blocks): the checksum, taken on every
    # call here instead of every 64th, sees it and the plan is made again
    other = gen.random_bcsr(96, 80, 0.0, seed=33, row_lengths=np.diff(two["A"]["b_row_ptr"])[::-1].tolist())
    assert other["nnzb"] == two["A"]["nnzb"] and not np.array_equal(other["b_col_idx"], two["A"]["b_col_idx"])
    two["rp"].copy_(to_dev(torch, other["b_row_ptr"].astype(np.int32), cuda))
    two["ci"].copy_(to_dev(torch, other["b_col_idx"].astype(np.int32), cuda))
    two["vals"].copy_(to_dev(torch, other["b_val"], cuda))
    two["A"] = other
    lib.smat_internal_plan_cache_check_every(C.c_uint64(1))
    got = drop_in(two)
    lib.smat_internal_plan_cache_check_every(C.c_uint64(0))
    assert cache_stats(smat)["rebuilt"] == s1["rebuilt"] + 1
    assert oracle.compare(got, oracle_ref(oracle, other, two["B"], two["N"]))[0] <= TOL_F16
    # the explicit way: clear the cache
    assert lib.smat_plan_cache_clear() == 0 and cache_stats(smat)["entries"] == 0
    # switched off: plain launches of the row-wise kernel, nothing kept
    monkeypatch.setenv("SMAT_PLAN_CACHE", "0")
    b = cache_stats(smat)["built"]
    assert oracle.compare(drop_in(two), oracle_ref(oracle, other, two["B"], two["N"]))[0] <= TOL_F16
    assert cache_stats(smat)["built"] == b and cache_stats(smat)["entries"] == 0
    monkeypatch.delenv("SMAT_PLAN_CACHE")
    # with SMAT_PLAN_CACHE=values the cached plan looks at the values too: a matrix with about one nonzero per block
    # goes through the compact kernel, the same bits as an explicit plan with attached values
    monkeypatch.setenv("SMAT_PLAN_CACHE", "values")
    d = gen.erdos_renyi(2048, 0.004)
    sp = setup(bcsr_of(smat, d), 128, 43)
    Cc, info = gpu_spmm_compact(smat, cuda, sp["A"], sp["B"], 128, kernel=0)
    assert info["kernel"] == COMPACT
    assert np.array_equal(drop_in(sp), Cc)
    lib.smat_plan_cache_clear()


def test_empty_matrix_and_empty_rows_write_zeros(smat, cuda, oracle):
    N = 72
    B = gen.dense_b(64, N, seed=1)
    empty = {"M": 48, "K": 64, "b_row_ptr": np.zeros(4, np.int32), "b_col_idx": np.zeros(0, np.int32),
             "b_val": np.zeros(0, np.uint16)}
    assert not gpu_spmm(smat, cuda, empty, B, N).any()
    assert not gpu_spmm(smat, cuda, empty, B, N, plan=True).any()
    A = gen.random_bcsr(6, 4, 0.0, seed=2, row_lengths=[0, 3, 0, 0, 1, 0])
    ref = oracle_ref(oracle, A, B, N)
    for plan in (False, True):
        C = gpu_spmm(smat, cuda, A, B, N, plan=plan)
        assert oracle.compare(C, ref)[0] <= TOL_F16
        assert not C.reshape(A["M"], N)[0:16].any() and not C.reshape(A["M"], N)[32:64].any()


@pytest.mark.parametrize("lengths", [
    [1, 2, 3, 4, 5, 63, 64, 65, 127, 128, 129, 0],   # odd/even tails, 64-block index refills
    [700, 1, 1, 1, 0, 2, 1, 1, 3, 1, 1, 1, 1, 1, 1, 1],  # one very long row: split by the plan
    [300, 290, 2, 2, 2, 2, 2, 2, 2, 2, 2, 2, 2, 2, 2, 2, 2, 2, 2, 2],  # two long rows
])
def test_skewed_rows_with_and_without_plan(smat, cuda, oracle, lengths):
    kb = max(max(lengths), 8)
    A = gen.random_bcsr(len(lengths), kb, 0.0, seed=len(lengths), row_lengths=lengths)
    N = 88
    B = gen.dense_b(A["K"], N, seed=33)
    ref = oracle_ref(oracle, A, B, N)
    c0 = gpu_spmm(smat, cuda, A, B, N, plan=False)
    c1 = gpu_spmm(smat, cuda, A, B, N, plan=True)
    assert oracle.compare(c0, ref)[0] <= TOL_F16
    assert oracle.compare(c1, ref)[0] <= TOL_F16
    c32 = gpu_spmm(smat, cuda, A, B, N, plan=True, c_f32=True)
    assert rel_err_f32(c32, ref) <= TOL_F32


@pytest.mark.parametrize("kernel", [3, 4])
def test_rowwise_kernel_power_law_rows_dealt_in_short_runs(smat, cuda, oracle, kernel):
    """R-MAT scale 14 through the row-wise kernel with a plan (B read in place, and from the slab-major copy): the
    list has the chunks of the long block rows first, and one run of workgroups per XCD would give the first XCD
    several times the mean, so the launch deals them in short runs.  1, 2 and 4 panels; the fp16 result carries the
    bits of the fp32 one rounded once."""
    import ctypes as C_
    d = gen.rmat(14, 16, seed=34)
    A = bcsr_of(smat, d)
    lens = np.diff(A["b_row_ptr"]).astype(np.int64)
    avg = lens[lens > 0].mean()
    chunk = (max(int(4.0 * avg + 0.5), 64) + 1) & ~1
    assert lens.max() > 2 * chunk                                   # some block row is split
    # the list as the plan builds it (chunks of the split rows, then the other rows), at two more than its pairs per item
    split = [min(chunk, n - b) for n in lens[lens > chunk] for b in range(0, n, chunk)]
    costs = np.array(split + list(lens[lens <= chunk]), np.uint64)
    costs = (costs + np.uint64(1)) // np.uint64(2) + np.uint64(2)
    prefix = np.concatenate([[0], np.cumsum(costs)]).astype(np.uint64)
    choose = smat.lib.smat_internal_choose_xcd_run
    choose.restype, choose.argtypes = C_.c_uint, [C_.c_void_p, C_.c_uint64, C_.c_int]
    for N in (64, 128, 256):
        n_panels = N // 64
        eighth = ((len(costs) * n_panels + 3) // 4 + 7) // 8
        if n_panels < 4:
            assert choose(prefix.ctypes.data, len(costs), n_panels) < eighth
        B = gen.dense_b(A["K"], N, seed=N + 3, dist="uniform")
        ref = oracle_ref(oracle, A, B, N)
        C = gpu_spmm(smat, cuda, A, B, N, plan=True, kernel=kernel)
        assert oracle.compare(C, ref)[0] <= TOL_F16
        C32 = gpu_spmm(smat, cuda, A, B, N, plan=True, kernel=kernel, c_f32=True)
        assert rel_err_f32(C32, ref) <= TOL_F32
        assert np.array_equal(C32.astype(np.float16).view(np.uint16), C)


@pytest.mark.parametrize("N", [32, 40, 64, 88, 128, 264])
def test_short_rows_with_a_plan_match_the_oracle_and_the_general_kernel(smat, cuda, oracle, N):
    """Rows of 0..10 blocks with a plan: the launcher takes the kernel that loads all operands of a row at once.
    Odd and even lengths, single blocks, empty rows, partial last panel (N % 32 != 0 and N % 64 != 0); without
    a plan the general row-wise kernel runs: same pairs, same order of the K = 32 steps, same bits."""
    lengths = [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 10, 1, 0, 9, 2, 10, 3, 0, 0, 7]
    A = gen.random_bcsr(len(lengths), 12, 0.0, seed=77, row_lengths=lengths)
    B = gen.dense_b(A["K"], N, seed=34)
    ref = oracle_ref(oracle, A, B, N)
    c_plan = gpu_spmm(smat, cuda, A, B, N, plan=True)
    assert oracle.compare(c_plan, ref)[0] <= TOL_F16
    assert np.array_equal(c_plan, gpu_spmm(smat, cuda, A, B, N, plan=False))
    c32 = gpu_spmm(smat, cuda, A, B, N, plan=True, c_f32=True)
    assert rel_err_f32(c32, ref) <= TOL_F32
    assert np.array_equal(c32, gpu_spmm(smat, cuda, A, B, N, plan=False, c_f32=True))


def test_rows_of_eleven_blocks_stay_with_the_general_kernel(smat, cuda, oracle):
    lengths = [11, 3, 10, 0, 1]
    A = gen.random_bcsr(len(lengths), 12, 0.0, seed=78, row_lengths=lengths)
    N = 64
    B = gen.dense_b(A["K"], N, seed=35)
    assert oracle.compare(gpu_spmm(smat, cuda, A, B, N, plan=True), oracle_ref(oracle, A, B, N))[0] <= TOL_F16


def test_plan_splits_long_rows(smat, cuda):
    lengths = [700] + [1] * 15
    A = gen.random_bcsr(16, 700, 0.0, seed=3, row_lengths=lengths)
    p = smat.Plan(A["b_row_ptr"], A["M"], A["K"], A["nnzb"], 64)
    info = p.info()
    p.close()
    assert info["split_rows"] == 1 and info["items"] > 16 and info["workspace_bytes"] > 0


SWEEP = 2


@pytest.mark.parametrize("mb,kb,density,N", [
    (9, 13, 0.35, 128),     # fewer block rows than one row group, one partial K chunk
    (40, 40, 0.15, 136),    # partial last panel, partial last row group
    (64, 33, 0.10, 256),    # K = 528: last chunk is 1 slab wide
    (33, 70, 0.05, 520),    # sparse enough that wavefronts get filler ops and blocks pair across chunks
    (32, 16, 1.00, 128),    # fully dense: every op is a pair
    (35, 3, 0.60, 8),       # narrowest N, K = 48: one partial chunk, most of the panel unused
    (70, 20, 0.30, 72),     # N just above one panel
    (130, 160, 1.00, 64),   # dense, ten chunks: 64 ops per wavefront and chunk, several descriptor windows
    (200, 300, 0.12, 192),  # four row groups, 19 chunks: the ring of stages wraps several times
    (64, 16, 0.50, 38408),  # 601 tiles on 256 CUs: a workgroup takes two or three tiles one after the other, last panel partial
    (140, 20, 0.30, 12808), # three row groups x 201 panels = 603 tiles, rounded up to 608 workgroup ids: ids without a tile
])
def test_sweep_kernel_matches_oracle(smat, cuda, oracle, mb, kb, density, N):
    A = gen.random_bcsr(mb, kb, density, seed=1000 + mb + kb)
    B = gen.dense_b(A["K"], N, seed=2000 + N, dist="normal")
    ref = oracle_ref(oracle, A, B, N)
    C = gpu_spmm(smat, cuda, A, B, N, plan=True, kernel=SWEEP)
    assert oracle.compare(C, ref)[0] <= TOL_F16
    C32 = gpu_spmm(smat, cuda, A, B, N, plan=True, kernel=SWEEP, c_f32=True)
    assert rel_err_f32(C32, ref) <= TOL_F32
    assert np.array_equal(C32.astype(np.float16).view(np.uint16), C)


def test_sweep_kernel_skewed_and_empty_rows(smat, cuda, oracle):
    lengths = [0, 90, 1, 0, 0, 3, 2, 64, 0, 17] + [0] * 30 + [5, 90]
    A = gen.random_bcsr(len(lengths), 90, 0.0, seed=4, row_lengths=lengths)
    N = 264
    B = gen.dense_b(A["K"], N, seed=8)
    ref = oracle_ref(oracle, A, B, N)
    C = gpu_spmm(smat, cuda, A, B, N, plan=True, kernel=SWEEP)
    assert oracle.compare(C, ref)[0] <= TOL_F16
    assert not C.reshape(A["M"], N)[0:16].any()


def test_unsorted_block_columns_take_the_row_wise_kernel(smat, cuda, oracle):
    """Block columns in descending order inside the block rows: the kernel choice left to the plan falls back to the
    row-wise kernel (which, like the reference, does not care about the order) instead of the sweep kernel."""
    A = gen.random_bcsr(512, 64, 0.2, seed=77)
    rp = A["b_row_ptr"]
    ci, val = A["b_col_idx"].copy(), A["b_val"].reshape(-1, 256).copy()
    for i in range(A["M"] // 16):
        ci[rp[i]:rp[i + 1]] = ci[rp[i]:rp[i + 1]][::-1]
        val[rp[i]:rp[i + 1]] = val[rp[i]:rp[i + 1]][::-1]
    N = 2048  # 8 row groups x 32 panels: the sweep kernel would be the plan's choice for ascending columns
    B = gen.dense_b(A["K"], N, seed=5)
    ref = oracle_ref(oracle, A, B, N)
    p = smat.Plan(rp, A["M"], A["K"], A["nnzb"], N, col_idx_host=A["b_col_idx"])
    assert p.info()["kernel"] == SWEEP
    p.close()
    p = smat.Plan(rp, A["M"], A["K"], A["nnzb"], N, col_idx_host=ci)
    assert p.info()["kernel"] == 1
    p.close()
    Ar = dict(A, b_col_idx=ci, b_val=val.reshape(-1))
    C = gpu_spmm(smat, cuda, Ar, B, N, plan=True)
    assert oracle.compare(C, ref)[0] <= TOL_F16


def test_sweep_kernel_keeps_non_finite_values_inside_their_block_row(smat, cuda, oracle):
    """An unpaired block shares its MFMA with a neighbouring block times zeros, a filler op multiplies two blocks by
    zeros: the plan takes those blocks from the same block row, so Inf in the values of one block row (times zero:
    NaN) does not reach any other row of C.  Every third block row is all Inf here; the others must come out as
    the oracle computes them (every row has at least two blocks)."""
    rng = np.random.default_rng(9)
    lengths = rng.integers(2, 9, size=130).tolist()  # few blocks per row over 100 block columns: many unpaired blocks and fillers
    A = gen.random_bcsr(130, 100, 0.0, seed=21, row_lengths=lengths)
    N = 128
    B = gen.dense_b(A["K"], N, seed=22, dist="normal")
    ref = oracle_ref(oracle, A, B, N).reshape(A["M"], N)
    val = A["b_val"].reshape(-1, 256).copy()
    rp = A["b_row_ptr"]
    bad_rows = np.arange(1, 130, 3)
    for r in bad_rows:
        val[rp[r]:rp[r + 1]] = 0x7C00  # +Inf
    Ainf = dict(A, b_val=val.reshape(-1))
    p = smat.Plan(rp, A["M"], A["K"], A["nnzb"], N, col_idx_host=A["b_col_idx"], kernel=SWEEP)
    info = p.info()
    p.close()
    assert info["sweep_ops"] > 0
    C = gpu_spmm(smat, cuda, Ainf, B, N, plan=True, kernel=SWEEP).reshape(A["M"], N)
    good = np.ones(A["M"], bool)
    for r in bad_rows:
        good[r * 16:r * 16 + 16] = False
    assert np.isfinite(C[good].view(np.float16)).all()
    assert oracle.compare(np.ascontiguousarray(C[good]), np.ascontiguousarray(ref[good]))[0] <= TOL_F16
    assert not np.isfinite(C[~good].view(np.float16)).any()  # Inf x B: Inf or NaN, as a block-by-block product gives


def test_sweep_needs_a_plan_with_col_idx(smat, cuda):
    A = gen.random_bcsr(4, 4, 0.5, seed=1)
    with pytest.raises(smat.SmatError):
        smat.Plan(A["b_row_ptr"], A["M"], A["K"], A["nnzb"], 128, col_idx_host=None, kernel=SWEEP)


def test_sweep_refuses_what_it_cannot_address(smat, cuda):
    """The sweep kernel addresses blocks in pairs and B with 32-bit offsets inside four columns: a single
    block is refused when the plan is made, K >= 2^28 at the launch (the buffers here are dummies that are
    never touched)."""
    import torch
    rp = np.array([0, 1], np.int32)
    ci = np.array([0], np.int32)
    with pytest.raises(smat.SmatError):
        smat.Plan(rp, 16, 64, 1, 128, col_idx_host=ci, kernel=SWEEP)
    M, K, N = 16, 1 << 28, 64
    rp = np.array([0, 2], np.int32)
    ci = np.array([0, 16], np.int32)
    plan = smat.Plan(rp, M, K, 2, 64, col_idx_host=ci, kernel=SWEEP)
    dummy = torch.zeros(4096, dtype=torch.int16, device=cuda)
    with pytest.raises(smat.SmatError):
        smat.spmm(dummy, to_dev(torch, rp, cuda), to_dev(torch, ci, cuda), dummy, dummy, M, N, K, 2, plan=plan, kernel=SWEEP)
    plan.close()


def test_b_ones_gives_row_sums(smat, cuda, oracle):
    # the reference fills B with 1.0 (common/matrix.h:38): every column of C is the row sum of A
    A = gen.random_bcsr(12, 12, 0.4, seed=77)
    N = 48
    B = np.full(A["K"] * N, 0x3C00, dtype=np.uint16)
    C = gpu_spmm(smat, cuda, A, B, N, c_f32=True)
    rp, ci, v = gen.bcsr_to_csr(A["M"], A["b_row_ptr"], A["b_col_idx"], A["b_val"])
    sums = np.zeros(A["M"], dtype=np.float64)
    np.add.at(sums, np.repeat(np.arange(A["M"]), np.diff(rp)), v.view(np.float16).astype(np.float64))
    assert np.allclose(C, sums[:, None], rtol=0, atol=1e-4)
    assert (C == C[:, :1]).all()


def test_config1_band_full_size(smat, cuda, oracle):
    d = gen.band(4096, 64)
    A = smat.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
    assert A.nnzb == 2284
    Ad = {"M": A.M, "K": A.K, "b_row_ptr": A.row_ptr, "b_col_idx": A.col_idx, "b_val": A.val}
    N = 128
    B = gen.dense_b(A.K, N, seed=0xB0000001, dist="uniform")
    ref = oracle.spmm_csr(d["M"], N, d["K"], d["row_ptr"], d["col_idx"], d["val"], B)  # from CSR: independent of blocking
    for plan in (False, True):
        C = gpu_spmm(smat, cuda, Ad, B, N, plan=plan)
        assert oracle.compare(C, ref)[0] <= TOL_F16


def test_config5_stencil_reduced_and_reordered(smat, cuda, oracle):
    d = gen.stencil27(16)  # 4096 rows
    N = 64
    B = gen.dense_b(d["K"], N, seed=0xB0000005, dist="uniform")
    ref = oracle.spmm_csr(d["M"], N, d["K"], d["row_ptr"], d["col_idx"], d["val"], B)
    A = smat.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
    Ad = {"M": A.M, "K": A.K, "b_row_ptr": A.row_ptr, "b_col_idx": A.col_idx, "b_val": A.val}
    C = gpu_spmm(smat, cuda, Ad, B, N, plan=True)
    assert oracle.compare(C, ref)[0] <= TOL_F16
    # reordered: P_r A P_c^T applied to P_c B gives P_r C
    pr, pc, _, _ = smat.reorder_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"])
    rp2, ci2, v2 = smat.permute_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], pr, pc)
    A2 = smat.csr_to_bcsr(d["M"], d["K"], rp2, ci2, v2)
    Bm = B.reshape(N, d["K"])
    B2 = np.ascontiguousarray(Bm[:, pc]).ravel()
    A2d = {"M": A2.M, "K": A2.K, "b_row_ptr": A2.row_ptr, "b_col_idx": A2.col_idx, "b_val": A2.val}
    C2 = gpu_spmm(smat, cuda, A2d, B2, N, plan=True)
    assert oracle.compare(C2, ref[pr])[0] <= TOL_F16


def test_plan_takes_the_sweep_kernel_only_when_it_fills_the_device(smat, cuda, oracle):
    import torch
    # 32 groups of 64 block rows, 10 % of the blocks: 8 panels of 64 columns make 256 workgroups
    A = gen.random_bcsr(2048, 32, 0.10, seed=77)
    M, K, nnzb = A["M"], A["K"], A["nnzb"]
    wide = smat.Plan(A["b_row_ptr"], M, K, nnzb, 512, col_idx_host=A["b_col_idx"])
    narrow = smat.Plan(A["b_row_ptr"], M, K, nnzb, 384, col_idx_host=A["b_col_idx"])
    assert wide.info()["kernel"] == SWEEP and narrow.info()["kernel"] == 1
    narrow.close()
    # too sparse (2 % of the blocks): row-wise whatever the width
    S = gen.random_bcsr(2048, 32, 0.02, seed=78)
    sparse = smat.Plan(S["b_row_ptr"], S["M"], S["K"], S["nnzb"], 512, col_idx_host=S["b_col_idx"])
    assert sparse.info()["kernel"] == 1
    sparse.close()
    # the plan made for N = 512, used with N = 512 (sweep) and with N = 128 (falls back to row-wise)
    vals, rp, ci = (to_dev(torch, A[k], cuda) for k in ("b_val", "b_row_ptr", "b_col_idx"))
    for N in (512, 128):
        B = gen.dense_b(K, N, seed=5 + N)
        C = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
        smat.spmm(vals, rp, ci, to_dev(torch, B, cuda), C, M, N, K, nnzb, plan=wide)
        torch.cuda.synchronize()
        rows = slice(0, 16 * 40)
        sub = {"M": 16 * 40, "K": K, "b_row_ptr": A["b_row_ptr"][:41], "b_col_idx": A["b_col_idx"][:A["b_row_ptr"][40]],
               "b_val": A["b_val"][:A["b_row_ptr"][40] * 256]}
        ref = oracle_ref(oracle, sub, B, N)
        assert oracle.compare(C.cpu().numpy().view(np.uint16)[rows], ref)[0] <= TOL_F16
    wide.close()


def test_config4_block_pruned_full_size_sampled_rows(smat, cuda, oracle):
    A = gen.block_pruned(8192, 0.10, 0.02)
    assert A["nnzb"] == 26214
    N = 4096
    B = gen.dense_b(8192, N, seed=0xB0000004, dist="normal")
    C = gpu_spmm(smat, cuda, A, B, N, plan=True, kernel=1).reshape(8192, N)
    # oracle on a sample of block rows (the full product is ~3e10 MACs on the CPU)
    rows = [0, 1, 17, 255, 256, 300, 511]
    rp = A["b_row_ptr"]
    sel = np.concatenate([np.arange(rp[r], rp[r + 1]) for r in rows])
    sub = {"M": 16 * len(rows), "K": 8192,
           "b_row_ptr": np.concatenate([[0], np.cumsum([rp[r + 1] - rp[r] for r in rows])]).astype(np.int32),
           "b_col_idx": A["b_col_idx"][sel],
           "b_val": A["b_val"].reshape(-1, 256)[sel].ravel()}
    ref = oracle_ref(oracle, sub, B, N)
    got = np.concatenate([C[16 * r:16 * r + 16] for r in rows])
    assert oracle.compare(got, ref)[0] <= TOL_F16
    # size-independent property: an independent launch without a plan gives the identical bits
    C2 = gpu_spmm(smat, cuda, A, B, N, plan=False).reshape(8192, N)
    assert np.array_equal(C, C2)
    # the sweep kernel (the plan's own choice for this matrix) pairs blocks differently, so its
    # fp32 sums may round differently: same tolerance against the oracle, and close to the other kernel
    C3 = gpu_spmm(smat, cuda, A, B, N, plan=True).reshape(8192, N)
    got3 = np.concatenate([C3[16 * r:16 * r + 16] for r in rows])
    assert oracle.compare(got3, ref)[0] <= TOL_F16
    d = np.abs(C3.view(np.float16).astype(np.float32) - C.view(np.float16).astype(np.float32)).max()
    assert d <= 2e-3 * np.abs(C.view(np.float16).astype(np.float32)).max()


def test_sweep_kernel_gives_the_same_bits_on_every_launch(smat, cuda):
    """The sweep kernel reuses an operand register set for the next op's LDS reads a few instructions after the
    MFMAs that read it were issued, and a workgroup reuses its LDS stages for its next tile: a late read or an
    early overwrite would show as launches of the same product that differ.  Headline size, 24 launches with one
    plan into fresh outputs, all compared bit for bit with the first."""
    import torch
    A = gen.block_pruned(8192, 0.10, 0.02)
    N = 4096
    B = gen.dense_b(8192, N, seed=0xB0000004, dist="normal")
    M, K, nnzb = A["M"], A["K"], A["nnzb"]
    vals, Bd = to_dev(torch, A["b_val"], cuda), to_dev(torch, B, cuda)
    rp, ci = to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda), to_dev(torch, A["b_col_idx"].astype(np.int32), cuda)
    p = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=SWEEP)
    first = None
    for launch in range(24):
        C = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
        smat.spmm(vals, rp, ci, Bd, C, M, N, K, nnzb, plan=p, kernel=SWEEP)
        torch.cuda.synchronize()
        if first is None:
            first = C
        else:
            assert torch.equal(C, first), f"launch {launch} differs from the first"
    p.close()


COMPACT = 5


def gpu_spmm_compact(smat, cuda, A, B_bits, N, c_f32=False, kernel=COMPACT, n_hint=None):
    """SpMM through a plan that has looked at the zero pattern of the values."""
    import torch
    M, K, nnzb = A["M"], A["K"], int(A["b_col_idx"].shape[0])
    vals = to_dev(torch, A["b_val"] if nnzb else np.zeros(8, np.uint16), cuda)
    rp = to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda)
    ci = to_dev(torch, A["b_col_idx"].astype(np.int32) if nnzb else np.zeros(1, np.int32), cuda)
    B = to_dev(torch, B_bits, cuda)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device=cuda) if c_f32 else \
        torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    p = smat.Plan(A["b_row_ptr"], M, K, nnzb, n_hint or N, col_idx_host=A["b_col_idx"], kernel=kernel)
    p.attach_values(vals, rp, ci)
    info = p.info()
    smat.spmm(vals, rp, ci, B, C, M, N, K, nnzb, plan=p, c_f32=c_f32, kernel=kernel)
    torch.cuda.synchronize()
    out = C.cpu().numpy()
    p.close()
    return (out if c_f32 else out.view(np.uint16)), info


def bcsr_of(smat, d):
    b = smat.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
    return {"M": b.M, "K": b.K, "b_row_ptr": b.row_ptr, "b_col_idx": b.col_idx, "b_val": b.val, "nnzb": b.nnzb}


@pytest.mark.parametrize("N", [8, 64, 72, 128, 264, 520])
def test_compact_kernel_sparse_blocks(smat, cuda, oracle, N):
    d = gen.erdos_renyi(1024, 0.004, seed=31 + N)          # about one nonzero per block
    A = bcsr_of(smat, d)
    B = gen.dense_b(A["K"], N, seed=N + 11, dist="normal")
    ref = oracle_ref(oracle, A, B, N)
    C, info = gpu_spmm_compact(smat, cuda, A, B, N)
    nz_cols = len(set(zip((np.repeat(np.arange(d["M"]), np.diff(d["row_ptr"])) // 16).tolist(), d["col_idx"].tolist())))
    assert info["compact_cols"] == nz_cols                  # one list entry per nonzero (block row, column)
    assert oracle.compare(C, ref)[0] <= TOL_F16
    C32, _ = gpu_spmm_compact(smat, cuda, A, B, N, c_f32=True)
    assert rel_err_f32(C32, ref) <= TOL_F32
    assert np.array_equal(C32.astype(np.float16).view(np.uint16), C)


def test_compact_kernel_dense_blocks_split_rows_and_auto(smat, cuda, oracle):
    # dense blocks (every column nonzero), one very long block row (split into chunks), empty rows
    lengths = [0, 300, 1, 0, 2, 0, 0, 7] + [3] * 24
    A = gen.random_bcsr(len(lengths), 320, 0.0, seed=6, row_lengths=lengths)
    N = 136
    B = gen.dense_b(A["K"], N, seed=2)
    ref = oracle_ref(oracle, A, B, N)
    C, info = gpu_spmm_compact(smat, cuda, A, B, N)
    assert info["compact_cols"] == 16 * A["nnzb"]
    assert oracle.compare(C, ref)[0] <= TOL_F16
    assert not C.reshape(A["M"], N)[0:16].any()
    # with SMAT_KERNEL_AUTO the plan keeps a dense kernel for dense blocks and takes the compact one for sparse blocks
    _, info_auto = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0)
    assert info_auto["kernel"] != COMPACT
    d = gen.rmat(11, 8, seed=3)
    As = bcsr_of(smat, d)
    Bs = gen.dense_b(As["K"], 128, seed=4, dist="uniform")
    Cs, info_s = gpu_spmm_compact(smat, cuda, As, Bs, 128, kernel=0, n_hint=256)
    assert info_s["kernel"] == COMPACT
    assert oracle.compare(Cs, oracle_ref(oracle, As, Bs, 128))[0] <= TOL_F16


def test_compact_kernel_needs_attached_values(smat, cuda):
    import torch
    A = gen.random_bcsr(4, 4, 0.5, seed=1)
    p = smat.Plan(A["b_row_ptr"], A["M"], A["K"], A["nnzb"], 64, col_idx_host=A["b_col_idx"])
    t = torch.zeros(A["M"] * 64, dtype=torch.int16, device=cuda)
    with pytest.raises(smat.SmatError, match="attach"):
        smat.spmm(t, t, t, t, t, A["M"], 64, A["K"], A["nnzb"], plan=p, kernel=COMPACT)
    p.close()


def test_compact_kernel_row_major_b(smat, cuda, oracle):
    """Row-major B (B[k*N + n]) skips the per-launch copy: same bits as with the reference layout."""
    import torch
    d = gen.erdos_renyi(2048, 0.003, seed=8)
    A = bcsr_of(smat, d)
    N = 200
    B = gen.dense_b(A["K"], N, seed=5, dist="normal")                      # column-major bits
    B_rm = np.ascontiguousarray(B.reshape(N, A["K"]).T).ravel()           # the same matrix, row-major
    M, K, nnzb = A["M"], A["K"], A["nnzb"]
    vals, rp, ci = to_dev(torch, A["b_val"], cuda), to_dev(torch, A["b_row_ptr"], cuda), to_dev(torch, A["b_col_idx"], cuda)
    p = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=COMPACT)
    p.attach_values(vals, rp, ci)
    out = []
    for bits, rm in ((B, False), (B_rm, True)):
        C = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
        smat.spmm(vals, rp, ci, to_dev(torch, bits, cuda), C, M, N, K, nnzb, plan=p, kernel=COMPACT, b_row_major=rm)
        torch.cuda.synchronize()
        out.append(C.cpu().numpy().view(np.uint16))
    assert np.array_equal(out[0], out[1])
    assert oracle.compare(out[0], oracle_ref(oracle, A, B, N))[0] <= TOL_F16
    with pytest.raises(smat.SmatError, match="row-major"):  # the dense kernels need a plan made for row-major B
        C = torch.zeros((M, N), dtype=torch.int16, device=cuda)
        smat.spmm(vals, rp, ci, to_dev(torch, B_rm, cuda), C, M, N, K, nnzb, plan=p, kernel=1, b_row_major=True)
    p.close()


@pytest.mark.parametrize("kernel", [1, 2, 3, 4])
def test_row_major_b_dense_kernels_bit_identical(smat, cuda, oracle, kernel):
    """Row-major B with the row-wise and sweep kernels: the same bits as the reference layout gives."""
    import torch
    A = gen.random_bcsr(70, 45, 0.2, seed=77)
    M, K, nnzb, N = A["M"], A["K"], A["nnzb"], 136
    B = gen.dense_b(K, N, seed=78, dist="normal")
    B_rm = np.ascontiguousarray(B.reshape(N, K).T).ravel()
    vals, rp, ci = to_dev(torch, A["b_val"], cuda), to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda), to_dev(torch, A["b_col_idx"].astype(np.int32), cuda)
    out = []
    for bits, rm in ((B, False), (B_rm, True)):
        p = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=kernel, b_row_major=rm)
        C = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
        smat.spmm(vals, rp, ci, to_dev(torch, bits, cuda), C, M, N, K, nnzb, plan=p, kernel=kernel, b_row_major=rm)
        torch.cuda.synchronize()
        out.append(C.cpu().numpy().view(np.uint16))
        p.close()
    assert np.array_equal(out[0], out[1])
    assert oracle.compare(out[0], oracle_ref(oracle, A, B, N))[0] <= TOL_F16


def test_compact_kernel_config2_full_size(smat, cuda, oracle):
    """Config 2 at its real size (16384 x 16384, 0.1 %, N = 256), whole result against the oracle."""
    d = gen.erdos_renyi(16384, 0.001)
    A = bcsr_of(smat, d)
    N = 256
    B = gen.dense_b(A["K"], N, seed=0xB0000002, dist="normal")
    C, info = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0)
    assert info["kernel"] == COMPACT and info["compact_cols"] <= int(d["row_ptr"][-1])
    assert oracle.compare(C, oracle_ref(oracle, A, B, N))[0] <= TOL_F16


@pytest.mark.parametrize("tq", [1, 2])
def test_compact_kernel_every_panel_width(smat, cuda, oracle, tq):
    """The compact kernel gathers the rows of B in two ways, by panel width (64 or 128 columns); the launcher
    picks the width from the sizes, so small inputs would only ever see the first.  Each is forced in turn here on the
    same inputs: N that ends inside a panel (at any multiple of 8 columns), fp16 and fp32 results, a block row
    long enough to be split (partial tiles through the workspace), empty rows, B row-major read in place."""
    import ctypes as C_
    import torch
    lib = smat.lib
    lib.smat_internal_compact_panel.argtypes = [C_.c_int]
    lib.smat_internal_compact_panel.restype = None
    lib.smat_internal_compact_panel(tq)
    try:
        d = gen.erdos_renyi(1024, 0.004, seed=77)               # about one nonzero per block, 1 to 3 steps per block row
        A = bcsr_of(smat, d)
        for N in (8, 72, 136, 264, 520):
            B = gen.dense_b(A["K"], N, seed=N + 5, dist="normal")
            ref = oracle_ref(oracle, A, B, N)
            C, _ = gpu_spmm_compact(smat, cuda, A, B, N)
            assert oracle.compare(C, ref)[0] <= TOL_F16
            C32, _ = gpu_spmm_compact(smat, cuda, A, B, N, c_f32=True)
            assert rel_err_f32(C32, ref) <= TOL_F32
            assert np.array_equal(C32.astype(np.float16).view(np.uint16), C)
        lengths = [0, 300, 1, 0, 2, 0, 0, 7] + [3] * 24         # dense blocks, one block row of 150 steps (split), empty rows
        A = gen.random_bcsr(len(lengths), 320, 0.0, seed=6, row_lengths=lengths)
        for N in (136, 392):
            B = gen.dense_b(A["K"], N, seed=2 + N)
            ref = oracle_ref(oracle, A, B, N)
            C, _ = gpu_spmm_compact(smat, cuda, A, B, N)
            assert oracle.compare(C, ref)[0] <= TOL_F16
            assert not C.reshape(A["M"], N)[0:16].any()
        # B row-major, read in place: the same bits as with the column-major B of the same values
        d = gen.rmat(11, 8, seed=3)
        A = bcsr_of(smat, d)
        N, M, K, nnzb = 200, A["M"], A["K"], A["nnzb"]
        B = gen.dense_b(K, N, seed=4, dist="uniform")
        C_col, _ = gpu_spmm_compact(smat, cuda, A, B, N)
        B_row = np.ascontiguousarray(B.reshape(N, K).T).reshape(-1)
        vals, rp, ci = (to_dev(torch, A["b_val"], cuda), to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda),
                        to_dev(torch, A["b_col_idx"].astype(np.int32), cuda))
        Bd = to_dev(torch, B_row, cuda)
        Cd = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
        p = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=COMPACT)
        p.attach_values(vals, rp, ci)
        smat.spmm(vals, rp, ci, Bd, Cd, M, N, K, nnzb, plan=p, kernel=COMPACT, b_row_major=True)
        torch.cuda.synchronize()
        p.close()
        assert np.array_equal(Cd.cpu().numpy().view(np.uint16), C_col)
        assert oracle.compare(C_col, oracle_ref(oracle, A, B, N))[0] <= TOL_F16
    finally:
        lib.smat_internal_compact_panel(0)


def test_compact_kernel_every_item_length_up_to_twenty_steps(smat, cuda, oracle):
    """Block row r has 2 (r + 1) dense blocks = r + 1 steps of 32 columns: every item length from 1 to 20 steps, so
    that an item ends at every position of the kernel's blocks of 8 steps (7, 8, 9, 15, 16, 17 ...), on both panel
    widths and with rows of B that the index loads past the end of an item still have to find valid."""
    import ctypes as C_
    lengths = [2 * (r + 1) for r in range(20)]
    A = gen.random_bcsr(len(lengths), 48, 0.0, seed=14, row_lengths=lengths)
    lib = smat.lib
    lib.smat_internal_compact_panel.argtypes = [C_.c_int]
    lib.smat_internal_compact_panel.restype = None
    try:
        for tq in (1, 2):
            lib.smat_internal_compact_panel(tq)
            for N in (64, 200):
                B = gen.dense_b(A["K"], N, seed=N + tq, dist="normal")
                C32, info = gpu_spmm_compact(smat, cuda, A, B, N, c_f32=True)
                assert info["compact_cols"] == 16 * A["nnzb"]
                assert rel_err_f32(C32, oracle_ref(oracle, A, B, N)) <= TOL_F32
    finally:
        lib.smat_internal_compact_panel(0)


def test_compact_kernel_power_law_rows(smat, cuda, oracle):
    """R-MAT scale 15: block rows of very different length, the longest split into chunks."""
    d = gen.rmat(15, 16, seed=21)
    A = bcsr_of(smat, d)
    N = 128
    B = gen.dense_b(A["K"], N, seed=9, dist="uniform")
    C, info = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0)
    assert info["kernel"] == COMPACT
    assert oracle.compare(C, oracle_ref(oracle, A, B, N))[0] <= TOL_F16
    # linearity in B, a size-independent property: A (2 B) = 2 (A B) bit for bit in the fp32 output
    # (scaling by two is exact in every product and every partial sum)
    B2 = (B.view(np.float16) * np.float16(2)).view(np.uint16)
    C32, _ = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0, c_f32=True)
    C32_2, _ = gpu_spmm_compact(smat, cuda, A, B2, N, kernel=0, c_f32=True)
    assert np.array_equal(C32 * np.float32(2), C32_2)


def test_compact_kernel_same_bits_however_the_items_are_dealt_to_the_xcds(smat, cuda, oracle):
    """The launch deals its workgroups to the XCDs in runs whose length it picks from the cost of the items (one
    run per XCD where that is balanced, short runs on lists like this one, R-MAT with its long block rows first).
    The deal decides where an item runs, never what it computes: every run length gives the bits of the launcher's
    own choice, on 1, 2 and 5 panels, with the split rows' partial tiles, and with a grid that the rounding to whole
    runs makes larger than the work."""
    import ctypes as C_
    lib = smat.lib
    lib.smat_internal_compact_run.argtypes, lib.smat_internal_compact_run.restype = [C_.c_int], None
    d = gen.rmat(14, 16, seed=33)
    A = bcsr_of(smat, d)
    rows = np.repeat(np.arange(d["M"], dtype=np.int64), np.diff(d["row_ptr"]))
    per_row = np.bincount(np.unique((rows // 16) * d["K"] + d["col_idx"]) // d["K"])   # nonzero columns per block row
    assert per_row.max() > max(4 * per_row[per_row > 0].mean(), 512) + 32                # some block row is split
    try:
        for N in (64, 128, 264):
            B = gen.dense_b(A["K"], N, seed=N + 1, dist="uniform")
            lib.smat_internal_compact_run(0)
            C, _ = gpu_spmm_compact(smat, cuda, A, B, N)
            assert oracle.compare(C, oracle_ref(oracle, A, B, N))[0] <= TOL_F16
            for run in (1, 3, 4, 16, 50, 64, 256, 1 << 20):
                lib.smat_internal_compact_run(run)
                C_run, _ = gpu_spmm_compact(smat, cuda, A, B, N)
                assert np.array_equal(C_run, C), (N, run)
    finally:
        lib.smat_internal_compact_run(0)


def test_attaching_values_times_the_deal_and_the_result_does_not_depend_on_it(smat, cuda, oracle):
    """smat_plan_attach_values times a few launches on zeros with different run lengths of the deal to the XCDs and
    keeps the fastest for launches at the plan's width.  Whatever it keeps is one of its candidates (the estimate's
    choice, an eighth of the launch, a half or a quarter of that), other widths go by the estimate, and the bits are
    those of a plan that measured nothing."""
    import ctypes as C_
    lib = smat.lib
    lib.smat_internal_compact_tune.argtypes, lib.smat_internal_compact_tune.restype = [C_.c_int], None
    lib.smat_internal_compact_last_run.restype = C_.c_int
    A = bcsr_of(smat, gen.erdos_renyi(4096, 0.004, seed=79))    # 256 block rows of about 16 steps
    n_items = A["M"] // 16
    try:
        for n_hint, N in ((256, 256), (512, 512), (512, 264)):
            B = gen.dense_b(A["K"], N, seed=N + 11, dist="normal")
            lib.smat_internal_compact_tune(0)
            C_plain, _ = gpu_spmm_compact(smat, cuda, A, B, N, n_hint=n_hint)
            run_plain = lib.smat_internal_compact_last_run()
            lib.smat_internal_compact_tune(1)
            C_timed, _ = gpu_spmm_compact(smat, cuda, A, B, N, n_hint=n_hint)
            run_timed = lib.smat_internal_compact_last_run()
            assert np.array_equal(C_timed, C_plain)
            assert oracle.compare(C_timed, oracle_ref(oracle, A, B, N))[0] <= TOL_F16
            eighth = ((n_items * ((N + 63) // 64) + 3) // 4 + 7) // 8
            assert run_plain == eighth                           # rows of one length: one run per XCD by the estimate
            if N == n_hint:
                assert run_timed in (eighth, eighth // 2, eighth // 4)
            else:
                assert run_timed == run_plain                    # measured for 512 columns, launched with 264
    finally:
        lib.smat_internal_compact_tune(1)


def test_plan_check_tells_patterns_apart(smat, cuda):
    """Two matrices of the same M, K and nnzb: the launch cannot tell them apart, smat_plan_check can."""
    A = gen.random_bcsr(20, 24, 0.25, seed=41)
    nnzb = A["nnzb"]
    ci2 = A["b_col_idx"].copy()
    ci2[0] = (ci2[0] + 16) % A["K"] if nnzb == 1 or (ci2[0] + 16) % A["K"] != ci2[1] else (ci2[0] + 32) % A["K"]
    plan = smat.Plan(A["b_row_ptr"], A["M"], A["K"], nnzb, 64, col_idx_host=A["b_col_idx"])
    plan.check(A["b_row_ptr"], A["b_col_idx"], A["M"], A["K"], nnzb)
    with pytest.raises(smat.SmatError, match="another block pattern"):
        plan.check(A["b_row_ptr"], ci2, A["M"], A["K"], nnzb)
    with pytest.raises(smat.SmatError, match="pass it"):
        plan.check(A["b_row_ptr"], None, A["M"], A["K"], nnzb)
    with pytest.raises(smat.SmatError, match="M/K/nnzb"):
        plan.check(A["b_row_ptr"], A["b_col_idx"], A["M"], A["K"] + 16, nnzb)
    plan.close()
    plan = smat.Plan(A["b_row_ptr"], A["M"], A["K"], nnzb, 64)  # made without column indices: row pointer only
    plan.check(A["b_row_ptr"], None, A["M"], A["K"], nnzb)
    plan.check(A["b_row_ptr"], ci2, A["M"], A["K"], nnzb)
    rp2 = A["b_row_ptr"].copy()
    i = int(np.argmax(np.diff(rp2) > 0))
    rp2[i + 1] -= 1 if i + 1 < rp2.size - 1 else 0
    if not np.array_equal(rp2, A["b_row_ptr"]):
        with pytest.raises(smat.SmatError, match="another block pattern"):
            plan.check(rp2, None, A["M"], A["K"], nnzb)
    plan.close()


MIXED = 6


def test_mixed_dispatch_half_dense_half_sparse_rows(smat, cuda, oracle):
    """Half the block rows hold dense blocks, half about one nonzero per block: the plan splits them at attach
    time, the row-wise kernel takes the first kind, the compact kernel the second, and C is whole."""
    A = gen.half_pruned_half_er(2048, 0.15, 0.004, seed=91)
    M, K, nnzb = A["M"], A["K"], A["nnzb"]
    N = 264
    B = gen.dense_b(K, N, seed=92, dist="normal")
    ref = oracle_ref(oracle, A, B, N)
    # left to itself the plan does not split a matrix this small: the dense rows are too few for the sweep kernel, and
    # the row-wise kernel (an extra launch, B in place) would not beat the compact kernel on them
    C_auto, info_auto = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0)
    assert info_auto["kernel"] == COMPACT and info_auto["mixed_dense_blocks"] == 0
    assert oracle.compare(C_auto, ref)[0] <= TOL_F16
    C, info = gpu_spmm_compact(smat, cuda, A, B, N, kernel=MIXED)   # the split asked for
    assert info["kernel"] == MIXED
    assert info["mixed_dense_blocks"] == A["dense_blocks"] and 0 < info["mixed_dense_items"] <= M // 32 + 8
    assert 0 < info["compact_cols"] < 3 * (nnzb - A["dense_blocks"])  # the list holds the sparse rows only
    assert oracle.compare(C, ref)[0] <= TOL_F16
    C32, _ = gpu_spmm_compact(smat, cuda, A, B, N, kernel=MIXED, c_f32=True)
    assert rel_err_f32(C32, ref) <= TOL_F32
    # each single kernel on the same matrix: same tolerance, and the rows each kernel of the mixed plan wrote
    # carry exactly the bits that kernel writes alone (same work items, same arithmetic)
    C_row, _ = gpu_spmm_compact(smat, cuda, A, B, N, kernel=1)
    C_cmp, _ = gpu_spmm_compact(smat, cuda, A, B, N, kernel=COMPACT)
    half = M // 2
    assert np.array_equal(C[:half], C_row[:half]) and np.array_equal(C[half:], C_cmp[half:])


def test_mixed_dispatch_falls_back_to_one_kernel(smat, cuda, oracle):
    """All rows of one kind: the plan keeps a single kernel (compact for sparse blocks, a dense one for full blocks)."""
    d = gen.erdos_renyi(1024, 0.004, seed=5)
    A = bcsr_of(smat, d)
    B = gen.dense_b(A["K"], 64, seed=6, dist="uniform")
    C, info = gpu_spmm_compact(smat, cuda, A, B, 64, kernel=0)
    assert info["kernel"] == COMPACT and info["mixed_dense_items"] == 0
    assert oracle.compare(C, oracle_ref(oracle, A, B, 64))[0] <= TOL_F16
    A = gen.random_bcsr(40, 40, 0.2, seed=7)
    B = gen.dense_b(A["K"], 64, seed=8, dist="uniform")
    C, info = gpu_spmm_compact(smat, cuda, A, B, 64, kernel=0)
    assert info["kernel"] in (1, 2) and info["compact_cols"] == 0
    assert oracle.compare(C, oracle_ref(oracle, A, B, 64))[0] <= TOL_F16
    with pytest.raises(smat.SmatError, match="SMAT_KERNEL_MIXED needs a plan"):
        gpu_spmm(smat, cuda, A, B, 64, plan=True, kernel=MIXED)


def test_values_checksum_tells_when_to_attach_again(smat, cuda, oracle):
    """The compact kernel multiplies the copy taken by attach_values: after an in-place update of the values the
    guard says so, the stale result is the old product, and attaching again gives the new one."""
    import torch
    d = gen.erdos_renyi(512, 0.01, seed=13)
    A = bcsr_of(smat, d)
    M, K, nnzb, N = A["M"], A["K"], A["nnzb"], 64
    B = gen.dense_b(K, N, seed=14, dist="uniform")
    vals, rp, ci = to_dev(torch, A["b_val"], cuda), to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda), to_dev(torch, A["b_col_idx"].astype(np.int32), cuda)
    Bd = to_dev(torch, B, cuda)
    p = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=COMPACT)
    p.attach_values(vals, rp, ci)
    assert p.values_current(vals)
    new_val = (A["b_val"].view(np.float16) * np.float16(2)).view(np.uint16)
    vals.copy_(to_dev(torch, new_val, cuda))
    torch.cuda.synchronize()
    assert not p.values_current(vals)
    p.attach_values(vals, rp, ci)
    assert p.values_current(vals)
    C = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    smat.spmm(vals, rp, ci, Bd, C, M, N, K, nnzb, plan=p, kernel=COMPACT)
    torch.cuda.synchronize()
    A2 = dict(A, b_val=new_val)
    assert oracle.compare(C.cpu().numpy().view(np.uint16), oracle_ref(oracle, A2, B, N))[0] <= TOL_F16
    # two values swapped inside one block: same multiset, another checksum
    v = new_val.copy()
    nz = np.flatnonzero(v)
    v[nz[0]], v[nz[-1]] = v[nz[-1]], v[nz[0]]
    if not np.array_equal(v, new_val):
        vals.copy_(to_dev(torch, v, cuda))
        torch.cuda.synchronize()
        assert not p.values_current(vals)
    p.close()
    plain = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, kernel=1)  # no copy of the values: always current
    assert plain.values_current(vals)
    plain.close()
