"""The benchmark configurations at their real sizes on the GPU: sampled block rows (the whole result where
the CPU oracle finishes in seconds) against the oracle, plus properties that do not depend on the size.

Bar as in test_gpu_spmm.py: max_j |C[i][j] - ref[i][j]| / ||ref[i][:]||_2 <= 1e-3 for the fp16 output."""
import numpy as np
import pytest

from smat_amd import generators as gen
from tests.test_gpu_spmm import TOL_F16, bcsr_of, gpu_spmm_compact, oracle_ref, to_dev

pytestmark = pytest.mark.gpu


def sample_rows(mb, n, extra=()):
    return np.unique(np.concatenate([np.linspace(0, mb - 1, min(mb, n)).astype(np.int64), np.asarray(extra, np.int64)]))


def check_sampled(oracle, A, B_bits, N, C_bits, rows):
    """Block rows `rows` of the fp16 result C_bits (M x N, uint16) against the oracle on those rows alone."""
    rp, ci = A["b_row_ptr"].astype(np.int64), A["b_col_idx"]
    sel = np.concatenate([np.arange(rp[r], rp[r + 1]) for r in rows])
    sub = {"M": 16 * len(rows), "K": A["K"],
           "b_row_ptr": np.concatenate([[0], np.cumsum([rp[r + 1] - rp[r] for r in rows])]).astype(np.int32),
           "b_col_idx": ci[sel], "b_val": A["b_val"].reshape(-1, 256)[sel].ravel()}
    ref = oracle_ref(oracle, sub, B_bits, N)
    got = np.concatenate([C_bits[16 * r:16 * r + 16] for r in rows])
    err = oracle.compare(got, ref)[0]
    assert err <= TOL_F16, err


@pytest.mark.timeout(600)
def test_config3_rmat_scale20_full_size(smat, cuda, oracle):
    """R-MAT scale 20, average degree 16, N = 128: 11 million blocks, 5.7 GB of block values (byte offsets
    beyond 2^31).  Blocked on the device; compact kernel (the plan's choice) and row-wise kernel."""
    import torch
    d = gen.rmat(20, 16)
    M, K, nnz = d["M"], d["K"], int(d["row_ptr"][-1])
    N = 128
    dev = smat.csr_to_bcsr_device(M, K, to_dev(torch, d["row_ptr"], cuda), to_dev(torch, d["col_idx"], cuda),
                                  to_dev(torch, d["val"], cuda), nnz)
    nnzb = dev.nnzb
    assert nnzb * 512 > 2**32
    host = dev.to_host()
    A = {"M": M, "K": K, "b_row_ptr": host.row_ptr, "b_col_idx": host.col_idx, "b_val": host.val, "nnzb": nnzb}
    mb = M // 16
    heaviest = int(np.argmax(np.diff(host.row_ptr)))
    rows = sample_rows(mb, 12, extra=(heaviest, mb - 1, mb - 2))  # the last rows read the highest offsets
    B = gen.dense_b(K, N, seed=0xB0000003, dist="uniform")
    B2 = (B.view(np.float16) * np.float16(2)).view(np.uint16)

    class Ptr:  # the arrays the device blocking returned, for smat.spmm / Plan.attach_values
        def __init__(self, p):
            self.p = p

        def data_ptr(self):
            return self.p
    vals, rp, ci = Ptr(dev.val), Ptr(dev.row_ptr), Ptr(dev.col_idx)
    Bd, B2d = to_dev(torch, B, cuda), to_dev(torch, B2, cuda)
    plan = smat.Plan(host.row_ptr, M, K, nnzb, N, col_idx_host=host.col_idx, kernel=0)
    plan.attach_values(vals, rp, ci)
    assert plan.info()["kernel"] == 5
    C = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    smat.spmm(vals, rp, ci, Bd, C, M, N, K, nnzb, plan=plan)
    torch.cuda.synchronize()
    check_sampled(oracle, A, B, N, C.cpu().numpy().view(np.uint16), rows)
    # linearity in B: A (2 B) = 2 (A B) bit for bit, fp16 output included (no result near the fp16 limits)
    C2 = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    smat.spmm(vals, rp, ci, B2d, C2, M, N, K, nnzb, plan=plan)
    torch.cuda.synchronize()
    c, c2 = C.view(torch.float16), C2.view(torch.float16)
    assert bool(torch.isfinite(c2).all()) and float(c.abs().max()) < 30000
    tiny = c.abs() < 2.0**-13  # twice a subnormal result may round differently
    assert bool(((c * 2 == c2) | tiny).all())
    plan.close()
    # row-wise kernel through the drop-in entry point (no plan): same sampled rows
    C.fill_(0x7E00)
    smat.spmm(vals, rp, ci, Bd, C, M, N, K, nnzb, drop_in=True)
    torch.cuda.synchronize()
    check_sampled(oracle, A, B, N, C.cpu().numpy().view(np.uint16), rows)
    dev.close()


@pytest.mark.timeout(900)
def test_config3_rmat_scale20_reordered_full_size(smat, cuda, oracle):
    """Config 3 in the form the benchmark states it: R-MAT scale 20 after both reorder passes (the permutations of
    a ten-minute smat_reorder_csr run, tests/golden/rmat_s20_deg16_perms.npz), then 16 x 16 BCSR: 8,076,241 blocks
    instead of 11,159,910.  The blocked structure has the recorded hash; sampled block rows (the heaviest and the
    last ones among them) against the oracle; A (2 B) = 2 (A B) over the whole result; and the result is the
    row-permuted product of the UNREORDERED matrix with the rows of B permuted back (on sampled rows)."""
    import json
    import os
    import torch
    import bench
    name = "rmat_s20_deg16_reordered_N128"
    bench.INFO.clear()
    A, B, N = bench.build_workload(name)
    want = json.load(open(bench.GOLDEN_STRUCTURE))[name]
    M, K, nnzb = A["M"], A["K"], A["nnzb"]
    assert (M, K, N, nnzb) == (want["M"], want["K"], want["N"], want["nnzb"]) and nnzb == 8076241
    assert bench.sha256_of(A["b_row_ptr"].astype(np.int32), A["b_col_idx"].astype(np.int32)) == want["pattern_sha256"]
    assert bench.INFO["perm_sha256"] == want["perm_sha256"]
    mb = M // 16
    heaviest = int(np.argmax(np.diff(A["b_row_ptr"])))
    rows = sample_rows(mb, 12, extra=(heaviest, mb - 1, mb - 2))
    B2 = (B.view(np.float16) * np.float16(2)).view(np.uint16)
    vals, Bd, B2d = to_dev(torch, A["b_val"], cuda), to_dev(torch, B, cuda), to_dev(torch, B2, cuda)
    rp, ci = to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda), to_dev(torch, A["b_col_idx"].astype(np.int32), cuda)
    plan = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=0)
    plan.attach_values(vals, rp, ci)
    assert plan.info()["kernel"] == 5
    C = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    smat.spmm(vals, rp, ci, Bd, C, M, N, K, nnzb, plan=plan)
    C2 = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    smat.spmm(vals, rp, ci, B2d, C2, M, N, K, nnzb, plan=plan)
    torch.cuda.synchronize()
    # the long block rows are at the front of the list: the launch deals its workgroups to the XCDs in short runs
    # (one run per XCD would be about 4,400 workgroups and leave one XCD with most of the steps)
    assert 0 < smat.lib.smat_internal_compact_last_run() <= 64
    plan.close()
    C_host = C.cpu().numpy().view(np.uint16)
    check_sampled(oracle, A, B, N, C_host, rows)
    c, c2 = C.view(torch.float16), C2.view(torch.float16)
    assert bool(torch.isfinite(c2).all()) and float(c.abs().max()) < 30000
    tiny = c.abs() < 2.0**-13
    assert bool(((c * 2 == c2) | tiny).all())
    del c, c2, C, C2, vals
    # against the matrix before the reorder: row i of the result is row perm_rows[i] of (A_original x B_back), where
    # B_back has the rows of B moved back to their old places.  Checked on the rows of the sampled block rows.
    z = np.load(bench.RMAT20_PERMS)
    pr, pc = z["perm_rows"].astype(np.int64), z["perm_cols"].astype(np.int64)
    d = gen.rmat(20, 16)
    Bm = B.reshape(N, K)
    B_back = np.empty_like(Bm)
    B_back[:, pc] = Bm
    new_rows = np.concatenate([np.arange(16 * r, 16 * r + 16) for r in rows])
    old_rows = pr[new_rows]
    lens = (d["row_ptr"][old_rows + 1] - d["row_ptr"][old_rows]).astype(np.int64)
    sel = np.concatenate([np.arange(d["row_ptr"][o], d["row_ptr"][o + 1]) for o in old_rows]) if lens.sum() else np.zeros(0, np.int64)
    sub_rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ref = oracle.spmm_csr(new_rows.size, N, K, sub_rp, d["col_idx"][sel], d["val"][sel], B_back.ravel())
    assert oracle.compare(np.ascontiguousarray(C_host[new_rows]), ref)[0] <= TOL_F16


def test_config2_reordered_full_size(smat, cuda, oracle):
    """Config 2 (16384 x 16384, 0.1 %, N = 256) after both reorder passes: whole result against the oracle,
    and equal to the product of the unpermuted matrix with rows and B permuted accordingly."""
    d = gen.erdos_renyi(16384, 0.001)
    pr, pc, sr, sc = smat.reorder_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], 16, 16, 0.5, True)
    rp, ci, v = smat.permute_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], pr, pc)
    A = bcsr_of(smat, {"M": d["M"], "K": d["K"], "row_ptr": rp, "col_idx": ci, "val": v})
    assert A["nnzb"] == sc[2] < bcsr_of(smat, d)["nnzb"]
    N = 256
    B = gen.dense_b(A["K"], N, seed=0xB0000002, dist="normal")
    C, info = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0)
    assert info["kernel"] == 5
    assert oracle.compare(C, oracle_ref(oracle, A, B, N))[0] <= TOL_F16
    # P_r A P_c times B  ==  P_r (A times (P_c B)): row i of the reordered product is row pr[i] of the
    # product of the original matrix with the rows of B moved back (same tolerance, other summation order)
    Bm = B.reshape(N, A["K"])                      # column-major: [n][k]
    B_back = np.empty_like(Bm)
    B_back[:, pc] = Bm                             # row pc[j] of the original B' is row j of B
    ref = oracle.spmm_csr(d["M"], N, d["K"], d["row_ptr"], d["col_idx"], d["val"], B_back.ravel())
    assert oracle.compare(C, ref[pr])[0] <= TOL_F16


@pytest.mark.parametrize("reordered", [False, True])
def test_config5_stencil_64_full_size(smat, cuda, oracle, reordered):
    """27-point stencil on a 64^3 grid (262,144 rows), N = 64: sampled block rows against the oracle."""
    d = gen.stencil27(64)
    if reordered:
        pr, pc, sr, sc = smat.reorder_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], 16, 16, 0.5, True)
        rp, ci, v = smat.permute_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], pr, pc)
        d = {"M": d["M"], "K": d["K"], "row_ptr": rp, "col_idx": ci, "val": v}
    A = bcsr_of(smat, d)
    N = 64
    B = gen.dense_b(A["K"], N, seed=0xB0000005, dist="uniform")
    C, info = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0)
    mb = A["M"] // 16
    check_sampled(oracle, A, B, N, C, sample_rows(mb, 40, extra=(1, mb - 2)))
    # the row-wise kernel on the same operands: close to it everywhere (other summation order)
    C1, _ = gpu_spmm_compact(smat, cuda, A, B, N, kernel=1)
    a, b = C.view(np.float16).astype(np.float32), C1.view(np.float16).astype(np.float32)
    assert np.abs(a - b).max() <= 2e-3 * np.abs(b).max()


def test_mixed_dispatch_full_size(smat, cuda, oracle):
    """8192 x 8192, upper half of the block rows dense blocks (10 % kept), lower half about one nonzero per
    block, N = 4096: the plan sends the upper half through the sweep kernel (its 256 block rows fill the device)
    and the lower half through the compact kernel."""
    A = gen.half_pruned_half_er(8192, 0.10, 0.001)
    N = 4096
    B = gen.dense_b(A["K"], N, seed=0xB0000006, dist="normal")
    C, info = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0)
    assert info["kernel"] == 6 and info["mixed_dense_blocks"] == A["dense_blocks"]
    assert info["sweep_ops"] > 0 and info["mixed_dense_items"] == 0  # sweep, not row-wise, for the dense rows
    mb = A["M"] // 16
    check_sampled(oracle, A, B, N, C, sample_rows(mb, 16, extra=(mb // 2 - 1, mb // 2, mb // 2 + 1)))


def test_mixed_dispatch_per_block(smat, cuda, oracle):
    """4096 x 4096, every block row holds dense blocks (10 % of the grid) and blocks of about one nonzero between them,
    N = 4096: no block row is of one kind, so the plan splits per BLOCK - a copy of the dense blocks through the sweep
    kernel, the columns of the other blocks added by the compact kernel - and the result is the product of the
    whole matrix (fp16 and fp32 C; row-major B; the same split when asked for by name)."""
    import torch
    A = gen.pruned_plus_er(4096, 0.10, 0.003)
    N = 4096
    M, K, nnzb = A["M"], A["K"], A["nnzb"]
    B = gen.dense_b(K, N, seed=0xB0000007, dist="normal")
    C, info = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0)
    assert info["kernel"] == 6 and info["mixed_dense_items"] == -1      # mixed, per block
    assert info["mixed_dense_blocks"] == A["dense_blocks"] and info["sweep_ops"] > 0
    assert 0 < info["compact_cols"] < 3 * (nnzb - A["dense_blocks"])     # the list holds the other blocks only
    mb = M // 16
    rows = sample_rows(mb, 24, extra=(0, 1, 63, 64, mb - 1))
    check_sampled(oracle, A, B, N, C, rows)
    C6, info6 = gpu_spmm_compact(smat, cuda, A, B, N, kernel=6)
    assert info6["mixed_dense_items"] == -1 and np.array_equal(C6, C)
    # fp32 C: only the summation order differs from one kernel over the whole matrix
    C32, _ = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0, c_f32=True)
    C32_one, info_one = gpu_spmm_compact(smat, cuda, A, B, N, kernel=2, c_f32=True)
    assert info_one["kernel"] == 2
    scale = np.sqrt((C32_one.astype(np.float64) ** 2).sum(axis=1)).max()
    assert np.abs(C32 - C32_one).max() <= 2e-6 * scale
    # the same through row-major B (the sweep kernel takes it from the plan's column-major copy, the compact kernel in place)
    B_rm = np.ascontiguousarray(B.reshape(N, K).T).ravel()
    vals, rp, ci = (to_dev(torch, A["b_val"], cuda), to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda),
                    to_dev(torch, A["b_col_idx"].astype(np.int32), cuda))
    p = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=0, b_row_major=True)
    p.attach_values(vals, rp, ci)
    assert p.info()["mixed_dense_items"] == -1
    Cd = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    smat.spmm(vals, rp, ci, to_dev(torch, B_rm, cuda), Cd, M, N, K, nnzb, plan=p, b_row_major=True)
    torch.cuda.synchronize()
    p.close()
    assert np.array_equal(Cd.cpu().numpy().view(np.uint16), C)


def test_sweep_kernel_unevenly_pruned_rows(smat, cuda, oracle):
    """8192 x 8192, dense blocks whose share falls from 18 % in the first block row to 2 % in the last, N = 4096: the
    sweep kernel's plan deals the block rows to its row groups by their block count (in order, the first group
    would hold 1.7 x the average), so the rows of C of one workgroup are scattered over the matrix.  Sampled block rows
    (the first and the last, the heaviest and an empty one if there is one) against the oracle, fp16 and fp32 C."""
    A = gen.block_pruned_skewed(8192, 0.18, 0.02)
    N = 4096
    M, K, nnzb = A["M"], A["K"], A["nnzb"]
    lens = np.diff(A["b_row_ptr"])
    assert lens.reshape(-1, 64).sum(1).max() > 1.5 * lens.sum() / 8
    B = gen.dense_b(K, N, seed=0xB0000008, dist="normal")
    C, info = gpu_spmm_compact(smat, cuda, A, B, N, kernel=0)
    assert info["kernel"] == 2 and info["sweep_ops"] > 0
    mb = M // 16
    rows = sample_rows(mb, 24, extra=(0, 1, 63, 64, mb - 1, int(np.argmax(lens)), int(np.argmin(lens))))
    check_sampled(oracle, A, B, N, C, rows)
    C32, _ = gpu_spmm_compact(smat, cuda, A, B, N, kernel=2, c_f32=True)
    assert np.array_equal(C32.astype(np.float16).view(np.uint16), C)


def test_config4_sweep_kernel_full_size_linearity_and_more_rows(smat, cuda, oracle):
    """Headline config through the plan's choice (the sweep kernel): 40 sampled block rows against the oracle
    (first and last of every row group among them), and A (2 B) = 2 (A B) bit for bit over the whole result."""
    import torch
    A = gen.block_pruned(8192, 0.10, 0.02)
    N = 4096
    M, K, nnzb = A["M"], A["K"], A["nnzb"]
    B = gen.dense_b(K, N, seed=0xB0000004, dist="normal")
    B2 = (B.view(np.float16) * np.float16(2)).view(np.uint16)
    vals, Bd, B2d = to_dev(torch, A["b_val"], cuda), to_dev(torch, B, cuda), to_dev(torch, B2, cuda)
    rp, ci = to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda), to_dev(torch, A["b_col_idx"].astype(np.int32), cuda)
    plan = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"])
    assert plan.info()["kernel"] == 2
    C = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    smat.spmm(vals, rp, ci, Bd, C, M, N, K, nnzb, plan=plan)
    C2 = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    smat.spmm(vals, rp, ci, B2d, C2, M, N, K, nnzb, plan=plan)
    torch.cuda.synchronize()
    plan.close()
    edges = [g * 64 + d for g in range(8) for d in (0, 63)]
    check_sampled(oracle, A, B, N, C.cpu().numpy().view(np.uint16), sample_rows(M // 16, 24, edges))
    c, c2 = C.view(torch.float16), C2.view(torch.float16)
    assert bool(torch.isfinite(c2).all()) and float(c.abs().max()) < 30000
    tiny = c.abs() < 2.0**-13  # twice a subnormal result may round differently
    assert bool(((c * 2 == c2) | tiny).all())
