"""Every kernel against the oracle on randomly drawn matrices and widths (fixed seeds): shapes that no hand-written
case names - block rows of 0 to 700 blocks side by side, N at any multiple of 8, row- and column-major B, plans with
and without attached values, fp16 and fp32 results.

Bar: max_j |C[i][j] - ref[i][j]| / ||ref[i][:]||_2 <= 1e-3 for fp16 C; 1e-5 for fp32 C (rows of 700 blocks sum
11,200 products, and every kernel has its own order of summation)."""
import numpy as np
import pytest

from smat_amd import generators as gen
from tests.test_gpu_spmm import TOL_F16, bcsr_of, oracle_ref, rel_err_f32, to_dev

pytestmark = pytest.mark.gpu

TOL_F32_LONG_ROWS = 1e-5


def draw_matrix(smat, rng):
    kind = rng.choice(["mask", "er", "rmat", "lengths", "uneven"])
    seed = int(rng.integers(1 << 30))
    if kind == "mask":
        return gen.random_bcsr(int(rng.integers(1, 200)), int(rng.integers(1, 200)), float(rng.choice([0.02, 0.1, 0.3, 0.9])), seed=seed)
    if kind == "er":
        return bcsr_of(smat, gen.erdos_renyi(16 * int(rng.integers(4, 300)), float(rng.choice([0.001, 0.004, 0.02])), seed=seed))
    if kind == "rmat":
        return bcsr_of(smat, gen.rmat(int(rng.integers(8, 13)), int(rng.choice([4, 16])), seed=seed))
    if kind == "lengths":
        n = int(rng.integers(1, 120))
        lengths = [int(x) for x in rng.choice([0, 0, 1, 2, 3, 5, 9, 10, 11, 40, 130, 700], size=n)]
        return gen.random_bcsr(n, max(max(lengths), 8), 0.0, seed=seed, row_lengths=lengths)
    return gen.block_pruned_skewed(16 * int(rng.integers(70, 400)), float(rng.choice([0.3, 0.6])), 0.02, seed=seed)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_matrices_every_kernel(smat, cuda, oracle, seed):
    import torch
    rng = np.random.default_rng(seed)
    done = 0
    for case in range(25):
        A = draw_matrix(smat, rng)
        M, K, nnzb = A["M"], A["K"], int(A["b_col_idx"].shape[0])
        if nnzb < 2:
            continue
        N = 8 * int(rng.integers(1, 70)) if rng.random() < 0.8 else int(rng.choice([64, 128, 256, 512, 1024]))
        B = gen.dense_b(K, N, seed=int(rng.integers(1 << 30)), dist=str(rng.choice(["normal", "uniform"])))
        ref = oracle_ref(oracle, A, B, N)
        vals, rp, ci = (to_dev(torch, A["b_val"], cuda), to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda),
                        to_dev(torch, A["b_col_idx"].astype(np.int32), cuda))
        for kernel in (0, 1, 2, 3, 4, 5, 6):
            c_f32 = bool(rng.random() < 0.5)
            row_major = bool(rng.random() < 0.3)
            attach = kernel in (5, 6) or (kernel == 0 and rng.random() < 0.7)
            what = (seed, case, M, K, N, nnzb, kernel, c_f32, row_major, attach)
            Bd = to_dev(torch, np.ascontiguousarray(B.reshape(N, K).T).ravel() if row_major else B, cuda)
            C = torch.full((M, N), float("nan"), dtype=torch.float32, device=cuda) if c_f32 else \
                torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
            p = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=kernel, b_row_major=row_major)
            try:
                if attach:
                    p.attach_values(vals, rp, ci)
                smat.spmm(vals, rp, ci, Bd, C, M, N, K, nnzb, plan=p, c_f32=c_f32, kernel=kernel, b_row_major=row_major)
                torch.cuda.synchronize()
            finally:
                p.close()
            out = C.cpu().numpy()
            if c_f32:
                assert rel_err_f32(out, ref) <= TOL_F32_LONG_ROWS, what
            else:
                assert oracle.compare(out.view(np.uint16), ref)[0] <= TOL_F16, what
            done += 1
    assert done >= 100
