"""Pins the oracle's CPU SpMM: dense float64 matmul, special cases, CSR-vs-blocked equality."""
import numpy as np
import pytest

from smat_amd import generators as gen


def dense_of(A):
    rp, ci, v = gen.bcsr_to_csr(A["M"], A["b_row_ptr"], A["b_col_idx"], A["b_val"])
    D = np.zeros((A["M"], A["K"]), dtype=np.float64)
    rows = np.repeat(np.arange(A["M"]), np.diff(rp))
    D[rows, ci] = v.view(np.float16).astype(np.float64)
    return D, (rp, ci, v)


@pytest.mark.parametrize("mb,kb,density,N,seed", [(3, 5, 0.5, 8, 1), (10, 7, 0.3, 24, 2), (16, 16, 0.1, 40, 3)])
def test_against_dense_float64(oracle, mb, kb, density, N, seed):
    A = gen.random_bcsr(mb, kb, density, seed)
    B = gen.dense_b(A["K"], N, seed + 10, dist="normal")
    D, (rp, ci, v) = dense_of(A)
    Bm = B.view(np.float16).reshape(N, A["K"]).T.astype(np.float64)  # column-major: (k, n) at [n*K + k]
    want = D @ Bm
    got_csr = oracle.spmm_csr(A["M"], N, A["K"], rp, ci, v, B)
    got_blk = oracle.spmm_bcsr(A["M"], N, A["K"], A["b_row_ptr"], A["b_col_idx"], A["b_val"], B)
    got_par = oracle.spmm_bcsr(A["M"], N, A["K"], A["b_row_ptr"], A["b_col_idx"], A["b_val"], B, threads=4)
    scale = np.abs(D) @ np.abs(Bm) + 1e-30
    for got in (got_csr, got_blk, got_par):
        assert (np.abs(got - want) / scale).max() < 1e-6  # fp32 accumulation of exactly representable products
    assert np.array_equal(got_blk, got_par)


def test_a_transposed_operand_would_fail(oracle):
    # guards against a transposed-block mistake: a single off-diagonal entry
    blk = np.zeros((16, 16), dtype=np.float16)
    blk[2, 9] = 1.0
    A = {"M": 16, "K": 16, "b_row_ptr": np.array([0, 1], np.int32), "b_col_idx": np.array([0], np.int32),
         "b_val": blk.view(np.uint16).ravel()}
    N = 8
    B = gen.dense_b(16, N, 5, dist="uniform")
    got = oracle.spmm_bcsr(16, N, 16, A["b_row_ptr"], A["b_col_idx"], A["b_val"], B)
    Bm = B.view(np.float16).reshape(N, 16).T.astype(np.float32)
    want = np.zeros((16, N), np.float32)
    want[2] = Bm[9]
    assert np.array_equal(got, want)


def test_row_major_b_option(oracle):
    A = gen.random_bcsr(4, 4, 0.6, 8)
    N = 16
    B = gen.dense_b(A["K"], N, 3)
    B_rm = np.ascontiguousarray(B.reshape(N, A["K"]).T).ravel()
    rp, ci, v = gen.bcsr_to_csr(A["M"], A["b_row_ptr"], A["b_col_idx"], A["b_val"])
    assert np.array_equal(oracle.spmm_csr(A["M"], N, A["K"], rp, ci, v, B),
                          oracle.spmm_csr(A["M"], N, A["K"], rp, ci, v, B_rm, b_row_major=True))


def test_b_ones_gives_row_sums_like_the_reference_harness(oracle):
    # the reference fills B with 1.0 (common/matrix.h:38) and its TEST_matrices checks CSR == blocked multiply
    A = gen.random_bcsr(6, 6, 0.4, 21)
    N = 8
    B = np.full(A["K"] * N, 0x3C00, dtype=np.uint16)
    rp, ci, v = gen.bcsr_to_csr(A["M"], A["b_row_ptr"], A["b_col_idx"], A["b_val"])
    c1 = oracle.spmm_csr(A["M"], N, A["K"], rp, ci, v, B)
    c2 = oracle.spmm_bcsr(A["M"], N, A["K"], A["b_row_ptr"], A["b_col_idx"], A["b_val"], B)
    assert np.allclose(c1, c2, rtol=0, atol=1e-5)
    assert (c1 == c1[:, :1]).all()


def test_compare_metric(oracle):
    ref = np.array([[3.0, 4.0], [0.0, 0.0]], dtype=np.float32)  # row norms 5 and 0
    c = np.array([[3.0, 4.5], [0.25, 0.0]], dtype=np.float16).view(np.uint16)
    rel, mx, mean = oracle.compare(c, ref)
    assert rel == pytest.approx(0.25)  # max(0.5/5, 0.25 absolute for the zero row)
    assert mx == pytest.approx(0.5) and mean == pytest.approx(0.75 / 4)


def write_el(path, M, rp, ci, v):
    """Edge list 'row col value' as CSR::read_from_edgelist (preprocess/src/general/csr.cpp:166-290) reads it."""
    vals = v.view(np.float16).astype(np.float64)
    with open(path, "w") as f:
        for i in range(M):
            for p in range(rp[i], rp[i + 1]):
                f.write(f"{i} {ci[p]} {vals[p]:.10g}\n")


@pytest.mark.parametrize("mb,density,N,seed", [(4, 0.5, 8, 11), (12, 0.2, 24, 12)])
def test_against_reference_csr_multiply(oracle, tmp_path, mb, density, N, seed):
    """The reference's own CSR::multiply (csr.cpp:47-63), compiled from the reference tree, on the same input."""
    import subprocess
    from tests.oracle_lib import ref_binary
    exe = ref_binary("ref_csr_multiply")
    if exe is None:
        pytest.skip("oracle/_ref/ref_csr_multiply not built (reference tree absent)")
    A = gen.random_bcsr(mb, mb, density, seed)  # square: the reference indexes B with A's row count
    rp, ci, v = gen.bcsr_to_csr(A["M"], A["b_row_ptr"], A["b_col_idx"], A["b_val"])
    # rows = last row + 1 and cols = largest column + 1 in the reference reader: pin both to M
    assert rp[A["M"]] > rp[A["M"] - 1] and ci.max() <= A["M"] - 1
    B = gen.dense_b(A["K"], N, seed + 1, dist="normal")
    write_el(tmp_path / "a.el", A["M"], rp, ci, v)
    B.view(np.float16).astype(np.float32).tofile(tmp_path / "b.f32")  # column-major, leading dimension K = M
    out = subprocess.run([exe, str(tmp_path / "a.el"), str(tmp_path / "b.f32"), str(N), "1", str(tmp_path / "c.f32")],
                         check=True, capture_output=True, text=True).stdout.split()
    rows, cols, nnz = int(out[0]), int(out[1]), int(out[2])
    assert rows == A["M"] and cols <= A["M"] and nnz == rp[A["M"]]
    c_ref = np.fromfile(tmp_path / "c.f32", dtype=np.float32).reshape(N, rows).T  # column-major M x N
    got = oracle.spmm_csr(A["M"], N, A["K"], rp, ci, v, B)
    scale = np.abs(c_ref).max(axis=1, keepdims=True) + 1e-30
    # same loop order; the two builds may differ in fused multiply-add contraction only
    assert (np.abs(got - c_ref) / scale).max() < 1e-6
