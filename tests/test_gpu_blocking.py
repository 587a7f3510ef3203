"""GPU blocking (CSR -> BCSR on the device) against the oracle's restatement of csrToBcsr
(src/cuda_hgemm/src/common/matrix.h:376-502) and against the host routine: every array bit for bit.
The oracle keeps two dense block maps, so it is the comparand where (M/16) x (K/16) cells fit."""
import numpy as np
import pytest

from smat_amd import generators as gen

pytestmark = pytest.mark.gpu


def device_blocking(smat, cuda, M, K, rp, ci, v):
    import torch
    rp_d = torch.from_numpy(np.ascontiguousarray(rp, np.int32)).to(cuda)
    ci_d = torch.from_numpy(np.ascontiguousarray(ci, np.int32) if len(ci) else np.zeros(1, np.int32)).to(cuda)
    v_d = torch.from_numpy((np.ascontiguousarray(v, np.uint16) if len(v) else np.zeros(1, np.uint16)).view(np.int16)).to(cuda)
    torch.cuda.synchronize()
    d = smat.csr_to_bcsr_device(M, K, rp_d, ci_d, v_d, int(rp[M]))
    out = d.to_host()
    d.close()
    return out


def check_same(smat, cuda, M, K, rp, ci, v, oracle=None):
    want = smat.csr_to_bcsr(M, K, rp, ci, v)
    got = device_blocking(smat, cuda, M, K, rp, ci, v)
    if oracle is not None:
        assert (M // 16) * (K // 16) <= 1 << 24
        o = oracle.csr_to_bcsr(M, K, rp, ci, v)
        assert got.counts == o["counts"]
        assert np.array_equal(got.row_ptr, o["row_ptr"]) and np.array_equal(got.col_idx, o["col_idx"])
        assert np.array_equal(got.val, o["val"])
    assert got.counts == want.counts
    assert np.array_equal(got.row_ptr, want.row_ptr)
    assert np.array_equal(got.col_idx, want.col_idx)
    assert np.array_equal(got.val, want.val)
    return want


def test_band_closed_form(smat, cuda, oracle):
    d = gen.band(4096, 64)
    b = check_same(smat, cuda, d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], oracle)
    assert b.nnzb == 2284


def test_erdos_renyi_and_stencil(smat, cuda, oracle):
    d = gen.erdos_renyi(4096, 0.002, seed=5)
    check_same(smat, cuda, d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], oracle)
    d = gen.stencil27(16)
    b = check_same(smat, cuda, d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], oracle)
    assert b.counts[1] > 0  # runs of three adjacent columns exist: the "dense" counter is exercised


def test_rmat_long_rows(smat, cuda, oracle):
    d = gen.rmat(13, 64, seed=11)  # the heaviest rows have far more than 512 entries: wavefront-per-row path
    assert np.diff(d["row_ptr"]).max() > 512
    check_same(smat, cuda, d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], oracle)


def test_unsorted_rows_duplicates_and_empty(smat, cuda, oracle):
    rng = np.random.default_rng(3)
    M, K = 96, 160
    rows = []
    for r in range(M):
        n = int(rng.integers(0, 40)) if r % 7 else 0       # some empty rows
        cols = rng.integers(0, K, n)
        if n > 4:
            cols[n // 2] = cols[0]                           # duplicates, far apart and adjacent
            cols[-1] = cols[-2]
        rows.append(cols)
    # one long row with duplicates in different 64-entry steps and inside one step
    long_cols = rng.integers(0, K, 1500)
    long_cols[700] = long_cols[3]
    long_cols[701] = long_cols[702]
    rows[5] = long_cols
    rp = np.zeros(M + 1, np.int32)
    rp[1:] = np.cumsum([len(c) for c in rows])
    ci = np.concatenate(rows).astype(np.int32)
    v = rng.integers(1, 0x3C00, len(ci)).astype(np.uint16)  # distinct-ish positive halfs: the winner of a duplicate shows
    check_same(smat, cuda, M, K, rp, ci, v, oracle)
    # all-empty matrix
    rp0 = np.zeros(33, np.int32)
    b = check_same(smat, cuda, 32, 48, rp0, np.zeros(0, np.int32), np.zeros(0, np.uint16), oracle)
    assert b.nnzb == 0


def test_rejects_bad_column(smat, cuda):
    rp = np.array([0, 1] + [1] * 15, np.int32)
    with pytest.raises(smat.SmatError):
        device_blocking(smat, cuda, 16, 16, rp, np.array([16], np.int32), np.array([1], np.uint16))
