"""CSR -> BCSR: closed forms, brute force on a dense bitmap, invariants, library == oracle bit for bit."""
import numpy as np
import pytest

from smat_amd import generators as gen


def dense_bitmap_bcsr(M, K, row_ptr, col_idx, val):
    """Independent statement in numpy: dense (M/16)x(K/16) bitmap, row-major numbering."""
    rows = np.repeat(np.arange(M), np.diff(row_ptr))
    mb, kb = M // 16, K // 16
    bitmap = np.zeros((mb, kb), dtype=bool)
    bitmap[rows // 16, col_idx // 16] = True
    brp = np.concatenate([[0], np.cumsum(bitmap.sum(axis=1))]).astype(np.int32)
    br, bc = np.nonzero(bitmap)
    rel = -np.ones((mb, kb), dtype=np.int64)
    rel[br, bc] = np.arange(br.size)
    vals = np.zeros(br.size * 256, dtype=np.uint16)
    idx = rel[rows // 16, col_idx // 16] * 256 + (rows % 16) * 16 + col_idx % 16
    for i, v in zip(idx, val):  # sequential: the later duplicate wins
        vals[i] = v
    return brp, (bc * 16).astype(np.int32), vals, bitmap, rel


def random_csr(M, K, nnz, seed, duplicates=True, sort=False):
    rng = np.random.default_rng(seed)
    r = rng.integers(0, M, nnz)
    c = rng.integers(0, K, nnz)
    if not duplicates:
        key = np.unique(r * K + c)
        r, c = key // K, key % K
        perm = rng.permutation(r.size)
        r, c = r[perm], c[perm]
    order = np.lexsort((c, r)) if sort else np.argsort(r, kind="stable")
    r, c = r[order], c[order]
    v = gen.f16_bits(rng.normal(size=r.size))
    v[v == 0] = 0x3C00
    row_ptr = np.zeros(M + 1, dtype=np.int32)
    np.add.at(row_ptr, r + 1, 1)
    return np.cumsum(row_ptr).astype(np.int32), c.astype(np.int32), v


@pytest.mark.parametrize("M,K,nnz,seed", [(16, 16, 5, 1), (64, 48, 300, 2), (512, 512, 4000, 3), (320, 1024, 20000, 4),
                                          (256, 256, 0, 5)])
def test_oracle_and_library_equal_brute_force(oracle, smat, M, K, nnz, seed):
    rp, ci, v = random_csr(M, K, nnz, seed)
    brp, bci, bv, bitmap, rel = dense_bitmap_bcsr(M, K, rp, ci, v)
    o = oracle.csr_to_bcsr(M, K, rp, ci, v)
    a = smat.csr_to_bcsr(M, K, rp, ci, v, want_maps=True)
    for got_rp, got_ci, got_v in ((o["row_ptr"], o["col_idx"], o["val"]), (a.row_ptr, a.col_idx, a.val)):
        assert np.array_equal(got_rp, brp) and np.array_equal(got_ci, bci) and np.array_equal(got_v, bv)
    # the dense maps: nonzero flag and running index == position in col_idx ("rel == ptr")
    assert np.array_equal(o["block_info"].reshape(bitmap.shape) != 0, bitmap)
    assert np.array_equal(o["rel_map"].reshape(bitmap.shape), rel)
    assert np.array_equal(a.block_info, o["block_info"]) and np.array_equal(a.rel_map, o["rel_map"])
    assert a.counts == o["counts"] and a.counts[0] == bci.size and a.counts[1] + a.counts[2] == a.counts[0]


def test_invariants_on_random_input(smat):
    rp, ci, v = random_csr(1024, 2048, 30000, 9, duplicates=False, sort=True)
    a = smat.csr_to_bcsr(1024, 2048, rp, ci, v)
    assert a.row_ptr[0] == 0 and (np.diff(a.row_ptr) >= 0).all() and a.row_ptr[-1] == a.nnzb
    assert (a.col_idx % 16 == 0).all()
    for br in range(1024 // 16):
        seg = a.col_idx[a.row_ptr[br]:a.row_ptr[br + 1]]
        assert (np.diff(seg) > 0).all()
    assert np.count_nonzero(a.val) == v.size  # no duplicates: every entry lands in exactly one cell


def test_dense_block_heuristic_counts(oracle, smat):
    # a block turns "dense" when three adjacent columns c-2, c-1, c with c % 4 in {2, 3} follow each other in a row
    M = K = 32
    rows = [0, 0, 0, 0, 17, 17, 17, 20, 20, 20]
    cols = [0, 1, 2, 20, 1, 2, 3, 4, 5, 6]  # row 0: 0,1,2 -> dense (c=2); row 17: 1,2,3 -> dense (c=3); row 20: 4,5,6 -> dense
    rp = np.zeros(M + 1, dtype=np.int32)
    np.add.at(rp, np.array(rows) + 1, 1)
    rp = np.cumsum(rp).astype(np.int32)
    ci = np.array(cols, dtype=np.int32)
    v = np.full(len(cols), 0x3C00, dtype=np.uint16)
    o = oracle.csr_to_bcsr(M, K, rp, ci, v)
    a = smat.csr_to_bcsr(M, K, rp, ci, v)
    # blocks: (0,0) dense, (0,1) sparse, (1,0) dense (row 17 promotes it; row 20 finds it already dense)
    assert o["counts"] == (3, 2, 1) and a.counts == (3, 2, 1)


def test_band_closed_form(smat, oracle):
    d = gen.band(4096, 64)
    assert d["row_ptr"][-1] == 4096 * 129 - 64 * 65 == 524224
    a = smat.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
    assert a.nnzb == 9 * 256 - 20 == 2284
    br = np.arange(256)
    assert np.array_equal(np.diff(a.row_ptr), np.minimum(br, 4) + np.minimum(255 - br, 4) + 1)
    for r in (0, 3, 100, 255):
        lo, hi = max(0, r - 4), min(255, r + 4)
        assert a.col_idx[a.row_ptr[r]:a.row_ptr[r + 1]].tolist() == list(range(16 * lo, 16 * hi + 16, 16))
    o = oracle.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
    assert np.array_equal(o["val"], a.val) and np.array_equal(o["col_idx"], a.col_idx)


def test_stencil_closed_forms(smat):
    d = gen.stencil27(16)
    assert d["row_ptr"][-1] == (3 * 16 - 2) ** 3
    d = gen.stencil27(64)
    assert d["row_ptr"][-1] == 190 ** 3 == 6859000
    a = smat.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
    assert a.nnzb == 10 * 190 * 190 == 361000
    assert set(np.unique(np.diff(a.row_ptr)).tolist()) <= {8, 12, 18, 27}


def test_block_pruned_mask_is_its_own_bcsr(smat):
    A = gen.block_pruned(1024, 0.10, 0.02, seed=77)
    rp, ci, v = gen.bcsr_to_csr(A["M"], A["b_row_ptr"], A["b_col_idx"], A["b_val"], drop_zeros=True)
    a = smat.csr_to_bcsr(A["M"], A["K"], rp, ci, v)
    assert a.nnzb == A["nnzb"] == round(0.1 * 64 * 64)
    assert np.array_equal(a.row_ptr, A["b_row_ptr"]) and np.array_equal(a.col_idx, A["b_col_idx"])
    assert np.array_equal(a.val, A["b_val"])


def test_bad_arguments(smat):
    rp = np.zeros(17, dtype=np.int32)
    with pytest.raises(smat.SmatError):
        smat.csr_to_bcsr(17, 16, rp, np.zeros(0, np.int32), np.zeros(0, np.uint16))
    rp2 = np.array([0] + [1] * 16, dtype=np.int32)
    with pytest.raises(smat.SmatError):
        smat.csr_to_bcsr(16, 16, rp2, np.array([16], np.int32), np.array([1], np.uint16))
