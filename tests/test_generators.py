"""Synthetic inputs: reproducibility and the closed forms the configurations promise."""
import numpy as np

from smat_amd import generators as gen


def test_counter_rng_is_reproducible_and_uniform():
    idx = np.arange(200000, dtype=np.uint64)
    a, b = gen.rand_u64(7, idx), gen.rand_u64(7, idx)
    assert np.array_equal(a, b) and not np.array_equal(a, gen.rand_u64(8, idx))
    assert int(gen.rand_u64(0, np.array([0], np.uint64))[0]) == 0xE220A8397B1DCDAF  # splitmix64(0) first output
    u = gen.rand_uniform(3, idx)
    assert 0 <= u.min() and u.max() < 1 and abs(u.mean() - 0.5) < 5e-3
    z = gen.rand_normal(3, idx)
    assert abs(z.mean()) < 1e-2 and abs(z.std() - 1) < 1e-2


def test_band_matches_reference_generator_pattern():
    d = gen.band(300, 5)
    rows = np.repeat(np.arange(300), np.diff(d["row_ptr"]))
    assert (np.abs(rows - d["col_idx"]) <= 5).all()
    assert d["row_ptr"][-1] == 300 * 11 - 5 * 6  # N(2b+1) - b(b+1)


def test_erdos_renyi_config2_shape():
    d = gen.erdos_renyi(16384, 0.001)
    nnz = int(d["row_ptr"][-1])
    assert 268435 - 300 < nnz <= 268435  # i.i.d. draws, duplicates merged
    for r in (0, 100, 16383):
        seg = d["col_idx"][d["row_ptr"][r]:d["row_ptr"][r + 1]]
        assert (np.diff(seg) > 0).all()


def test_rmat_small_is_skewed_and_deduplicated():
    d = gen.rmat(scale=12, avg_degree=16)
    deg = np.diff(d["row_ptr"])
    assert d["M"] == 4096 and deg.sum() <= 16 * 4096 and deg.max() > 20 * deg.mean()
    rows = np.repeat(np.arange(4096), deg)
    key = rows.astype(np.int64) * 4096 + d["col_idx"]
    assert np.unique(key).size == key.size


def test_block_pruned_config4_shape():
    A = gen.block_pruned(8192, 0.10, 0.02)
    assert A["nnzb"] == 26214 and A["b_row_ptr"][-1] == 26214 and A["b_val"].size == 26214 * 256
    v = A["b_val"][:256 * 500].view(np.float16).astype(np.float64)
    assert abs(v.std() - 0.02) < 1e-3 and np.count_nonzero(v) > 0.99 * v.size
    lens = np.diff(A["b_row_ptr"])
    assert 20 < lens.min() and lens.max() < 90


def test_stencil_values():
    d = gen.stencil27(4)
    rows = np.repeat(np.arange(64), np.diff(d["row_ptr"]))
    v = d["val"].view(np.float16).astype(np.float32)
    assert (v[rows == d["col_idx"]] == 26).all() and (v[rows != d["col_idx"]] == -1).all()
    assert d["row_ptr"][-1] == 10 ** 3  # (3n-2)^3


def test_pruned_plus_er_holds_both_kinds_of_blocks_in_every_row():
    A = gen.pruned_plus_er(2048, 0.10, 0.003)
    top = gen.block_pruned(2048, 0.10, 0.02, 0x5A170007)
    mb = 128
    rp, ci = A["b_row_ptr"], A["b_col_idx"]
    assert A["dense_blocks"] == top["nnzb"] and A["nnzb"] > 2 * top["nnzb"] and rp[-1] == A["nnzb"]
    vals = A["b_val"].reshape(-1, 256)
    full = ((vals & 0x7FFF) != 0).sum(axis=1) > 200          # a dense block; the others hold a handful of entries
    assert full.sum() == top["nnzb"] and ((vals[~full] & 0x7FFF) != 0).sum(axis=1).max() <= 8
    for r in range(mb):
        seg = ci[rp[r]:rp[r + 1]]
        assert (np.diff(seg) > 0).all() and (seg % 16 == 0).all()
        kinds = full[rp[r]:rp[r + 1]]
        assert kinds.any() and (~kinds).any()                 # no block row of one kind
        dense_cols = seg[kinds]
        assert np.array_equal(dense_cols, top["b_col_idx"][top["b_row_ptr"][r]:top["b_row_ptr"][r + 1]])
