"""Row reordering: the library against fixtures recorded from the compiled reference
(tests/golden/reorder/*.npz, made by tests/golden/make_reorder_golden.py) and, when
oracle/_ref/Matrix_Blocking is present, against the reference program run live."""
import glob
import os
import subprocess

import numpy as np
import pytest

from smat_amd import generators as gen
from tests.oracle_lib import ref_binary

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "reorder", "*.npz")))


def reordered_edges(rows, row_ptr, col_idx, perm):
    rp = row_ptr.astype(np.int64)
    cnt = np.diff(rp)[perm]
    new_rows = np.repeat(np.arange(rows), cnt)
    new_cols = np.concatenate([col_idx[rp[p]:rp[p + 1]] for p in perm]) if rows else np.zeros(0, np.int64)
    return new_rows, new_cols


def test_fixtures_exist():
    assert len(FIXTURES) >= 10


def check_fixture(smat, path):
    d = np.load(path)
    rows, cols = int(d["rows"]), int(d["cols"])
    for k, (cb, rb, tau) in enumerate(d["params"]):
        g, perm, stats = smat.reorder_rows(rows, cols, d["row_ptr"], d["col_idx"], int(cb), int(rb),
                                           float(np.float32(tau)))
        assert np.array_equal(g, d[f"grouping_{k}"]), (k, "grouping")
        assert np.array_equal(stats, d[f"stats_{k}"]), (k, "counters")
        nr, nc = reordered_edges(rows, d["row_ptr"], d["col_idx"], perm)
        assert np.array_equal(nr, d[f"reordered_rows_{k}"]) and np.array_equal(nc, d[f"reordered_cols_{k}"])
        assert np.array_equal(np.sort(perm), np.arange(rows))


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p)[:-4] for p in FIXTURES])
def test_grouping_permutation_and_counters_match_reference(smat, path):
    check_fixture(smat, path)


# The scan over the later rows runs in batches on several threads for large matrices (rows looked at in
# parallel against the current pattern, results applied in row order up to the first merge).  These settings
# send the small recorded matrices through that path: a few rows one by one behind every merge, then batches
# of a handful of rows, so that merges fall into batches at every position.
BATCHED = [dict(SMAT_REORDER_THREADS="4", SMAT_REORDER_SERIAL_ROWS="4", SMAT_REORDER_FIRST_BATCH="16"),
           dict(SMAT_REORDER_THREADS="3", SMAT_REORDER_SERIAL_ROWS="1", SMAT_REORDER_FIRST_BATCH="8"),
           dict(SMAT_REORDER_THREADS="2", SMAT_REORDER_SERIAL_ROWS="1", SMAT_REORDER_FIRST_BATCH="1")]


@pytest.mark.parametrize("env", BATCHED, ids=["4x16", "3x8", "2x1"])
@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p)[:-4] for p in FIXTURES])
def test_fixtures_through_the_batched_scan(smat, monkeypatch, path, env):
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    check_fixture(smat, path)


def run_reference(tmp_path, r, c, cb, rb, tau):
    binary = ref_binary("Matrix_Blocking")
    el = tmp_path / "case.el"
    order = np.lexsort((c, r))
    el.write_text("\n".join(f"{a} {b}" for a, b in zip(r[order].tolist(), c[order].tolist())) + "\n")
    out = tmp_path / "stats.txt"
    subprocess.run([binary, "-f", str(el), "-a", "5", "-b", str(cb), "-B", str(rb), "-F", "1", "-t", repr(tau),
                    "-v", "0", "-o", str(out)], check=True, stdout=subprocess.DEVNULL)
    fields = (tmp_path / "stats.txt.g").read_text().strip().split(",")
    return np.array([int(x) for x in fields[1:] if x], dtype=np.int64)


@pytest.mark.skipif(ref_binary("Matrix_Blocking") is None, reason="oracle/_ref/Matrix_Blocking not built")
@pytest.mark.parametrize("seed", range(6))
def test_live_against_reference_program(smat, tmp_path, seed):
    rng = np.random.default_rng(seed)
    rows, cols = int(rng.integers(50, 1500)), int(rng.integers(50, 3000))
    nnz = int(rows * rng.uniform(1, 12))
    key = np.unique(rng.integers(0, rows, nnz) * cols + rng.integers(0, cols, nnz))
    r, c = key // cols, key % cols
    # duplicate some row patterns so merges happen
    src = rng.integers(0, rows, rows // 3)
    extra_r, extra_c = [], []
    for dst_row, s in enumerate(src):
        m = r == s
        extra_r.append(np.full(int(m.sum()), (dst_row * 7) % rows))
        extra_c.append(c[m])
    key = np.unique(np.concatenate([r] + extra_r) * cols + np.concatenate([c] + extra_c))
    r, c = key // cols, key % cols
    if r.max() != rows - 1:
        rows = int(r.max()) + 1
    cb, rb, tau = [(16, 16, 0.5), (8, 16, 0.5), (16, 16, 0.2), (5, 4, 0.6), (16, 16, 0.8), (1, 2, 0.5)][seed]
    want = run_reference(tmp_path, r, c, cb, rb, tau)
    row_ptr = np.zeros(rows + 1, dtype=np.int64)
    np.add.at(row_ptr, r + 1, 1)
    g, perm, _ = smat.reorder_rows(rows, int(c.max()) + 1, np.cumsum(row_ptr), c, cb, rb, float(np.float32(tau)))
    assert np.array_equal(g, want)


@pytest.mark.skipif(ref_binary("Matrix_Blocking") is None, reason="oracle/_ref/Matrix_Blocking not built")
def test_live_against_reference_program_stencil_32k_rows(smat, tmp_path):
    """A structured matrix two orders of magnitude larger than the recorded fixtures (the 64-cubed stencil,
    262,144 rows, was compared once by hand: identical grouping, 0.32 s here against 7.5 s there)."""
    d = gen.stencil27(32)
    rows = int(d["M"])
    r = np.repeat(np.arange(rows), np.diff(d["row_ptr"]))
    c = d["col_idx"].astype(np.int64)
    want = run_reference(tmp_path, r, c, 16, 16, 0.5)
    g, perm, _ = smat.reorder_rows(rows, int(d["K"]), d["row_ptr"].astype(np.int64), c, 16, 16, 0.5)
    assert np.array_equal(g, want)


@pytest.mark.skipif(ref_binary("Matrix_Blocking") is None, reason="oracle/_ref/Matrix_Blocking not built")
@pytest.mark.parametrize("threads", ["1", "default", "4x64"])
def test_live_against_reference_program_power_law_16k_rows(smat, tmp_path, monkeypatch, threads):
    """R-MAT rows: the set of candidate rows of a group grows to thousands of entries (the reference trims it
    only in some shapes of its tree), most rows are farther away than all of them, and distances repeat.  That
    is where the shortcuts of the candidate set act (no-op insertions, the place of a key found from the last
    key with the same distance), and 16,384 rows are enough for the threaded scan to switch itself on."""
    if threads == "1":
        monkeypatch.setenv("SMAT_REORDER_THREADS", "1")
    elif threads == "4x64":
        for k, v in dict(SMAT_REORDER_THREADS="4", SMAT_REORDER_SERIAL_ROWS="8", SMAT_REORDER_FIRST_BATCH="64").items():
            monkeypatch.setenv(k, v)
    d = gen.rmat(14, 16)
    r = np.repeat(np.arange(int(d["M"])), np.diff(d["row_ptr"]))
    c = d["col_idx"].astype(np.int64)
    rows = int(r.max()) + 1  # rows behind the last nonempty one do not exist in an edge list
    want = run_reference(tmp_path, r, c, 16, 16, 0.5)
    g, perm, _ = smat.reorder_rows(rows, int(d["K"]), d["row_ptr"].astype(np.int64)[:rows + 1], c, 16, 16, 0.5)
    assert np.array_equal(g, want)


def test_threaded_scan_gives_the_single_thread_result_at_32k_rows(smat, monkeypatch):
    """Both passes of 32,768 R-MAT rows with the default thread count against one thread."""
    d = gen.rmat(15, 16)
    got = smat.reorder_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], 16, 16, 0.5, True)
    monkeypatch.setenv("SMAT_REORDER_THREADS", "1")
    want = smat.reorder_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], 16, 16, 0.5, True)
    for a, b in zip(got, want):
        assert np.array_equal(a, b)


TWO_PASS = sorted(glob.glob(os.path.join(HERE, "golden", "reorder_two_pass", "*.npz")))


def check_two_pass(smat, rows, cols, row_ptr, col_idx, cb, rb, tau, want):
    """smat_reorder_csr (row pass, then the same pass on the transpose of the row-permuted pattern) against
    the two runs of the reference program, src/reorder.py:107-182: per pass the reordered edge list, the
    counters, and that the permutation sorts the rows by the GROUPING line."""
    M, K = rows + 5, cols + 3  # trailing empty rows / columns: not in an edge list, they keep their place
    rp = np.concatenate([row_ptr, np.full(5, row_ptr[-1])]).astype(np.int32)
    pr, pc, sr, sc = smat.reorder_csr(M, K, rp, col_idx, cb, rb, tau, do_cols=True)
    assert np.array_equal(np.sort(pr), np.arange(M)) and np.array_equal(np.sort(pc), np.arange(K))
    assert np.array_equal(pr[rows:], np.arange(rows, M)) and np.array_equal(pc[cols:], np.arange(cols, K))
    pr, pc = pr[:rows], pc[:cols]
    # row pass
    nr, nc = reordered_edges(rows, row_ptr, col_idx, pr)
    assert np.array_equal(nr, want["row_pass_el"][:, 0]) and np.array_equal(nc, want["row_pass_el"][:, 1])
    assert np.array_equal(sr, want["stats_rows"])
    assert np.all(np.diff(want["grouping_rows"][pr]) >= 0)
    # column pass: the rows of the transpose are the columns; its edge list after the pass is
    # (new column, new row) sorted by new column, the new rows of a column ascending
    inv_c = np.empty(cols, np.int64)
    inv_c[pc] = np.arange(cols)
    t_rows, t_cols = inv_c[nc], nr
    order = np.lexsort((t_cols, t_rows))
    assert np.array_equal(t_rows[order], want["col_pass_el"][:, 0]) and np.array_equal(t_cols[order], want["col_pass_el"][:, 1])
    assert np.array_equal(sc, want["stats_cols"])
    assert want["grouping_cols"].size == cols and np.all(np.diff(want["grouping_cols"][pc]) >= 0)


def test_two_pass_fixtures_exist():
    assert len(TWO_PASS) >= 5


@pytest.mark.parametrize("path", TWO_PASS, ids=[os.path.basename(p)[:-4] for p in TWO_PASS])
def test_column_pass_matches_reference_on_the_transposed_row_permuted_edge_list(smat, path):
    d = np.load(path)
    cb, rb, tau = d["params"]
    check_two_pass(smat, int(d["rows"]), int(d["cols"]), d["row_ptr"], d["col_idx"], int(cb), int(rb), float(np.float32(tau)), d)


@pytest.mark.skipif(ref_binary("Matrix_Blocking") is None, reason="oracle/_ref/Matrix_Blocking not built")
@pytest.mark.parametrize("seed", range(4))
def test_two_pass_live_against_reference_program(smat, tmp_path, seed):
    import sys
    sys.path.insert(0, os.path.join(HERE, "golden"))
    import make_reorder_golden as mk
    rng = np.random.default_rng(100 + seed)
    rows, cols = int(rng.integers(100, 900)), int(rng.integers(100, 1200))
    nnz = int(rows * rng.uniform(2, 10))
    key = np.unique(np.concatenate([rng.integers(0, rows, nnz) * cols + rng.integers(0, cols, nnz),
                                    [(rows - 1) * cols + cols - 1]]))
    r, c = key // cols, key % cols
    cb, rb, tau = [(16, 16, 0.5), (8, 16, 0.5), (16, 16, 0.3), (4, 6, 0.6)][seed]
    (g1, el1, st1), (g2, el2, st2) = mk.run_two_pass(r, c, cb, rb, tau, str(tmp_path))
    row_ptr = np.zeros(rows + 1, dtype=np.int64)
    np.add.at(row_ptr, r + 1, 1)
    want = {"row_pass_el": el1, "col_pass_el": el2, "stats_rows": st1, "stats_cols": st2, "grouping_rows": g1, "grouping_cols": g2}
    check_two_pass(smat, rows, cols, np.cumsum(row_ptr), c, cb, rb, float(np.float32(tau)), want)


def test_two_pass_flow_and_permute(smat):
    d = gen.stencil27(10)  # 1000 rows -> padded to 1008
    M = K = 1008
    rp = np.concatenate([d["row_ptr"], np.full(8, d["row_ptr"][-1])]).astype(np.int32)
    pr, pc, sr, sc = smat.reorder_csr(M, K, rp, d["col_idx"], 16, 16, 0.5, do_cols=True)
    assert np.array_equal(np.sort(pr), np.arange(M)) and np.array_equal(np.sort(pc), np.arange(K))
    assert np.array_equal(pr[1000:], np.arange(1000, M)) and np.array_equal(pc[1000:], np.arange(1000, K))
    # row pass alone equals the single-pass API on the 1000 real rows
    g, perm, stats = smat.reorder_rows(1000, 1000, d["row_ptr"], d["col_idx"], 16, 16, 0.5)
    assert np.array_equal(pr[:1000], perm) and np.array_equal(sr, stats)
    # permuting keeps every entry: value multiset per (old row, old col) is preserved
    rp2, ci2, v2 = smat.permute_csr(M, K, rp, d["col_idx"], d["val"], pr, pc)
    assert rp2[-1] == rp[-1]
    inv_c = np.empty(K, np.int64)
    inv_c[pc] = np.arange(K)
    for new_r in (0, 17, 500, 999):
        old = pr[new_r]
        want = sorted(zip(inv_c[d["col_idx"][rp[old]:rp[old + 1]]].tolist(), d["val"][rp[old]:rp[old + 1]].tolist()))
        got = list(zip(ci2[rp2[new_r]:rp2[new_r + 1]].tolist(), v2[rp2[new_r]:rp2[new_r + 1]].tolist()))
        assert got == want
    # the point of the exercise: fewer nonzero blocks than the natural order here? (not guaranteed in general,
    # so only the bookkeeping is asserted) -- the block count reported by the pass equals the BCSR of its output
    a_rows_only = smat.csr_to_bcsr(M, K, *smat.permute_csr(M, K, rp, d["col_idx"], d["val"], pr, None))
    assert a_rows_only.nnzb == sr[2]


def test_bad_arguments(smat):
    with pytest.raises(smat.SmatError):
        smat.reorder_rows(2, 4, np.array([0, 2, 3]), np.array([3, 1, 0]), 16, 16, 0.5)  # unsorted row
    with pytest.raises(smat.SmatError):
        smat.reorder_rows(1, 4, np.array([0, 1]), np.array([0]), 0, 16, 0.5)
    with pytest.raises(smat.SmatError):
        smat.permute_csr(16, 16, np.zeros(17, np.int32), np.zeros(0, np.int32), np.zeros(0, np.uint16),
                         np.zeros(16, np.int64), None)  # not a permutation
