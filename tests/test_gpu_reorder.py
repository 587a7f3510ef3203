"""The reorder fixtures replayed on the GPU box: the permutation inside a group comes from std::sort's
order of equal keys, which depends on the C++ library of the machine the tests run on."""
import os

import numpy as np
import pytest

from tests.test_reorder import FIXTURES, TWO_PASS, check_two_pass, reordered_edges

pytestmark = pytest.mark.gpu
ROW_PASS = [p for p in FIXTURES if os.path.basename(p)[:-4] in ("er_1024", "stencil_12", "rmat_12", "clustered_2000", "er_gaps_500")]


def test_enough_fixtures():
    assert len(ROW_PASS) >= 4 and len(TWO_PASS) >= 3


@pytest.mark.parametrize("path", ROW_PASS, ids=[os.path.basename(p)[:-4] for p in ROW_PASS])
def test_row_pass_fixture_on_this_machine(smat, path):
    d = np.load(path)
    rows, cols = int(d["rows"]), int(d["cols"])
    for k, (cb, rb, tau) in enumerate(d["params"]):
        g, perm, stats = smat.reorder_rows(rows, cols, d["row_ptr"], d["col_idx"], int(cb), int(rb), float(np.float32(tau)))
        assert np.array_equal(g, d[f"grouping_{k}"]) and np.array_equal(stats, d[f"stats_{k}"])
        nr, nc = reordered_edges(rows, d["row_ptr"], d["col_idx"], perm)
        assert np.array_equal(nr, d[f"reordered_rows_{k}"]) and np.array_equal(nc, d[f"reordered_cols_{k}"])


@pytest.mark.parametrize("path", TWO_PASS, ids=[os.path.basename(p)[:-4] for p in TWO_PASS])
def test_two_pass_fixture_on_this_machine(smat, path):
    d = np.load(path)
    cb, rb, tau = d["params"]
    check_two_pass(smat, int(d["rows"]), int(d["cols"]), d["row_ptr"], d["col_idx"], int(cb), int(rb), float(np.float32(tau)), d)


@pytest.mark.parametrize("path", ROW_PASS[:3], ids=[os.path.basename(p)[:-4] for p in ROW_PASS[:3]])
def test_row_pass_fixture_through_the_threaded_scan_on_this_machine(smat, monkeypatch, path):
    """The same fixtures through the batched scan on helper threads (small batches, so that merges fall into
    them): thread creation, spinning helpers and the ordered application on this machine's cores."""
    for k, v in dict(SMAT_REORDER_THREADS="8", SMAT_REORDER_SERIAL_ROWS="2", SMAT_REORDER_FIRST_BATCH="32").items():
        monkeypatch.setenv(k, v)
    test_row_pass_fixture_on_this_machine(smat, path)


def test_threaded_scan_gives_the_single_thread_result_at_32k_rows(smat, monkeypatch):
    """32,768 R-MAT rows with this machine's default thread count against one thread."""
    from smat_amd import generators as gen
    d = gen.rmat(15, 16)
    rows = int(np.flatnonzero(np.diff(d["row_ptr"]))[-1]) + 1
    args = (rows, int(d["K"]), d["row_ptr"].astype(np.int64)[:rows + 1], d["col_idx"].astype(np.int64), 16, 16, 0.5)
    g_many, perm_many, stats_many = smat.reorder_rows(*args)
    monkeypatch.setenv("SMAT_REORDER_THREADS", "1")
    g_one, perm_one, stats_one = smat.reorder_rows(*args)
    assert np.array_equal(g_many, g_one) and np.array_equal(perm_many, perm_one) and np.array_equal(stats_many, stats_one)
