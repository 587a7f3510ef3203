"""Command-line tools: Matrix_Blocking writes the same files as the reference program; hgemm runs the
matrix-load -> block -> SpMM -> verify flow on the GPU."""
import filecmp
import os
import subprocess

import numpy as np
import pytest

from smat_amd import generators as gen
from tests.oracle_lib import ref_binary

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "smat_amd", "bin")


def write_el(path, d):
    rows = np.repeat(np.arange(int(d["rows"])), np.diff(d["row_ptr"]))
    path.write_text("\n".join(f"{a} {b}" for a, b in zip(rows.tolist(), d["col_idx"].tolist())) + "\n")


def run_blocking(binary, el, out, cb, rb, tau):
    subprocess.run([binary, "-f", str(el), "-a", "5", "-b", str(cb), "-B", str(rb), "-F", "1", "-t", str(tau),
                    "-v", "0", "-o", str(out)], check=True, stdout=subprocess.DEVNULL)


@pytest.mark.parametrize("case,k", [("clustered_800", 0), ("er_gaps_500", 1), ("stencil_8", 2)])
def test_matrix_blocking_cli_matches_fixture(tmp_path, case, k):
    d = np.load(os.path.join(ROOT, "tests", "golden", "reorder", case + ".npz"))
    cb, rb, tau = d["params"][k]
    el = tmp_path / "case.el"
    write_el(el, d)
    run_blocking(os.path.join(BIN, "Matrix_Blocking"), el, tmp_path / "st.txt", int(cb), int(rb), tau)
    fields = (tmp_path / "st.txt.g").read_text().strip().split(",")
    assert fields[0] == "GROUPING"
    assert [int(x) for x in fields[1:] if x] == d[f"grouping_{k}"].tolist()
    out = np.loadtxt(tmp_path / "case_reordered.el", dtype=np.int64, ndmin=2)
    assert np.array_equal(out[:, 0], d[f"reordered_rows_{k}"]) and np.array_equal(out[:, 1], d[f"reordered_cols_{k}"])


@pytest.mark.skipif(ref_binary("Matrix_Blocking") is None, reason="oracle/_ref/Matrix_Blocking not built")
def test_matrix_blocking_cli_files_identical_to_reference_program(tmp_path):
    d = np.load(os.path.join(ROOT, "tests", "golden", "reorder", "rmat_10.npz"))
    for who, binary in (("mine", os.path.join(BIN, "Matrix_Blocking")), ("ref", ref_binary("Matrix_Blocking"))):
        (tmp_path / who).mkdir()
        write_el(tmp_path / who / "case.el", d)
        run_blocking(binary, tmp_path / who / "case.el", tmp_path / who / "st.txt", 8, 16, 0.5)
    assert filecmp.cmp(tmp_path / "mine" / "st.txt.g", tmp_path / "ref" / "st.txt.g", shallow=False)
    assert filecmp.cmp(tmp_path / "mine" / "case_reordered.el", tmp_path / "ref" / "case_reordered.el", shallow=False)


def write_mtx(path, d, n_rows=None):
    rows = np.repeat(np.arange(d["M"]), np.diff(d["row_ptr"]))
    vals = d["val"].view(np.float16).astype(np.float64)
    with open(path, "w") as f:
        f.write("%%MatrixMarket matrix coordinate real general\n")
        f.write(f"{n_rows or d['M']} {n_rows or d['K']} {rows.size}\n")
        f.write("\n".join(f"{r + 1} {c + 1} {v!r}" for r, c, v in zip(rows.tolist(), d["col_idx"].tolist(), vals.tolist())))
        f.write("\n")


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [[], ["-reorder"], ["-use_plan=false"], ["-kernel=2", "-n_mult=32"]])
def test_hgemm_flow_with_check(tmp_path, extra):
    d = gen.stencil27(10)  # 1000 rows: the loader pads to 1008
    mtx = tmp_path / "stencil10.mtx"
    write_mtx(mtx, d)
    cmd = [os.path.join(BIN, "hgemm"), f"-filename={mtx}", "-n_mult=9", "-enable_check", "-random_b",
           "-warmup_iterations=1", "-profiling_iterations=3", "-sleep_duration=1"] + extra
    run = subprocess.run(cmd, cwd=tmp_path, capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr[-2000:]
    assert "PASS" in run.stderr and "1008 x 1008" in run.stderr and "Done" in run.stderr
    assert (tmp_path / "results_smat.csv").read_text().startswith(str(mtx) + ",")


@pytest.mark.gpu
def test_hgemm_reads_binary_container(tmp_path):
    """The text parse can be done once, ahead of time: hgemm takes the SMATBIN1 file smat_convert writes."""
    d = gen.stencil27(10)
    mtx = tmp_path / "stencil10.mtx"
    write_mtx(mtx, d)
    subprocess.run([os.path.join(BIN, "smat_convert"), "-in", str(mtx), "-out", str(tmp_path / "stencil10.smat")],
                   check=True, stdout=subprocess.DEVNULL)
    cmd = [os.path.join(BIN, "hgemm"), f"-filename={tmp_path / 'stencil10.smat'}", "-n_mult=9", "-enable_check",
           "-random_b", "-warmup_iterations=1", "-profiling_iterations=3", "-sleep_duration=1", "-use_plan"]
    run = subprocess.run(cmd, cwd=tmp_path, capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr[-2000:]
    assert "PASS" in run.stderr and "1008 x 1008" in run.stderr
    # same flow with the blocking done on the GPU: same block counts in the log, same verdict
    run2 = subprocess.run(cmd + ["-gpu_blocking"], cwd=tmp_path, capture_output=True, text=True, timeout=120)
    assert run2.returncode == 0, run2.stderr[-2000:]
    assert "PASS" in run2.stderr and "Blocking on the GPU" in run2.stderr
    blocks = [ln.split("]")[-1] for ln in run.stderr.splitlines() if "nonzero blocks," in ln]
    blocks2 = [ln.split("]")[-1] for ln in run2.stderr.splitlines() if "nonzero blocks," in ln]
    assert blocks and blocks == blocks2


@pytest.mark.gpu
def test_hgemm_lineplot_sweeps_n(tmp_path):
    """createLinePlot of the reference harness (common/tester.h:211-267): one "N, ms" line per N = 8*mult."""
    d = gen.stencil27(10)
    mtx = tmp_path / "stencil10.mtx"
    write_mtx(mtx, d)
    cmd = [os.path.join(BIN, "hgemm"), f"-filename={mtx}", "-random_b", "-warmup_iterations=1", "-profiling_iterations=2",
           "-sleep_duration=1", "-lineplot", "-lineplot_from=14", "-lineplot_to=30", "-lineplot_step=5"]
    run = subprocess.run(cmd, cwd=tmp_path, capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr[-2000:]
    lines = (tmp_path / "results_smat.csv").read_text().strip().splitlines()
    assert [int(ln.split(",")[0]) for ln in lines] == [112, 152, 192, 232]
    assert all(float(ln.split(",")[1]) > 0 for ln in lines)


@pytest.mark.gpu
def test_hgemm_check_fails_on_a_nan_in_the_result(tmp_path):
    """The verify step treats a result that is not a number as a gross error: one NaN planted in C ends the run with
    FAIL and a non-zero status (a maximum taken with std::max alone would never see it)."""
    d = gen.stencil27(10)
    mtx = tmp_path / "stencil10.mtx"
    write_mtx(mtx, d)
    cmd = [os.path.join(BIN, "hgemm"), f"-filename={mtx}", "-n_mult=9", "-enable_check", "-random_b",
           "-warmup_iterations=1", "-profiling_iterations=1", "-sleep_duration=1", "-poison_check"]
    run = subprocess.run(cmd, cwd=tmp_path, capture_output=True, text=True, timeout=120)
    assert run.returncode != 0
    assert "FAIL" in run.stderr and "PASS" not in run.stderr and "not finite" in run.stderr
