"""Regenerates tests/golden/reorder/*.npz from the compiled reference reorderer.

Run in the build container (needs oracle/_ref/Matrix_Blocking, i.e. `make -C oracle ref`):

    python tests/golden/make_reorder_golden.py

For every case it writes a seeded edge list, runs
`Matrix_Blocking -f <case>.el -a 5 -b <col_block> -B <row_block> -F 1 -t <tau> -v 0 -o <out>`
(the command line of src/reorder.py:131-132), and stores, as plain arrays,
the input CSR pattern, the GROUPING line of `<out>.g`, the row order of
`<case>_reordered.el`, and the integer statistics comparison_counter,
merge_counter, VBR_nzblocks_count and VBR_longest_row from the stats file.
Only data is stored; nothing of the reference's code.

It also records the two-pass flow of src/reorder.py:107-182 into tests/golden/reorder_two_pass/*.npz:
the program on <case>.el, then on the transpose of <case>_reordered.el ((u, v) -> (v, u), lines sorted,
src/reorder.py:82-104), with both GROUPING lines, both reordered edge lists and both sets of counters.
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from smat_amd import generators as gen  # noqa: E402

REF_BIN = os.path.join(ROOT, "oracle", "_ref", "Matrix_Blocking")
OUT_DIR = os.path.join(HERE, "reorder")


def er_pattern(rows, cols, nnz, seed):
    idx = np.arange(nnz, dtype=np.uint64)
    r = (gen.rand_u64(seed, idx * np.uint64(2)) % np.uint64(rows)).astype(np.int64)
    c = (gen.rand_u64(seed, idx * np.uint64(2) + np.uint64(1)) % np.uint64(cols)).astype(np.int64)
    key = np.unique(r * cols + c)
    return key // cols, key % cols


def clustered_pattern(rows, cols, templates, per_row_noise, seed):
    """Rows are noisy copies of a few template rows scattered far apart: exercises merges,
    the distance-cache skip and the candidate-set top-up."""
    t_cols = [np.unique((gen.rand_u64(seed + 17 * t, np.arange(24, dtype=np.uint64)) % np.uint64(cols)).astype(np.int64))
              for t in range(templates)]
    which = (gen.rand_u64(seed ^ 0x33, np.arange(rows, dtype=np.uint64)) % np.uint64(templates)).astype(np.int64)
    rr, cc = [], []
    for r in range(rows):
        base = t_cols[which[r]]
        drop = gen.rand_uniform(seed ^ 0x55, np.arange(r * 64, r * 64 + base.size, dtype=np.uint64)) < 0.15
        extra = (gen.rand_u64(seed ^ 0x77, np.arange(r * 8, r * 8 + per_row_noise, dtype=np.uint64)) % np.uint64(cols)).astype(np.int64)
        c = np.unique(np.concatenate([base[~drop], extra]))
        rr.append(np.full(c.size, r, dtype=np.int64))
        cc.append(c)
    return np.concatenate(rr), np.concatenate(cc)


def csr_pattern(d):
    rows = np.repeat(np.arange(d["M"], dtype=np.int64), np.diff(d["row_ptr"]))
    return rows, d["col_idx"].astype(np.int64)


def rmat_small(scale, deg, seed):
    d = gen.rmat(scale=scale, avg_degree=deg, seed=seed)
    return csr_pattern(d)


def with_gaps(rows_cols, every):
    """Empties every `every`-th row (keeps the last row so the row count is unchanged)."""
    r, c = rows_cols
    keep = (r % every != 1) | (r == r.max())
    return r[keep], c[keep]


CASES = {
    # name: (pattern builder, [(col_block, row_block, tau), ...])
    "er_256": (lambda: er_pattern(256, 256, 2048, 11), [(16, 16, 0.5), (8, 16, 0.5), (16, 16, 0.1), (3, 3, 0.6)]),
    "er_1024": (lambda: er_pattern(1024, 1024, 16384, 12), [(16, 16, 0.5), (8, 16, 0.5), (16, 16, 0.9)]),
    "er_4096_sparse": (lambda: er_pattern(4096, 4096, 16384, 13), [(16, 16, 0.5), (8, 16, 0.5)]),
    "er_rect_600x900": (lambda: er_pattern(600, 900, 6000, 14), [(16, 16, 0.5), (4, 8, 0.4)]),
    "er_gaps_500": (lambda: with_gaps(er_pattern(500, 500, 5000, 15), 7), [(16, 16, 0.5), (8, 16, 0.7)]),
    "band_512_bw8": (lambda: csr_pattern(gen.band(512, 8)), [(16, 16, 0.5), (8, 16, 0.5), (16, 16, 0.1)]),
    "stencil_8": (lambda: csr_pattern(gen.stencil27(8)), [(16, 16, 0.5), (8, 16, 0.5), (3, 3, 0.6)]),
    "stencil_12": (lambda: csr_pattern(gen.stencil27(12)), [(16, 16, 0.5), (16, 16, 0.1)]),
    "rmat_8": (lambda: rmat_small(8, 8, 21), [(16, 16, 0.5), (8, 16, 0.5), (3, 3, 0.6)]),
    "rmat_10": (lambda: rmat_small(10, 8, 22), [(16, 16, 0.5), (8, 16, 0.5), (16, 16, 0.1)]),
    "rmat_12": (lambda: rmat_small(12, 6, 23), [(16, 16, 0.5), (8, 16, 0.5)]),
    "clustered_800": (lambda: clustered_pattern(800, 2048, 9, 2, 31), [(16, 16, 0.5), (8, 16, 0.5), (16, 16, 0.3), (16, 5, 0.5)]),
    "clustered_2000": (lambda: clustered_pattern(2000, 4096, 40, 1, 32), [(16, 16, 0.5), (16, 16, 0.7), (4, 7, 0.5)]),
}


def write_el(path, r, c):
    order = np.lexsort((c, r))
    with open(path, "w") as f:
        f.write("\n".join(f"{a} {b}" for a, b in zip(r[order].tolist(), c[order].tolist())))
        f.write("\n")


def run_reference(r, c, col_block, row_block, tau, workdir):
    el = os.path.join(workdir, "case.el")
    out = os.path.join(workdir, "stats.txt")
    write_el(el, r, c)
    subprocess.run([REF_BIN, "-f", el, "-a", "5", "-b", str(col_block), "-B", str(row_block), "-F", "1",
                    "-t", repr(tau), "-v", "0", "-o", out], check=True, stdout=subprocess.DEVNULL)
    with open(out + ".g") as f:
        fields = f.read().strip().split(",")
    assert fields[0] == "GROUPING"
    grouping = np.array([int(x) for x in fields[1:] if x != ""], dtype=np.int64)
    with open(out) as f:
        header = f.readline().strip().split(",")
        values = f.readline().strip().split(",")
    stats = dict(zip(header, values))
    reordered = np.loadtxt(os.path.join(workdir, "case_reordered.el"), dtype=np.int64, ndmin=2)
    return grouping, reordered, np.array([int(stats["comparison_counter"]), int(stats["merge_counter"]),
                                          int(stats["VBR_nzblocks_count"]), int(stats["VBR_longest_row"])],
                                         dtype=np.int64)


TWO_PASS = {
    # name: (case of CASES, col_block, row_block, tau)
    "er_256": ("er_256", 16, 16, 0.5),
    "er_rect_600x900": ("er_rect_600x900", 16, 16, 0.5),
    "er_gaps_500": ("er_gaps_500", 16, 16, 0.5),
    "stencil_8": ("stencil_8", 16, 16, 0.5),
    "rmat_10": ("rmat_10", 16, 16, 0.5),
    "clustered_800_b8": ("clustered_800", 8, 16, 0.5),
}


def run_two_pass(r, c, col_block, row_block, tau, workdir):
    """Both runs of the reference program; returns per pass (grouping, reordered edge list, counters)."""
    first = run_reference(r, c, col_block, row_block, tau, workdir)
    reordered = first[1]
    second_dir = os.path.join(workdir, "t")
    os.makedirs(second_dir)
    second = run_reference(reordered[:, 1], reordered[:, 0], col_block, row_block, tau, second_dir)  # write_el sorts the lines
    return first, second


def main_two_pass():
    out_dir = os.path.join(HERE, "reorder_two_pass")
    os.makedirs(out_dir, exist_ok=True)
    for name, (case, cb, rb, tau) in TWO_PASS.items():
        r, c = CASES[case][0]()
        order = np.lexsort((c, r))
        r, c = r[order], c[order]
        rows = int(r.max()) + 1
        row_ptr = np.zeros(rows + 1, dtype=np.int64)
        np.add.at(row_ptr, r + 1, 1)
        with tempfile.TemporaryDirectory() as wd:
            (g1, el1, st1), (g2, el2, st2) = run_two_pass(r, c, cb, rb, tau, wd)
        np.savez_compressed(os.path.join(out_dir, name + ".npz"), rows=np.int64(rows), cols=np.int64(c.max() + 1),
                            row_ptr=np.cumsum(row_ptr).astype(np.int32), col_idx=c.astype(np.int32),
                            params=np.array([cb, rb, tau], dtype=np.float64),
                            grouping_rows=g1.astype(np.int32), grouping_cols=g2.astype(np.int32),
                            row_pass_el=el1.astype(np.int32), col_pass_el=el2.astype(np.int32),
                            stats_rows=st1, stats_cols=st2)
        print(f"two-pass {name} b={cb} B={rb} tau={tau}: rows={rows} stats {st1.tolist()} then {st2.tolist()}")


def main():
    if not os.path.exists(REF_BIN):
        sys.exit(f"{REF_BIN} missing: run `make -C oracle ref` first")
    os.makedirs(OUT_DIR, exist_ok=True)
    for name, (builder, params) in CASES.items():
        r, c = builder()
        order = np.lexsort((c, r))
        r, c = r[order], c[order]
        rows = int(r.max()) + 1
        row_ptr = np.zeros(rows + 1, dtype=np.int64)
        np.add.at(row_ptr, r + 1, 1)
        row_ptr = np.cumsum(row_ptr)
        store = {"rows": np.int64(rows), "cols": np.int64(c.max() + 1), "row_ptr": row_ptr.astype(np.int32),
                 "col_idx": c.astype(np.int32), "params": np.array(params, dtype=np.float64)}
        for k, (cb, rb, tau) in enumerate(params):
            with tempfile.TemporaryDirectory() as wd:
                grouping, reordered, stats = run_reference(r, c, cb, rb, tau, wd)
            store[f"grouping_{k}"] = grouping.astype(np.int32)
            # the reordered edge list has one line per nonzero, "newrow col", rows ascending;
            # keep only the columns (the row structure follows from the permutation) as a checksum-free exact record
            store[f"reordered_rows_{k}"] = reordered[:, 0].astype(np.int32)
            store[f"reordered_cols_{k}"] = reordered[:, 1].astype(np.int32)
            store[f"stats_{k}"] = stats
            print(f"{name} b={cb} B={rb} tau={tau}: rows={rows} nnz={c.size} stats={stats.tolist()}")
        np.savez_compressed(os.path.join(OUT_DIR, name + ".npz"), **store)


if __name__ == "__main__":
    main()
    main_two_pass()
