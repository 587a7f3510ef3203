"""Adds to structure_hashes.json what the REFERENCE program makes of the reordered benchmark matrices.

Run in the build container (needs oracle/_ref/Matrix_Blocking, i.e. `make -C oracle ref`):

    python tests/golden/make_reference_structures.py [name ...]

For every workload below it writes the pattern of the generated matrix as an edge list, runs the reference's
`Matrix_Blocking -a 5 -b 16 -B 16 -F 1 -t 0.5` on it and then on the transpose of `<case>_reordered.el`
(the two runs of src/reorder.py:131-132,174-175), takes the pattern that comes out of the second run
((new column, new row) per line), blocks it 16 x 16 and records under "reference" in the workload's entry:
the SHA-256 of that row_ptr / col_idx (int32), the number of blocks and the four counters of each pass.
Only the reference program's output is used for this: the repository's own reorder is not run here.
tests/test_structure_hashes.py and bench.py then compare what the library produces with these records.
"""
import json
import os
import subprocess
import sys
import tempfile
import time

import numpy as np
import pandas as pd

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from smat_amd import generators as gen  # noqa: E402

REF_BIN = os.path.join(ROOT, "oracle", "_ref", "Matrix_Blocking")
OUT = os.path.join(HERE, "structure_hashes.json")

# workload -> generator of the CSR whose pattern is reordered
WORKLOADS = {
    "er_16384_0.1pct_reordered_N256": lambda: gen.erdos_renyi(16384, 0.001),
    "stencil27_64_reordered_N64": lambda: gen.stencil27(64),
    "rmat_s15_deg16_reordered_N128": lambda: gen.rmat(15, 16),
    "rmat_s16_deg16_reordered_N128": lambda: gen.rmat(16, 16),
    "rmat_s17_deg16_reordered_N128": lambda: gen.rmat(17, 16),
}


def sha256_of(*arrays):
    import hashlib
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def write_el(path, r, c):
    order = np.lexsort((c, r))
    pd.DataFrame({"r": r[order], "c": c[order]}).to_csv(path, sep=" ", header=False, index=False)


def run_pass(r, c, workdir):
    """One run of the reference program on the edge list (r, c); returns the reordered edge list and the counters."""
    os.makedirs(workdir, exist_ok=True)
    el, out = os.path.join(workdir, "case.el"), os.path.join(workdir, "stats.txt")
    write_el(el, r, c)
    subprocess.run([REF_BIN, "-f", el, "-a", "5", "-b", "16", "-B", "16", "-F", "1", "-t", "0.5", "-v", "0", "-o", out],
                   check=True, stdout=subprocess.DEVNULL)
    with open(out) as f:
        stats = dict(zip(f.readline().strip().split(","), f.readline().strip().split(",")))
    e = pd.read_csv(os.path.join(workdir, "case_reordered.el"), sep=" ", header=None, usecols=[0, 1]).to_numpy(np.int64)
    counters = [int(stats[k]) for k in ("comparison_counter", "merge_counter", "VBR_nzblocks_count", "VBR_longest_row")]
    return e[:, 0], e[:, 1], counters


def block_pattern(rows, cols, M):
    """BCSR row_ptr / col_idx (absolute first column of each block, matrix.h:455) of a pattern."""
    key = np.unique((rows // 16) * (1 << 32) + (cols // 16))
    br, bc = key >> 32, key & 0xFFFFFFFF
    row_ptr = np.zeros(M // 16 + 1, np.int64)
    np.add.at(row_ptr, br + 1, 1)
    return np.cumsum(row_ptr).astype(np.int32), (bc * 16).astype(np.int32)


def main():
    if not os.path.exists(REF_BIN):
        sys.exit(f"{REF_BIN} missing: run `make -C oracle ref` first")
    names = sys.argv[1:] or list(WORKLOADS)
    for name in names:
        d = WORKLOADS[name]()
        r = np.repeat(np.arange(d["M"], dtype=np.int64), np.diff(d["row_ptr"]))
        c = d["col_idx"].astype(np.int64)
        t0 = time.perf_counter()
        with tempfile.TemporaryDirectory() as wd:
            nr, nc, st_rows = run_pass(r, c, os.path.join(wd, "rows"))          # lines: new row, old column
            t_mid = time.perf_counter()
            tr, tc, st_cols = run_pass(nc, nr, os.path.join(wd, "cols"))        # transpose; lines: new column, new row
        rp, ci = block_pattern(tc, tr, d["M"])
        data = json.load(open(OUT))  # read here, not at the start: a run takes minutes
        entry = data.setdefault(name, {})
        entry["reference"] = {
            "program": "oracle/_ref/Matrix_Blocking -a 5 -b 16 -B 16 -F 1 -t 0.5, on the pattern and then on the transpose "
                       "of its reordered edge list",
            "nnzb": int(ci.size), "pattern_sha256": sha256_of(rp, ci), "stats_rows": st_rows, "stats_cols": st_cols,
            "seconds": [round(t_mid - t0, 1), round(time.perf_counter() - t_mid, 1)],
        }
        print(name, entry["reference"], flush=True)
        with open(OUT, "w") as f:
            json.dump(data, f, indent=1, sort_keys=True)
            f.write("\n")


if __name__ == "__main__":
    main()
