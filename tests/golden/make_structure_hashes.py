"""Writes structure_hashes.json: SHA-256 of the blocked structure (row_ptr, col_idx as int32) and of the row and
column permutations of every benchmark workload, computed by this build on the machine the file is made on.

    python tests/golden/make_structure_hashes.py [--perm-file rmat_scale20_perms.npz]

The tests and bench.py recompute the same hashes wherever they run (the GPU machine's host code and its
device-side blocking) and compare: the structure must be the same bit for bit on every machine.  The reordered
R-MAT scale 20 workload needs the permutations of an earlier smat_amd.reorder_csr run (ten minutes on eight
threads): they are read from rmat_s20_deg16_perms.npz next to this file unless --perm-file names another file.
The "reference" records inside the entries (what the reference's own program made of the same patterns) are
written by make_reference_structures.py and carried over here."""
import argparse
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import bench  # noqa: E402

WORKLOADS = ["band_4096_bw64_N128", "er_16384_0.1pct_N256", "er_16384_0.1pct_reordered_N256", "rmat_s20_deg16_N128",
             "rmat_s20_deg16_reordered_N128", "block_pruned_8192_10pct_N4096", "half_pruned_half_er_8192_N4096", "pruned_plus_er_8192_N4096", "block_pruned_skewed_8192_N4096",
             "stencil27_64_N64", "stencil27_64_reordered_N64", "rmat_s15_deg16_reordered_N128", "rmat_s16_deg16_reordered_N128",
             "rmat_s17_deg16_reordered_N128"]
OUT = os.path.join(HERE, "structure_hashes.json")


def entry(name):
    bench.INFO.clear()
    A, _, N = bench.build_workload(name, want_b=False)
    e = {"M": int(A["M"]), "K": int(A["K"]), "N": int(N), "nnzb": int(A["nnzb"]),
         "pattern_sha256": bench.sha256_of(A["b_row_ptr"].astype(np.int32), A["b_col_idx"].astype(np.int32)),
         "values_sha256": bench.sha256_of(np.ascontiguousarray(A["b_val"]))}
    if "perm_sha256" in bench.INFO:
        e["perm_sha256"] = bench.INFO["perm_sha256"]
    return e


def keep_reference(new, old):
    """The "reference" record of an entry is written by make_reference_structures.py: carried over."""
    if old and "reference" in old:
        new["reference"] = old["reference"]
    return new


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--perm-file", default=None)
    args = ap.parse_args()
    bench.PERM_FILE = args.perm_file
    old = json.load(open(OUT)) if os.path.exists(OUT) else {}
    out = {}
    for name in WORKLOADS:
        out[name] = keep_reference(entry(name), old.get(name))
        print(name, out[name], flush=True)
    with open(OUT, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")


if __name__ == "__main__":
    main()
