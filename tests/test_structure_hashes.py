"""The blocked structure of every benchmark workload, and the permutations of the reordered ones, against the
hashes recorded in tests/golden/structure_hashes.json (made by tests/golden/make_structure_hashes.py on the
build machine).  Run without a GPU it checks this machine's host code; marked gpu it checks the GPU machine's
host code (its C++ library decides the order of equal keys in the reorder's sorts) and the device-side blocking."""
import json
import os

import numpy as np
import pytest

import bench

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = json.load(open(os.path.join(HERE, "golden", "structure_hashes.json")))
# the reordered R-MAT scale 20 workload (permutations from tests/golden/rmat_s20_deg16_perms.npz) takes minutes to
# build on few cores: it runs with the GPU tests only, here and in tests/test_gpu_full_size.py
NAMES = [n for n in sorted(GOLDEN) if n != "rmat_s20_deg16_reordered_N128"]
REFERENCE_DERIVED = [n for n in sorted(GOLDEN) if "reference" in GOLDEN[n]]


def check(name):
    bench.INFO.clear()
    A, _, N = bench.build_workload(name, want_b=False)
    want = GOLDEN[name]
    assert (int(A["M"]), int(A["K"]), int(N), int(A["nnzb"])) == (want["M"], want["K"], want["N"], want["nnzb"])
    assert bench.sha256_of(A["b_row_ptr"].astype(np.int32), A["b_col_idx"].astype(np.int32)) == want["pattern_sha256"]
    assert bench.sha256_of(np.ascontiguousarray(A["b_val"])) == want["values_sha256"]
    if "perm_sha256" in want:
        assert bench.INFO["perm_sha256"] == want["perm_sha256"]
    res = bench.structure_against_golden(name, A)
    assert res is not None and res["ok"] and not res["differs"]
    if "reference" in want:
        # the reference's own program, run on this pattern and then on the transpose of its output, ends with the
        # same blocked structure and reports the same counters (comparisons, merges, blocks, longest row) per pass
        ref = want["reference"]
        assert res["equals_reference_program"]
        assert want["pattern_sha256"] == ref["pattern_sha256"] and want["nnzb"] == ref["nnzb"]
        assert bench.INFO["reorder_counters"] == [ref["stats_rows"], ref["stats_cols"]]
    return A


def test_fixture_covers_every_config():
    assert len(GOLDEN) >= 9 and "rmat_s20_deg16_reordered_N128" in GOLDEN
    assert all(len(e["pattern_sha256"]) == 64 for e in GOLDEN.values())
    # the reordered forms of configs 2 and 5 at full size and of config 3 at reduced scales are pinned to the
    # output of the reference's reorder program
    assert {"er_16384_0.1pct_reordered_N256", "stencil27_64_reordered_N64", "rmat_s15_deg16_reordered_N128",
            "rmat_s16_deg16_reordered_N128"} <= set(REFERENCE_DERIVED)


@pytest.mark.parametrize("name", NAMES)
def test_structure_matches_the_recorded_hashes(name):
    check(name)


def test_a_changed_structure_is_reported():
    A, _, _ = bench.build_workload("band_4096_bw64_N128", want_b=False)
    A = dict(A, b_col_idx=A["b_col_idx"].copy())
    A["b_col_idx"][5] += 16
    res = bench.structure_against_golden("band_4096_bw64_N128", A)
    assert not res["ok"] and res["differs"] == ["pattern_sha256"]


@pytest.mark.gpu
@pytest.mark.timeout(900)
@pytest.mark.parametrize("name", NAMES)
def test_structure_on_the_gpu_machine(smat, cuda, name):
    check(name)


@pytest.mark.gpu
@pytest.mark.parametrize("gen_name,args,workload", [("band", (4096, 64), "band_4096_bw64_N128"),
                                                    ("erdos_renyi", (16384, 0.001), "er_16384_0.1pct_N256"),
                                                    ("stencil27", (64,), "stencil27_64_N64"),
                                                    ("rmat", (20, 16), "rmat_s20_deg16_N128")])
def test_device_blocking_gives_the_recorded_structure(smat, cuda, gen_name, args, workload):
    import torch
    from smat_amd import generators as gen
    d = getattr(gen, gen_name)(*args)
    rp = torch.from_numpy(d["row_ptr"].astype(np.int32)).to(cuda)
    ci = torch.from_numpy(d["col_idx"].astype(np.int32)).to(cuda)
    v = torch.from_numpy(np.ascontiguousarray(d["val"]).view(np.int16)).to(cuda)
    dev = smat.csr_to_bcsr_device(d["M"], d["K"], rp, ci, v, int(d["row_ptr"][d["M"]]))
    b = dev.to_host()
    dev.close()
    want = GOLDEN[workload]
    assert b.nnzb == want["nnzb"]
    assert bench.sha256_of(b.row_ptr.astype(np.int32), b.col_idx.astype(np.int32)) == want["pattern_sha256"]
    assert bench.sha256_of(np.ascontiguousarray(b.val)) == want["values_sha256"]
