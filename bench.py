#!/usr/bin/env python3
"""Headline benchmark: block-sparse SpMM on one MI355X.

A "step" is one SpMM launch C = A_bcsr x B over inputs already resident in HBM.
Default workload = the block-pruned configuration the metric is quoted on:
A 8192 x 8192 fp16, 16x16 block mask with 10% of the blocks kept (dense inside,
N(0, 0.02)), B 8192 x 4096 fp16 N(0,1), fp16 C.  The work list (plan) is built
once, outside the timed region, like the reference builds its BCSR once; it also
looks at the block values once (which columns of the blocks are nonzero).

Prints ONE JSON line: effective GFLOP/s = 2 * nnzb * 256 * N / t, the roofline
fraction of the SpMM kernel (timed with HIP events on the launch stream), and a
CPU baseline (the oracle's blocked loop nest on the host cores, bounded sample).
"""
import argparse
import ctypes as C
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

KERNEL_NAMES = {1: "rowwise", 2: "sweep", 3: "rowwise", 5: "compact", 6: "mixed"}


def profiled(workload, kernel_id):
    """HBM traffic per launch (bytes) and MFMA-busy share that rocprofv3 counted for this kernel on this
    workload, read from the committed summary profiles/spmm_<kernel>_<workload>.md (lines
    `traffic_bytes_per_launch: <number>` and `mfma_busy: <number>`), with the file as `source`.
    Nothing is returned for a pair that has no summary: counters are never measured inside this run."""
    import re
    path = os.path.join(ROOT, "profiles", f"spmm_{KERNEL_NAMES.get(kernel_id, kernel_id)}_{workload}.md")
    if not os.path.exists(path):
        return {}
    text = open(path).read()
    out = {}
    for key in ("traffic_bytes_per_launch", "mfma_busy"):
        m = re.search(rf"^{key}:\s*([0-9.eE+]+)", text, re.M)
        if m:
            out[key] = float(m.group(1))
    if out:
        out["source"] = os.path.relpath(path, ROOT)
    return out


def sha256_of(*arrays):
    import hashlib
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def verify_sample(A, B, N, C_bits, n_sample=24, tol=1e-3):
    """The result of the last timed launch against the CPU oracle on block rows spread over the matrix
    (first, last, and evenly spaced ones between).  Returns the worst error relative to the row L2 norm;
    the caller fails the run above `tol` (fp16 output of an fp32-accumulated product)."""
    from tests.oracle_lib import load_oracle
    oracle = load_oracle()
    rp, ci = A["b_row_ptr"], A["b_col_idx"]
    mb = A["M"] // 16
    rows = np.unique(np.linspace(0, mb - 1, min(mb, n_sample)).astype(np.int64))
    keep = np.concatenate([np.arange(rp[r], rp[r + 1]) for r in rows]).astype(np.int64)
    sub_rp = np.concatenate([[0], np.cumsum([rp[r + 1] - rp[r] for r in rows])]).astype(np.int32)
    want = oracle.spmm_bcsr(16 * rows.size, N, A["K"], sub_rp, ci[keep], A["b_val"].reshape(-1, 256)[keep].ravel(), B,
                            threads=max(1, min(16, os.cpu_count() or 1, oracle.max_threads())))
    got = np.concatenate([C_bits[16 * r:16 * r + 16] for r in rows])
    rel, max_abs, _ = oracle.compare(got, want)
    return {"block_rows": int(rows.size), "blocks": int(keep.size), "max_rel_to_row_l2": float(f"{rel:.3e}"),
            "max_abs": float(f"{max_abs:.3e}"), "tolerance": tol, "ok": bool(rel <= tol and np.isfinite(rel))}


GOLDEN_STRUCTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "golden", "structure_hashes.json")


def structure_against_golden(name, A):
    """Compares the blocked structure (and the permutations of a reordered workload) with the hashes recorded
    when the fixture file was made on another machine and, where the entry holds one, with the structure the
    reference's own reorder program produced for this workload.  None if the workload has no entry."""
    if not os.path.exists(GOLDEN_STRUCTURE):
        return None
    want = json.load(open(GOLDEN_STRUCTURE)).get(name)
    if want is None:
        return None
    got = {"nnzb": int(A["nnzb"]),
           "pattern_sha256": sha256_of(A["b_row_ptr"].astype(np.int32), A["b_col_idx"].astype(np.int32)),
           "values_sha256": sha256_of(np.ascontiguousarray(A["b_val"]))}
    if "perm_sha256" in want:
        got["perm_sha256"] = INFO.get("perm_sha256")
    res = {"ok": all(got[k] == want[k] for k in got), "fixture": "tests/golden/structure_hashes.json",
           "differs": [k for k in got if got[k] != want[k]]}
    ref = want.get("reference")
    if ref is not None:
        # what the reference's own reorder program, run twice on this pattern, made of it (recorded by
        # tests/golden/make_reference_structures.py): same blocked structure, same counters per pass
        same = got["pattern_sha256"] == ref["pattern_sha256"] and got["nnzb"] == ref["nnzb"]
        counters = INFO.get("reorder_counters")
        if counters is not None:
            same = same and counters == [ref["stats_rows"], ref["stats_cols"]]
        res["equals_reference_program"] = bool(same)
        res["ok"] = res["ok"] and bool(same)
        if not same:
            res["differs"].append("reference")
    return res


RMAT20_PERMS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "golden", "rmat_s20_deg16_perms.npz")
INFO = {}  # facts about the generated workload that go into the config of the result line
PERM_FILE = None


def build_workload(name, want_b=True):
    from smat_amd import generators as gen
    import smat_amd
    if name == "block_pruned_8192_10pct_N4096":
        A = gen.block_pruned(8192, 0.10, 0.02)
        N, bdist, bseed = 4096, "normal", 0xB0000004
    elif name == "half_pruned_half_er_8192_N4096":
        # two kinds of block rows in one matrix (dense blocks above, about one nonzero per block below): mixed dispatch
        A = gen.half_pruned_half_er(8192, 0.10, 0.001)
        N, bdist, bseed = 4096, "normal", 0xB0000006
    elif name == "pruned_plus_er_8192_N4096":
        # both kinds of blocks in every block row (dense blocks, about one nonzero per block between them): mixed dispatch per block
        A = gen.pruned_plus_er(8192, 0.10, 0.001)
        N, bdist, bseed = 4096, "normal", 0xB0000007
    elif name == "block_pruned_skewed_8192_N4096":
        # a weight whose rows were pruned unevenly (18 % of the blocks kept in the first block row, 2 % in the last): the
        # sweep kernel's plan deals the block rows to its row groups by their block count
        A = gen.block_pruned_skewed(8192, 0.18, 0.02)
        N, bdist, bseed = 4096, "normal", 0xB0000008
    elif name == "band_4096_bw64_N128":
        d = gen.band(4096, 64)
        b = smat_amd.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
        A = {"M": b.M, "K": b.K, "b_row_ptr": b.row_ptr, "b_col_idx": b.col_idx, "b_val": b.val, "nnzb": b.nnzb}
        N, bdist, bseed = 128, "uniform", 0xB0000001
    elif name in ("stencil27_64_N64", "stencil27_64_reordered_N64"):
        d = gen.stencil27(64)
        b = smat_amd.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
        if "reordered" in name:
            t0 = time.perf_counter()
            pr, pc, sr, sc = smat_amd.reorder_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], 16, 16, 0.5, True)
            INFO["reorder_s"] = round(time.perf_counter() - t0, 3)
            INFO["reorder_counters"] = [np.asarray(sr).tolist(), np.asarray(sc).tolist()]
            INFO["nnzb_before_reorder"] = int(b.nnzb)
            INFO["perm_sha256"] = sha256_of(np.asarray(pr, np.int64), np.asarray(pc, np.int64))
            rp, ci, v = smat_amd.permute_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], pr, pc)
            b = smat_amd.csr_to_bcsr(d["M"], d["K"], rp, ci, v)
        A = {"M": b.M, "K": b.K, "b_row_ptr": b.row_ptr, "b_col_idx": b.col_idx, "b_val": b.val, "nnzb": b.nnzb}
        N, bdist, bseed = 64, "uniform", 0xB0000005
    elif name in ("er_16384_0.1pct_N256", "er_16384_0.1pct_reordered_N256"):
        d = gen.erdos_renyi(16384, 0.001)
        b = smat_amd.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
        if "reordered" in name:
            # row pass, then column pass on the transpose (-a 5 -b 16 -B 16 -F 1 -t 0.5), timed apart
            t0 = time.perf_counter()
            pr, pc, sr, sc = smat_amd.reorder_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], 16, 16, 0.5, True)
            INFO["reorder_s"] = round(time.perf_counter() - t0, 3)
            INFO["reorder_counters"] = [np.asarray(sr).tolist(), np.asarray(sc).tolist()]
            INFO["nnzb_before_reorder"] = int(b.nnzb)
            INFO["perm_sha256"] = sha256_of(np.asarray(pr, np.int64), np.asarray(pc, np.int64))
            rp, ci, v = smat_amd.permute_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], pr, pc)
            b = smat_amd.csr_to_bcsr(d["M"], d["K"], rp, ci, v)
        A = {"M": b.M, "K": b.K, "b_row_ptr": b.row_ptr, "b_col_idx": b.col_idx, "b_val": b.val, "nnzb": b.nnzb}
        N, bdist, bseed = 256, "normal", 0xB0000002
    elif re.fullmatch(r"rmat_s(\d+)_deg16(_reordered)?_N128", name):
        scale = int(re.fullmatch(r"rmat_s(\d+)_deg16(_reordered)?_N128", name).group(1))
        d = gen.rmat(scale, 16)
        if "reordered" not in name:
            b = smat_amd.csr_to_bcsr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"])
        else:
            if scale == 20:
                # the reorder of 2^20 rows takes ten minutes on eight host threads (an hour on one): its permutations
                # come from a file (npz with perm_rows, perm_cols, reorder_s) written by an earlier smat_amd.reorder_csr
                # run; the one in tests/golden/ unless --perm-file names another
                z = np.load(PERM_FILE or RMAT20_PERMS)
                pr, pc = z["perm_rows"], z["perm_cols"]
                INFO["reorder_s"] = float(z["reorder_s"])
                INFO["reorder_counters"] = [z["stats_rows"].tolist(), z["stats_cols"].tolist()] if "stats_rows" in z else None
            else:
                t0 = time.perf_counter()
                pr, pc, sr, sc = smat_amd.reorder_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], 16, 16, 0.5, True)
                INFO["reorder_s"] = round(time.perf_counter() - t0, 3)
                INFO["reorder_counters"] = [np.asarray(sr).tolist(), np.asarray(sc).tolist()]
            rows_of = np.repeat(np.arange(d["M"], dtype=np.int64), np.diff(d["row_ptr"]))
            INFO["nnzb_before_reorder"] = int(np.unique((rows_of >> 4) * (d["K"] >> 4) + (d["col_idx"] >> 4)).size)  # without the block values
            del rows_of
            INFO["perm_sha256"] = sha256_of(np.asarray(pr, np.int64), np.asarray(pc, np.int64))
            rp, ci, v = smat_amd.permute_csr(d["M"], d["K"], d["row_ptr"], d["col_idx"], d["val"], pr, pc)
            b = smat_amd.csr_to_bcsr(d["M"], d["K"], rp, ci, v)
        A = {"M": b.M, "K": b.K, "b_row_ptr": b.row_ptr, "b_col_idx": b.col_idx, "b_val": b.val, "nnzb": b.nnzb}
        N, bdist, bseed = 128, "uniform", 0xB0000003
    else:
        raise SystemExit(f"unknown workload {name}")
    B = gen.dense_b(A["K"], N, seed=bseed, dist=bdist) if want_b else None
    return A, B, N


def algorithmic_bytes(A, N, c_bytes=2):
    """Every operand touched once: blocks (512 B values + 4 B index), row pointer, B, C."""
    mb = A["M"] // 16
    return A["nnzb"] * 516 + (mb + 1) * 4 + 2 * A["K"] * N + c_bytes * A["M"] * N


def cpu_baseline(A, B, N, target_s=12.0):
    """Oracle blocked SpMM (fp32 accumulate) on the host cores over a leading slice of block rows."""
    from tests.oracle_lib import load_oracle
    oracle = load_oracle()
    threads = max(1, min(16, os.cpu_count() or 1, oracle.max_threads()))
    rp = A["b_row_ptr"]
    mb = A["M"] // 16

    def run(nrows):
        sub_rp = rp[:nrows + 1].astype(np.int32)
        nb = int(sub_rp[-1])
        t0 = time.perf_counter()
        oracle.spmm_bcsr(16 * nrows, N, A["K"], sub_rp, A["b_col_idx"][:nb], A["b_val"][:nb * 256], B,
                         threads=threads)
        return time.perf_counter() - t0, nb

    probe_rows = min(mb, 2 * threads)
    t_probe, nb_probe = run(probe_rows)
    # the widening of B to fp32 is a fixed cost of the oracle; the sample is sized on the loop nest
    rows = int(min(mb, max(probe_rows, probe_rows * target_s / max(t_probe, 1e-3))))
    t, nb = run(rows)
    gflops = 2.0 * nb * 256 * N / t / 1e9
    return {"value": round(gflops, 3), "unit": "GFLOP/s", "cores": threads, "kind": "port",
            "sample": f"first {rows} of {mb} block rows ({nb} blocks) of the same workload, {t:.2f} s, "
                      f"OpenMP over block rows, includes widening B to fp32"}


def cpu_baseline_reference(A, B, N, target_s=10.0):
    """The reference's own serial CSR::multiply (preprocess/src/general/csr.cpp:47-63), compiled from the
    reference tree into oracle/_ref/, on a leading principal submatrix of A (it indexes B with A's row
    count, so the sample has to be square) and the matching rows of B, all N columns."""
    import subprocess
    import tempfile
    from tests.oracle_lib import ref_binary
    from smat_amd import generators as gen
    exe = ref_binary("ref_csr_multiply")
    if exe is None:
        return None
    mb = min(A["M"], A["K"]) // 16
    K = A["K"]
    Bf = B.view(np.float16).reshape(N, K)  # column-major: row n of this view is column n of B

    def run(rb):
        rp, ci = A["b_row_ptr"], A["b_col_idx"]
        keep = np.concatenate([np.arange(rp[r], rp[r + 1])[ci[rp[r]:rp[r + 1]] < 16 * rb] for r in range(rb)]) \
            if rb else np.zeros(0, np.int64)
        sub_rp = np.zeros(rb + 1, np.int32)
        for r in range(rb):
            sub_rp[r + 1] = sub_rp[r] + int((ci[rp[r]:rp[r + 1]] < 16 * rb).sum())
        sub = {"M": 16 * rb, "b_row_ptr": sub_rp, "b_col_idx": ci[keep], "b_val": A["b_val"].reshape(-1, 256)[keep].ravel()}
        crp, cci, cv = gen.bcsr_to_csr(sub["M"], sub["b_row_ptr"], sub["b_col_idx"], sub["b_val"])
        nz = cv != 0
        vals = cv.view(np.float16).astype(np.float64)
        rows = np.repeat(np.arange(sub["M"]), np.diff(crp))
        with tempfile.TemporaryDirectory() as d:
            with open(os.path.join(d, "a.el"), "w") as f:
                f.write("".join(f"{r} {c} {v:.10g}\n" for r, c, v in zip(rows[nz], cci[nz], vals[nz])))
                f.write(f"{sub['M'] - 1} {sub['M'] - 1} 0\n")  # pins rows = cols = 16 * rb in the reference reader
            np.ascontiguousarray(Bf[:, :16 * rb]).astype(np.float32).tofile(os.path.join(d, "b.f32"))
            out = subprocess.run([exe, os.path.join(d, "a.el"), os.path.join(d, "b.f32"), str(N), "1"],
                                 check=True, capture_output=True, text=True).stdout.split()
        return float(out[3]), int(nz.sum())

    rb = min(mb, 32)
    t, nnz = run(rb)
    while t < target_s / 4 and rb < mb:  # nnz of a principal submatrix grows with rb squared
        rb = int(min(mb, max(rb + 1, rb * min(4.0, (target_s / max(t, 1e-3)) ** 0.5))))
        t, nnz = run(rb)
    return {"value": round(2.0 * nnz * N / t / 1e9, 3), "unit": "GFLOP/s", "cores": 1, "kind": "reference",
            "sample": f"leading {16 * rb} x {16 * rb} submatrix of A ({nnz} nonzeros) times the matching {16 * rb} x {N} "
                      f"rows of B, {t:.2f} s, reference CSR::multiply (serial, fp32), flops = 2*nnz*N"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="block_pruned_8192_10pct_N4096")
    ap.add_argument("--kernel", type=int, default=0, help="0 auto, 1 rowwise, 2 sweep, 3 rowwise reading B in place, 5 compact, 6 mixed (rowwise + compact by block row)")
    ap.add_argument("--no-plan", action="store_true")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-static-mix", action="store_true", help="skip the static-schedule micro-benchmark that the sweep kernel is compared with")
    ap.add_argument("--no-verify", action="store_true", help="skip the check of sampled block rows against the CPU oracle")
    ap.add_argument("--no-attach-values", action="store_true",
                    help="do not let the plan look at the block values (the compact kernel, id 5, needs them)")
    ap.add_argument("--b-row-major", action="store_true",
                    help="hand B over row-major (B[k*N + n], the SMAT_B_ROW_MAJOR option) instead of the reference's column-major layout")
    ap.add_argument("--perm-file", default=None, help="npz with perm_rows / perm_cols / reorder_s for the reordered R-MAT workload (default: tests/golden/rmat_s20_deg16_perms.npz)")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (a kernel of known HBM traffic, "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one MI355X: run with --gpus 1 (this build has no multi-GPU path)")

    import torch
    import smat_amd
    from smat_amd._lib import lib, check

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    global PERM_FILE
    PERM_FILE = args.perm_file
    A, B, N = build_workload(args.workload)
    M, K, nnzb = A["M"], A["K"], A["nnzb"]

    def dev_i16(a):
        return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).to(dev)

    vals, Bd = dev_i16(A["b_val"]), dev_i16(B)
    if args.b_row_major:
        Bd = Bd.view(N, K).t().contiguous()  # generators hand out the reference layout: N columns of K values
    rp = torch.from_numpy(A["b_row_ptr"].astype(np.int32)).to(dev)
    ci = torch.from_numpy(A["b_col_idx"].astype(np.int32)).to(dev)
    Cd = torch.zeros((M, N), dtype=torch.int16, device=dev)
    plan = None
    if not args.no_plan:
        plan = smat_amd.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=args.kernel)

    if plan is not None and not args.no_attach_values:
        plan.attach_values(vals, rp, ci)  # one-off look at the zero pattern of the blocks (not timed, like the plan)

    def step():
        smat_amd.spmm(vals, rp, ci, Bd, Cd, M, N, K, nnzb, plan=plan, kernel=args.kernel, b_row_major=args.b_row_major)

    if args.calibration_copy_mib:
        src = torch.ones(args.calibration_copy_mib << 19, dtype=torch.int16, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads and writes calibration_copy_mib MiB each
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # HIP events on the stream the kernels are launched on (the null stream)
    ev0, ev1 = C.c_void_p(), C.c_void_p()
    check(lib.smat_event_create(C.byref(ev0)))
    check(lib.smat_event_create(C.byref(ev1)))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    check(lib.smat_event_record(ev0, None))
    for _ in range(args.steps):
        step()
    check(lib.smat_event_record(ev1, None))
    check(lib.smat_event_synchronize(ev1))
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms = C.c_float()
    check(lib.smat_event_elapsed_ms(ev0, ev1, C.byref(ms)))
    kernel_ms = ms.value / args.steps
    lib.smat_event_destroy(ev0)
    lib.smat_event_destroy(ev1)

    # every launch on its own: event pairs around single launches (the gaps between launches are not in them)
    n_single = min(args.steps, 50)
    pairs = []
    for _ in range(n_single):
        e0, e1 = C.c_void_p(), C.c_void_p()
        check(lib.smat_event_create(C.byref(e0)))
        check(lib.smat_event_create(C.byref(e1)))
        check(lib.smat_event_record(e0, None))
        step()
        check(lib.smat_event_record(e1, None))
        pairs.append((e0, e1))
    torch.cuda.synchronize()
    singles = []
    for e0, e1 in pairs:
        check(lib.smat_event_elapsed_ms(e0, e1, C.byref(ms)))
        singles.append(ms.value)
        lib.smat_event_destroy(e0)
        lib.smat_event_destroy(e1)
    singles = np.array(singles)

    # the result of the last launch against the CPU oracle, before anything is reported
    check_result = None
    if not args.no_verify:
        check_result = verify_sample(A, B, N, Cd.cpu().numpy().view(np.uint16))

    peak = C.c_double()
    check(lib.smat_bench_mfma_peak(C.byref(peak)))

    flops = 2.0 * nnzb * 256 * N
    qbytes = algorithmic_bytes(A, N)
    value = flops / (wall_ms * 1e-3) / 1e9
    ach_tflops = flops / (kernel_ms * 1e-3) / 1e12
    ach_gbs = qbytes / (kernel_ms * 1e-3) / 1e9
    mfma_bound = (flops / (PEAK_FP16_TFLOPS * 1e12)) >= (qbytes / (PEAK_HBM_GBS * 1e9))
    if mfma_bound:
        roof = {"bound": "mfma", "achieved": round(ach_tflops, 2), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(ach_tflops / PEAK_FP16_TFLOPS, 4)}
    else:
        roof = {"bound": "hbm", "achieved": round(ach_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(ach_gbs / PEAK_HBM_GBS, 4)}
    kernel_id = (plan.info()["kernel"] if plan is not None else 1) if args.kernel == 0 else args.kernel
    if kernel_id == 4:
        kernel_id = 1
    prof = profiled(args.workload, kernel_id)
    roof["traffic"] = prof.get("traffic_bytes_per_launch")
    if prof:
        roof["profile_source"] = prof["source"]
        if "mfma_busy" in prof:
            roof["mfma_busy_rocprof"] = prof["mfma_busy"]
    roof["kernel_ms"] = round(kernel_ms, 5)
    if roof["traffic"]:
        # the rate of the bytes that the profiled launch moved beyond the L2 (part of them served by the memory-side
        # cache): below the algorithmic rate where a kernel does not read the zeros inside the blocks
        roof["traffic_gbs"] = round(roof["traffic"] / (kernel_ms * 1e-3) / 1e9, 1)
    roof["kernel_ms_single_launch"] = {"n": int(singles.size), "median": round(float(np.median(singles)), 5),
                                       "min": round(float(singles.min()), 5), "max": round(float(singles.max()), 5)}
    roof["measured_mfma_peak_tflops"] = round(peak.value, 1)
    if mfma_bound and peak.value > 0:
        roof["frac_of_measured_mfma_peak"] = round(ach_tflops / peak.value, 4)
    if kernel_id == 2 and not args.no_static_mix:
        # what the sweep kernel's data flow delivers on a static schedule (smat_bench_static_mix), on this device, now
        mix = {}
        for key, variant in (("lds_reads_and_mfma", 0), ("full_mix_a_in_l2", 1), ("full_mix", 2),
                             ("full_mix_a_in_l2_barrier_per_8_ops", 3), ("full_mix_barrier_per_8_ops", 4)):
            t = C.c_double()
            check(lib.smat_bench_static_mix(variant, C.byref(t)))
            mix[key] = round(t.value, 1)
        roof["static_mix_tflops"] = mix["full_mix"]
        roof["frac_of_static_mix"] = round(ach_tflops / mix["full_mix"], 4) if mix["full_mix"] > 0 else None
        roof["static_mix_variants_tflops"] = mix
    roof["algorithmic_flops"] = flops
    roof["algorithmic_bytes"] = qbytes
    roof["hbm_gbs_at_algorithmic_bytes"] = round(ach_gbs, 1)

    out = {
        "metric": "effective SpMM GFLOP/s + % of fp16 MFMA/HBM roofline, 1x MI355X",
        "value": round(value, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": args.workload, "M": M, "K": K, "N": N, "nnzb": nnzb, "block": 16,
                   "c_dtype": "f16", "b_layout": "row-major" if args.b_row_major else "column-major (reference)", "plan": None if plan is None else plan.info(),
                   "pattern_sha256": sha256_of(A["b_row_ptr"].astype(np.int32), A["b_col_idx"].astype(np.int32)), **INFO},
        "roofline": roof,
        "verified": check_result,
        "structure_vs_fixture": structure_against_golden(args.workload, A),
    }
    if not args.no_cpu_baseline:
        port = cpu_baseline(A, B, N)
        ref = cpu_baseline_reference(A, B, N)
        out["cpu_baseline"] = ref if ref is not None else port
        if ref is not None:
            out["cpu_baseline_all_cores"] = port
    print(json.dumps(out))
    if out["structure_vs_fixture"] is not None and not out["structure_vs_fixture"]["ok"]:
        raise SystemExit(f"bench.py: the blocked structure differs from the recorded one: {out['structure_vs_fixture']}")
    if check_result is not None and not check_result["ok"]:
        raise SystemExit(f"bench.py: the result of the last launch differs from the CPU oracle: {check_result}")


if __name__ == "__main__":
    main()
