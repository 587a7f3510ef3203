"""The entry point that allocates nothing (smat_spmm_bcsr_f16_static) against the existing entry point that
runs the same kernels on plan-owned scratch (smat_spmm_bcsr_f16_ex with a SMAT_KERNEL_ROWWISE_PACKED plan):
bit-identical fp16 output, on two calls in a row, the second with a smaller input (the array keeps the first
call's contents)."""
import ctypes as C

import numpy as np
import pytest

from smat_amd import generators as gen

pytestmark = pytest.mark.gpu
ROWWISE_PACKED = 4


def to_dev(torch, a, cuda):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16) if a.dtype == np.uint16 else np.ascontiguousarray(a)).to(cuda)


def alloc_counts():
    from smat_amd._lib import lib
    out = (C.c_int64 * 2)()
    lib.smat_internal_alloc_counts(out)
    return out[0], out[1]


def run_both(smat, cuda, A, B_bits, N):
    import torch
    from smat_amd._lib import lib, check
    M, K, nnzb = A["M"], A["K"], A["nnzb"]
    vals, Bd = to_dev(torch, A["b_val"], cuda), to_dev(torch, B_bits, cuda)
    rp, ci = to_dev(torch, A["b_row_ptr"].astype(np.int32), cuda), to_dev(torch, A["b_col_idx"].astype(np.int32), cuda)
    # existing entry point: plan-owned copy of B
    counts_before_plan = alloc_counts()
    C_ref = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    plan = smat.Plan(A["b_row_ptr"], M, K, nnzb, N, col_idx_host=A["b_col_idx"], kernel=ROWWISE_PACKED)
    assert plan.info()["split_rows"] == 0 and plan.info()["b_pack_bytes"] == K * N * 2
    smat.spmm(vals, rp, ci, Bd, C_ref, M, N, K, nnzb, plan=plan, kernel=ROWWISE_PACKED)
    torch.cuda.synchronize()
    plan.close()
    # the entry point under test: no plan, no allocation.  Witnesses: the library's own count of its device
    # allocations and releases (every one of them goes through the counted wrappers of devmem.h), and the free
    # device memory the driver reports (which a hipMalloc inside the library would lower, whoever made it).
    C_new = torch.full((M, N), 0x7E00, dtype=torch.int16, device=cuda)
    torch.cuda.synchronize()
    after_plan = alloc_counts()
    assert after_plan[0] > counts_before_plan[0], "the counters do not see the plan's allocations"
    # the first call on a device loads the kernels' code and looks up the fixed array (both the runtime's doing,
    # once per process): the free memory is read after it
    check(lib.smat_spmm_bcsr_f16_static(vals.data_ptr(), rp.data_ptr(), ci.data_ptr(), Bd.data_ptr(), C_new.data_ptr(),
                                        M, N, K, nnzb, None))
    torch.cuda.synchronize()
    assert alloc_counts() == after_plan, "smat_spmm_bcsr_f16_static allocated or released device memory"
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        check(lib.smat_spmm_bcsr_f16_static(vals.data_ptr(), rp.data_ptr(), ci.data_ptr(), Bd.data_ptr(), C_new.data_ptr(),
                                            M, N, K, nnzb, None))
    torch.cuda.synchronize()
    assert alloc_counts() == after_plan, "smat_spmm_bcsr_f16_static allocated or released device memory"
    assert torch.cuda.mem_get_info()[0] >= free_before
    return C_ref.cpu().numpy().view(np.uint16), C_new.cpu().numpy().view(np.uint16)


def test_static_entry_point_matches_the_plan_owned_scratch_twice(smat, cuda, oracle):
    # first call: 96 x 80 blocks, N = 264 (partial panel); second call: smaller in every dimension
    for mb, kb, density, N, seed in ((96, 80, 0.2, 264, 5), (40, 33, 0.3, 72, 6)):
        A = gen.random_bcsr(mb, kb, density, seed=seed)
        B = gen.dense_b(A["K"], N, seed=seed + 50, dist="normal")
        ref, new = run_both(smat, cuda, A, B, N)
        assert np.array_equal(ref, new)
        want = oracle.spmm_bcsr(A["M"], N, A["K"], A["b_row_ptr"], A["b_col_idx"], A["b_val"], B, threads=8)
        assert oracle.compare(new, want)[0] <= 1e-3  # relative to the row L2 norm


def test_static_entry_point_rejects_a_b_beyond_its_scratch(smat, cuda):
    import torch
    from smat_amd._lib import lib
    dummy = torch.zeros(4096, dtype=torch.int16, device=cuda)
    M, K, N = 16, 8192, 4104  # K * N * 2 bytes just above 64 MiB
    rc = lib.smat_spmm_bcsr_f16_static(dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(),
                                       M, N, K, 1, None)
    assert rc == -5 and b"exceeds the fixed scratch" in lib.smat_last_error()
