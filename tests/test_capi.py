"""The C ABI: every function declared in include/smat.h is exported and bound; argument checks that
need no GPU return the documented status."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "smat.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(smat_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_drop_in_entry_point():
    names = declared_functions()
    assert "smat_spmm_bcsr_f16" in names and "smat_spmm_bcsr_f16_ex" in names and len(names) >= 30


def test_every_declared_symbol_is_exported_and_bound(smat):
    from smat_amd._lib import SIGNATURES, library_path
    handle = C.CDLL(library_path())
    for name in declared_functions():
        assert hasattr(handle, name), f"{name} declared in smat.h but not exported"
        assert name in SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(SIGNATURES) == declared_functions()


def test_library_is_in_tree_and_has_device_code(smat):
    from smat_amd._lib import library_path
    path = library_path()
    assert path.startswith(ROOT)
    blob = open(path, "rb").read()
    assert b"gfx950" in blob and b"spmm_sweep_kernel" in blob and b"spmm_rowwise_kernel" in blob


def test_shape_checks_fail_before_any_device_work(smat):
    from smat_amd._lib import lib
    buf = np.zeros(64, dtype=np.uint16)
    p = buf.ctypes.data_as(C.c_void_p)
    assert lib.smat_spmm_bcsr_f16(p, p, p, p, p, 16, 12, 16, 1, None, None) == -1  # N % 8
    assert b"multiple of 8" in lib.smat_last_error()
    assert lib.smat_spmm_bcsr_f16(p, p, p, p, p, 17, 8, 16, 1, None, None) == -1   # M % 16
    assert lib.smat_spmm_bcsr_f16(p, None, p, p, p, 16, 8, 16, 1, None, None) == -1  # NULL row_ptr
    assert lib.smat_spmm_bcsr_f16(None, p, None, p, p, 16, 8, 16, 1, None, None) == -1  # nnzb > 0 without vals
    assert smat.lib.smat_version().startswith(b"smat-amd")


def test_plan_argument_checks(smat):
    rp = np.array([0, 1, 3], dtype=np.int32)
    with pytest.raises(smat.SmatError):  # nnzb does not match row_ptr
        smat.Plan(rp, 32, 32, 5, 64)
    with pytest.raises(smat.SmatError):  # n_hint not a multiple of 8
        smat.Plan(rp, 32, 32, 3, 12)
    with pytest.raises(smat.SmatError):  # col_idx not a block column
        smat.Plan(rp, 32, 32, 3, 64, col_idx_host=np.array([0, 8, 16], np.int32))


def test_sweep_plan_refuses_columns_that_do_not_ascend(smat):
    """The sweep kernel pairs neighbouring blocks of a block row by the K chunk they sit in: columns that are not
    strictly ascending inside a block row are refused when such a plan is asked for (before any device work)."""
    from smat_amd import generators as gen
    A = gen.random_bcsr(64, 160, 0.1, seed=3)
    rp, ci = A["b_row_ptr"], A["b_col_idx"].copy()
    for i in range(64):  # the columns of every block row in descending order
        ci[rp[i]:rp[i + 1]] = ci[rp[i]:rp[i + 1]][::-1]
    for kernel in (smat.KERNEL_SWEEP, smat.KERNEL_MIXED):
        with pytest.raises(smat.SmatError) as err:
            smat.Plan(rp, A["M"], A["K"], A["nnzb"], 4096, col_idx_host=ci, kernel=kernel)
        assert err.value.code == -1 and "ascending" in str(err.value)
    dup = A["b_col_idx"].copy()
    dup[rp[5] + 1] = dup[rp[5]]  # a repeated column is no better
    with pytest.raises(smat.SmatError):
        smat.Plan(rp, A["M"], A["K"], A["nnzb"], 4096, col_idx_host=dup, kernel=smat.KERNEL_SWEEP)
