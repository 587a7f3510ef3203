"""Host-side mirror of the reference's matrix-load -> reorder/block -> SpMM flow.

Thin wrappers over the C ABI: numpy arrays for host data, torch CUDA tensors
(only as device memory) for the SpMM operands.
"""
import ctypes as C
from dataclasses import dataclass

import numpy as np

from ._lib import SpmmOpts, check, lib

BS = 16
KERNEL_AUTO, KERNEL_ROWWISE, KERNEL_SWEEP, KERNEL_ROWWISE_DIRECT, KERNEL_ROWWISE_PACKED, KERNEL_COMPACT = 0, 1, 2, 3, 4, 5
KERNEL_MIXED = 6
C_F16, C_F32 = 0, 1


def _take(ptr, n, dtype):
    """Copy n elements out of a library-owned buffer, then free it."""
    if n:
        arr = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), shape=(n,)).copy()
    else:
        arr = np.zeros(0, dtype=dtype)
    lib.smat_host_free(ptr)
    return arr


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def mtx_read(path):
    """Matrix Market -> CSR (loader semantics of mmio_allinone). Returns dict."""
    M, K, nnz, sym, ref = C.c_size_t(), C.c_size_t(), C.c_size_t(), C.c_int(), C.c_int()
    rp, ci, v = C.c_void_p(), C.c_void_p(), C.c_void_p()
    check(lib.smat_mtx_read(str(path).encode(), C.byref(M), C.byref(K), C.byref(nnz), C.byref(sym),
                            C.byref(rp), C.byref(ci), C.byref(v), C.byref(ref)))
    return {
        "M": M.value, "K": K.value, "nnz": nnz.value, "symmetric": bool(sym.value),
        "row_ptr": _take(rp, M.value + 1, np.int32),
        "col_idx": _take(ci, nnz.value, np.int32),
        "val": _take(v, nnz.value, np.uint16),
    }


def bin_write_csr(path, M, K, row_ptr, col_idx, val, perm_rows=None, perm_cols=None):
    """CSR (+ optional permutations) -> SMATBIN1 container."""
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    col_idx = np.ascontiguousarray(col_idx, dtype=np.int32)
    val = np.ascontiguousarray(val, dtype=np.uint16)
    pr = None if perm_rows is None else np.ascontiguousarray(perm_rows, dtype=np.int64)
    pc = None if perm_cols is None else np.ascontiguousarray(perm_cols, dtype=np.int64)
    check(lib.smat_bin_write_csr(str(path).encode(), M, K, _p(row_ptr), _p(col_idx), _p(val), _p(pr), _p(pc)))


def bin_write_bcsr(path, M, K, b_row_ptr, b_col_idx, b_val, perm_rows=None, perm_cols=None):
    """16x16 BCSR (+ optional permutations) -> SMATBIN1 container."""
    b_row_ptr = np.ascontiguousarray(b_row_ptr, dtype=np.int32)
    b_col_idx = np.ascontiguousarray(b_col_idx, dtype=np.int32)
    b_val = np.ascontiguousarray(b_val, dtype=np.uint16)
    pr = None if perm_rows is None else np.ascontiguousarray(perm_rows, dtype=np.int64)
    pc = None if perm_cols is None else np.ascontiguousarray(perm_cols, dtype=np.int64)
    check(lib.smat_bin_write_bcsr(str(path).encode(), M, K, len(b_col_idx), _p(b_row_ptr), _p(b_col_idx), _p(b_val),
                                  _p(pr), _p(pc)))


def bin_read(path):
    """SMATBIN1 container -> dict(kind, M, K, n, row_ptr, col_idx, val, perm_rows, perm_cols)."""
    kind, M, K, n = C.c_int(), C.c_size_t(), C.c_size_t(), C.c_size_t()
    rp, ci, v, pr, pc = C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p(), C.c_void_p()
    check(lib.smat_bin_read(str(path).encode(), C.byref(kind), C.byref(M), C.byref(K), C.byref(n), C.byref(rp),
                            C.byref(ci), C.byref(v), C.byref(pr), C.byref(pc)))
    rows = M.value if kind.value == 1 else M.value // BS
    per = 1 if kind.value == 1 else 256
    return {
        "kind": kind.value, "M": M.value, "K": K.value, "n": n.value,
        "row_ptr": _take(rp, rows + 1, np.int32), "col_idx": _take(ci, n.value, np.int32),
        "val": _take(v, n.value * per, np.uint16),
        "perm_rows": _take(pr, M.value, np.int64) if pr.value else None,
        "perm_cols": _take(pc, K.value, np.int64) if pc.value else None,
    }


def mtx_write(path, M, K, row_ptr, col_idx, val):
    """CSR -> Matrix Market coordinate real general, entries in storage order."""
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    col_idx = np.ascontiguousarray(col_idx, dtype=np.int32)
    val = np.ascontiguousarray(val, dtype=np.uint16)
    check(lib.smat_mtx_write(str(path).encode(), M, K, _p(row_ptr), _p(col_idx), _p(val)))


@dataclass
class Bcsr:
    M: int
    K: int
    row_ptr: np.ndarray  # int32 [M/16+1]
    col_idx: np.ndarray  # int32 [nnzb], absolute first column of each block
    val: np.ndarray      # uint16 (fp16 bits) [nnzb*256]
    counts: tuple        # (nonzero, "dense", "sparse") blocks
    block_info: np.ndarray = None
    rel_map: np.ndarray = None

    @property
    def nnzb(self):
        return int(self.col_idx.shape[0])


def csr_to_bcsr(M, K, row_ptr, col_idx, val, want_maps=False):
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    col_idx = np.ascontiguousarray(col_idx, dtype=np.int32)
    val = np.ascontiguousarray(val, dtype=np.uint16)
    counts = (C.c_int64 * 3)()
    brp, bci, bv = C.c_void_p(), C.c_void_p(), C.c_void_p()
    info, rel = C.c_void_p(), C.c_void_p()
    check(lib.smat_csr_to_bcsr(M, K, _p(row_ptr), _p(col_idx), _p(val), counts, C.byref(brp), C.byref(bci),
                               C.byref(bv), C.byref(info) if want_maps else None,
                               C.byref(rel) if want_maps else None))
    nnzb = counts[0]
    out = Bcsr(M, K, _take(brp, M // BS + 1, np.int32), _take(bci, nnzb, np.int32),
               _take(bv, nnzb * 256, np.uint16), tuple(counts))
    if want_maps:
        cells = (M // BS) * (K // BS)
        out.block_info = _take(info, cells, np.int32)
        out.rel_map = _take(rel, cells, np.int32)
    return out


class DeviceBcsr:
    """BCSR arrays in device memory, as returned by smat_csr_to_bcsr_device (freed on close)."""

    def __init__(self, M, K, row_ptr, col_idx, val, counts):
        self.M, self.K, self.counts = M, K, counts
        self.row_ptr, self.col_idx, self.val = row_ptr, col_idx, val  # device addresses (ints)

    @property
    def nnzb(self):
        return int(self.counts[0])

    def to_host(self):
        rp = np.empty(self.M // BS + 1, np.int32)
        ci = np.empty(self.nnzb, np.int32)
        v = np.empty(self.nnzb * 256, np.uint16)
        check(lib.smat_memcpy_d2h(_p(rp), self.row_ptr, rp.nbytes))
        if self.nnzb:
            check(lib.smat_memcpy_d2h(_p(ci), self.col_idx, ci.nbytes))
            check(lib.smat_memcpy_d2h(_p(v), self.val, v.nbytes))
        return Bcsr(self.M, self.K, rp, ci, v, tuple(self.counts))

    def close(self):
        for a in ("row_ptr", "col_idx", "val"):
            if getattr(self, a):
                lib.smat_free(getattr(self, a))
                setattr(self, a, None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def csr_to_bcsr_device(M, K, row_ptr_dev, col_idx_dev, val_dev, nnz):
    """CSR -> BCSR on the GPU; the three inputs are device tensors (anything with .data_ptr())."""
    counts = (C.c_int64 * 3)()
    brp, bci, bv = C.c_void_p(), C.c_void_p(), C.c_void_p()
    ptr = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None  # noqa: E731
    check(lib.smat_csr_to_bcsr_device(M, K, ptr(row_ptr_dev), ptr(col_idx_dev), ptr(val_dev), nnz, counts,
                                      C.byref(brp), C.byref(bci), C.byref(bv)))
    return DeviceBcsr(M, K, brp.value, bci.value, bv.value, tuple(counts))


def reorder_rows(rows, cols, row_ptr, col_idx, col_block=16, row_block=16, tau=0.5):
    """One pass of the row clustering. Returns (grouping, perm, stats)."""
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int64)
    col_idx = np.ascontiguousarray(col_idx, dtype=np.int64)
    grouping = np.empty(rows, dtype=np.int64)
    perm = np.empty(rows, dtype=np.int64)
    stats = np.zeros(4, dtype=np.int64)
    check(lib.smat_reorder_rows(rows, cols, _p(row_ptr), _p(col_idx), col_block, row_block, tau,
                                _p(grouping), _p(perm), _p(stats)))
    return grouping, perm, stats


def reorder_csr(M, K, row_ptr, col_idx, col_block=16, row_block=16, tau=0.5, do_cols=True):
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    col_idx = np.ascontiguousarray(col_idx, dtype=np.int32)
    pr = np.empty(M, dtype=np.int64)
    pc = np.empty(K, dtype=np.int64)
    sr = np.zeros(4, dtype=np.int64)
    sc = np.zeros(4, dtype=np.int64)
    check(lib.smat_reorder_csr(M, K, _p(row_ptr), _p(col_idx), col_block, row_block, tau, int(do_cols),
                               _p(pr), _p(pc), _p(sr), _p(sc)))
    return pr, pc, sr, sc


def permute_csr(M, K, row_ptr, col_idx, val, perm_rows=None, perm_cols=None):
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    col_idx = np.ascontiguousarray(col_idx, dtype=np.int32)
    val = np.ascontiguousarray(val, dtype=np.uint16)
    pr = None if perm_rows is None else np.ascontiguousarray(perm_rows, dtype=np.int64)
    pc = None if perm_cols is None else np.ascontiguousarray(perm_cols, dtype=np.int64)
    orp, oci, ov = C.c_void_p(), C.c_void_p(), C.c_void_p()
    check(lib.smat_permute_csr(M, K, _p(row_ptr), _p(col_idx), _p(val), _p(pr), _p(pc),
                               C.byref(orp), C.byref(oci), C.byref(ov)))
    nnz = int(row_ptr[M])
    return _take(orp, M + 1, np.int32), _take(oci, nnz, np.int32), _take(ov, nnz, np.uint16)


class Plan:
    """Per-matrix work list (built once, outside any timed loop)."""

    def __init__(self, row_ptr_host, M, K, nnzb, n_hint, col_idx_host=None, kernel=KERNEL_AUTO, b_row_major=False):
        self._h = C.c_void_p()
        rp = np.ascontiguousarray(row_ptr_host, dtype=np.int32)
        ci = None if col_idx_host is None else np.ascontiguousarray(col_idx_host, dtype=np.int32)
        opts = SpmmOpts(1 if b_row_major else 0, 0, kernel, 0, None)
        check(lib.smat_plan_create(C.byref(self._h), _p(rp), _p(ci), M, K, nnzb, n_hint, C.byref(opts)))
        self._rp_host = rp

    def check(self, row_ptr_host, col_idx_host, M, K, nnzb):
        """Raises SmatError unless the plan was made from this block pattern (fingerprint of the host arrays)."""
        rp = np.ascontiguousarray(row_ptr_host, dtype=np.int32)
        ci = None if col_idx_host is None else np.ascontiguousarray(col_idx_host, dtype=np.int32)
        check(lib.smat_plan_check(self._h, _p(rp), _p(ci), M, K, nnzb))

    def values_current(self, vals_dev):
        """False when the block values have changed since attach_values (the compact kernel works from a copy)."""
        cur = C.c_int()
        check(lib.smat_plan_values_current(self._h, C.c_void_p(vals_dev.data_ptr()), C.byref(cur)))
        return bool(cur.value)

    def attach_values(self, vals_dev, row_ptr_dev, col_idx_dev):
        """Let the plan list the nonzero columns of the blocks (device tensors of the same matrix)."""
        ptr = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None  # noqa: E731
        check(lib.smat_plan_attach_values(self._h, ptr(vals_dev), ptr(row_ptr_dev), ptr(col_idx_dev), _p(self._rp_host)))

    @property
    def handle(self):
        return self._h

    def info(self):
        out = (C.c_int64 * 12)()
        check(lib.smat_plan_info(self._h, out))
        keys = ("kernel", "items", "split_rows", "chunk", "workspace_bytes", "panel", "sweep_ops", "sweep_records",
                "b_pack_bytes", "compact_cols", "mixed_dense_items", "mixed_dense_blocks")
        return dict(zip(keys, out))

    def close(self):
        if self._h:
            lib.smat_plan_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def spmm(vals, row_ptr, col_idx, B, C_out, M, N, K, nnzb, plan=None, c_f32=False, kernel=KERNEL_AUTO,
         stream=None, drop_in=False, b_row_major=False):
    """Launch the SpMM on device tensors (anything with .data_ptr()).

    drop_in=True calls the positional drop-in entry point (smat_spmm_bcsr_f16) with
    NULL block_info / rel_map; otherwise the options entry point."""
    ptr = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None  # noqa: E731
    if drop_in:
        check(lib.smat_spmm_bcsr_f16(ptr(vals), ptr(row_ptr), ptr(col_idx), ptr(B), ptr(C_out), M, N, K, nnzb,
                                     None, None))
        return
    opts = SpmmOpts(1 if b_row_major else 0, C_F32 if c_f32 else C_F16, kernel, 0,
                    C.c_void_p(stream) if stream else None)
    check(lib.smat_spmm_bcsr_f16_ex(ptr(vals), ptr(row_ptr), ptr(col_idx), ptr(B), ptr(C_out), M, N, K, nnzb,
                                    C.byref(opts), plan.handle if plan is not None else None))
