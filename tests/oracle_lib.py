"""ctypes access to oracle/liboracle.so -- the CPU checker. Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "liboracle.so")
REF_DIR = os.path.join(ORACLE_DIR, "_ref")

_vp, _i64, _int = C.c_void_p, C.c_int64, C.c_int
_pp = C.POINTER(C.c_void_p)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


class Oracle:
    def __init__(self, handle):
        self.h = handle
        h = handle
        h.orc_f64_to_f16.restype = C.c_uint16
        h.orc_f64_to_f16.argtypes = [C.c_double]
        h.orc_f16_to_f32.restype = C.c_float
        h.orc_f16_to_f32.argtypes = [C.c_uint16]
        h.orc_f16_to_f32_array.argtypes = [_vp, _vp, _i64]
        h.orc_f64_to_f16_array.argtypes = [_vp, _vp, _i64]
        h.orc_mtx_read.restype = _int
        h.orc_mtx_read.argtypes = [C.c_char_p, C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_int),
                                   _pp, _pp, _pp]
        h.orc_free.argtypes = [_vp]
        h.orc_csr_to_bcsr.restype = _int
        h.orc_csr_to_bcsr.argtypes = [_i64, _i64, _vp, _vp, _vp, C.POINTER(_i64), _pp, _pp, _pp, _pp, _pp]
        h.orc_spmm_csr_f32.argtypes = [_i64, _i64, _i64, _vp, _vp, _vp, _vp, _int, _vp]
        h.orc_spmm_bcsr_f32.argtypes = [_i64, _i64, _i64, _vp, _vp, _vp, _vp, _int, _vp, _int]
        h.orc_compare_f16_vs_f32.argtypes = [_vp, _vp, _i64, _i64, _vp]
        h.orc_max_threads.restype = _int

    def _take(self, ptr, n, dtype):
        if n:
            a = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), shape=(n,)).copy()
        else:
            a = np.zeros(0, dtype=dtype)
        self.h.orc_free(ptr)
        return a

    def f64_to_f16(self, x):
        x = np.ascontiguousarray(x, dtype=np.float64)
        out = np.empty(x.shape, dtype=np.uint16)
        self.h.orc_f64_to_f16_array(_p(x), _p(out), x.size)
        return out

    def f16_to_f32(self, h):
        h = np.ascontiguousarray(h, dtype=np.uint16)
        out = np.empty(h.shape, dtype=np.float32)
        self.h.orc_f16_to_f32_array(_p(h), _p(out), h.size)
        return out

    def mtx_read(self, path):
        m, n, nnz, sym = _i64(), _i64(), _i64(), _int()
        rp, ci, v = C.c_void_p(), C.c_void_p(), C.c_void_p()
        rc = self.h.orc_mtx_read(str(path).encode(), C.byref(m), C.byref(n), C.byref(nnz), C.byref(sym),
                                 C.byref(rp), C.byref(ci), C.byref(v))
        if rc != 0:
            return {"rc": rc}
        return {"rc": 0, "M": m.value, "K": n.value, "nnz": nnz.value, "symmetric": bool(sym.value),
                "row_ptr": self._take(rp, m.value + 1, np.int32), "col_idx": self._take(ci, nnz.value, np.int32),
                "val": self._take(v, nnz.value, np.uint16)}

    def csr_to_bcsr(self, M, K, row_ptr, col_idx, val):
        row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
        col_idx = np.ascontiguousarray(col_idx, dtype=np.int32)
        val = np.ascontiguousarray(val, dtype=np.uint16)
        counts = (_i64 * 3)()
        brp, bci, bv, info, rel = (C.c_void_p() for _ in range(5))
        rc = self.h.orc_csr_to_bcsr(M, K, _p(row_ptr), _p(col_idx), _p(val), counts, C.byref(brp), C.byref(bci),
                                    C.byref(bv), C.byref(info), C.byref(rel))
        assert rc == 0
        nnzb = counts[0]
        cells = (M // 16) * (K // 16)
        return {"counts": tuple(counts), "row_ptr": self._take(brp, M // 16 + 1, np.int32),
                "col_idx": self._take(bci, nnzb, np.int32), "val": self._take(bv, nnzb * 256, np.uint16),
                "block_info": self._take(info, cells, np.int32), "rel_map": self._take(rel, cells, np.int32)}

    def spmm_csr(self, M, N, K, row_ptr, col_idx, val, B, b_row_major=False):
        row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
        col_idx = np.ascontiguousarray(col_idx, dtype=np.int32)
        val = np.ascontiguousarray(val, dtype=np.uint16)
        B = np.ascontiguousarray(B, dtype=np.uint16)
        out = np.empty((M, N), dtype=np.float32)
        self.h.orc_spmm_csr_f32(M, N, K, _p(row_ptr), _p(col_idx), _p(val), _p(B), int(b_row_major), _p(out))
        return out

    def spmm_bcsr(self, M, N, K, b_row_ptr, b_col_idx, b_val, B, b_row_major=False, threads=1):
        b_row_ptr = np.ascontiguousarray(b_row_ptr, dtype=np.int32)
        b_col_idx = np.ascontiguousarray(b_col_idx, dtype=np.int32)
        b_val = np.ascontiguousarray(b_val, dtype=np.uint16)
        B = np.ascontiguousarray(B, dtype=np.uint16)
        out = np.empty((M, N), dtype=np.float32)
        self.h.orc_spmm_bcsr_f32(M, N, K, _p(b_row_ptr), _p(b_col_idx), _p(b_val), _p(B), int(b_row_major),
                                 _p(out), int(threads))
        return out

    def compare(self, c_f16_bits, ref_f32):
        """(max |d| / row L2 norm, max abs, mean abs) of an fp16 result against the fp32 reference."""
        c = np.ascontiguousarray(c_f16_bits, dtype=np.uint16)
        r = np.ascontiguousarray(ref_f32, dtype=np.float32)
        out = np.zeros(3, dtype=np.float64)
        self.h.orc_compare_f16_vs_f32(_p(c), _p(r), r.shape[0], r.shape[1], _p(out))
        return tuple(out)

    def max_threads(self):
        return self.h.orc_max_threads()


def load_oracle():
    if not os.path.exists(ORACLE_SO):  # built by __graft_entry__.build(); build here only if nothing is there
        subprocess.run(["make", "-C", ORACLE_DIR], check=True, stdout=subprocess.DEVNULL)
    return Oracle(C.CDLL(ORACLE_SO))


def ref_binary(name):
    """Path of a reference program compiled into oracle/_ref/, or None."""
    path = os.path.join(REF_DIR, name)
    return path if os.path.exists(path) else None
