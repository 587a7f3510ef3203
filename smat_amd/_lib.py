"""ctypes binding of libsmat_amd.so (every symbol declared in include/smat.h)."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))


def library_path():
    """The in-tree library."""
    return os.path.join(_HERE, "libsmat_amd.so")


class SmatError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"smat error {code}: {message}")
        self.code = code


class SpmmOpts(C.Structure):
    _fields_ = [
        ("b_layout", C.c_int32),
        ("c_dtype", C.c_int32),
        ("kernel", C.c_int32),
        ("reserved", C.c_int32),
        ("stream", C.c_void_p),
    ]


_vp, _sz, _i64, _int = C.c_void_p, C.c_size_t, C.c_int64, C.c_int
_pp = C.POINTER(C.c_void_p)
_pi64 = C.POINTER(C.c_int64)

# name -> (restype, argtypes); the test-suite checks this table against smat.h
SIGNATURES = {
    "smat_last_error": (C.c_char_p, []),
    "smat_version": (C.c_char_p, []),
    "smat_spmm_bcsr_f16": (_int, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp, _vp]),
    "smat_plan_cache_clear": (_int, []),
    "smat_spmm_bcsr_f16_ex": (_int, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, C.POINTER(SpmmOpts), _vp]),
    "smat_spmm_bcsr_f16_static": (_int, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp]),
    "smat_plan_values_current": (_int, [_vp, _vp, C.POINTER(C.c_int)]),
    "smat_plan_check": (_int, [_vp, _vp, _vp, _sz, _sz, _sz]),
    "smat_plan_create": (_int, [_pp, _vp, _vp, _sz, _sz, _sz, _sz, C.POINTER(SpmmOpts)]),
    "smat_plan_attach_values": (_int, [_vp, _vp, _vp, _vp, _vp]),
    "smat_plan_destroy": (_int, [_vp]),
    "smat_plan_info": (_int, [_vp, _pi64]),
    "smat_mtx_read": (_int, [C.c_char_p, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_int),
                              _pp, _pp, _pp, C.POINTER(_int)]),
    "smat_host_free": (None, [_vp]),
    "smat_bin_write_csr": (_int, [C.c_char_p, _sz, _sz, _vp, _vp, _vp, _vp, _vp]),
    "smat_bin_write_bcsr": (_int, [C.c_char_p, _sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp]),
    "smat_bin_read": (_int, [C.c_char_p, C.POINTER(_int), C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz),
                              _pp, _pp, _pp, _pp, _pp]),
    "smat_mtx_write": (_int, [C.c_char_p, _sz, _sz, _vp, _vp, _vp]),
    "smat_csr_to_bcsr": (_int, [_sz, _sz, _vp, _vp, _vp, _pi64, _pp, _pp, _pp, _pp, _pp]),
    "smat_csr_to_bcsr_device": (_int, [_sz, _sz, _vp, _vp, _vp, _sz, _pi64, _pp, _pp, _pp]),
    "smat_reorder_rows": (_int, [_i64, _i64, _vp, _vp, _i64, _i64, C.c_float, _vp, _vp, _vp]),
    "smat_reorder_csr": (_int, [_sz, _sz, _vp, _vp, _i64, _i64, C.c_float, _int, _vp, _vp, _vp, _vp]),
    "smat_permute_csr": (_int, [_sz, _sz, _vp, _vp, _vp, _vp, _vp, _pp, _pp, _pp]),
    "smat_device_count": (_int, [C.POINTER(_int)]),
    "smat_set_device": (_int, [_int]),
    "smat_device_name": (_int, [_int, C.c_char_p, _sz]),
    "smat_device_attr": (_int, [_int, _pi64, _pi64, _pi64, _pi64]),
    "smat_malloc": (_int, [_pp, _sz]),
    "smat_free": (_int, [_vp]),
    "smat_memcpy_h2d": (_int, [_vp, _vp, _sz]),
    "smat_memcpy_d2h": (_int, [_vp, _vp, _sz]),
    "smat_memcpy_d2d": (_int, [_vp, _vp, _sz]),
    "smat_memset": (_int, [_vp, _int, _sz]),
    "smat_device_synchronize": (_int, []),
    "smat_stream_create": (_int, [_pp]),
    "smat_stream_destroy": (_int, [_vp]),
    "smat_stream_synchronize": (_int, [_vp]),
    "smat_event_create": (_int, [_pp]),
    "smat_event_destroy": (_int, [_vp]),
    "smat_event_record": (_int, [_vp, _vp]),
    "smat_event_synchronize": (_int, [_vp]),
    "smat_event_elapsed_ms": (_int, [_vp, _vp, C.POINTER(C.c_float)]),
    "smat_bench_mfma_peak": (_int, [C.POINTER(C.c_double)]),
    "smat_bench_static_mix": (_int, [_int, C.POINTER(C.c_double)]),
}


def _load():
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C smat_amd/csrc`). There is no CPU fallback."
        )
    # PyTorch wheels carry their own HIP runtime (same SONAME as the system one).  Two
    # runtimes in one process cannot both open the GPU, so when torch is installed it
    # is imported first and this library binds to the runtime torch already loaded.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    handle = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
    return handle


lib = _load()


def check(code):
    if code != 0:
        raise SmatError(code, lib.smat_last_error().decode())
