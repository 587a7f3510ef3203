"""smat_amd: MI355X (gfx950) block-sparse SpMM, C = A_bcsr(16x16, fp16) x B(fp16).

The compute path is the HIP library ``libsmat_amd.so`` (C ABI in ``include/smat.h``);
this package is the thin Python mirror used by the tests and by ``bench.py``.
Importing it never falls back to a CPU implementation: if the shared library is
missing, loading raises.
"""
from ._lib import lib, SmatError, library_path  # noqa: F401
from .host import (  # noqa: F401
    KERNEL_AUTO,
    KERNEL_ROWWISE,
    KERNEL_SWEEP,
    KERNEL_ROWWISE_DIRECT,
    KERNEL_ROWWISE_PACKED,
    KERNEL_COMPACT,
    KERNEL_MIXED,
    Bcsr,
    Plan,
    csr_to_bcsr,
    bin_write_csr,
    bin_write_bcsr,
    bin_read,
    mtx_write,
    csr_to_bcsr_device,
    DeviceBcsr,
    mtx_read,
    permute_csr,
    reorder_csr,
    reorder_rows,
    spmm,
)

__all__ = [
    "lib", "SmatError", "library_path", "Bcsr", "Plan", "csr_to_bcsr", "bin_write_csr", "bin_write_bcsr", "bin_read", "mtx_write", "csr_to_bcsr_device", "DeviceBcsr", "mtx_read",
    "permute_csr", "reorder_csr", "reorder_rows", "spmm",
    "KERNEL_AUTO", "KERNEL_ROWWISE", "KERNEL_SWEEP", "KERNEL_ROWWISE_DIRECT", "KERNEL_ROWWISE_PACKED", "KERNEL_COMPACT", "KERNEL_MIXED",
]
