"""ctypes loader for the HIP kernel library.  No fallback: a missing library is an error."""
from __future__ import annotations

import ctypes as C
from pathlib import Path

_PKG = Path(__file__).resolve().parent
KERNEL_LIB_PATH = _PKG / "libpie_hip_kernels.so"
ABI_VERSION = 3   # PIE_HIP_ABI_VERSION of include/pie_hip_kernels.h this module was written against

_kernels = None


class KernelLibraryMissing(RuntimeError):
    pass


def kernels() -> C.CDLL:
    """Load libpie_hip_kernels.so (built by `python -m pie_amd.build`)."""
    global _kernels
    if _kernels is None:
        if not KERNEL_LIB_PATH.exists():
            raise KernelLibraryMissing(
                f"{KERNEL_LIB_PATH} is not built; run `python -m pie_amd.build` "
                "(there is no CPU or PyTorch fallback for these ops)")
        lib = C.CDLL(str(KERNEL_LIB_PATH))
        lib.pie_hip_abi_version.restype = C.c_int
        got = lib.pie_hip_abi_version()
        if got != ABI_VERSION:
            raise KernelLibraryMissing(
                f"{KERNEL_LIB_PATH} has ABI version {got}, expected {ABI_VERSION}; rebuild it")
        _kernels = lib
    return _kernels
