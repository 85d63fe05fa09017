"""The C-ABI libraries load and export every symbol their headers declare (no GPU calls)."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def declared(header: Path, prefix: str):
    text = re.sub(r"/\*.*?\*/", "", header.read_text(), flags=re.S)
    return sorted(set(re.findall(rf"\b({prefix}\w+)\s*\(", text)))


def test_kernel_library_exports_declared_symbols():
    lib_path = ROOT / "pie_amd" / "libpie_hip_kernels.so"
    if not lib_path.exists():
        from pie_amd import build

        build.build_kernels()
    lib = ctypes.CDLL(str(lib_path))
    names = declared(ROOT / "include" / "pie_hip_kernels.h", "pie_hip_")
    assert len(names) >= 4
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared but not exported: {missing}"
    lib.pie_hip_abi_version.restype = ctypes.c_int
    from pie_amd._lib import ABI_VERSION

    assert lib.pie_hip_abi_version() == ABI_VERSION


def test_missing_library_is_loud(monkeypatch, tmp_path):
    from pie_amd import _lib

    monkeypatch.setattr(_lib, "_kernels", None)
    monkeypatch.setattr(_lib, "KERNEL_LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(_lib.KernelLibraryMissing):
        _lib.kernels()
