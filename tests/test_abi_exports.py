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
    # header macro, Python mirror, Rust constant and the built library agree
    header = (ROOT / "include" / "pie_hip_kernels.h").read_text()
    assert int(re.search(r"#define\s+PIE_HIP_ABI_VERSION\s+(\d+)", header).group(1)) == ABI_VERSION
    rs = _rust_sources()
    assert int(re.search(r"pub const PIE_HIP_ABI_VERSION: c_int = (\d+);", rs).group(1)) == ABI_VERSION


def test_rust_constants_match_the_header():
    """Every PIE_HIP_* integer macro of the kernel header exists in the Rust crate with the same
    value (formats, KV storage kinds, RoPE pairings, sampler kinds, status codes)."""
    header = re.sub(r"/\*.*?\*/", "", (ROOT / "include" / "pie_hip_kernels.h").read_text(), flags=re.S)
    rs = _rust_sources()
    macros = dict(re.findall(r"#define\s+(PIE_HIP_[A-Z0-9_]+)\s+(-?\d+)\s*$", header, flags=re.M))
    for body in re.findall(r"enum\s*\{(.*?)\}", header, flags=re.S):
        macros.update(re.findall(r"(PIE_HIP_[A-Z0-9_]+)\s*=\s*(-?\d+)", body))
    consts = dict(re.findall(r"pub const (PIE_HIP_[A-Z0-9_]+): c_int = (-?\d+);", rs))
    assert len(macros) >= 15
    missing = sorted(set(macros) - set(consts))
    assert not missing, f"header macros without a Rust constant: {missing}"
    wrong = {k: (macros[k], consts[k]) for k in macros if int(macros[k]) != int(consts[k])}
    assert not wrong, wrong


def _rust_sources() -> str:
    src = ROOT / "pie_amd" / "rust" / "pie-driver-hip" / "src"
    return (src / "lib.rs").read_text() + "\n" + (src / "sys.rs").read_text()


def test_generated_rust_declarations_are_up_to_date_and_cover_the_header():
    """src/sys.rs is what gen_sys.py makes of the current header, and it binds every declared
    entry point."""
    import subprocess
    import sys

    gen = ROOT / "pie_amd" / "rust" / "pie-driver-hip" / "gen_sys.py"
    assert subprocess.run([sys.executable, str(gen), "--check"]).returncode == 0, \
        "include/pie_hip_kernels.h changed: run pie_amd/rust/pie-driver-hip/gen_sys.py"
    rs = _rust_sources()
    bound = set(re.findall(r"pub fn (pie_hip_\w+)\s*\(", rs))
    names = set(declared(ROOT / "include" / "pie_hip_kernels.h", "pie_hip_"))
    assert names <= bound, sorted(names - bound)
    # the ready callback may be null on the C side
    assert "ready_cb: Option<ReadyCb>" in rs


def test_missing_library_is_loud(monkeypatch, tmp_path):
    from pie_amd import _lib

    monkeypatch.setattr(_lib, "_kernels", None)
    monkeypatch.setattr(_lib, "KERNEL_LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(_lib.KernelLibraryMissing):
        _lib.kernels()


def test_rust_bindings_name_only_exported_symbols_with_matching_arity():
    """The (uncompiled) Rust FFI declarations under pie_amd/rust bind functions that the two
    libraries really export, with as many parameters as the C headers declare."""
    rs = re.sub(r"//[^\n]*", "", _rust_sources())
    decls = re.findall(r"pub fn (pie_\w+)\s*\((.*?)\)\s*(?:->[^;]+)?;", rs, flags=re.S)
    assert len(decls) >= 15
    headers = ""
    for h in ("pie_hip_kernels.h", "pie_driver_abi.h"):
        headers += re.sub(r"/\*.*?\*/", "", (ROOT / "include" / h).read_text(), flags=re.S)
    kernels = ctypes.CDLL(str(ROOT / "pie_amd" / "libpie_hip_kernels.so"))
    driver_path = ROOT / "pie_amd" / "libpie_driver_hip.so"
    driver = ctypes.CDLL(str(driver_path)) if driver_path.exists() else None

    def arity(params: str) -> int:
        params = params.strip()
        if not params or params == "void":
            return 0
        depth, n = 0, 1
        for ch in params:
            depth += ch in "(<"
            depth -= ch in ")>"
            n += ch == "," and depth == 0
        return n - (1 if params.rstrip().endswith(",") else 0)

    for name, params in decls:
        lib = driver if name.startswith("pie_driver_") else kernels
        if lib is not None:
            assert hasattr(lib, name), name
        m = re.search(rf"\b{name}\s*\((.*?)\)\s*;", headers, flags=re.S)
        assert m, f"{name} is not declared in include/"
        assert arity(params) == arity(m.group(1)), name
