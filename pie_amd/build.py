"""Build the gfx950 kernel library and the C++ host driver, in-tree.

`python -m pie_amd.build` compiles every `.hip` file under `pie_amd/csrc/` with
hipcc for gfx950 only and links `pie_amd/libpie_hip_kernels.so`.  Objects are
cached under `build/` keyed on source mtimes; `force=True` recompiles everything.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "pie_amd" / "csrc"
INCLUDE = ROOT / "include"
OBJ_DIR = ROOT / "build" / "obj"
KERNEL_LIB = ROOT / "pie_amd" / "libpie_hip_kernels.so"
DRIVER_SRC = CSRC / "driver"
DRIVER_LIB = ROOT / "pie_amd" / "libpie_driver_hip.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    # Packed-FP32 VALU forms are disabled for every device compile.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def _newer(target: Path, deps: list[Path]) -> bool:
    if not target.exists():
        return False
    t = target.stat().st_mtime
    return all(d.stat().st_mtime <= t for d in deps)


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + proc.stderr)
        raise RuntimeError(f"build step failed: {cmd[0]} ... {cmd[-1]}")
    # hipcc's host pass warns that it does not know the packed-fp32 feature; drop that.
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if err.strip():
        sys.stderr.write(err + "\n")


def hip_sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build_kernels(force: bool = False, jobs: int | None = None) -> Path:
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    headers = sorted(CSRC.glob("*.h")) + sorted(INCLUDE.glob("*.h"))
    todo = []
    objs = []
    for src in hip_sources():
        obj = OBJ_DIR / (src.stem + ".o")
        objs.append(obj)
        if force or not _newer(obj, [src] + headers):
            todo.append([HIPCC, *HIP_FLAGS, "-c", str(src), "-o", str(obj)])
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_run, todo))
    if force or todo or not KERNEL_LIB.exists():
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(KERNEL_LIB),
              *map(str, objs)])
    return KERNEL_LIB


def build_driver(force: bool = False, jobs: int | None = None) -> Path:
    """The C++ host driver (`pie_driver_hip_run_inproc` and friends), linked against the
    kernel library next to it."""
    obj_dir = OBJ_DIR / "driver"
    obj_dir.mkdir(parents=True, exist_ok=True)
    headers = sorted(DRIVER_SRC.glob("*.hpp")) + sorted(INCLUDE.glob("*.h"))
    todo, objs = [], []
    for src in sorted(DRIVER_SRC.glob("*.hip")):
        obj = obj_dir / (src.stem + ".o")
        objs.append(obj)
        if force or not _newer(obj, [src] + headers):
            todo.append([HIPCC, *HIP_FLAGS, f"-I{DRIVER_SRC}", "-c", str(src), "-o", str(obj)])
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_run, todo))
    if force or todo or not DRIVER_LIB.exists() or not _newer(DRIVER_LIB, [KERNEL_LIB]):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(DRIVER_LIB),
              *map(str, objs), f"-L{KERNEL_LIB.parent}", "-lpie_hip_kernels",
              "-Wl,-rpath,$ORIGIN", "-lpthread"])
    return DRIVER_LIB


def build_all(force: bool = False) -> None:
    build_kernels(force=force)
    build_driver(force=force)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
    print(KERNEL_LIB)
    print(DRIVER_LIB)
