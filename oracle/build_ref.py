"""Build the reference's own host sampler and BRLE decoder into oracle/_ref/ (TEST
INFRASTRUCTURE ONLY).

Sources are compiled where they lie in the reference tree — driver/portable/src/sampler.cpp and
driver/cuda/src/brle.cpp, both plain C++20 with no dependency outside the standard library — with
the small `extern "C"` shim oracle/ref_shim.cpp in front; nothing is copied, and no header, library
or generated file is stood in for.  Also built: the reference's own BRLE unit test
(driver/cuda/tests/test_brle.cpp) as oracle/_ref/ref_test_brle, which tests run once.

The rest of the reference's CPU path (driver/portable: plan.cpp, graph_*.cpp, executor) needs ggml
from llama.cpp and header libraries fetched at configure time and is not buildable here.

Outputs only under oracle/_ref/ (git-ignored).  Without the reference tree this does nothing and
returns None; tests that need the library skip."""
from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
REF = Path(os.environ.get("PIE_REFERENCE_DIR", "/root/reference"))
OUT = HERE / "_ref"
LIB = OUT / "libpie_ref.so"
BRLE_TEST = OUT / "ref_test_brle"

SAMPLER = REF / "driver" / "portable" / "src" / "sampler.cpp"
BRLE = REF / "driver" / "cuda" / "src" / "brle.cpp"
BRLE_TEST_SRC = REF / "driver" / "cuda" / "tests" / "test_brle.cpp"


def available() -> bool:
    return SAMPLER.exists() and BRLE.exists()


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(map(str, cmd)) + "\n" + proc.stdout + proc.stderr)
        raise RuntimeError("reference build failed")


def build(force: bool = False):
    """Returns the library path, or None when the reference tree is absent (an existing build,
    e.g. one that travelled to another machine, is then used as it is)."""
    if not available():
        return LIB if LIB.exists() else None
    deps = [SAMPLER, BRLE, HERE / "ref_shim.cpp", Path(__file__)]
    if not force and LIB.exists() and all(d.stat().st_mtime <= LIB.stat().st_mtime for d in deps):
        return LIB
    OUT.mkdir(exist_ok=True)
    # CMake Release flags (the reference sets no others: no fast-math, no -march), x86-64 baseline
    flags = ["-std=c++20", "-O3", "-DNDEBUG", "-fPIC", f"-I{SAMPLER.parent}", f"-I{BRLE.parent}"]
    _run(["g++", *flags, "-shared", "-o", str(LIB), str(HERE / "ref_shim.cpp"), str(SAMPLER), str(BRLE)])
    if BRLE_TEST_SRC.exists():
        _run(["g++", *flags, "-o", str(BRLE_TEST), str(BRLE_TEST_SRC), str(BRLE)])
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
