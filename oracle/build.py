"""Compile the C oracle (test infrastructure) into oracle/libpie_oracle.so.

Plain gcc, no fast-math and no FMA contraction, so every float operation is the
IEEE one the source spells out.  OpenMP only parallelises independent rows.
"""
from __future__ import annotations

import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
LIB = HERE / "libpie_oracle.so"


def build(force: bool = False) -> Path:
    srcs = sorted((HERE / "src").glob("*.c"))
    deps = srcs + sorted((HERE / "src").glob("*.h"))
    if not force and LIB.exists() and all(d.stat().st_mtime <= LIB.stat().st_mtime for d in deps):
        return LIB
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp", "-ffp-contract=off",
           "-fno-fast-math", "-Wall", "-Wextra", "-o", str(LIB), *map(str, srcs), "-lm"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("oracle build failed")
    if proc.stderr.strip():
        sys.stderr.write(proc.stderr)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
