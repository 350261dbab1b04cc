"""Builds the C restatement of the CPU oracle (oracle/qworacle_c.c -> oracle/libqworacle.so) with gcc.
Test infrastructure only: tests, the smoke check and the benchmark's CPU-baseline leg load it."""
from __future__ import annotations

import pathlib
import shutil
import subprocess

HERE = pathlib.Path(__file__).resolve().parent
SRC = HERE / "qworacle_c.c"
LIB = HERE / "libqworacle.so"


def build(verbose: bool = False) -> pathlib.Path:
    gcc = shutil.which("gcc")
    if gcc is None:
        raise RuntimeError("gcc not found; the oracle's C restatement cannot be built")
    cmd = [gcc, "-O2", "-std=c11", "-fPIC", "-shared", "-ffp-contract=off", "-fopenmp", "-o", str(LIB), str(SRC), "-lm"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"gcc failed:\n{res.stderr[-4000:]}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build(verbose=True)
