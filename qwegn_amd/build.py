"""Builds libqwhip.so (gfx950 code objects + the C ABI) in-tree with hipcc."""
from __future__ import annotations

import concurrent.futures
import pathlib
import shutil
import subprocess

PKG = pathlib.Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libqwhip.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-ffp-contract=off",
    # scalar kernel arguments arrive in SGPRs instead of through a load at the start of every wave (see qw_launch_scalar)
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
]


def sources() -> list[pathlib.Path]:
    return sorted(CSRC.glob("*.hip"))


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not pathlib.Path(exe).exists():
        raise RuntimeError("hipcc not found; libqwhip cannot be built")
    return exe


def _compile(src: pathlib.Path, obj: pathlib.Path) -> None:
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{res.stderr[-6000:]}")


def build_lib(jobs: int = 8, verbose: bool = False) -> pathlib.Path:
    """Compiles every csrc/*.hip for gfx950 and links libqwhip.so. Always recompiles."""
    LIB_DIR.mkdir(exist_ok=True)
    objdir = PKG / "build"
    objdir.mkdir(exist_ok=True)
    srcs = sources()
    objs = [objdir / (s.stem + ".o") for s in srcs]
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, min(jobs, len(srcs)))) as ex:
        list(ex.map(_compile, srcs, objs))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(LIB_PATH), *map(str, objs)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr[-6000:]}")
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


HOST_TESTS = PKG / "host" / "host_tests"


def build_host_tests(verbose: bool = False) -> pathlib.Path:
    """Compiles the C++ host operator layer's test program (plain host C++ through hipcc's clang) against libqwhip.so."""
    cmd = [_hipcc(), "-x", "c++", "-std=c++17", "-O2", str(PKG / "host" / "host_tests.cpp"), "-x", "none", "-o", str(HOST_TESTS),
           "-L", str(LIB_DIR), "-lqwhip", "-Wl,-rpath,$ORIGIN/../lib"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"host_tests build failed:\n{res.stderr[-6000:]}")
    if verbose:
        print(f"built {HOST_TESTS}")
    return HOST_TESTS


if __name__ == "__main__":
    build_lib(verbose=True)
    build_host_tests(verbose=True)
