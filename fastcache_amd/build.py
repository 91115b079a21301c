"""Build recipe for libfastcache_hip.so (hipcc, gfx950 only).

``python -m fastcache_amd.build`` compiles every ``csrc/*.hip`` file into one shared library
next to this file.  hipcc cross-compiles without a GPU, so the library is built on the
development host and travels with the source tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libfastcache_hip.so"
OBJ_DIR = PKG_DIR / "csrc" / "build"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
DEVICE_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-fPIC",
    "-std=c++17",
    # packed-fp32 instructions are kept out of every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile_one(src: Path, verbose: bool) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    extra = os.environ.get("FC_EXTRA_HIPCC_FLAGS", "").split()      # e.g. -DCP_R=16 for tuning runs
    cmd = [HIPCC, *DEVICE_FLAGS, *extra, "-c", str(src), "-o", str(obj)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{res.stdout}\n{res.stderr}")
    return obj


def build_library(verbose: bool = False, jobs: int = 4) -> Path:
    """Compile and link the library unconditionally; returns its path."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile_one(s, verbose), srcs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(verbose="-q" not in sys.argv)
    print(f"built {path}")
