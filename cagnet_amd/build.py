"""Build recipe of libcagnet_amd.so: hipcc, gfx950 code objects only, no torch in the link.

    python -m cagnet_amd.build          # compile every csrc/*.hip and link cagnet_amd/lib/libcagnet_amd.so

The library is built in-tree so that it travels with the source tree; nothing is compiled at
import time and nothing falls back to another implementation when the library is missing.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
OBJ_DIR = LIB_DIR / "obj"
LIB_PATH = LIB_DIR / "libcagnet_amd.so"

ARCH = "gfx950"
# Packed-fp32 instruction selection is switched off for every kernel; the flag is a device-side
# target feature, the host pass only warns that it does not know it.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "-fPIC",
    f"--offload-arch={ARCH}",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-warning-option",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: libcagnet_amd.so cannot be built")
    return exe


def sources() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


def _compile_one(src: Path) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stdout}\n{proc.stderr}")
    noise = "is not a recognized feature for this target"
    warnings = "\n".join(l for l in proc.stderr.splitlines() if l.strip() and noise not in l)
    if warnings:
        print(f"[cagnet_amd.build] {src.name}:\n{warnings}", file=sys.stderr)
    return obj


def build_library(jobs: int | None = None, verbose: bool = True) -> Path:
    """Compile and link unconditionally (also when a built library is already there)."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC_DIR}")
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile_one, srcs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(tmp), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[cagnet_amd.build] built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
