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
    "-Wno-inline-asm", "-Wno-int-to-pointer-cast",  # the asm statements that set m0 name it as clobbered; clang notes that it is a reserved register
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: libcagnet_amd.so cannot be built")
    return exe


def sources() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


# Host-side AddressSanitizer + UndefinedBehaviorSanitizer build (the device code is compiled as usual): every
# -fsanitize= sits directly behind -Xarch_host so that it reaches the host pass only.
SAN_LIB_PATH = LIB_DIR / "libcagnet_amd_hostsan.so"
SAN_OBJ_DIR = LIB_DIR / "obj_hostsan"
HOST_SANITIZE_FLAGS = ["-g", "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
                       "-Xarch_host", "-fno-sanitize-recover=undefined", "-Xarch_host", "-fno-omit-frame-pointer"]


def _compile_one(src: Path, sanitize: bool = False) -> Path:
    obj = (SAN_OBJ_DIR if sanitize else OBJ_DIR) / (src.stem + ".o")
    flags = [f for f in HIPCC_FLAGS if f != "-O3"] + ["-O1"] + HOST_SANITIZE_FLAGS if sanitize else HIPCC_FLAGS
    cmd = [_hipcc(), *flags, "-c", str(src), "-o", str(obj)]
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


def kernel_resources(source: str = "spmm.hip", match: str = "spmm_tile_kernel") -> dict:
    """Registers and scratch of the kernels of csrc/<source> whose names contain `match`, from the compiler's own
    resource notes (the device pass only, to assembly text).  {mangled name: {"vgpr_count", "vgpr_spill_count",
    "sgpr_spill_count", "private_segment_fixed_size"}}.  The tile kernels keep their accumulators in fixed registers
    across inline-asm statements; that only holds while the register allocator spills nothing around them."""
    import re
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        out = Path(tmp) / "kernels.s"
        cmd = [_hipcc(), *HIPCC_FLAGS, "--offload-device-only", "-S", str(CSRC_DIR / source), "-o", str(out)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {source}:\n{proc.stderr}")
        text = out.read_text()
    found = {}
    for block in re.split(r"\n  - \.agpr_count:", text)[1:]:
        name = re.search(r"\.name:\s+(\S+)", block)
        if not name or match not in name.group(1):
            continue
        keys = ("vgpr_count", "vgpr_spill_count", "sgpr_spill_count", "private_segment_fixed_size")
        found[name.group(1)] = {k: int(re.search(rf"\.{k}:\s+(\d+)", block).group(1)) for k in keys}
    return found


def build_host_sanitized(jobs: int | None = None) -> Path:
    """The same sources with the host code instrumented by ASan and UBSan, as
    lib/libcagnet_amd_hostsan.so.  It is only ever linked into a sanitized test driver
    (tests/abi_host_driver.cpp); the product never loads it."""
    SAN_OBJ_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda src: _compile_one(src, True), srcs))
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-Xarch_host", "-fsanitize=address", "-Xarch_host",
           "-fsanitize=undefined", "-o", str(SAN_LIB_PATH), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"sanitized link failed:\n{proc.stdout}\n{proc.stderr}")
    return SAN_LIB_PATH


SAN_DRIVER_SRC = PKG_DIR.parent / "tests" / "abi_host_driver.cpp"
SAN_DRIVER_PATH = LIB_DIR / "abi_host_driver"


def build_host_driver() -> Path:
    """tests/abi_host_driver.cpp compiled with ASan + UBSan and linked against the sanitized library (built
    first).  The program carries the sanitizer runtime itself, so it runs without any preloading."""
    lib = build_host_sanitized()
    rocm = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))
    clang = rocm / "llvm" / "bin" / "clang++"
    cmd = [str(clang), "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-fno-omit-frame-pointer", "-D__HIP_PLATFORM_AMD__", f"-I{rocm / 'include'}", f"-I{PKG_DIR.parent / 'include'}",
           str(SAN_DRIVER_SRC), "-o", str(SAN_DRIVER_PATH), str(lib), f"-L{rocm / 'lib'}", "-lamdhip64",
           f"-Wl,-rpath,{LIB_DIR}", f"-Wl,-rpath,{rocm / 'lib'}"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"sanitized driver build failed:\n{proc.stdout}\n{proc.stderr}")
    return SAN_DRIVER_PATH


if __name__ == "__main__":
    if "--host-sanitize" in sys.argv[1:]:
        print(build_host_driver())
    else:
        build_library()
