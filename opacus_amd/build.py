"""Builds ``libdpsgd_hip.so`` (the HIP kernels behind the C ABI of ``include/dpk.h``).

``python -m opacus_amd.build`` cross-compiles every ``csrc/*.hip`` for gfx950 with
hipcc and links them into ``opacus_amd/lib/libdpsgd_hip.so``. No GPU is needed to
build. Nothing here is called at import time: the library is built ahead of use and
``opacus_amd._lib`` only loads what is there.
"""

from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libdpsgd_hip.so"
OBJ_DIR = PKG_DIR / "build"

ARCH = "gfx950"
# -packed-fp32-ops is switched off: the compiler must not form v_pk_*_f32 from
# ordinary float code.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unknown-warning-option",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built")
    return exe


def _compile_one(src: Path, extra: list[str]) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{res.stdout}\n{res.stderr}")
    return obj


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build_library(verbose: bool = True, extra_flags: list[str] | None = None, jobs: int | None = None) -> Path:
    """Compiles all sources (always, even when a library is present) and links them."""
    extra = list(extra_flags or [])
    OBJ_DIR.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    jobs = jobs or min(8, len(srcs), os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile_one(s, extra), srcs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
