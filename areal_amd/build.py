"""Compile the gfx950 kernels into ``areal_amd/libareal_amd.so`` with hipcc.

Run as ``python -m areal_amd.build``.  The library is built in-tree so that it
travels with the source tree; nothing is compiled at import time.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libareal_amd.so"
ARCH = "gfx950"

HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # keep hipcc from forming packed-fp32 instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# the library links against the HIP runtime only
LINK_LIBS: list[str] = []


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build_library(verbose: bool = True, jobs: int = 4) -> Path:
    """Compile every ``csrc/*.hip`` and link the shared library.  Always rebuilds."""
    hipcc = _hipcc()
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    srcs = sources()
    objs = [obj_dir / (s.stem + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        if verbose:
            print(f"[areal_amd.build] hipcc {src.name}", flush=True)
        _run([hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)])

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs), *LINK_LIBS])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[areal_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    sys.exit(0)
