"""Builds the gfx950 kernel library (``pippy_amd/lib/libpippy_amd.so``) with hipcc.

The library is a plain C-ABI shared object (see ``include/pippy_amd.h``); it does not link against
torch.  ``build()`` always recompiles; everything else only loads what is already built.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libpippy_amd.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed-fp32 VALU forms are switched off for every device compilation unit
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


def _compile_one(src: Path, obj: Path) -> None:
    cmd = [HIPCC, *HIP_FLAGS, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stderr}")


def build(verbose: bool = True, jobs: int | None = None) -> Path:
    """Compile every ``csrc/*.hip`` for gfx950 and link the shared library."""
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    obj_dir = LIB_DIR / "obj"
    obj_dir.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC_DIR}")
    objs = [obj_dir / (s.stem + ".o") for s in srcs]
    jobs = jobs or min(8, len(srcs), os.cpu_count() or 1)
    if verbose:
        print(f"[pippy_amd] hipcc {ARCH}: {len(srcs)} sources, {jobs} jobs", file=sys.stderr)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_compile_one, srcs, objs))
    link = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB_PATH),
            *map(str, objs)]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"[pippy_amd] built {LIB_PATH}", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build()
