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
DEFAULT_LIB_PATH = LIB_DIR / "libpippy_amd.so"
# PIPPY_AMD_LIB points the loader at another build of the library (a measurement variant made with
# ``python -m pippy_amd._build --define ... --out ...``); the default build never sets it
LIB_PATH = Path(os.environ.get("PIPPY_AMD_LIB") or DEFAULT_LIB_PATH).resolve()

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed-fp32 VALU forms are switched off for every device compilation unit
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


def _compile_one(src: Path, obj: Path, defines: tuple = ()) -> None:
    cmd = [HIPCC, *HIP_FLAGS, *("-D" + d for d in defines), "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stderr}")


def build(verbose: bool = True, jobs: int | None = None, defines: tuple = (), out: Path | None = None) -> Path:
    """Compile every ``csrc/*.hip`` for gfx950 and link the shared library.  ``defines`` (``NAME=VALUE``
    strings) and ``out`` make a variant of the library beside the default one."""
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    lib_path = Path(out).resolve() if out else DEFAULT_LIB_PATH
    if defines and lib_path == DEFAULT_LIB_PATH:
        raise ValueError("a build with extra defines needs an output path of its own (out=...)")
    lib_path.parent.mkdir(parents=True, exist_ok=True)
    obj_dir = LIB_DIR / ("obj" if lib_path == DEFAULT_LIB_PATH else "obj_" + lib_path.stem)
    obj_dir.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC_DIR}")
    objs = [obj_dir / (s.stem + ".o") for s in srcs]
    jobs = jobs or min(8, len(srcs), os.cpu_count() or 1)
    if verbose:
        print(f"[pippy_amd] hipcc {ARCH}: {len(srcs)} sources, {jobs} jobs", file=sys.stderr)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda so: _compile_one(so[0], so[1], tuple(defines)), zip(srcs, objs)))
    link = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(lib_path),
            *map(str, objs)]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"[pippy_amd] built {lib_path}", file=sys.stderr)
    return lib_path


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--define", action="append", default=[], metavar="NAME=VALUE",
                    help="extra preprocessor definition (a measurement variant; needs --out)")
    ap.add_argument("--out", default=None, help="path of the shared library to write (default: the package's own)")
    a = ap.parse_args()
    build(defines=tuple(a.define), out=a.out)
