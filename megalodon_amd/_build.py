"""Compile the gfx950 C-ABI library ``lib/libmegalodon_hip.so`` with hipcc.

The library has no PyTorch dependency: it is plain HIP behind ``extern "C"``
entry points (``include/megalodon_hip.h``), so a single ``hipcc -shared``
invocation per translation unit is the whole build.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libmegalodon_hip.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed-fp32 VALU forms are disabled for every device translation unit
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-Wno-ignored-optimization-argument",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile(src: Path, obj_dir: Path, extra: list[str], force: bool = True) -> Path:
    obj = obj_dir / (src.stem + ".o")
    if not force and obj.exists():
        deps = [src, *CSRC.glob("*.hpp"), PKG_DIR.parent / "include" / "megalodon_hip.h"]
        if all(obj.stat().st_mtime > d.stat().st_mtime for d in deps):
            return obj
    cmd = [HIPCC, *FLAGS, *extra, "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{r.stdout}\n{r.stderr}")
    return obj


def build_library(verbose: bool = True, extra: list[str] | None = None, jobs: int = 8,
                  force: bool = True) -> Path:
    """Compile every ``csrc/*.hip`` and link ``libmegalodon_hip.so``.  With
    ``force=False`` objects newer than their source and the shared headers are
    reused (developer iterations only)."""
    extra = list(extra or [])
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    srcs = sources()
    if verbose:
        print(f"[megalodon_amd] hipcc {ARCH}: {', '.join(s.name for s in srcs)}", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, obj_dir, extra, force), srcs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[megalodon_amd] built {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    args = sys.argv[1:]
    incremental = "--incremental" in args
    build_library(extra=[a for a in args if a != "--incremental"], force=not incremental)
