"""Build libtessera_gfx950.so (hipcc, --offload-arch=gfx950) in-tree.

``python -m tessera_amd.build`` or ``tessera_amd.build.build_library()``.
Every translation unit under ``csrc/*.hip`` is compiled to an object in
``csrc/build/`` (in parallel) and linked into ``lib/libtessera_gfx950.so``.
hipcc cross-compiles without a GPU present.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = CSRC / "build"
LIB = PKG / "lib" / "libtessera_gfx950.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed-fp32 VALU forms are disabled for every HIP translation unit.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def _compile(src: Path, force: bool) -> Path:
    obj = OBJ / (src.stem + ".o")
    deps = [src] + list(CSRC.glob("*.h")) + [PKG.parent / "include" / "tessera_gfx950.h"]
    if not force and obj.exists() and all(obj.stat().st_mtime >= d.stat().st_mtime for d in deps):
        return obj
    cmd = [HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_library(force: bool = True, jobs: int = 8) -> Path:
    """Compile and link the library; returns its path.  ``force`` recompiles
    every unit even when an up-to-date object exists."""
    OBJ.mkdir(parents=True, exist_ok=True)
    LIB.parent.mkdir(parents=True, exist_ok=True)
    srcs = sorted(CSRC.glob("*.hip"))
    if not srcs:
        raise RuntimeError("no HIP sources found")
    with ThreadPoolExecutor(max_workers=min(jobs, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build_library(force="--incremental" not in sys.argv))
