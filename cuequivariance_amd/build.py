"""Build recipe: compiles the HIP sources into ``libcueq_amd.so`` for gfx950 with hipcc.

``python -m cuequivariance_amd.build`` (or ``__graft_entry__.build()``) compiles every
translation unit to an object file in ``cuequivariance_amd/_build`` (in parallel, only
the stale ones unless ``force``) and links them.  Cross-compiles without a GPU.
"""

from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
BUILD = PKG / "_build"
LIB = PKG / "libcueq_amd.so"

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# Packed fp32 instructions are disabled for every device compile of this library.
COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip")) + sorted((CSRC / "generated").glob("*.hip"))


def _stale(src: Path, obj: Path) -> bool:
    if not obj.exists():
        return True
    newest = max([src.stat().st_mtime] + [h.stat().st_mtime for h in list(CSRC.glob("*.h")) + [ROOT / "include" / "cueq_amd.h"]])
    return obj.stat().st_mtime < newest


def _compile(src: Path, obj: Path) -> None:
    cmd = [HIPCC, *COMMON_FLAGS, "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{r.stdout}\n{r.stderr}")


def build_library(force: bool = False, jobs: int | None = None, verbose: bool = True) -> Path:
    BUILD.mkdir(exist_ok=True)
    sys.path.insert(0, str(ROOT))
    from cuequivariance_amd.codegen import registry as _registry

    _registry.generate()
    srcs = sources()
    todo = []
    for s in srcs:
        obj = BUILD / (s.stem + ".o")
        if force or _stale(s, obj):
            todo.append((s, obj))
    jobs = jobs or min(8, max(1, (os.cpu_count() or 2)))
    if verbose and todo:
        print(f"[cueq_amd] compiling {len(todo)} file(s) for gfx950", file=sys.stderr, flush=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for f in [ex.submit(_compile, s, o) for s, o in todo]:
            f.result()
    objs = [str(BUILD / (s.stem + ".o")) for s in srcs]
    if todo or not LIB.exists():
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *objs]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    # fused kernels of the registered fully connected products: separate small objects next to the library
    from cuequivariance_amd import jit as _jit

    _jit.prebuild_fully_connected(force)
    return LIB


if __name__ == "__main__":
    build_library(force="--force" in sys.argv)
    print(LIB)
