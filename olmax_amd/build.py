"""Builds libolmax_hip.so (hand-written gfx950 kernels + C ABI) in-tree with hipcc.

Every ``.hip`` file under ``csrc/`` is compiled to an object in parallel and the objects
are linked into ``olmax_amd/libolmax_hip.so``.  No GPU is needed: hipcc cross-compiles.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
OBJ = HERE / "csrc" / "build"
LIB = HERE / "libolmax_hip.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffast-math" if False else "-fno-fast-math",
    "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    "-Wno-inline-asm",
    "-Wno-unknown-warning-option",
    "-I", str(CSRC),
    "-I", str(HERE.parent / "include"),
]


def _compile(src: Path, force: bool) -> Path:
    obj = OBJ / (src.stem + ".o")
    deps = [src] + list(CSRC.glob("*.h")) + list((HERE.parent / "include").glob("*.h"))
    if not force and obj.exists() and all(obj.stat().st_mtime > d.stat().st_mtime for d in deps):
        return obj
    cmd = [HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{r.stderr[-4000:]}")
    return obj


def build_all(force: bool = True, jobs: int = 8) -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    srcs = sorted(CSRC.glob("*.hip"))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    return LIB


if __name__ == "__main__":
    p = build_all(force="--force" in sys.argv)
    print(p)
