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


FFI_SRC = HERE / "ffi" / "olmax_ffi.cc"
FFI_LIB = HERE / "libolmax_ffi.so"


def xla_ffi_include_dir():
    """Directory that holds xla/ffi/api/ffi.h (it ships inside jaxlib), or None.  $OLMAX_XLA_FFI_INCLUDE
    overrides the lookup through jax.ffi.include_dir()."""
    cand = os.environ.get("OLMAX_XLA_FFI_INCLUDE")
    if not cand:
        try:
            import jax.ffi  # noqa: WPS433 - optional dependency, absent in this image

            cand = jax.ffi.include_dir()
        except Exception:
            return None
    return cand if cand and (Path(cand) / "xla" / "ffi" / "api" / "ffi.h").exists() else None


def build_ffi_adapter():
    """Compile the XLA-FFI adapter (ffi/olmax_ffi.cc -> libolmax_ffi.so, linked against
    libolmax_hip.so) when the XLA FFI headers are installed; returns the library path, or None
    (with a note on stderr) when they are not.  Nothing stands in for missing headers."""
    inc = xla_ffi_include_dir()
    if inc is None:
        print("olmax_amd.build: XLA FFI headers (xla/ffi/api/ffi.h, shipped with jaxlib) not found: "
              "libolmax_ffi.so not built", file=sys.stderr)
        return None
    cmd = [HIPCC, "-x", "c++", "-D__HIP_PLATFORM_AMD__", "-O2", "-std=c++17", "-fPIC", "-shared", "-I", inc,
           "-I", str(HERE.parent / "include"), "-I", "/opt/rocm/include", str(FFI_SRC), "-o", str(FFI_LIB),
           "-L", str(HERE), "-lolmax_hip", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {FFI_SRC.name}:\n{r.stderr[-4000:]}")
    return FFI_LIB


if __name__ == "__main__":
    p = build_all(force="--force" in sys.argv)
    print(p)
    build_ffi_adapter()
