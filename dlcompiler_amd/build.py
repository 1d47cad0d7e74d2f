"""Compile the gfx950 kernels in ``csrc/`` into ``lib/libdlblas_hip.so`` with hipcc.

Run ``python -m dlcompiler_amd.build`` (cross-compiles without a GPU).  Every ``*.hip`` file
becomes one object; objects are rebuilt only when the source or a header is newer, unless
``force`` is set.
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
OBJ_DIR = LIB_DIR / "obj"
LIB_PATH = LIB_DIR / "libdlblas_hip.so"
INCLUDE_DIR = PKG_DIR.parent / "include"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar fp32
# code; the host pass prints a harmless "not a recognized feature" note for it.
DEVICE_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _sources() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


def _headers() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.h")) + sorted(INCLUDE_DIR.glob("*.h"))


def _stale(target: Path, deps: list[Path]) -> bool:
    if not target.exists():
        return True
    t = target.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps)


def _compile_one(src: Path, obj: Path, verbose: bool) -> None:
    cmd = [HIPCC, *DEVICE_FLAGS, f"-I{INCLUDE_DIR}", "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build_library(force: bool = False, verbose: bool = False, jobs: int | None = None) -> Path:
    """Build (or rebuild) the shared library and return its path."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    headers = _headers()
    todo = []
    objs = []
    for src in _sources():
        obj = OBJ_DIR / (src.stem + ".o")
        objs.append(obj)
        if force or _stale(obj, [src, *headers]):
            todo.append((src, obj))
    if todo:
        jobs = jobs or min(8, len(todo))
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            list(pool.map(lambda so: _compile_one(so[0], so[1], verbose), todo))
    if todo or force or _stale(LIB_PATH, objs):
        cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB_PATH),
               *map(str, objs)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(force="--force" in sys.argv, verbose=True)
    print(path)
