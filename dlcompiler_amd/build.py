"""Compile the gfx950 kernels in ``csrc/`` into ``lib/libdlblas_hip.so`` with hipcc.

Run ``python -m dlcompiler_amd.build`` (cross-compiles without a GPU).  Every ``*.hip`` file
becomes one object; objects are rebuilt only when the source or a header is newer, unless
``force`` is set.

The compiler's per-kernel resource report (registers, scratch, spills) is collected for every
object and written next to it.  Several kernels issue their loads through inline assembly with
hand-counted ``s_waitcnt`` values: a register the allocator spills or copies through scratch
memory between such a load and its wait would be read before the data has landed, and scratch
traffic would also change the vector-memory counts the waits assume.  The build therefore fails
when one of those kernels reports scratch memory or spilled vector registers.
"""
from __future__ import annotations

import json
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
OBJ_DIR = LIB_DIR / "obj"
LIB_PATH = LIB_DIR / "libdlblas_hip.so"
# measurement kernels that bench.py times; a library of their own, not part of the operator ABI
PROBE_SRC = CSRC_DIR / "bench" / "probe.hip"
PROBE_LIB_PATH = LIB_DIR / "libdlblas_bench_probe.so"
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
    # the direct-to-LDS helpers list m0 (a reserved register) among their clobbers on purpose
    "-Wno-inline-asm",
    "-Rpass-analysis=kernel-resource-usage",
]

# kernels whose loads and waits are issued by hand: no scratch, no spilled vector registers
HAND_SCHEDULED = ("moe_gemm", "prefill_attn_kernel", "paged_decode_split_kernel")


def _sources() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


def _headers() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.h")) + sorted(INCLUDE_DIR.glob("*.h"))


def _stale(target: Path, deps: list[Path]) -> bool:
    if not target.exists():
        return True
    t = target.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps)


_REMARK = re.compile(r"remark:\s+(.*?)\s*\[-Rpass-analysis=kernel-resource-usage\]")
_FIELDS = {"VGPRs": "vgprs", "AGPRs": "agprs", "TotalSGPRs": "sgprs",
           "ScratchSize [bytes/lane]": "scratch_bytes", "VGPRs Spill": "vgpr_spills",
           "SGPRs Spill": "sgpr_spills", "Occupancy [waves/SIMD]": "occupancy",
           "LDS Size [bytes/block]": "lds_bytes"}


def parse_resource_remarks(stderr: str) -> dict[str, dict[str, int]]:
    """``{mangled kernel name: {vgprs, agprs, sgprs, scratch_bytes, vgpr_spills, ...}}`` from the
    ``-Rpass-analysis=kernel-resource-usage`` remarks of one hipcc run."""
    kernels: dict[str, dict[str, int]] = {}
    cur = None
    for line in stderr.splitlines():
        m = _REMARK.search(line)
        if not m:
            continue
        key, _, val = m.group(1).partition(":")
        key, val = key.strip(), val.strip()
        if key == "Function Name":
            cur = kernels.setdefault(val, {})
        elif cur is not None and key in _FIELDS and val.lstrip("-").isdigit():
            cur[_FIELDS[key]] = int(val)
    return kernels


def check_hand_scheduled(kernels: dict[str, dict[str, int]], source_text: str = "") -> list[str]:
    """Names (with the offending figures) of hand-scheduled kernels that use scratch or spill.

    The check fails closed: a source that defines a hand-scheduled kernel (its tag appears in
    ``source_text``) must yield at least one parsed report for it, and every such report must
    carry both figures -- a compiler that prints the remarks differently, or not at all, stops
    the build instead of passing it."""
    bad = []
    for tag in HAND_SCHEDULED:
        if tag in source_text and not any(tag in name for name in kernels):
            bad.append(f"{tag}: defined in the source but no resource report was parsed for it")
    for name, r in kernels.items():
        if any(tag in name for tag in HAND_SCHEDULED):
            if "scratch_bytes" not in r or "vgpr_spills" not in r:
                bad.append(f"{name}: resource report lacks the scratch or spill figure")
            elif r["scratch_bytes"] or r["vgpr_spills"]:
                bad.append(f"{name}: scratch {r['scratch_bytes']} B/lane, "
                           f"{r['vgpr_spills']} spilled VGPRs")
    return bad


def _compile_one(src: Path, obj: Path, verbose: bool) -> None:
    cmd = [HIPCC, *DEVICE_FLAGS, f"-I{INCLUDE_DIR}", "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = ("is not a recognized feature for this target", "-Rpass-analysis=kernel-resource-usage")
    lines = proc.stderr.splitlines()
    keep, skip = [], 0
    for l in lines:
        if any(n in l for n in noise):
            skip = 2 if "-Rpass-analysis" in l and "Function Name" in l else 0
            continue
        if skip and (l.lstrip().startswith(("|", "^")) or re.match(r"\s*\d+ \|", l)):
            skip -= 1  # the source excerpt printed under a remark
            continue
        keep.append(l)
    err = "\n".join(keep)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    kernels = parse_resource_remarks(proc.stderr)
    report = obj.with_suffix(".resources.json")
    report.write_text(json.dumps(kernels, indent=1, sort_keys=True))
    bad = check_hand_scheduled(kernels, src.read_text())
    if bad:
        obj.unlink(missing_ok=True)
        raise RuntimeError(f"{src.name}: hand-scheduled kernels must not spill or use scratch:\n  "
                           + "\n  ".join(bad))
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
    build_probe_library(force)
    return LIB_PATH


def build_probe_library(force: bool = False) -> Path:
    """Build ``libdlblas_bench_probe.so`` (the measurement kernels bench.py times)."""
    deps = [PROBE_SRC, *PROBE_SRC.parent.glob("*.h"), *_headers()]
    if force or _stale(PROBE_LIB_PATH, deps):
        cmd = [HIPCC, *[f for f in DEVICE_FLAGS if not f.startswith("-Rpass")], f"-I{INCLUDE_DIR}",
               "-shared", str(PROBE_SRC), "-o", str(PROBE_LIB_PATH)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {PROBE_SRC.name}:\n{proc.stderr}")
    return PROBE_LIB_PATH


def kernel_resources() -> dict[str, dict[str, int]]:
    """The resource reports of the last build of every object, merged."""
    merged: dict[str, dict[str, int]] = {}
    for rep in sorted(OBJ_DIR.glob("*.resources.json")):
        merged.update(json.loads(rep.read_text()))
    return merged


if __name__ == "__main__":
    path = build_library(force="--force" in sys.argv, verbose=True)
    print(path)
