"""Builds the native artefacts in-tree: `btb_amd/libbtb_hip.so` (the HIP kernels and their C ABI, for gfx950) with
hipcc, and `oracle/libbtb_oracle.so` (the CPU checker) with gcc. hipcc cross-compiles, so this runs where no GPU is.

    python -m btb_amd.build            # both
    python -m btb_amd.build hip        # the product library only
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libbtb_hip.so")
OBJ = os.path.join(HERE, "csrc", "obj")
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "libbtb_oracle.so")

ARCH = "gfx950"

# -packed-fp32-ops: v_pk_{add,mul,fma}_f32 are never emitted; -ffp-contract=off: every fused multiply-add in the
# kernels is an explicit fmaf, so the compiler fuses nothing on its own (the summation order is part of the contract)
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the HIP library cannot be built")


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _fresh(src: str, obj: str) -> bool:
    """whether obj is newer than its source and every header the sources share"""
    if not os.path.exists(obj):
        return False
    deps = [src] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    deps.append(os.path.join(ROOT, "include", "btb_hip.h"))
    return all(os.path.getmtime(d) <= os.path.getmtime(obj) for d in deps)


def _compile(src: str, incremental: bool = False) -> str:
    obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
    if incremental and _fresh(src, obj):
        return obj
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(ln for ln in r.stderr.splitlines() if noise not in ln)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_hip(jobs: int = 8, incremental: bool = False) -> str:
    """compile every csrc/*.hip for gfx950 and link libbtb_hip.so; returns its path. `incremental` (a developer's
    shortcut, `python -m btb_amd.build hip --incremental`) skips sources whose object is newer than they and the
    headers are"""
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, incremental), sources()))
    tmp = LIB + ".tmp"
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, LIB)
    return LIB


def build_oracle() -> str:
    """the CPU oracle's C restatement (test infrastructure) as a shared library"""
    r = subprocess.run(["make", "-C", ORACLE_DIR, "-B", "libbtb_oracle.so"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"oracle build failed:\n{r.stdout}\n{r.stderr}")
    return ORACLE_LIB


def main(argv: list[str]) -> int:
    incremental = "--incremental" in argv
    what = [a for a in argv[1:] if not a.startswith("--")] or ["hip", "oracle"]
    if "hip" in what:
        print(build_hip(incremental=incremental))
    if "oracle" in what:
        print(build_oracle())
    return 0


if __name__ == "__main__":
    raise SystemExit(main(sys.argv))
