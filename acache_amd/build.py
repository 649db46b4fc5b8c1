"""Build ``libacache_hip.so`` (gfx950) in-tree with hipcc.

``python -m acache_amd.build`` compiles every ``csrc/*.hip`` to an object file
(in parallel) and links them into ``acache_amd/libacache_hip.so``.  The build
needs no GPU: hipcc cross-compiles for gfx950.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = CSRC / "_obj"
LIB = PKG / "libacache_hip.so"

# packed-fp32 code generation is switched off for every HIP translation unit
HIP_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++20", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]
PER_FILE_FLAGS = {
    # the RoPE rotation must not be contracted into fused multiply-adds
    "relocate.hip": ["-ffp-contract=off"],
    "rope_scatter.hip": ["-ffp-contract=off"],
}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm toolchain is required to build libacache_hip.so")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build(verbose: bool = True, jobs: int | None = None) -> Path:
    hipcc = _hipcc()
    OBJ.mkdir(exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    if not sources:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    objs = [OBJ / (s.stem + ".o") for s in sources]

    def compile_one(pair):
        src, obj = pair
        cmd = [hipcc, *HIP_FLAGS, *PER_FILE_FLAGS.get(src.name, []), "-c", str(src), "-o", str(obj)]
        if verbose:
            print("[acache_amd.build] hipcc", src.name, flush=True)
        _run(cmd)

    jobs = jobs or min(8, len(sources), os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(sources, objs)))
    tmp = LIB.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)])
    os.replace(tmp, LIB)
    if verbose:
        print(f"[acache_amd.build] linked {LIB} ({LIB.stat().st_size >> 10} KiB)", flush=True)
    return LIB


if __name__ == "__main__":
    build()
