"""Build libquick_ssm_hip.so (gfx950) in-tree with hipcc.

    python -m quick_ssm_amd.build            # compile every source, link the shared library

hipcc cross-compiles for gfx950 without a GPU.  Objects go to quick_ssm_amd/csrc/build/, the
library to quick_ssm_amd/libquick_ssm_hip.so, which is what quick_ssm_amd._lib loads.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
SRC_DIR = PKG_DIR / "csrc"
OBJ_DIR = SRC_DIR / "build"
LIB_PATH = PKG_DIR / "libquick_ssm_hip.so"
SOURCES = ("scan_fwd.hip", "scan_bwd.hip", "gates.hip", "rmsnorm.hip", "colsum.hip", "scan_api.hip")

# Packed-fp32 VALU forms are kept out of the generated code on purpose.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libquick_ssm_hip.so cannot be built")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("command failed: " + " ".join(cmd))
    noise = "packed-fp32-ops' is not a recognized feature"
    for line in (proc.stdout + proc.stderr).splitlines():
        if line.strip() and noise not in line:
            sys.stderr.write(line + "\n")


def build(verbose: bool = True, extra_flags: list[str] | None = None) -> Path:
    """Compile all HIP sources for gfx950 and link the C-ABI shared library."""
    hipcc = _hipcc()
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    flags = HIPCC_FLAGS + list(extra_flags or [])
    jobs = []
    for name in SOURCES:
        src = SRC_DIR / name
        obj = OBJ_DIR / (src.stem + ".o")
        jobs.append(([hipcc, *flags, "-c", str(src), "-o", str(obj)], obj))
    if verbose:
        print(f"[quick_ssm_amd.build] hipcc {' '.join(flags)}", flush=True)
    with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1)) as pool:
        list(pool.map(lambda job: _run(job[0]), jobs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *[str(o) for _, o in jobs]])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[quick_ssm_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build()
