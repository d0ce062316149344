"""Build libsyncopate_hip.so (gfx950) in-tree with hipcc.

    python -m syncopate_amd.build            # compile every csrc/*.hip and link

hipcc cross-compiles for gfx950 without a GPU.  The library is linked without
an rpath to a ROCm tree: at run time ``syncopate_amd._lib`` imports torch first,
so the HIP runtime torch already loaded (same soname) is the one the kernels
launch on and torch's stream handles are valid in it.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB_NAME = "libsyncopate_hip.so"
LIB_PATH = CSRC / LIB_NAME
ARCH = "gfx950"

# -packed-fp32-ops is off: hipcc must not form v_pk_*_f32 from scalar float code.
DEVICE_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build libsyncopate_hip.so")
    return exe


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass of hipcc does not know the AMDGPU target feature and says so
    err = "\n".join(
        line for line in proc.stderr.splitlines() if "packed-fp32-ops" not in line
    )
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        print(err, file=sys.stderr)


def build_library(jobs: int = 4, verbose: bool = True) -> Path:
    """Compile all HIP sources and link the shared library; always recompiles."""
    hipcc = _hipcc()
    obj_dir = CSRC / "build"
    obj_dir.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC}")

    def compile_one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        _run([hipcc, *DEVICE_FLAGS, "-c", str(src), "-o", str(obj)])
        if verbose:
            print(f"[syncopate_amd.build] compiled {src.name}")
        return obj

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        objs = list(pool.map(compile_one, srcs))

    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[syncopate_amd.build] linked {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
