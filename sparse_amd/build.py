"""Build the gfx950 C-ABI library ``sparse_amd/csrc/libsparse_hip.so`` with hipcc.

Run as ``python -m sparse_amd.build``.  hipcc cross-compiles without a GPU, so this runs
anywhere the ROCm toolchain is installed; the resulting ``.so`` is loaded by
``sparse_amd._lib`` and is never rebuilt implicitly at import time.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"
LIB_NAME = "libsparse_hip.so"
ARCH = "gfx950"

SOURCES = [
    "runtime.hip",
    "router.hip",
    "permute.hip",
    "swiglu_decode.hip",
    "swiglu_prefill.hip",
    "ffn_tiled.hip",
    "ffn.hip",
    "combine.hip",
    "layout.hip",
]

# Packed-fp32 VALU ops are switched off for the device pass; the host pass does not know
# the feature and says so, which is harmless.
HIP_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def lib_path() -> Path:
    return CSRC / LIB_NAME


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; the ROCm toolchain is required to build libsparse_hip.so")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), proc.stdout, proc.stderr))
    # the host pass prints one "not a recognized feature" line per flag; drop those
    for line in proc.stderr.splitlines():
        if "packed-fp32-ops" in line or not line.strip():
            continue
        print(line, file=sys.stderr)


def build(verbose: bool = True, jobs: int | None = None) -> Path:
    hipcc = _hipcc()
    obj_dir = CSRC / "build"
    obj_dir.mkdir(exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)

    def compile_one(name: str) -> str:
        obj = obj_dir / (name + ".o")
        cmd = [hipcc, *HIP_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", "-c", str(CSRC / name), "-o", str(obj)]
        if verbose:
            print("[sparse_amd.build] hipcc -c", name, flush=True)
        _run(cmd)
        return str(obj)

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    out = lib_path()
    tmp = out.with_suffix(".so.tmp")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", str(tmp)])
    os.replace(tmp, out)
    if verbose:
        print("[sparse_amd.build] wrote", out, flush=True)
    return out


if __name__ == "__main__":
    build()
