"""Build the gfx950 C-ABI library ``sparse_amd/csrc/libsparse_hip.so`` with hipcc.

Run as ``python -m sparse_amd.build``.  hipcc cross-compiles without a GPU, so this runs
anywhere the ROCm toolchain is installed; the resulting ``.so`` is loaded by
``sparse_amd._lib`` and is never rebuilt implicitly at import time.
"""
from __future__ import annotations

import os
import re
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
    "swiglu_prefill_merged.hip",
    "ffn_tiled.hip",
    "ffn.hip",
    "combine.hip",
    "rs_predict.hip",
    "layout.hip",
    "mfma_probe.hip",
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


# Kernels whose pipelines wait for a *counted* number of vector-memory operations.  A register
# spill adds scratch loads and stores to that count, so a build in which one of these kernels
# uses scratch memory is refused.
NO_SCRATCH = {"swiglu_prefill.hip": ("prefill_ffn_kernel",),
              "swiglu_prefill_merged.hip": ("prefill_merged_kernel",)}
RESOURCE_REMARKS = "-Rpass-analysis=kernel-resource-usage"


def scratch_by_kernel(remarks: str) -> dict[str, int]:
    """``{mangled kernel name: scratch bytes per lane}`` from hipcc's resource-usage remarks."""
    out: dict[str, int] = {}
    name = None
    for line in remarks.splitlines():
        if "remark: Function Name:" in line:
            name = line.split("Function Name:", 1)[1].split("[", 1)[0].strip()
        elif "ScratchSize [bytes/lane]:" in line and name is not None:
            out[name] = int(line.split("ScratchSize [bytes/lane]:", 1)[1].split("[", 1)[0])
    return out


def check_no_scratch(source: str, remarks: str) -> None:
    wanted = NO_SCRATCH.get(source, ())
    if not wanted:
        return
    table = scratch_by_kernel(remarks)
    for kernel in wanted:
        hits = {n: b for n, b in table.items() if kernel in n}
        if not hits:
            raise RuntimeError(f"{source}: no resource remarks for {kernel}; cannot check its scratch use")
        bad = {n: b for n, b in hits.items() if b != 0}
        if bad:
            raise RuntimeError(f"{source}: {kernel} uses scratch memory {bad}; its counted waits assume none")


def lib_path() -> Path:
    return CSRC / LIB_NAME


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; the ROCm toolchain is required to build libsparse_hip.so")
    return exe


def _run(cmd: list[str]) -> str:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), proc.stdout, proc.stderr))
    # the host pass prints one "not a recognized feature" line per flag; drop those, and the
    # resource remarks (with the source excerpts clang prints under each of them)
    quiet = RESOURCE_REMARKS in cmd
    for line in proc.stderr.splitlines():
        if "packed-fp32-ops" in line or not line.strip():
            continue
        if quiet and ("remark:" in line or re.match(r"\s*\d*\s*\|", line)):
            continue
        print(line, file=sys.stderr)
    return proc.stderr


def build(verbose: bool = True, jobs: int | None = None) -> Path:
    hipcc = _hipcc()
    obj_dir = CSRC / "build"
    obj_dir.mkdir(exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)

    def compile_one(name: str) -> str:
        obj = obj_dir / (name + ".o")
        cmd = [hipcc, *HIP_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", "-c", str(CSRC / name), "-o", str(obj)]
        if name in NO_SCRATCH:
            cmd.insert(1, RESOURCE_REMARKS)
        if verbose:
            print("[sparse_amd.build] hipcc -c", name, flush=True)
        check_no_scratch(name, _run(cmd))
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
