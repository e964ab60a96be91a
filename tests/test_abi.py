"""The C-ABI library loads and exports every symbol ``include/sparse_hip.h`` declares.
No compute calls here: this runs without a GPU."""
import ctypes
import re
from pathlib import Path

import pytest

from sparse_amd import _lib

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "sparse_hip.h"


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(sparse_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("sparse_hip_gate_topk", "sparse_hip_permute_build", "sparse_hip_grouped_swiglu_decode",
                 "sparse_hip_grouped_swiglu_prefill", "sparse_hip_combine", "sparse_hip_shared_expert",
                 "sparse_hip_expert_upload_async", "sparse_hip_event_query", "sparse_hip_stream_wait_event",
                 "sparse_hip_version", "sparse_hip_arch"):
        assert must in names


def test_library_exports_every_declared_symbol():
    assert _lib.LIB_PATH.exists(), "build with `python -m sparse_amd.build` first"
    raw = ctypes.CDLL(str(_lib.LIB_PATH))
    missing = [n for n in declared_symbols() if not hasattr(raw, n)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_binding_covers_every_declared_symbol():
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_identity_and_error_channel():
    lib = _lib.load()
    assert lib.sparse_hip_version() == _lib.ABI_VERSION
    assert lib.sparse_hip_arch() == b"gfx950"
    # argument validation happens before any HIP call, so it works without a GPU
    rc = lib.sparse_hip_gate_topk(None, 0, 4, 300, 4, 0, 0, None, None, None)
    assert rc == -1
    assert b"gate_topk" in lib.sparse_hip_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc, "sparse_hip_gate_topk")
    assert lib.sparse_hip_permute_ws_bytes(4096, 6, 64) == 16 * 64 * 4
    assert lib.sparse_hip_permute_ws_bytes(8, 4, 60) == 60 * 4


def test_struct_layouts_match_the_header():
    # sparse_hip_experts: ptr, u64, ptr, 4 x i32 ; sparse_hip_seglist: 2 ptr, i32, 256 x i16
    assert ctypes.sizeof(_lib.Experts) == 8 + 8 + 8 + 16
    assert ctypes.sizeof(_lib.SegList) == 8 + 8 + 4 + 2 * 256 + 2 * 256 + 4  # tail padding to 8


def test_documented_ctypes_binding_is_current():
    """The binding shown to the reference's maintainers compiles as Python, names the library's current ABI
    version and calls only symbols the header declares (the GPU suite executes it)."""
    text = (ROOT / "INTEGRATION.md").read_text()
    block = re.search(r"```python\n(.*?)```", text[text.index("## Seam 2"):], re.S).group(1)
    compile(block, "INTEGRATION.md:seam-2", "exec")
    assert f"sparse_hip_version() == {_lib.ABI_VERSION}" in block
    assert f"ABI version {_lib.ABI_VERSION}" in text
    header_text = HEADER.read_text()
    assert f"#define SPARSE_HIP_ABI_VERSION {_lib.ABI_VERSION}" in header_text
    used = set(re.findall(r"_lib\.(sparse_hip_[a-z0-9_]+)", block)) | set(re.findall(r'"(sparse_hip_[a-z0-9_]+)"', block))
    assert used and used <= set(declared_symbols()), sorted(used - set(declared_symbols()))
    # struct mirrors in the block have the library's layout
    ns = {}
    exec(re.search(r"class Experts.*?\n\n", block, re.S).group(0), {"C": ctypes}, ns)
    exec(re.search(r"class SegList.*?\n\n", block, re.S).group(0), {"C": ctypes}, ns)
    assert ctypes.sizeof(ns["Experts"]) == ctypes.sizeof(_lib.Experts)
    assert ctypes.sizeof(ns["SegList"]) == ctypes.sizeof(_lib.SegList)
