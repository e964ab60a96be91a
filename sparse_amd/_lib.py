"""ctypes binding of ``libsparse_hip.so`` (the C ABI declared in ``include/sparse_hip.h``).

The library is loaded from ``sparse_amd/csrc/``; it is never built here.  A missing
library raises ``SparseHipMissing`` -- there is no CPU fallback behind these entry points.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "csrc" / "libsparse_hip.so"

F32 = 0
BF16 = 1
F16 = 2
MAX_EXPERTS = 256
MAX_TOPK = 16
DECODE_MAX_TOKENS = 32
ENOTREADY = 1
ABI_VERSION = 3
PERMUTE_STATIC_MAX_TOKENS = 65536


class SparseHipMissing(RuntimeError):
    """libsparse_hip.so has not been built (run ``python -m sparse_amd.build``)."""


class SparseHipError(RuntimeError):
    """A C-ABI call returned a failure code."""


class Experts(C.Structure):
    """``sparse_hip_experts``."""

    _fields_ = [
        ("slab_dev", C.c_void_p),
        ("slot_stride", C.c_uint64),
        ("expert_slot_dev", C.c_void_p),
        ("num_experts", C.c_int32),
        ("hidden", C.c_int32),
        ("inter", C.c_int32),
        ("dtype", C.c_int32),
    ]


class SegList(C.Structure):
    """``sparse_hip_seglist``."""

    _fields_ = [
        ("eids_dev", C.c_void_p),
        ("count_dev", C.c_void_p),
        ("n", C.c_int32),
        ("eids", C.c_int16 * MAX_EXPERTS),
        ("slots", C.c_int16 * MAX_EXPERTS),
    ]


_vp, _i, _sz = C.c_void_p, C.c_int, C.c_size_t

# name -> (restype, argtypes); every symbol include/sparse_hip.h declares
SIGNATURES = {
    "sparse_hip_version": (_i, []),
    "sparse_hip_arch": (C.c_char_p, []),
    "sparse_hip_last_error": (C.c_char_p, []),
    "sparse_hip_router_logits": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "sparse_hip_gate_topk": (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "sparse_hip_gate_topk_grouped": (_i, [_vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "sparse_hip_gate_topk_scaled": (_i, [_vp, _i, _i, _i, _i, _i, _i, _i, C.c_float, _i, _vp, _vp, _vp, _vp]),
    "sparse_hip_pseudo_logits": (_i, [_vp, _i, _vp, _i, _i, _i, C.c_float, C.c_float, _vp, _vp]),
    "sparse_hip_topk": (_i, [_vp, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "sparse_hip_route_decode": (
        _i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "sparse_hip_route_decode_packed": (
        _i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "sparse_hip_route_decode_packed_shared": (
        _i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i,
             _vp, _vp]),
    "sparse_hip_shared_gate_up": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "sparse_hip_permute_ws_bytes": (_sz, [_i, _i, _i]),
    "sparse_hip_permute_build": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "sparse_hip_permute_build_static": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "sparse_hip_grouped_swiglu_decode": (
        _i, [C.POINTER(Experts), _vp, _vp, _vp, _vp, C.POINTER(SegList), _i, _i, _vp, _vp, _vp]),
    "sparse_hip_prefill_ws_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "sparse_hip_grouped_swiglu_prefill": (
        _i, [C.POINTER(Experts), _vp, _vp, _vp, _vp, C.POINTER(SegList), _i, _i, _vp, _vp, _vp, _vp]),
    "sparse_hip_moe_ffn_prefill_ws_bytes": (_sz, [_i, _i, _i, _i, _i, _i]),
    "sparse_hip_moe_ffn_prefill": (
        _i, [C.POINTER(Experts), _vp, _vp, _vp, _vp, C.POINTER(SegList), _i, _i, _vp, _vp,
             _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp]),
    "sparse_hip_moe_ffn_decode": (
        _i, [C.POINTER(Experts), _vp, _vp, _vp, _vp, C.POINTER(SegList), _i, _i, _vp, _vp,
             _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp]),
    "sparse_hip_moe_ffn_decode_combine": (
        _i, [C.POINTER(Experts), _vp, _vp, _vp, _vp, _vp, C.POINTER(SegList), _i, _i, _vp, _vp,
             _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp]),
    "sparse_hip_decode_split_counter_offset": (_sz, [_i, _i]),
    "sparse_hip_decode_split_ws_bytes": (_sz, [_i, _i]),
    "sparse_hip_decode_split_parts": (_i, [_i]),
    "sparse_hip_combine_split": (_i, [_vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _vp, _vp]),
    "sparse_hip_shared_expert": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "sparse_hip_combine": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "sparse_hip_expert_upload_async": (_i, [_vp, _vp, _sz, _vp, _vp]),
    "sparse_hip_event_create": (_i, [_i, C.POINTER(_vp)]),
    "sparse_hip_event_destroy": (_i, [_vp]),
    "sparse_hip_event_record": (_i, [_vp, _vp]),
    "sparse_hip_event_query": (_i, [_vp]),
    "sparse_hip_stream_wait_event": (_i, [_vp, _vp]),
    "sparse_hip_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(C.c_float)]),
    "sparse_hip_stream_create": (_i, [C.POINTER(_vp)]),
    "sparse_hip_stream_destroy": (_i, [_vp]),
    "sparse_hip_stream_synchronize": (_i, [_vp]),
    "sparse_hip_host_alloc": (_i, [_sz, C.POINTER(_vp)]),
    "sparse_hip_host_free": (_i, [_vp]),
    "sparse_hip_tile_weight": (_i, [_vp, _vp, _i, _i, _i, _i, _vp]),
    "sparse_hip_calib_copy": (_i, [_vp, _vp, _sz, _vp]),
    "sparse_hip_rs_predict": (_i, [_vp, _i, _i, _i, _vp, _vp, _i, _vp, _vp, _i, _vp, _vp, _vp]),
    "sparse_hip_rs_dense": (_i, [_vp, _i, _i, _i, _vp, _vp, _i, _i, _vp, _vp, _vp]),
    "sparse_hip_rs_layernorm": (_i, [_vp, _i, _i, _i, _i, _i, _vp, _vp, C.c_float, _vp, _vp]),
    "sparse_hip_rs_features": (_i, [_vp, _i, _i, _i, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "sparse_hip_rs_softmax": (_i, [_vp, _i, _i, _vp, _vp]),
    "sparse_hip_prefill_drain_waits": (_i, [_i]),
    "sparse_hip_prefill_clock_probe": (_i, [_vp]),
    "sparse_hip_mfma_probe": (_i, [_i, _i, _vp, C.POINTER(C.c_double), C.POINTER(C.c_double), _vp]),
    "sparse_hip_profile_enable": (_i, [_i]),
    "sparse_hip_profile_reset": (_i, []),
    "sparse_hip_profile_read": (_i, [_i, C.POINTER(C.c_double), C.POINTER(C.c_int64)]),
    "sparse_hip_kernel_name": (C.c_char_p, [_i]),
}

KERNELS = ("router_logits", "gate_topk", "permute", "decode_gateup", "decode_down", "prefill_gateup",
           "prefill_down", "tiled_gateup", "tiled_down", "combine", "route_decode")

_lib = None


def load() -> C.CDLL:
    """Load the library once and bind every declared symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise SparseHipMissing(
            f"{LIB_PATH} not found: build it with `python -m sparse_amd.build` "
            "(hipcc --offload-arch=gfx950); there is no CPU fallback for the MoE kernels")
    lib = C.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means the .so is stale
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.sparse_hip_version()
    if got != ABI_VERSION:
        raise SparseHipError(f"libsparse_hip.so has ABI version {got}, the binding expects {ABI_VERSION}")
    _lib = lib
    return lib


def last_error() -> str:
    return load().sparse_hip_last_error().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    """Raise the Python exception that matches a failure code (ValueError for a bad
    argument, RuntimeError for a HIP failure), as the reference raises from Python."""
    if rc == 0:
        return
    msg = f"{what}: {last_error()} (code {rc})"
    if rc == -1:
        raise ValueError(msg)
    raise SparseHipError(msg)
