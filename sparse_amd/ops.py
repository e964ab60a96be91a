"""Operator-level Python wrappers over the C ABI.

PyTorch supplies device memory (``Tensor.data_ptr()``) and the current HIP stream; all
arithmetic happens in ``libsparse_hip.so``.  Every wrapper takes its outputs and
workspaces from the caller (or allocates them with torch when ``None`` is passed) and
launches asynchronously on ``torch.cuda.current_stream()``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lru import LruTable
from ._lib import BF16, F16, F32, DECODE_MAX_TOKENS, Experts, SegList


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return BF16
    if dtype == torch.float16:
        return F16
    if dtype == torch.float32:
        return F32
    raise ValueError(f"unsupported dtype {dtype}: the MoE kernels take bfloat16, float16 or float32")


HALF_DTYPES = (torch.bfloat16, torch.float16)   # the 16-bit formats of the MFMA kernels


def _need_half(t: torch.Tensor, name: str) -> None:
    _need(t, name)
    if t.dtype not in HALF_DTYPES:
        raise ValueError(f"{name} must be bfloat16 or float16, got {t.dtype}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must be a device tensor")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


# --------------------------------------------------------------------------- router
def router_logits(x: torch.Tensor, wg: torch.Tensor, wsg: Optional[torch.Tensor] = None,
                  logits_dtype: Optional[torch.dtype] = None,
                  out: Optional[torch.Tensor] = None,
                  shared_gate_out: Optional[torch.Tensor] = None):
    """``gate(x)`` (and ``shared_expert_gate(x)`` when ``wsg`` is given)."""
    lib = _lib.load()
    T, H = x.shape
    E = wg.shape[0]
    _need(x, "x")
    _need(wg, "wg", x.dtype, (E, H))
    ldt = logits_dtype or x.dtype
    if out is None:
        out = torch.empty((T, E), device=x.device, dtype=ldt)
    _need(out, "logits", ldt, (T, E))
    if wsg is not None:
        _need(wsg, "wsg", x.dtype)
        if wsg.numel() != H:
            raise ValueError("wsg must hold H elements")
        if shared_gate_out is None:
            shared_gate_out = torch.empty((T,), device=x.device, dtype=x.dtype)
    rc = lib.sparse_hip_router_logits(_ptr(x), _ptr(wg), _ptr(wsg), dtype_code(x.dtype), dtype_code(ldt),
                                      T, H, E, _ptr(out), _ptr(shared_gate_out), _stream())
    _lib.check(rc, "sparse_hip_router_logits")
    return out, shared_gate_out


def gate_topk(logits: torch.Tensor, k: int, renorm: bool = False, out_dtype: Optional[torch.dtype] = None,
              topv: Optional[torch.Tensor] = None, topi: Optional[torch.Tensor] = None,
              n_group: int = 1, topk_group: int = 1, scale: float = 1.0,
              pseudo_logits: Optional[torch.Tensor] = None):
    """Fused softmax(fp32) + top-k: returns ``(topv [T,k] out_dtype, topi [T,k] int64)``.
    With ``n_group > 1`` only experts of the ``topk_group`` best groups keep their probability
    (DeepSeek-V2's group-limited selection); the others enter the top-k with 0.  ``scale`` (the
    gate's routed scaling factor) multiplies the weights in fp32 before they are rounded;
    ``pseudo_logits`` [T,E] fp32, if given, receives -inf except log(weight) at the selected experts."""
    lib = _lib.load()
    _need(logits, "logits")
    T, E = logits.shape
    odt = out_dtype or logits.dtype
    if topv is None:
        topv = torch.empty((T, k), device=logits.device, dtype=odt)
    if topi is None:
        topi = torch.empty((T, k), device=logits.device, dtype=torch.int64)
    _need(topv, "topv", odt, (T, k))
    _need(topi, "topi", torch.int64, (T, k))
    if pseudo_logits is not None:
        _need(pseudo_logits, "pseudo logits", torch.float32, (T, E))
    rc = lib.sparse_hip_gate_topk_scaled(_ptr(logits), dtype_code(logits.dtype), T, E, int(k), int(bool(renorm)),
                                         int(n_group), int(topk_group), float(scale), dtype_code(odt), _ptr(topv),
                                         _ptr(topi), _ptr(pseudo_logits), _stream())
    _lib.check(rc, "sparse_hip_gate_topk_scaled")
    return topv, topi


def pseudo_logits(topv: torch.Tensor, topi: torch.Tensor, num_experts: int, eps: float = 1e-12,
                  fill: float = float("-inf"), out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out [T,E]`` fp32 = ``fill`` except ``log(max(topv, eps))`` at ``topi`` (utils/eval_core.py:9490-9499,
    :11137-11155)."""
    lib = _lib.load()
    _need(topv, "topv")
    T, K = topv.shape
    _need(topi, "topi", torch.int64, (T, K))
    if out is None:
        out = torch.empty((T, int(num_experts)), device=topv.device, dtype=torch.float32)
    _need(out, "pseudo logits", torch.float32, (T, int(num_experts)))
    rc = lib.sparse_hip_pseudo_logits(_ptr(topv), dtype_code(topv.dtype), _ptr(topi), T, K, int(num_experts),
                                      float(eps), float(fill), _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_pseudo_logits")
    return out


def topk_values(values: torch.Tensor, k: int, renorm: bool = False, out_dtype: Optional[torch.dtype] = None,
                topv: Optional[torch.Tensor] = None, topi: Optional[torch.Tensor] = None):
    """Top-k of given fp32 probabilities (no softmax), descending, ties to the lower index:
    returns ``(topv [T,k] out_dtype, topi [T,k] int64)``."""
    lib = _lib.load()
    _need(values, "values", torch.float32)
    T, E = values.shape
    odt = out_dtype or torch.float32
    if topv is None:
        topv = torch.empty((T, k), device=values.device, dtype=odt)
    if topi is None:
        topi = torch.empty((T, k), device=values.device, dtype=torch.int64)
    _need(topv, "topv", odt, (T, k))
    _need(topi, "topi", torch.int64, (T, k))
    rc = lib.sparse_hip_topk(_ptr(values), T, E, int(k), int(bool(renorm)), dtype_code(odt), _ptr(topv), _ptr(topi),
                             _stream())
    _lib.check(rc, "sparse_hip_topk")
    return topv, topi


# --------------------------------------------------------------------------- permute
class Permutation:
    """Outputs of ``permute_build`` (all int32 device tensors)."""

    __slots__ = ("perm", "inv_perm", "seg_offsets", "active_eids", "n_active", "ws")

    def __init__(self, T: int, K: int, E: int, device) -> None:
        self.perm = torch.empty((T * K,), device=device, dtype=torch.int32)
        self.inv_perm = torch.empty((T * K,), device=device, dtype=torch.int32)
        self.seg_offsets = torch.empty((E + 1,), device=device, dtype=torch.int32)
        self.active_eids = torch.empty((E,), device=device, dtype=torch.int32)
        self.n_active = torch.empty((1,), device=device, dtype=torch.int32)
        nbytes = _lib.load().sparse_hip_permute_ws_bytes(T, K, E)
        self.ws = torch.empty((max(1, nbytes // 4),), device=device, dtype=torch.int32)


def permute_build(topi: torch.Tensor, num_experts: int, out: Optional[Permutation] = None) -> Permutation:
    lib = _lib.load()
    _need(topi, "topi", torch.int64)
    T, K = topi.shape
    if out is None:
        out = Permutation(T, K, num_experts, topi.device)
    rc = lib.sparse_hip_permute_build(_ptr(topi), T, K, int(num_experts), _ptr(out.perm), _ptr(out.inv_perm),
                                      _ptr(out.seg_offsets), _ptr(out.active_eids), _ptr(out.n_active),
                                      _ptr(out.ws), _stream())
    _lib.check(rc, "sparse_hip_permute_build")
    return out


def route_decode(x: torch.Tensor, wg: torch.Tensor, wsg: Optional[torch.Tensor], k: int, renorm: bool,
                 logits: torch.Tensor, shared_gate: Optional[torch.Tensor], topv: torch.Tensor,
                 topi: torch.Tensor, perm: Permutation, counter: torch.Tensor) -> None:
    """Router logits + top-k + permutation in one launch (T <= 32).  ``counter`` is a zeroed
    int32[1] the kernel uses to find its last workgroup and leaves at zero."""
    lib = _lib.load()
    T, H = x.shape
    E = wg.shape[0]
    _need(x, "x")
    _need(wg, "wg", x.dtype, (E, H))
    _need(logits, "logits", None, (T, E))
    _need(topv, "topv", x.dtype, (T, k))
    _need(topi, "topi", torch.int64, (T, k))
    _need(counter, "counter", torch.int32, (1,))
    if wsg is not None:
        _need(wsg, "wsg", x.dtype)
        _need(shared_gate, "shared gate logits", x.dtype, (T,))
    rc = lib.sparse_hip_route_decode(_ptr(x), _ptr(wg), _ptr(wsg), dtype_code(x.dtype), dtype_code(logits.dtype),
                                     T, H, E, int(k), int(bool(renorm)), _ptr(logits), _ptr(shared_gate),
                                     _ptr(topv), _ptr(topi), _ptr(perm.perm), _ptr(perm.inv_perm),
                                     _ptr(perm.seg_offsets), _ptr(perm.active_eids), _ptr(perm.n_active),
                                     _ptr(counter), _stream())
    _lib.check(rc, "sparse_hip_route_decode")


ROUTE_PACKED_MAX_TOKENS = 16
ROUTE_PACKED_ROWS = 64


def pack_router_gate(wg: torch.Tensor, wsg: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """The gate matrix ``route_decode_packed`` reads: 64 rows of the weights' 16-bit dtype (the E
    gate rows, then the shared-expert gate vector when there is one, then zeros) in the tiled
    weight layout, flattened.  ``None`` when the shapes do not fit (more than 64 rows, H not a
    multiple of 64, fp32): the caller then stays on ``route_decode``."""
    from .weights import tile_weight
    E, H = wg.shape
    rows = E + (1 if wsg is not None else 0)
    if wg.dtype not in HALF_DTYPES or H % 64 or rows > ROUTE_PACKED_ROWS:
        return None
    full = torch.zeros((ROUTE_PACKED_ROWS, H), dtype=wg.dtype, device=wg.device)
    full[:E] = wg
    if wsg is not None:
        full[E] = wsg.reshape(-1).to(wg.dtype)
    return tile_weight(full).contiguous()


def route_decode_packed(x: torch.Tensor, gate_packed: torch.Tensor, num_experts: int, has_shared_gate: bool, k: int,
                        renorm: bool, logits: torch.Tensor, shared_gate: Optional[torch.Tensor], topv: torch.Tensor,
                        topi: torch.Tensor, perm: Permutation, shared_up=None) -> None:
    """Router logits + top-k + permutation of up to 16 bf16 or fp16 tokens by one workgroup, on the
    matrix ``pack_router_gate`` made.  ``shared_up = (gate_w, up_w, inter_out)``: the same launch
    also computes the shared expert's SiLU(gate x) * (up x) into ``inter_out [T, Is]`` (tiled
    weights ``[Is, H]``, Is a multiple of 32), on the part of the device routing leaves idle."""
    lib = _lib.load()
    T, H = x.shape
    E = int(num_experts)
    _need_half(x, "x")
    _need(gate_packed, "packed gate", x.dtype, (ROUTE_PACKED_ROWS * H,))
    _need(logits, "logits", None, (T, E))
    _need(topv, "topv", x.dtype, (T, k))
    _need(topi, "topi", torch.int64, (T, k))
    if has_shared_gate:
        _need(shared_gate, "shared gate logits", x.dtype, (T,))
    common = (_ptr(x), _ptr(gate_packed), int(bool(has_shared_gate)), dtype_code(x.dtype), dtype_code(logits.dtype),
              T, H, E, int(k),
              int(bool(renorm)), _ptr(logits), _ptr(shared_gate), _ptr(topv), _ptr(topi), _ptr(perm.perm),
              _ptr(perm.inv_perm), _ptr(perm.seg_offsets), _ptr(perm.active_eids), _ptr(perm.n_active))
    if shared_up is None:
        _lib.check(lib.sparse_hip_route_decode_packed(*common, _stream()), "sparse_hip_route_decode_packed")
        return
    gw, uw, inter = shared_up
    Is = int(gw.shape[0])
    _need(gw, "shared gate_proj", x.dtype, (Is, H))
    _need(uw, "shared up_proj", x.dtype, (Is, H))
    _need(inter, "shared inter_ws", x.dtype, (T, Is))
    _lib.check(lib.sparse_hip_route_decode_packed_shared(*common, _ptr(gw), _ptr(uw), Is, _ptr(inter), _stream()),
               "sparse_hip_route_decode_packed_shared")


def shared_gate_up(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor, inter_out: torch.Tensor) -> None:
    """The shared expert's SiLU(gate x) * (up x) for up to 16 bf16 or fp16 tokens, by the kernel code
    ``route_decode_packed(shared_up=...)`` runs beside the routing (same bits)."""
    T, H = x.shape
    Is = int(gate_w.shape[0])
    _need_half(x, "x")
    _need(gate_w, "shared gate_proj", x.dtype, (Is, H))
    _need(up_w, "shared up_proj", x.dtype, (Is, H))
    _need(inter_out, "shared inter_ws", x.dtype, (T, Is))
    _lib.check(_lib.load().sparse_hip_shared_gate_up(_ptr(x), _ptr(gate_w), _ptr(up_w), dtype_code(x.dtype), T, H, Is,
                                                     _ptr(inter_out), _stream()), "sparse_hip_shared_gate_up")


# --------------------------------------------------------------------------- experts
def make_experts(slab: torch.Tensor, expert_slot: torch.Tensor, num_experts: int, hidden: int, inter: int,
                 slot_stride_bytes: Optional[int] = None) -> Experts:
    """Describe a weight slab ``[slots, 3*I*H]`` (gate | up | down per slot)."""
    _need(slab, "slab")
    _need(expert_slot, "expert_slot", torch.int32, (num_experts,))
    es = slab.element_size()
    stride = slot_stride_bytes if slot_stride_bytes is not None else 3 * hidden * inter * es
    return Experts(slab.data_ptr(), stride, expert_slot.data_ptr(), num_experts, hidden, inter,
                   dtype_code(slab.dtype))


def seglist_device(perm: Permutation, max_segments: int) -> SegList:
    """Segment list read on the device: the active experts in ascending id."""
    s = SegList()
    s.eids_dev = perm.active_eids.data_ptr()
    s.count_dev = perm.n_active.data_ptr()
    s.n = int(max_segments)
    return s


def seglist_host(eids: Sequence[int], slots: Optional[Sequence[int]] = None) -> SegList:
    """Segment list passed by value, in the given execution order; ``slots[i]`` is the slab
    slot holding ``eids[i]`` (default: slot == expert id)."""
    s = SegList()
    s.eids_dev = None
    s.count_dev = None
    s.n = len(eids)
    if s.n > _lib.MAX_EXPERTS:
        raise ValueError("too many segments")
    for i, e in enumerate(eids):
        s.eids[i] = int(e)
        s.slots[i] = int(e) if slots is None else int(slots[i])
    return s


def grouped_swiglu(experts: Experts, x: torch.Tensor, topv: torch.Tensor, perm: Permutation, segs: SegList,
                   inter_ws: torch.Tensor, parts: torch.Tensor, *, decode: Optional[bool] = None,
                   tile_ws: Optional[torch.Tensor] = None) -> None:
    """Routed-expert FFN over the segments in ``segs``; rows land in ``parts`` (permuted order)."""
    lib = _lib.load()
    T, H = x.shape
    K = topv.shape[1]
    _need(x, "x")
    _need(topv, "topv", x.dtype, (T, K))
    _need(inter_ws, "inter_ws", x.dtype, (T * K, experts.inter))
    _need(parts, "parts", x.dtype, (T * K, H))
    if H != experts.hidden:
        raise ValueError(f"x has hidden {H}, the expert slab has {experts.hidden}")
    use_decode = (T <= DECODE_MAX_TOKENS) if decode is None else bool(decode)
    if use_decode:
        rc = lib.sparse_hip_grouped_swiglu_decode(C.byref(experts), _ptr(x), _ptr(topv), _ptr(perm.perm),
                                                  _ptr(perm.seg_offsets), C.byref(segs), T, K, _ptr(inter_ws),
                                                  _ptr(parts), _stream())
        _lib.check(rc, "sparse_hip_grouped_swiglu_decode")
        return
    if tile_ws is None:
        tile_ws = prefill_tile_ws(T, K, experts.num_experts, H, experts.inter, x.device)
    rc = lib.sparse_hip_grouped_swiglu_prefill(C.byref(experts), _ptr(x), _ptr(topv), _ptr(perm.perm),
                                               _ptr(perm.seg_offsets), C.byref(segs), T, K, _ptr(inter_ws),
                                               _ptr(parts), _ptr(tile_ws), _stream())
    _lib.check(rc, "sparse_hip_grouped_swiglu_prefill")


_TILE_WS = LruTable.from_env("SPARSE_HIP_WORKSPACE_CACHE", 8)


def prefill_tile_ws(T: int, K: int, num_segments: int, hidden: int, inter: int, device) -> torch.Tensor:
    """Tile-map workspace of the prefill kernels, cached per shape (launches on one stream
    reuse it in order)."""
    def make() -> torch.Tensor:
        nbytes = _lib.load().sparse_hip_prefill_ws_bytes(T, K, num_segments, hidden, inter)
        return torch.empty((max(16, nbytes),), device=device, dtype=torch.uint8)

    return _TILE_WS.get_or_make((T, K, num_segments, hidden, inter, str(device)), make)


def shared_expert(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor,
                  shared_gate: Optional[torch.Tensor], inter_ws: torch.Tensor, out: torch.Tensor,
                  inter_ready: bool = False) -> None:
    """The shared expert.  ``inter_ready``: ``inter_ws`` already holds SiLU(gate x) * (up x)
    (bf16 calls of up to 32 tokens), only the down projection runs."""
    lib = _lib.load()
    T, H = x.shape
    Is = gate_w.shape[0]
    _need(x, "x")
    _need(gate_w, "shared gate_proj", x.dtype, (Is, H))
    _need(up_w, "shared up_proj", x.dtype, (Is, H))
    _need(down_w, "shared down_proj", x.dtype, (H, Is))
    _need(inter_ws, "shared inter_ws", x.dtype, (T, Is))
    _need(out, "shared out", x.dtype, (T, H))
    if shared_gate is not None:
        _need(shared_gate, "shared gate logits", x.dtype)
        if shared_gate.numel() != T:
            raise ValueError("shared gate logits must hold T elements")
    rc = lib.sparse_hip_shared_expert(_ptr(x), None if inter_ready else _ptr(gate_w),
                                      None if inter_ready else _ptr(up_w), _ptr(down_w), _ptr(shared_gate),
                                      dtype_code(x.dtype), T, H, Is, _ptr(inter_ws), _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_shared_expert")


def combine(parts: torch.Tensor, perm: Permutation, shared: Optional[torch.Tensor], T: int, K: int,
            out: torch.Tensor) -> None:
    lib = _lib.load()
    H = parts.shape[1]
    _need(parts, "parts", None, (T * K, H))
    _need(out, "out", parts.dtype, (T, H))
    if shared is not None:
        _need(shared, "shared", parts.dtype, (T, H))
    rc = lib.sparse_hip_combine(_ptr(parts), _ptr(perm.inv_perm), _ptr(shared), dtype_code(parts.dtype), T, K, H,
                                _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_combine")


def combine_split(parts: torch.Tensor, perm: Permutation, split_ws: torch.Tensor, nparts: int,
                  shared_gate: Optional[torch.Tensor], T: int, K: int, out: torch.Tensor) -> None:
    """``combine`` for a decode call whose shared down projection was left as ``nparts`` fp32
    partial sums in ``split_ws`` (``moe_ffn_decode(split_ws=...)``)."""
    lib = _lib.load()
    H = parts.shape[1]
    _need_half(parts, "parts")
    _need(parts, "parts", parts.dtype, (T * K, H))
    _need(out, "out", parts.dtype, (T, H))
    _need(split_ws, "split workspace", torch.float32)
    if split_ws.numel() < int(nparts) * T * H:
        raise ValueError("split workspace is too small for this T and H")
    if shared_gate is not None:
        _need(shared_gate, "shared gate logits", parts.dtype, (T,))
    rc = lib.sparse_hip_combine_split(_ptr(parts), _ptr(perm.inv_perm), _ptr(split_ws), int(nparts), _ptr(shared_gate),
                                      dtype_code(parts.dtype), T, K, H, _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_combine_split")


# --------------------------------------------------------------------------- residency
class Event:
    """A HIP event owned through the C ABI (no timing unless asked)."""

    def __init__(self, timing: bool = False) -> None:
        h = C.c_void_p()
        _lib.check(_lib.load().sparse_hip_event_create(int(timing), C.byref(h)), "sparse_hip_event_create")
        self.handle = h.value

    def record(self, stream: Optional[int] = None) -> None:
        _lib.check(_lib.load().sparse_hip_event_record(self.handle, _stream() if stream is None else stream),
                   "sparse_hip_event_record")

    def query(self) -> bool:
        rc = _lib.load().sparse_hip_event_query(self.handle)
        if rc == _lib.ENOTREADY:
            return False
        _lib.check(rc, "sparse_hip_event_query")
        return True

    def wait(self, stream: Optional[int] = None) -> None:
        """Make ``stream`` (default: torch's current stream) wait; the host does not block."""
        _lib.check(_lib.load().sparse_hip_stream_wait_event(_stream() if stream is None else stream, self.handle),
                   "sparse_hip_stream_wait_event")

    def elapsed_ms(self, end: "Event") -> float:
        ms = C.c_float()
        _lib.check(_lib.load().sparse_hip_event_elapsed_ms(self.handle, end.handle, C.byref(ms)),
                   "sparse_hip_event_elapsed_ms")
        return float(ms.value)

    def __del__(self) -> None:
        try:
            if self.handle:
                _lib.load().sparse_hip_event_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class SideStream:
    """A non-blocking HIP stream at the default priority, for expert uploads."""

    def __init__(self) -> None:
        h = C.c_void_p()
        _lib.check(_lib.load().sparse_hip_stream_create(C.byref(h)), "sparse_hip_stream_create")
        self.handle = h.value

    def synchronize(self) -> None:
        _lib.check(_lib.load().sparse_hip_stream_synchronize(self.handle), "sparse_hip_stream_synchronize")

    def __del__(self) -> None:
        try:
            if self.handle:
                _lib.load().sparse_hip_stream_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def expert_upload_async(dst_dev_ptr: int, src_host_ptr: int, nbytes: int, stream: int,
                        event: Optional[Event]) -> None:
    rc = _lib.load().sparse_hip_expert_upload_async(dst_dev_ptr, src_host_ptr, nbytes, stream,
                                                    None if event is None else event.handle)
    _lib.check(rc, "sparse_hip_expert_upload_async")


def host_alloc(nbytes: int) -> int:
    p = C.c_void_p()
    _lib.check(_lib.load().sparse_hip_host_alloc(nbytes, C.byref(p)), "sparse_hip_host_alloc")
    return p.value


def host_free(ptr: int) -> None:
    _lib.check(_lib.load().sparse_hip_host_free(ptr), "sparse_hip_host_free")


# --------------------------------------------------------------------------- measurement
def calib_copy(src: torch.Tensor, dst: torch.Tensor) -> None:
    """Plain device copy of a known size: the yardstick the hardware byte counters of a
    profiler run are scaled with."""
    _need(src, "src")
    _need(dst, "dst", src.dtype, tuple(src.shape))
    nbytes = src.numel() * src.element_size()
    _lib.check(_lib.load().sparse_hip_calib_copy(_ptr(src), _ptr(dst), nbytes, _stream()), "sparse_hip_calib_copy")


def profile_enable(on: bool) -> None:
    _lib.check(_lib.load().sparse_hip_profile_enable(int(bool(on))), "sparse_hip_profile_enable")


def profile_reset() -> None:
    _lib.check(_lib.load().sparse_hip_profile_reset(), "sparse_hip_profile_reset")


def profile_read() -> dict:
    """``{kernel: (total_ms, launches, device function name)}`` for every kernel id."""
    lib = _lib.load()
    out = {}
    for kid, name in enumerate(_lib.KERNELS):
        ms, n = C.c_double(), C.c_int64()
        _lib.check(lib.sparse_hip_profile_read(kid, C.byref(ms), C.byref(n)), "sparse_hip_profile_read")
        out[name] = (float(ms.value), int(n.value), lib.sparse_hip_kernel_name(kid).decode())
    return out


def rs_predict(x: torch.Tensor, w1: torch.Tensor, b1: torch.Tensor, w2: torch.Tensor, b2: torch.Tensor,
               hidden_ws: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Routing-scout forward pass: ``softmax(w2 relu(w1 x + b1) + b2)`` in fp32, with fp32 parameters
    whose BatchNorm is already folded into ``w1`` / ``b1``.  Returns ``pred [T, E]``."""
    T, H = x.shape
    D, E = w1.shape[0], w2.shape[0]
    _need(x, "x")
    _need(w1, "w1", torch.float32, (D, H))
    _need(b1, "b1", torch.float32, (D,))
    _need(w2, "w2", torch.float32, (E, D))
    _need(b2, "b2", torch.float32, (E,))
    if hidden_ws is None:
        hidden_ws = torch.empty((T, D), device=x.device, dtype=torch.float32)
    if out is None:
        out = torch.empty((T, E), device=x.device, dtype=torch.float32)
    _need(hidden_ws, "hidden workspace", torch.float32)
    _need(out, "pred", torch.float32, (T, E))
    if hidden_ws.numel() < T * D:
        raise ValueError("hidden workspace is too small")
    rc = _lib.load().sparse_hip_rs_predict(_ptr(x), dtype_code(x.dtype), T, H, _ptr(w1), _ptr(b1), D, _ptr(w2),
                                           _ptr(b2), E, _ptr(hidden_ws), _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_rs_predict")
    return out


RS_ACT = {"none": 0, "relu": 1, "gelu": 2}


def rs_dense(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, act: str = "none",
             residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``act(x w^T + b) (+ residual)`` in fp32: one Linear of a routing-scout predictor with the
    activation and the residual connection that follow it.  ``x [T, H]`` in any supported dtype, fp32
    parameters, fp32 result ``[T, D]``."""
    T, H = x.shape
    D = w.shape[0]
    _need(x, "x")
    _need(w, "w", torch.float32, (D, H))
    _need(b, "b", torch.float32, (D,))
    if residual is not None:
        _need(residual, "residual", torch.float32, (T, D))
    if out is None:
        out = torch.empty((T, D), device=x.device, dtype=torch.float32)
    _need(out, "out", torch.float32, (T, D))
    rc = _lib.load().sparse_hip_rs_dense(_ptr(x), dtype_code(x.dtype), T, H, _ptr(w), _ptr(b), D, RS_ACT[act],
                                         _ptr(residual) if residual is not None else None, _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_rs_dense")
    return out


def rs_layernorm(x: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor, eps: float, width: Optional[int] = None,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """LayerNorm over the first ``width`` columns of ``x [T, ld_in]`` (all of them by default) into fp32
    rows ``out [T, ld_out]`` (as wide as ``x`` by default); columns past ``width`` come out zero."""
    T, ld_in = x.shape
    H = ld_in if width is None else int(width)
    _need(x, "x")
    _need(gamma, "gamma", torch.float32, (H,))
    _need(beta, "beta", torch.float32, (H,))
    if out is None:
        out = torch.empty((T, ld_in), device=x.device, dtype=torch.float32)
    _need(out, "out", torch.float32)
    if out.dim() != 2 or out.shape[0] != T:
        raise ValueError("out must be [T, ld_out]")
    rc = _lib.load().sparse_hip_rs_layernorm(_ptr(x), dtype_code(x.dtype), T, H, ld_in, int(out.shape[1]),
                                             _ptr(gamma), _ptr(beta), float(eps), _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_rs_layernorm")
    return out


def rs_features(x: torch.Tensor, topi: torch.Tensor, topv: torch.Tensor, num_experts: int,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``[float(x) | routing weights rescaled to sum 1 at the chosen experts | zero padding]`` as fp32
    rows whose length is H + E rounded up to a multiple of 8: what a predictor of the
    ``hidden_router_topk`` kind reads."""
    T, H = x.shape
    K, E = int(topi.shape[1]), int(num_experts)
    ld = (H + E + 7) // 8 * 8
    _need(x, "x")
    _need(topi, "topi", torch.int64, (T, K))
    _need(topv, "topv", x.dtype, (T, K))
    if out is None:
        out = torch.empty((T, ld), device=x.device, dtype=torch.float32)
    _need(out, "out", torch.float32, (T, ld))
    rc = _lib.load().sparse_hip_rs_features(_ptr(x), dtype_code(x.dtype), T, H, _ptr(topi), _ptr(topv), K, E, ld,
                                            _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_rs_features")
    return out


def rs_softmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row softmax of fp32 ``logits [T, E]``."""
    T, E = logits.shape
    _need(logits, "logits", torch.float32)
    if out is None:
        out = torch.empty_like(logits)
    _need(out, "out", torch.float32, (T, E))
    rc = _lib.load().sparse_hip_rs_softmax(_ptr(logits), T, E, _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_rs_softmax")
    return out


def prefill_clock_probe(counters: Optional[torch.Tensor]) -> None:
    """Point the prefill-size FFN kernel's clock probe at ``counters`` (two int64 in device memory, which
    the caller zeroes: [0] collects shader-clock cycles, [1] ticks of the constant 100 MHz clock, summed
    over workgroups), or switch it off with ``None``.  A measurement aid; the reference has no such thing."""
    if counters is not None:
        _need(counters, "counters", torch.int64, (2,))
    _lib.check(_lib.load().sparse_hip_prefill_clock_probe(_ptr(counters)), "sparse_hip_prefill_clock_probe")


def prefill_shader_clock_mhz(counters: torch.Tensor) -> float:
    """Average shader clock of a busy compute unit over the launches the probe has seen."""
    cyc, ticks = (int(v) for v in counters.tolist())
    return 100.0 * cyc / ticks if ticks else 0.0


def mfma_probe(from_lds: bool, iters: int = 20000, device="cuda:0") -> Tuple[float, float]:
    """``(TFLOP/s, shader clock in MHz)`` of a loop of bf16 16x16x32 MFMAs on the prefill kernel's wavefront
    tile, eight wavefronts per compute unit, operands in registers or (``from_lds``) with the activation
    fragments read from LDS every k step.  A measurement aid; the reference has no such thing."""
    counters = torch.zeros(4, dtype=torch.int64, device=device)
    tflops, mhz = C.c_double(0.0), C.c_double(0.0)
    with torch.cuda.device(counters.device):
        _lib.check(_lib.load().sparse_hip_mfma_probe(int(bool(from_lds)), int(iters), _ptr(counters), C.byref(tflops),
                                                     C.byref(mhz), _stream()), "sparse_hip_mfma_probe")
    return float(tflops.value), float(mhz.value)


def moe_ffn_prefill(experts: Experts, x: torch.Tensor, topv: torch.Tensor, perm: Permutation, segs: SegList,
                    inter_ws: torch.Tensor, parts: torch.Tensor, shared_w=None,
                    shared_gate: Optional[torch.Tensor] = None, shared_inter_ws: Optional[torch.Tensor] = None,
                    shared_out: Optional[torch.Tensor] = None, tile_ws: Optional[torch.Tensor] = None) -> None:
    """Routed experts + shared expert of a prefill-size call as one launch per projection (bf16 or
    fp16): routed and shared tiles share the launches' tails.  ``shared_w`` None: routed experts only;
    an empty ``segs``: the shared expert only.  Bit-identical to ``grouped_swiglu`` + ``shared_expert``."""
    lib = _lib.load()
    T, H = x.shape
    K = topv.shape[1]
    _need_half(x, "x")
    _need(topv, "topv", x.dtype, (T, K))
    _need(inter_ws, "inter_ws", x.dtype, (T * K, experts.inter))
    _need(parts, "parts", x.dtype, (T * K, H))
    if H != experts.hidden:
        raise ValueError(f"x has hidden {H}, the expert slab has {experts.hidden}")
    Is = 0
    gw = uw = dw = None
    if shared_w is not None:
        gw, uw, dw = shared_w
        Is = gw.shape[0]
        _need(gw, "shared gate_proj", x.dtype, (Is, H))
        _need(uw, "shared up_proj", x.dtype, (Is, H))
        _need(dw, "shared down_proj", x.dtype, (H, Is))
        _need(shared_inter_ws, "shared inter_ws", x.dtype, (T, Is))
        _need(shared_out, "shared out", x.dtype, (T, H))
        if shared_gate is not None:
            _need(shared_gate, "shared gate logits", x.dtype)
            if shared_gate.numel() != T:
                raise ValueError("shared gate logits must hold T elements")
    if tile_ws is None:
        tile_ws = moe_ffn_prefill_ws(T, K, experts.num_experts, H, experts.inter, Is, x.device)
    rc = lib.sparse_hip_moe_ffn_prefill(C.byref(experts), _ptr(x), _ptr(topv), _ptr(perm.perm),
                                        _ptr(perm.seg_offsets), C.byref(segs), T, K, _ptr(inter_ws), _ptr(parts),
                                        _ptr(gw), _ptr(uw), _ptr(dw), _ptr(shared_gate), Is,
                                        _ptr(shared_inter_ws), _ptr(shared_out), _ptr(tile_ws), _stream())
    _lib.check(rc, "sparse_hip_moe_ffn_prefill")


def moe_ffn_prefill_ws(T: int, K: int, num_segments: int, hidden: int, inter: int, shared_inter: int,
                       device) -> torch.Tensor:
    """Tile-queue workspace of ``moe_ffn_prefill``, cached per shape (launches on one stream reuse it
    in order)."""
    def make() -> torch.Tensor:
        nbytes = _lib.load().sparse_hip_moe_ffn_prefill_ws_bytes(T, K, num_segments, hidden, inter, shared_inter)
        return torch.empty((max(256, nbytes),), device=device, dtype=torch.uint8)

    return _TILE_WS.get_or_make(("merged", T, K, num_segments, hidden, inter, shared_inter, str(device)), make)


def moe_ffn_decode(experts: Experts, x: torch.Tensor, topv: torch.Tensor, perm: Permutation, segs: SegList,
                   inter_ws: torch.Tensor, parts: torch.Tensor, shared_w, shared_gate: Optional[torch.Tensor],
                   shared_inter_ws: torch.Tensor, shared_out: torch.Tensor,
                   split_ws: Optional[torch.Tensor] = None, shared_inter_ready: bool = False) -> None:
    """Routed experts + shared expert of a decode call in one launch pair (bf16 or fp16, T <= 32).
    ``split_ws`` (from ``decode_split_workspace``) lets the shared down projection spread its
    long reduction over four workgroups per tile.  ``shared_inter_ready``: ``shared_inter_ws``
    already holds the shared expert's SiLU(gate x) * (up x) (``route_decode_packed`` computed it
    beside the routing), so its gate and up projections are not run again."""
    lib = _lib.load()
    T, H = x.shape
    K = topv.shape[1]
    gw, uw, dw = shared_w
    Is = gw.shape[0]
    _need_half(x, "x")
    _need(topv, "topv", x.dtype, (T, K))
    _need(inter_ws, "inter_ws", x.dtype, (T * K, experts.inter))
    _need(parts, "parts", x.dtype, (T * K, H))
    _need(gw, "shared gate_proj", x.dtype, (Is, H))
    _need(uw, "shared up_proj", x.dtype, (Is, H))
    _need(dw, "shared down_proj", x.dtype, (H, Is))
    _need(shared_inter_ws, "shared inter_ws", x.dtype, (T, Is))
    _need(shared_out, "shared out", x.dtype, (T, H))
    if split_ws is not None:
        _need(split_ws, "split workspace", torch.float32)
        if split_ws.numel() * 4 < int(lib.sparse_hip_decode_split_ws_bytes(T, H)):
            raise ValueError("split workspace is too small for this T and H")
    rc = lib.sparse_hip_moe_ffn_decode(C.byref(experts), _ptr(x), _ptr(topv), _ptr(perm.perm),
                                       _ptr(perm.seg_offsets), C.byref(segs), T, K, _ptr(inter_ws), _ptr(parts),
                                       None if shared_inter_ready else _ptr(gw),
                                       None if shared_inter_ready else _ptr(uw), _ptr(dw), _ptr(shared_gate), Is,
                                       _ptr(shared_inter_ws), _ptr(shared_out), _ptr(split_ws), _stream())
    _lib.check(rc, "sparse_hip_moe_ffn_decode")


def decode_split_workspace(T: int, H: int, device) -> torch.Tensor:
    """fp32 workspace for ``moe_ffn_decode(split_ws=...)``: the partial sums of the shared down
    projection, ``[parts, T, H]``, followed by the per-tile arrival counters of
    ``moe_ffn_decode_combine``, which start out (and are always left) at zero."""
    lib = _lib.load()
    n = int(lib.sparse_hip_decode_split_ws_bytes(int(T), int(H)))
    return torch.zeros((n + 3) // 4, dtype=torch.float32, device=device)


def moe_ffn_decode_combine(experts: Experts, x: torch.Tensor, topv: torch.Tensor, perm: Permutation, segs: SegList,
                           inter_ws: torch.Tensor, parts: torch.Tensor, shared_w, shared_gate: Optional[torch.Tensor],
                           shared_inter_ws: torch.Tensor, split_ws: torch.Tensor, out: torch.Tensor,
                           shared_inter_ready: bool = False) -> None:
    """``moe_ffn_decode`` with the combine step folded into the down projection's launch:
    writes the layer's expert output ``out [T,H]`` (routed sum + shared expert)."""
    lib = _lib.load()
    T, H = x.shape
    K = topv.shape[1]
    gw, uw, dw = shared_w
    Is = gw.shape[0]
    _need_half(x, "x")
    _need(topv, "topv", x.dtype, (T, K))
    _need(inter_ws, "inter_ws", x.dtype, (T * K, experts.inter))
    _need(parts, "parts", x.dtype, (T * K, H))
    _need(gw, "shared gate_proj", x.dtype, (Is, H))
    _need(uw, "shared up_proj", x.dtype, (Is, H))
    _need(dw, "shared down_proj", x.dtype, (H, Is))
    _need(shared_inter_ws, "shared inter_ws", x.dtype, (T, Is))
    _need(out, "out", x.dtype, (T, H))
    _need(split_ws, "split workspace", torch.float32)
    if split_ws.numel() * 4 < int(lib.sparse_hip_decode_split_ws_bytes(T, H)):
        raise ValueError("split workspace is too small for this T and H")
    rc = lib.sparse_hip_moe_ffn_decode_combine(
        C.byref(experts), _ptr(x), _ptr(topv), _ptr(perm.perm), _ptr(perm.inv_perm), _ptr(perm.seg_offsets),
        C.byref(segs), T, K, _ptr(inter_ws), _ptr(parts), None if shared_inter_ready else _ptr(gw),
        None if shared_inter_ready else _ptr(uw), _ptr(dw), _ptr(shared_gate), Is,
        _ptr(shared_inter_ws), _ptr(split_ws), _ptr(out), _stream())
    _lib.check(rc, "sparse_hip_moe_ffn_decode_combine")


def decode_split_parts(shared_inter: int) -> int:
    """Parts the fused decode call cuts the shared down projection into when it is given a
    workspace (1: it is not cut and ``shared_out`` is written as usual)."""
    return int(_lib.load().sparse_hip_decode_split_parts(int(shared_inter)))
