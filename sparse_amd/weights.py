"""Expert weight storage: HBM slot slab and pinned-host arena.

One slot holds one routed expert as three matrices back to back,
``gate [I,H] | up [I,H] | down [H,I]`` (the module layout of the reference,
utils/eval_core.py:5115-5123, made contiguous so that one expert is one H2D copy), each
stored in the kernels' tiled order (``tile_weight``) so that weight streaming is a run of
contiguous wave loads.
All-resident layers use ``E`` slots with the identity slot table; cached layers use
``capacity (+ staging)`` slots and rewrite ``expert_slot`` as experts move.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence, Tuple

import torch

from . import ops

ExpertWeights = Tuple[torch.Tensor, torch.Tensor, torch.Tensor]


def expert_numel(hidden: int, inter: int) -> int:
    return 3 * hidden * inter


def tile_weight(w: torch.Tensor) -> torch.Tensor:
    """Row-major ``[R, K]`` -> the library's tiled layout, flattened (R % 16 == 0, K % 64 == 0).

    Element (row, k) goes to ``(row//16)*16*K + (k//64)*1024 + ((k//8)%2)*512 +
    ((k//16)%4)*128 + (row%16)*8 + k%8``: per 16-row group and 64-wide k block, the
    order is (8-k half, k quarter, row, k within 8)."""
    R, K = w.shape
    if R % 16 or K % 64:
        raise ValueError(f"tiled weights need rows % 16 == 0 and cols % 64 == 0, got {tuple(w.shape)}")
    v = w.reshape(R // 16, 16, K // 64, 4, 2, 8)       # [group, row, block, quarter, half, k8]
    return v.permute(0, 2, 4, 3, 1, 5).reshape(-1)      # [group, block, half, quarter, row, k8]


def untile_weight(flat: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    """Inverse of ``tile_weight``."""
    v = flat.reshape(rows // 16, cols // 64, 2, 4, 16, 8)
    return v.permute(0, 4, 1, 3, 2, 5).reshape(rows, cols)


def pack_expert_into(dst_row: torch.Tensor, weights: ExpertWeights, hidden: int, inter: int) -> None:
    """Copy (gate, up, down), each tiled, into one flat slot row."""
    gw, uw, dw = weights
    if tuple(gw.shape) != (inter, hidden) or tuple(uw.shape) != (inter, hidden) or tuple(dw.shape) != (hidden, inter):
        raise ValueError(
            f"expert weights must be gate/up [{inter},{hidden}] and down [{hidden},{inter}], got "
            f"{tuple(gw.shape)}, {tuple(uw.shape)}, {tuple(dw.shape)}")
    n = hidden * inter
    dst_row[0:n].copy_(tile_weight(gw))
    dst_row[n:2 * n].copy_(tile_weight(uw))
    dst_row[2 * n:3 * n].copy_(tile_weight(dw))


class HostExpertArena:
    """All routed experts of a layer in pinned host memory, one row per expert id."""

    def __init__(self, experts: Sequence[ExpertWeights], hidden: int, inter: int, dtype: torch.dtype,
                 pin: bool = True) -> None:
        self.hidden, self.inter, self.dtype = hidden, inter, dtype
        self.num_experts = len(experts)
        numel = expert_numel(hidden, inter)
        self._pinned_ptr = None
        if pin:
            # hipHostMalloc of the exact size: torch's pinned allocator rounds every block up
            # to a power of two, which nearly doubles a 1.1 GB layer
            esize = torch.empty((), dtype=dtype).element_size()
            nbytes = self.num_experts * numel * esize
            self._pinned_ptr = ops.host_alloc(nbytes)
            buf = (ctypes.c_uint8 * nbytes).from_address(self._pinned_ptr)
            self.rows = torch.frombuffer(buf, dtype=torch.uint8).view(dtype).view(self.num_experts, numel)
        else:
            self.rows = torch.empty((self.num_experts, numel), dtype=dtype)
        for e, w in enumerate(experts):
            pack_expert_into(self.rows[e], tuple(t.to(dtype) for t in w), hidden, inter)
        self.expert_bytes = self.rows[0].numel() * self.rows.element_size()

    def __del__(self) -> None:
        ptr, self._pinned_ptr = getattr(self, "_pinned_ptr", None), None
        if ptr:
            self.rows = None
            try:
                ops.host_free(ptr)
            except Exception:
                pass

    def host_ptr(self, eid: int) -> int:
        return self.rows[eid].data_ptr()


class ExpertSlab:
    """``num_slots`` expert slots in HBM plus the device-side expert -> slot table."""

    def __init__(self, num_slots: int, num_experts: int, hidden: int, inter: int, dtype: torch.dtype,
                 device: torch.device) -> None:
        self.hidden, self.inter, self.dtype = hidden, inter, dtype
        self.num_slots, self.num_experts = num_slots, num_experts
        self.data = torch.empty((num_slots, expert_numel(hidden, inter)), dtype=dtype, device=device)
        self.expert_bytes = self.data[0].numel() * self.data.element_size()
        # host mirror of the table; pushed to the device whenever it changes
        self.slot_of = [-1] * num_experts
        self.expert_slot = torch.zeros((num_experts,), dtype=torch.int32, device=device)

    @classmethod
    def resident(cls, experts: Sequence[ExpertWeights], hidden: int, inter: int, dtype: torch.dtype,
                 device: torch.device) -> "ExpertSlab":
        """All experts resident, slot == expert id."""
        slab = cls(len(experts), len(experts), hidden, inter, dtype, device)
        for e, w in enumerate(experts):
            pack_expert_into(slab.data[e], tuple(t.detach() for t in w), hidden, inter)
            slab.slot_of[e] = e
        slab.push_table()
        return slab

    def slot_ptr(self, slot: int) -> int:
        return self.data.data_ptr() + slot * self.expert_bytes

    def push_table(self) -> None:
        table = torch.tensor([max(0, s) for s in self.slot_of], dtype=torch.int32)
        self.expert_slot.copy_(table)
