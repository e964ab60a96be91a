"""Process-wide state the MoE blocks share, and the counters they report.

``SparseContext`` keeps the subset of the reference's class-level registry
(utils/eval_core.py:2349-3375) that the layer path reads: the phase / call-id protocol a
decode loop drives (:2394-2395, :3259-3263), the layer registry through which layer *l*
reaches layer *l+1*'s cache (:2768-2770, :10940), the RS predictor bank (:5209-5213) and
the routing cache.  ``Metrics`` is the subset of the reference's counters (:1688-2347)
that the cache / prefetch / EPIPE machinery updates.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

import torch


@dataclass
class DistEnv:
    """``DistEnv(rank, world, local_rank, device)`` (reference :140-145).  One GPU: world 1."""

    rank: int = 0
    world: int = 1
    local_rank: int = 0
    device: torch.device = torch.device("cuda:0")


@dataclass
class Metrics:
    cache_hit_count: int = 0
    prefetch_hit_count: int = 0
    cache_miss_count: int = 0
    demand_h2d_bytes: int = 0
    prefetch_h2d_bytes: int = 0
    prefetch_issued_count: int = 0
    prefetch_admitted_count: int = 0
    prefetch_wasted_count: int = 0
    prefetch_completed_count: int = 0
    prefetch_complete_before_use_count: int = 0
    prefetch_budget_zero_count: int = 0
    prefetch_budget_positive_count: int = 0
    rs_next_layer_pred_calls: int = 0
    rs_mlp_calls: int = 0
    # device time of the three segments of a layer call, accumulated while
    # SPARSE_EXPERT_TIMING=1 (utils/eval_core.py:1837-1840, :14655-14676)
    moe_router_ms: float = 0.0
    moe_expert_ms: float = 0.0
    moe_shared_ms: float = 0.0
    moe_timing_calls: int = 0
    # ms the compute lane spent in demand copies during decode (reference :1764-1766): filled from the
    # timed copies by `harvest_timings`; the RS executors' demand stage reads it against
    # SPARSE_EPIPE_RS_DEMAND_STAGE_THRESHOLD_MS
    demand_h2d_exposed_decode_ms: float = 0.0
    sampled_demand_h2d_exposed_decode_ms: float = 0.0
    counters: Dict[str, float] = field(default_factory=dict)
    # (kind, layer, expert) in issue order: kind in hit | prefetch_hit | miss
    events: Optional[List[Tuple[str, int, int]]] = None
    # when set, every expert upload is bracketed by a timing event pair on its lane
    time_copies: bool = False
    # deferred timing: (start_event, end_event, tag, layer[, stage])
    pending_events: List[Tuple[Any, ...]] = field(default_factory=list)
    timings_ms: Dict[str, float] = field(default_factory=dict)
    timings_n: Dict[str, int] = field(default_factory=dict)

    def bump(self, name: str, value: float = 1) -> None:
        self.counters[name] = self.counters.get(name, 0) + value

    def hit_rate(self) -> float:
        total = self.cache_hit_count + self.prefetch_hit_count + self.cache_miss_count
        return (self.cache_hit_count + self.prefetch_hit_count) / total if total else 0.0

    def harvest_timings(self) -> Dict[str, float]:
        """Read deferred event pairs (call after a device synchronisation)."""
        for start, end, tag, _layer, *rest in self.pending_events:
            ms = start.elapsed_ms(end)
            self.timings_ms[tag] = self.timings_ms.get(tag, 0.0) + ms
            self.timings_n[tag] = self.timings_n.get(tag, 0) + 1
            if tag == "compute_h2d_ms" and rest and rest[0] == "decode":
                self.demand_h2d_exposed_decode_ms += ms
        self.pending_events.clear()
        return self.timings_ms


class SparseContext:
    """Class-level registry; a harness sets ``current_phase`` and calls
    ``begin_runtime_call`` before every pass over the layer stack."""

    layer_blocks: Dict[int, Any] = {}
    current_phase: str = "none"          # "prefill" | "decode" | "none"
    runtime_call_id: int = -1
    current_moe_layer_idx: int = -1
    rs_bank: Optional[List[Any]] = None   # rs_bank[l] predicts layer l from layer l-1's input
    rs_bank_layout: str = "next_layer"
    rs_bank_source_layers: List[int] = []
    routing_cache: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
    prefill_scp_transient_demoted_for_decode: bool = False
    staging: Optional[Any] = None          # forecast staging engine (sparse_amd.staging.BoundedRS) while installed

    @classmethod
    def register_layer_block(cls, layer_idx: int, block: Any) -> None:
        cls.layer_blocks[int(layer_idx)] = block

    @classmethod
    def begin_runtime_call(cls, call_id: int) -> None:
        cls.runtime_call_id = int(call_id)
        cls.routing_cache = {}

    @classmethod
    def set_rs_bank(cls, modules: List[Any], source_layers: Optional[List[int]] = None) -> None:
        """``modules[l]`` (or None) is the predictor of layer l's experts from the input of
        layer ``source_layers[l]`` (default l-1; a layer only prefetches for the next one
        when that entry names it)."""
        cls.rs_bank = list(modules)
        cls.rs_bank_layout = "next_layer"
        cls.rs_bank_source_layers = (
            [int(s) for s in source_layers] if source_layers is not None else [l - 1 for l in range(len(modules))])

    @classmethod
    def finalize_prefetch_all(cls) -> None:
        """Count the last prefetch cycle of every layer (reference :3055-3061)."""
        for blk in cls.layer_blocks.values():
            blk._finalize_prev_group_prefetch()

    @classmethod
    def reset(cls) -> None:
        cls.layer_blocks = {}
        cls.current_phase = "none"
        cls.runtime_call_id = -1
        cls.current_moe_layer_idx = -1
        cls.rs_bank = None
        cls.rs_bank_layout = "next_layer"
        cls.rs_bank_source_layers = []
        cls.routing_cache = {}
        cls.prefill_scp_transient_demoted_for_decode = False
        cls.staging = None
