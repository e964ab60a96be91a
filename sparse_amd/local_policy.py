"""Cost-aware local readiness policy (the reference's ``utils/lightweight_policy.py``).

A per-layer helper, fed with explicit cost estimates, that bends two decisions of the
offloaded path without any device work or communication:

* prefetch scoring -- a candidate that is not resident is discounted by the share of its
  copy time that already fits under compute the layer is known to have available, so the
  budget goes to experts whose load would otherwise be exposed
  (hooked where the reference hooks it, utils/eval_core.py:10428-10430, :10993-10996);
* the residual choice of the RS residual scan -- among late prefetches and stageable
  misses pick the one whose copy overlaps most with the ready experts' compute, or none
  when the overlap is not worth the split (:12320-12348).

``CostProfile`` reads the reference's JSON schema (version 1: ``rank_defaults`` plus optional
per-rank and per-layer overrides of the six cost fields).  ``measure_costs`` fills such a
profile from measurements on the running MI355X.
"""
from __future__ import annotations

import hashlib
import json
import math
import time
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Dict, Iterable, List, Mapping, Optional, Sequence, Set, Tuple

COST_FIELDS = ("h2d_bytes_per_ms", "h2d_latency_ms", "expert_ms", "item_ms", "next_attention_ms",
               "split_overhead_ms")


@dataclass(frozen=True)
class Costs:
    bandwidth: float      # host-to-device bytes per millisecond
    latency: float        # fixed cost of one copy, ms
    expert: float         # compute per routed expert (group), ms
    item: float           # compute per routed row, ms
    attention: float      # the next layer's attention, ms (time a prefetch may hide behind)
    split: float          # overhead of splitting a call around a residual, ms

    @classmethod
    def from_dict(cls, values: Mapping[str, Any]) -> "Costs":
        numbers = [float(values[name]) for name in COST_FIELDS]
        if any((not math.isfinite(v)) or v < 0 for v in numbers) or numbers[0] <= 0:
            raise ValueError("local policy costs must be finite/nonnegative, with positive H2D bandwidth")
        return cls(*numbers)

    def compute(self, groups: int, items: int) -> float:
        return self.expert * groups + self.item * items


class CostProfile:
    """Cost table with the override order defaults < rank < layer < layer-and-rank."""

    def __init__(self, path: Any, world: int) -> None:
        raw = Path(path).read_bytes()
        self.data = json.loads(raw)
        declared = self.data.get("calibrated")
        if self.data.get("schema_version") != 1 or self.data.get("world_size") != world \
                or not isinstance(declared, bool):
            raise ValueError("local cost profile schema/world/calibration declaration mismatch")
        self.digest = hashlib.sha256(raw).hexdigest()
        self._resolved: Dict[Tuple[int, int], Costs] = {}

    def cost(self, rank: int, layer: int) -> Costs:
        key = (rank, layer)
        found = self._resolved.get(key)
        if found is None:
            merged = dict(self.data["rank_defaults"])
            merged.update(self.data.get("rank_overrides", {}).get(str(rank), {}))
            per_layer = self.data.get("layers", {}).get(str(layer), {})
            merged.update(per_layer.get("defaults", {}))
            merged.update(per_layer.get("rank_overrides", {}).get(str(rank), {}))
            found = self._resolved[key] = Costs.from_dict(merged)
        return found


class LocalPolicy:
    def __init__(self, profile: CostProfile, rank: int, layer: int, expert_bytes: Mapping[int, int],
                 local_candidates: Iterable[int], *, prefetch: bool = True, route: bool = True,
                 feedback: bool = True) -> None:
        self.profile, self.cost = profile, profile.cost(rank, layer)
        self.rank, self.layer = rank, layer
        self.transfer = {int(e): self.cost.latency + n / self.cost.bandwidth for e, n in expert_bytes.items()}
        self.local_candidates = frozenset(local_candidates)
        self.prefetch, self.route, self.feedback = bool(prefetch), bool(route), bool(feedback)
        self.reset()

    def reset(self) -> None:
        self.ready_ms = 0.0      # compute of the ready experts seen by the last residual scan
        self.window_ms = 0.0     # time a prefetch issued now has before its layer runs
        self.route_key = self.route_table = None
        self.stats: Dict[str, float] = dict(
            prefetch_calls=0, candidate_scores=0, feedback_updates=0, route_calls=0, route_table_rebuilds=0,
            residual_calls=0, prefetch_host_ms=0.0, route_host_ms=0.0, residual_host_ms=0.0)

    def scores(self, values: Mapping[int, float], residents: Set[int]) -> Mapping[int, float]:
        """Discount non-resident candidates; resident scores keep their units (they are
        retention values compared against the same thresholds as before)."""
        if not self.prefetch:
            return values
        t0 = time.perf_counter()
        covered = self.ready_ms if self.feedback else 0.0
        adjusted: Dict[int, float] = {}
        for eid, score in values.items():
            if eid in residents:
                adjusted[eid] = score
                continue
            copy_ms = self.transfer[eid]
            window = min(self.window_ms, copy_ms)
            gain = min(window, max(0.0, copy_ms - covered))
            # no window estimate: keep the score rather than switch prefetching off
            adjusted[eid] = score * gain / window if window > 0 else score
        self.stats["prefetch_calls"] += 1
        self.stats["candidate_scores"] += len(values)
        self.stats["prefetch_host_ms"] += (time.perf_counter() - t0) * 1e3
        return adjusted

    def observe_ready(self, groups: int, items: int) -> None:
        if self.feedback:
            self.ready_ms = self.cost.compute(groups, items)
            self.stats["feedback_updates"] += 1

    def residual(self, ready_groups: int, ready_items: int,
                 candidates: Sequence[Tuple[int, int, str]]) -> Optional[Tuple[int, str]]:
        """``candidates`` are ``(segment index, expert id, kind)`` in the executor's own order
        (late prefetches first); the first of equally good ones wins, and none is chosen
        unless its overlap exceeds the split overhead."""
        t0 = time.perf_counter()
        ready = self.cost.compute(ready_groups, ready_items)
        best, benefit = None, self.cost.split
        for index, eid, kind in candidates:
            overlap = min(ready, self.transfer[eid])
            if overlap > benefit:
                best, benefit = (index, kind), overlap
        self.stats["residual_calls"] += 1
        self.stats["residual_host_ms"] += (time.perf_counter() - t0) * 1e3
        return best

    def summary(self) -> Dict[str, Any]:
        return {**self.stats, "profile_sha256": self.profile.digest, "calibrated": self.profile.data["calibrated"],
                "prefetch": self.prefetch, "route": self.route, "feedback": self.feedback,
                "metadata_collectives": 0, "device_to_host_copies": 0}


def install_lightweight_policies(profile: CostProfile, *, prefetch: bool = True, route: bool = True,
                                 feedback: bool = True) -> List[LocalPolicy]:
    """Give every registered offloaded block its policy (reference :17745-17756).  On one GPU
    no expert has a cheaper local replica, so ``local_candidates`` is empty and the routing
    part of the policy has nothing to do."""
    from .context import SparseContext
    if SparseContext.rs_bank_layout != "next_layer":
        raise ValueError("local readiness policy currently requires adjacent-layer probability RS")
    made = []
    for layer, block in sorted(SparseContext.layer_blocks.items()):
        res = getattr(block, "residency", None)
        if res is None:
            continue
        if block.planner_mode != "rs_prefetch" or block.cache_policy != "lru":
            raise ValueError("local readiness policy requires original router, RS prefetch, CPU offload, LRU "
                             "and no oracle/SKVS")
        sizes = {int(e): int(res.expert_bytes) for e in block.local_expert_ids}
        res.light_policy = LocalPolicy(profile, block.rank, layer, sizes, (), prefetch=prefetch, route=route,
                                       feedback=feedback)
        made.append(res.light_policy)
    return made


def measure_costs(block: Any, batches: Sequence[int] = (1, 4, 8, 16, 32), repeats: int = 20,
                  expert_bytes: Optional[int] = None) -> Dict[str, float]:
    """Measure the cost fields on the running GPU with an all-resident block of the layer
    shape in question.  Copy rate and latency: a pinned-host to HBM copy of one expert's
    bytes against a 4 KiB one.  Compute: the routed grouped-FFN launch timed at several
    decode batch sizes, fitted by least squares to ``expert_ms * experts + item_ms * rows``
    (both clamped at zero).  ``next_attention_ms`` and ``split_overhead_ms`` are set to the
    smallest launch time seen: in an attention-free stack that is all a prefetch can hide
    behind besides the routed compute, and roughly what one more launch boundary costs."""
    import numpy as np
    import torch
    from . import ops
    if getattr(block, "residency", None) is not None:
        raise ValueError("measure_costs needs a block with expert_offload='gpu'")
    stream = torch.cuda.current_stream().cuda_stream
    start, end = ops.Event(timing=True), ops.Event(timing=True)

    def timed(fn, n):
        fn()
        torch.cuda.synchronize()
        start.record(stream)
        for _ in range(n):
            fn()
        end.record(stream)
        torch.cuda.synchronize()
        return start.elapsed_ms(end) / n

    elem = 4 if block.dtype == torch.float32 else 2
    nbytes = int(expert_bytes) if expert_bytes else 3 * block.hidden_size * block.inter_size * elem
    host = ops.host_alloc(nbytes)
    try:
        dev = torch.empty(nbytes, dtype=torch.uint8, device=block.device)
        full_ms = timed(lambda: ops.expert_upload_async(dev.data_ptr(), host, nbytes, stream, None), repeats)
        latency_ms = timed(lambda: ops.expert_upload_async(dev.data_ptr(), host, 4096, stream, None), repeats)
        torch.cuda.synchronize()
    finally:
        ops.host_free(host)
    bandwidth = nbytes / max(full_ms - latency_ms, 1e-6)

    rows_a, rows_t = [], []
    gen = torch.Generator().manual_seed(7)
    for T in batches:
        x = torch.randn(T, block.hidden_size, generator=gen).to(block.dtype).to(block.device)
        ws = block._workspace(T)
        block._route(x, ws)
        offsets = ws.perm.seg_offsets.cpu().tolist()
        experts = sum(1 for e in range(block.num_experts) if offsets[e + 1] > offsets[e])
        t = timed(lambda: ops.grouped_swiglu(block._experts_desc, x, ws.topv, ws.perm, ws.segs_dev, ws.inter,
                                             ws.parts), repeats)
        rows_a.append((experts, T * block.top_k))
        rows_t.append(t)
    sol, *_ = np.linalg.lstsq(np.asarray(rows_a, dtype=np.float64), np.asarray(rows_t, dtype=np.float64), rcond=None)
    expert_ms, item_ms = (max(0.0, float(v)) for v in sol)
    if expert_ms == 0.0 and item_ms == 0.0:
        expert_ms = min(rows_t) / max(1, rows_a[0][0])
    floor = float(min(rows_t))
    return dict(h2d_bytes_per_ms=float(bandwidth), h2d_latency_ms=float(latency_ms), expert_ms=expert_ms,
                item_ms=item_ms, next_attention_ms=floor, split_overhead_ms=floor)


def write_profile(path: Any, costs: Mapping[str, float], *, calibrated: bool, provenance: str = "") -> None:
    Path(path).write_text(json.dumps(dict(
        schema_version=1, world_size=1, calibrated=bool(calibrated), provenance=provenance,
        rank_defaults={k: float(costs[k]) for k in COST_FIELDS}, rank_overrides={}, layers={}), indent=2))
