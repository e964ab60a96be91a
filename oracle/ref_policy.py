"""CPU oracle of the cost-aware local readiness policy.  TEST INFRASTRUCTURE ONLY: only
``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import
this.

Restates utils/lightweight_policy.py of the reference as plain functions over plain
numbers (no classes, no timers), so that the product's classes can be checked against an
independent formulation:

  transfer_ms        :62-63     latency + bytes / bandwidth
  compute_ms         :33-34     expert * groups + item * items
  resolve_costs      :47-56     override order defaults < rank < layer < layer-and-rank
  adjusted_scores    :76-99     discount of non-resident prefetch candidates
  choose_residual    :106-118   residual with the largest coverable copy, first one on ties

Pinned by the reference's own known-answer tests (tests/test_lightweight_policy.py:31-44,
:46-54), restated in tests/test_local_policy.py, and by closed-form cases there.
"""
from __future__ import annotations

from typing import Dict, Iterable, Mapping, Optional, Sequence, Set, Tuple

FIELDS = ("h2d_bytes_per_ms", "h2d_latency_ms", "expert_ms", "item_ms", "next_attention_ms", "split_overhead_ms")


def resolve_costs(data: Mapping, rank: int, layer: int) -> Dict[str, float]:
    out = dict(data["rank_defaults"])
    out.update(data.get("rank_overrides", {}).get(str(rank), {}))
    lay = data.get("layers", {}).get(str(layer), {})
    out.update(lay.get("defaults", {}))
    out.update(lay.get("rank_overrides", {}).get(str(rank), {}))
    return {k: float(out[k]) for k in FIELDS}


def transfer_ms(costs: Mapping[str, float], nbytes: float) -> float:
    return costs["h2d_latency_ms"] + nbytes / costs["h2d_bytes_per_ms"]


def compute_ms(costs: Mapping[str, float], groups: int, items: int) -> float:
    return costs["expert_ms"] * groups + costs["item_ms"] * items


def adjusted_scores(costs: Mapping[str, float], expert_bytes: Mapping[int, float], values: Mapping[int, float],
                    residents: Set[int], window_ms: float, ready_ms: float, feedback: bool = True) -> Dict[int, float]:
    cover = ready_ms if feedback else 0.0
    out = {}
    for eid, score in values.items():
        if eid in residents:
            out[eid] = score
            continue
        t = transfer_ms(costs, expert_bytes[eid])
        window = min(window_ms, t)
        gain = min(window, max(0.0, t - cover))
        out[eid] = score * gain / window if window > 0 else score
    return out


def choose_residual(costs: Mapping[str, float], expert_bytes: Mapping[int, float], ready_groups: int,
                    ready_items: int, candidates: Sequence[Tuple[int, int, str]]) -> Optional[Tuple[int, str]]:
    ready = compute_ms(costs, ready_groups, ready_items)
    best, benefit = None, costs["split_overhead_ms"]
    for index, eid, kind in candidates:
        overlap = min(ready, transfer_ms(costs, expert_bytes[eid]))
        if overlap > benefit:
            best, benefit = (index, kind), overlap
    return best
