"""CPU oracle of the staging ownership rules.  TEST INFRASTRUCTURE ONLY: only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import this.

Restates utils/rs_staging.py:52-94 (what a demand lookup sees while copies are staged for a
layer call) as one function over plain data, so that it shares no structure with the
product's ``DemandCacheView``: the resident cache is a recency-ordered list of
``(expert, payload)`` (index 0 = least recently used), the staged copies a dict
``expert -> [payload, used]``.

Pinned by (tests/test_staging.py): the reference's own known-answer tests, restated --
tests/test_rs_staging.py:60-66 (a wrong forecast neither evicts nor reorders), :94-99
(a resident hit has precedence over a staged shadow), :134-145 (all 64 access sequences
over two residents), :152-180 (first-use order of staged experts).  Candidate selection
is ``oracle/ref_rs.select_candidates``.  Both are also checked against vectors recorded from
the reference's own modules (tests/golden/make_staging_golden.py, tests/test_staging_golden.py).
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple


def lookup(resident: List[Tuple[int, Any]], staged: Dict[int, list], used_order: List[int], expert: int,
           touch: bool = True) -> Optional[Any]:
    """``DemandCacheView.get`` (touch) / ``.peek`` (no touch).  Mutates ``resident`` recency,
    the staged ``used`` flags and ``used_order`` exactly as the reference does."""
    for i, (eid, payload) in enumerate(resident):
        if eid == expert:
            if touch:
                resident.append(resident.pop(i))
            return payload
    entry = staged.get(int(expert))
    if entry is None:
        return None
    if touch and not entry[1]:
        entry[1] = True
        used_order.append(int(expert))
    return entry[0]


def has(resident: List[Tuple[int, Any]], staged: Dict[int, list], expert: int) -> bool:
    return any(eid == expert for eid, _ in resident) or int(expert) in staged
