"""CPU oracle of the expert-weight caches.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may
import this; the product's own cache is ``sparse_amd/cache.py``.

Restates ``ExpertWeightCache`` (utils/eval_core.py:3669-3881) and
``EpipePrefillExtraCache`` (:3884-3950) with a plain Python list as the recency order
(index 0 = least recently used), so that it shares no data structure with the product.

Pinned by (tests/test_cache.py):
  - the reference's own known-answer cases: access moves an entry to the MRU end and a
    staged-but-unused expert changes nothing (tests/test_rs_staging.py:60-66), eviction
    victim is the oldest entry and ``resident_ids()`` lists oldest first (:152-180), all 64
    access sequences over two residents (:134-145);
  - the independent LRU replay counts of tests/test_scp_cache_replay.py:52-61, :89-98
    (loads / hits / eviction with capacity 1 / zero capacity);
  - textbook LRU by brute force (an OrderedDict model) on random traces without pins,
    and the 4-class victim rule on hand-built pinned / protected / transient states;
  - golden traces written by running the reference's own class (extracted from its
    source, tests/golden/make_residency_golden.py) on random operation sequences.
"""
from __future__ import annotations

from typing import Any, List, Optional, Set, Tuple


class _Slot:
    def __init__(self, eid: int, payload: Any, pinned: bool, transient: bool) -> None:
        self.eid, self.payload, self.pinned, self.transient = eid, payload, pinned, transient


class RefExpertWeightCache:
    def __init__(self, capacity: int) -> None:
        self.capacity = int(capacity)
        self.order: List[_Slot] = []  # least recently used first
        self.last_evicted_transient = False

    # -- helpers
    def _find(self, eid: int) -> int:
        for i, s in enumerate(self.order):
            if s.eid == eid:
                return i
        return -1

    def _to_mru(self, i: int) -> _Slot:
        s = self.order.pop(i)
        self.order.append(s)
        return s

    # -- :3686-3704
    def get(self, eid: int):
        if self.capacity <= 0:
            return None
        i = self._find(eid)
        return None if i < 0 else self._to_mru(i).payload

    def peek(self, eid: int):
        if self.capacity <= 0:
            return None
        i = self._find(int(eid))
        return None if i < 0 else self.order[i].payload

    def has(self, eid: int) -> bool:
        return self._find(eid) >= 0

    # -- :3706-3746
    def unpin_all(self) -> None:
        for s in self.order:
            s.pinned = False

    def clear(self) -> None:
        self.order = []
        self.last_evicted_transient = False

    def unpin(self, eid: int) -> None:
        i = self._find(eid)
        if i >= 0:
            self.order[i].pinned = False

    def promote_hot(self, eid: int) -> None:
        i = self._find(eid)
        if i >= 0:
            self._to_mru(i)

    def resident_ids(self) -> List[int]:
        return [s.eid for s in self.order]

    def discard(self, eid: int) -> bool:
        i = self._find(int(eid))
        if i < 0:
            return False
        self.order.pop(i)
        return True

    def evictable_prefetch_ids(self, protect_ids: Optional[Set[int]] = None) -> List[int]:
        protect = protect_ids or set()
        return [int(s.eid) for s in self.order if not s.pinned and s.eid not in protect]

    def prefetch_free_slots(self) -> int:
        return max(0, self.capacity - len(self.order))

    # -- :3748-3801
    def put(self, eid: int, payload, pinned: bool = False, prefer_hot: bool = False,
            protect_ids: Optional[Set[int]] = None, prefill_scp_transient: bool = False) -> Optional[int]:
        if self.capacity <= 0:
            return None
        i = self._find(eid)
        if i >= 0:
            s = self._to_mru(i)
            s.payload = payload
            s.pinned = s.pinned or bool(pinned)
            s.transient = bool(s.transient or prefill_scp_transient)
            return None
        self.order.append(_Slot(eid, payload, bool(pinned), bool(prefill_scp_transient)))
        protect = protect_ids or set()
        evicted = None
        was_transient = False
        while len(self.order) > self.capacity:
            tests = (
                lambda s: (not s.pinned) and int(s.eid) not in protect and s.transient,
                lambda s: (not s.pinned) and int(s.eid) not in protect,
                lambda s: (not s.pinned) and s.transient,
                lambda s: not s.pinned,
                lambda s: True,
            )
            victim = None
            for ok in tests:
                victim = next((j for j, s in enumerate(self.order) if ok(s)), None)
                if victim is not None:
                    break
            gone = self.order.pop(victim)
            evicted, was_transient = int(gone.eid), bool(gone.transient)
        self.last_evicted_transient = was_transient
        return evicted

    def last_evicted_was_prefill_scp_transient(self) -> bool:
        return bool(self.last_evicted_transient)

    # -- :3803-3841
    def admit_prefetch(self, eid: int, payload, *, protect_ids: Optional[Set[int]] = None,
                       preferred_victim: Optional[int] = None) -> bool:
        if self.capacity <= 0:
            return False
        i = self._find(eid)
        if i >= 0:
            s = self._to_mru(i)
            s.payload, s.pinned = payload, True
            return True
        if len(self.order) < self.capacity:
            self.order.append(_Slot(eid, payload, True, False))
            return True
        evictable = self.evictable_prefetch_ids(protect_ids or set())
        if not evictable:
            return False
        victim = evictable[0]
        if preferred_victim is not None and int(preferred_victim) in evictable:
            victim = int(preferred_victim)
        self.discard(victim)
        self.order.append(_Slot(eid, payload, True, False))
        return True

    # -- :3843-3881
    def is_prefill_scp_transient(self, eid: int) -> bool:
        i = self._find(int(eid))
        return bool(self.order[i].transient) if i >= 0 else False

    def clear_prefill_scp_transient(self, eid: int) -> bool:
        i = self._find(int(eid))
        if i < 0 or not self.order[i].transient:
            return False
        self.order[i].transient = False
        return True

    def prefill_scp_transient_ids(self) -> List[int]:
        return [int(s.eid) for s in self.order if s.transient]

    def reset_request_metadata(self, *, unpin: bool = True, demote_hot: bool = False) -> None:
        if unpin:
            self.unpin_all()

    def demote_prefill_scp_transients(self) -> int:
        ids = self.prefill_scp_transient_ids()
        for eid in ids:  # each one in turn becomes the oldest entry
            s = self.order.pop(self._find(eid))
            s.pinned = False
            self.order.insert(0, s)
        return len(ids)

    def occupancy(self):
        n = len(self.order)
        return dict(capacity=self.capacity, resident=n, hot=0, transient_demand=n, transient_prefetch=0,
                    prefill_scp_transient=len(self.prefill_scp_transient_ids()))


class RefEpipePrefillExtraCache:
    """:3884-3950."""

    def __init__(self, capacity: int) -> None:
        self.capacity = max(0, int(capacity))
        self.order: List[Tuple[int, Any, int]] = []  # (eid, payload, nbytes), oldest first

    def _find(self, eid: int) -> int:
        return next((i for i, s in enumerate(self.order) if s[0] == int(eid)), -1)

    def has(self, eid: int) -> bool:
        return self._find(eid) >= 0

    def get(self, eid: int):
        if self.capacity <= 0:
            return None
        i = self._find(eid)
        if i < 0:
            return None
        s = self.order.pop(i)
        self.order.append(s)
        return s[1]

    def peek(self, eid: int):
        if self.capacity <= 0:
            return None
        i = self._find(eid)
        return None if i < 0 else self.order[i][1]

    def put(self, eid: int, payload, *, nbytes: int = 0):
        eid = int(eid)
        if self.capacity <= 0:
            return False, False, None
        i = self._find(eid)
        if i >= 0:
            self.order.pop(i)
            self.order.append((eid, payload, max(0, int(nbytes))))
            return True, True, None
        evicted = None
        if len(self.order) >= self.capacity:
            evicted = self.order.pop(0)[0]
        self.order.append((eid, payload, max(0, int(nbytes))))
        return True, False, evicted

    def clear(self) -> int:
        n = len(self.order)
        self.order = []
        return n

    def resident_ids(self) -> List[int]:
        return [s[0] for s in self.order]

    def resident_count(self) -> int:
        return len(self.order)

    def resident_nbytes(self) -> int:
        return sum(s[2] for s in self.order)


# ---------------------------------------------------------------------------------------
# Tiered cache (utils/eval_core.py:3953-4338).  One list per tier, least recently used
# first; an entry is a ``_Slot``.  Pinned by tests/test_cache.py: golden traces produced by
# the reference's own class on random operation sequences (tests/golden/tiered_ops.json,
# written by tests/golden/make_residency_golden.py) -- return values, resident order, tier
# occupancy and the "last evicted was a prefill transient" flag after every operation --
# and the capacity split (:4843-4890) on the full grid of small cache sizes.
# ---------------------------------------------------------------------------------------
HOT, DEMAND, PREFETCH = 0, 1, 2


class RefTieredExpertWeightCache:
    def __init__(self, capacity: int, hot_capacity: int, prefetch_reserved: int = 1) -> None:
        self.capacity = int(capacity)
        self.hot_capacity = max(0, min(int(hot_capacity), int(capacity)))
        transient = max(0, self.capacity - self.hot_capacity)
        self.prefetch_capacity = 0 if transient <= 0 else max(0, min(int(prefetch_reserved), transient))
        self.demand_capacity = max(0, transient - self.prefetch_capacity)
        self.tiers: List[List[_Slot]] = [[], [], []]
        self.last_evicted_transient = False

    # -- helpers
    def _where(self, eid: int) -> Tuple[int, int]:
        for t in (HOT, DEMAND, PREFETCH):
            for i, s in enumerate(self.tiers[t]):
                if s.eid == eid:
                    return t, i
        return -1, -1

    def _remove(self, eid: int) -> Optional[_Slot]:
        t, i = self._where(eid)
        return None if t < 0 else self.tiers[t].pop(i)

    def _append(self, t: int, slot: _Slot) -> None:
        self.tiers[t] = [s for s in self.tiers[t] if s.eid != slot.eid] + [slot]

    def _evict_down_to(self, t: int, cap: int, protect: Optional[Set[int]]) -> Optional[int]:
        """:3978-4013."""
        protect = protect or set()
        tier = self.tiers[t]
        evicted, transient = None, False
        while len(tier) > cap:
            rules = (lambda s: not s.pinned and s.eid not in protect and s.transient,
                     lambda s: not s.pinned and s.eid not in protect,
                     lambda s: not s.pinned and s.transient,
                     lambda s: not s.pinned,
                     lambda s: True)
            idx = next(i for rule in rules for i, s in enumerate(tier) if rule(s))
            victim = tier.pop(idx)
            evicted, transient = victim.eid, bool(victim.transient)
        self.last_evicted_transient = transient
        return evicted

    def _insert_hot(self, eid: int, payload, protect: Optional[Set[int]] = None) -> Optional[int]:
        """:4021-4048."""
        if self.hot_capacity <= 0:
            return self.put(eid, payload, pinned=False, prefer_hot=False, protect_ids=protect)
        for t in (DEMAND, PREFETCH):
            self.tiers[t] = [s for s in self.tiers[t] if s.eid != eid]
        self._append(HOT, _Slot(eid, payload, False, False))
        guard = protect or set()
        evicted = None
        while len(self.tiers[HOT]) > self.hot_capacity:
            hot = self.tiers[HOT]
            rules = (lambda s: not s.pinned and s.eid not in guard, lambda s: not s.pinned, lambda s: True)
            idx = next(i for rule in rules for i, s in enumerate(hot) if rule(s))
            old = hot.pop(idx)
            self._append(DEMAND, _Slot(old.eid, old.payload, False, old.transient))
            evicted = self._evict_down_to(DEMAND, self.demand_capacity, protect)
        return evicted

    # -- lookups :4050-4089
    def get(self, eid: int):
        t, i = self._where(eid)
        if t < 0:
            return None
        slot = self.tiers[t].pop(i)
        self.tiers[t].append(slot)
        return slot.payload

    def peek(self, eid: int):
        t, i = self._where(int(eid))
        return None if t < 0 else self.tiers[t][i].payload

    def has(self, eid: int) -> bool:
        return self._where(eid)[0] >= 0

    def resident_ids(self) -> List[int]:
        return [s.eid for t in (HOT, DEMAND, PREFETCH) for s in self.tiers[t]]

    # -- :4091-4150
    def discard(self, eid: int) -> bool:
        return self._remove(int(eid)) is not None

    def unpin_all(self) -> None:
        for t in (PREFETCH, DEMAND):
            for s in self.tiers[t]:
                s.pinned = False

    def clear(self) -> None:
        self.tiers = [[], [], []]
        self.last_evicted_transient = False

    def unpin(self, eid: int) -> None:
        t, i = self._where(eid)
        if t in (PREFETCH, DEMAND):
            self.tiers[t][i].pinned = False

    def promote_hot(self, eid: int) -> None:
        t, i = self._where(eid)
        if t == HOT:
            self.tiers[HOT].append(self.tiers[HOT].pop(i))
        elif t >= 0:
            self._insert_hot(eid, self.tiers[t][i].payload)

    def evictable_prefetch_ids(self, protect_ids: Optional[Set[int]] = None) -> List[int]:
        protect = protect_ids or set()
        return [s.eid for t in (PREFETCH, DEMAND) for s in self.tiers[t] if not s.pinned and s.eid not in protect]

    def prefetch_free_slots(self) -> int:
        return max(0, self.prefetch_capacity - len(self.tiers[PREFETCH]))

    # -- :4152-4202
    def put(self, eid: int, payload, pinned: bool = False, prefer_hot: bool = False,
            protect_ids: Optional[Set[int]] = None, prefill_scp_transient: bool = False) -> Optional[int]:
        if self.capacity <= 0:
            return None
        if prefer_hot and self.hot_capacity > 0:
            return self._insert_hot(eid, payload, protect_ids)
        t, i = self._where(eid)
        if t >= 0:
            slot = self.tiers[t].pop(i)
            slot.payload = payload
            if t != HOT:
                slot.pinned = slot.pinned or bool(pinned)
                slot.transient = bool(slot.transient or prefill_scp_transient)
            self.tiers[t].append(slot)
            return self._evict_down_to(PREFETCH, self.prefetch_capacity, protect_ids) if t == PREFETCH else None
        slot = _Slot(eid, payload, bool(pinned), bool(prefill_scp_transient))
        if pinned:
            self.tiers[PREFETCH].append(slot)
            return self._evict_down_to(PREFETCH, self.prefetch_capacity, protect_ids)
        self.tiers[DEMAND].append(slot)
        return self._evict_down_to(DEMAND, self.demand_capacity, protect_ids)

    # -- :4204-4270
    def admit_prefetch(self, eid: int, payload, *, protect_ids: Optional[Set[int]] = None,
                       preferred_victim: Optional[int] = None) -> bool:
        if self.capacity <= 0:
            return False
        t, i = self._where(eid)
        if t == HOT:
            self.tiers[HOT].append(self.tiers[HOT].pop(i))
            return True
        if t >= 0:
            slot = self.tiers[t].pop(i)
            slot.payload, slot.pinned = payload, True
            self.tiers[t].append(slot)
            return True
        protect = protect_ids or set()
        hint = None if preferred_victim is None else int(preferred_victim)
        for t, cap in ((PREFETCH, self.prefetch_capacity), (DEMAND, self.demand_capacity)):
            tier = self.tiers[t]
            if len(tier) >= cap:
                victims = [s.eid for s in tier if s.eid not in protect and not s.pinned]
                if not victims:
                    continue
                gone = hint if hint in victims else victims[0]
                self.tiers[t] = tier = [s for s in tier if s.eid != gone]
            tier.append(_Slot(eid, payload, True, False))
            return True
        return False

    # -- :4272-4338
    def is_prefill_scp_transient(self, eid: int) -> bool:
        t, i = self._where(int(eid))
        return t >= 0 and bool(self.tiers[t][i].transient)

    def clear_prefill_scp_transient(self, eid: int) -> bool:
        t, i = self._where(int(eid))
        if t >= 0 and self.tiers[t][i].transient:
            self.tiers[t][i].transient = False
            return True
        return False

    def prefill_scp_transient_ids(self) -> List[int]:
        return [s.eid for t in (HOT, DEMAND, PREFETCH) for s in self.tiers[t] if s.transient]

    def reset_request_metadata(self, *, unpin: bool = True, demote_hot: bool = False) -> None:
        if unpin:
            self.unpin_all()
        if demote_hot and self.tiers[HOT]:
            for s in list(self.tiers[HOT]):
                self._append(DEMAND, _Slot(s.eid, s.payload, False, False))
            self.tiers[HOT] = []
            self._evict_down_to(DEMAND, self.demand_capacity, set())

    def demote_prefill_scp_transients(self) -> int:
        ids = self.prefill_scp_transient_ids()
        for eid in ids:
            slot = self._remove(eid)
            slot.pinned = False
            self.tiers[DEMAND].insert(0, slot)
        if ids:
            self._evict_down_to(DEMAND, self.demand_capacity, set())
        return len(ids)

    def occupancy_counts(self) -> List[int]:
        return [len(self.tiers[HOT]), len(self.tiers[DEMAND]), len(self.tiers[PREFETCH]),
                len(self.prefill_scp_transient_ids())]


def ref_tiered_capacity_split(expert_cache: int, prefetch_enabled: bool, prefetch_reserved: int = 0,
                              prefetch_extra_capacity: int = 0) -> Tuple[int, int, int]:
    """(total, hot, reserved) -- utils/eval_core.py:4843-4890."""
    base = int(expert_cache)
    extra = max(0, int(prefetch_extra_capacity)) if prefetch_enabled else 0
    if base <= 1:
        return base + extra, 0, 0
    budget = 4 if base >= 12 else 3 if base >= 8 else max(2, base // 3)
    budget = min(budget, max(1, base - 1))
    reserved = max(0, int(prefetch_reserved)) if prefetch_enabled else 0
    if reserved > 0 and extra <= 0:
        budget = min(max(1, base - 1), budget + reserved)
    reserved = min(reserved, max(0, budget))
    return base + extra, max(1, base - budget), reserved
