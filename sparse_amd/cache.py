"""Host-side residency policy for expert weights in HBM.

``ExpertWeightCache`` keeps the interface and the observable behaviour of the reference's
plain LRU with pinning and active replacement (utils/eval_core.py:3661-3881): same
methods, same recency order, same victim choice, so hit/miss/eviction sequences are
identical for identical access sequences.  The payload of an entry is whatever the block
stores for a resident expert -- here the index of the HBM slot that holds its weights.

Recency order is the insertion order of a ``dict`` (oldest first); "touch" is
pop-and-reinsert.
"""
from __future__ import annotations

from typing import Any, Dict, Iterable, List, Optional, Set, Tuple


class CacheEntry:
    __slots__ = ("payload", "pinned", "hot", "prefill_scp_transient")

    def __init__(self, payload: Any, pinned: bool = False, hot: bool = False,
                 prefill_scp_transient: bool = False) -> None:
        self.payload = payload
        self.pinned = pinned
        self.hot = hot
        self.prefill_scp_transient = prefill_scp_transient


class ExpertWeightCache:
    """LRU over expert ids with pin / protect aware eviction (reference :3669-3881)."""

    def __init__(self, capacity: int) -> None:
        self.capacity = int(capacity)
        self._entries: Dict[int, CacheEntry] = {}
        self._last_evicted_transient = False

    # ---- lookups ------------------------------------------------------------
    def _touch(self, expert_id: int) -> CacheEntry:
        entry = self._entries.pop(expert_id)
        self._entries[expert_id] = entry
        return entry

    def get(self, expert_id: int):
        """Payload of a resident expert, which becomes most recently used (:3686-3693)."""
        if self.capacity <= 0 or expert_id not in self._entries:
            return None
        return self._touch(expert_id).payload

    def peek(self, expert_id: int):
        if self.capacity <= 0:
            return None
        entry = self._entries.get(int(expert_id))
        return entry.payload if entry is not None else None

    def has(self, expert_id: int) -> bool:
        return expert_id in self._entries

    def resident_ids(self) -> List[int]:
        """Oldest first."""
        return list(self._entries)

    def __len__(self) -> int:
        return len(self._entries)

    # ---- metadata -----------------------------------------------------------
    def unpin(self, expert_id: int) -> None:
        entry = self._entries.get(expert_id)
        if entry is not None:
            entry.pinned = False

    def unpin_all(self) -> None:
        for entry in self._entries.values():
            entry.pinned = False

    def promote_hot(self, expert_id: int) -> None:
        """In the plain LRU "hot" only means most recently used (:3720-3722)."""
        if expert_id in self._entries:
            self._touch(expert_id)

    def clear(self) -> None:
        self._entries.clear()
        self._last_evicted_transient = False

    def discard(self, expert_id: int) -> bool:
        return self._entries.pop(int(expert_id), None) is not None

    def evictable_prefetch_ids(self, protect_ids: Optional[Set[int]] = None) -> List[int]:
        """Unpinned, unprotected residents, oldest first (:3734-3743)."""
        protect = protect_ids or ()
        return [int(k) for k, v in self._entries.items() if not v.pinned and k not in protect]

    def prefetch_free_slots(self) -> int:
        return max(0, self.capacity - len(self._entries))

    # ---- insertion ----------------------------------------------------------
    def _pick_victim(self, protect: Iterable[int]) -> int:
        """Oldest entry of the best non-empty class, classes in the order
        unpinned+unprotected+transient, unpinned+unprotected, unpinned+transient,
        unpinned, anything (:3770-3791)."""
        best: List[Optional[int]] = [None, None, None, None]
        oldest = None
        for k, v in self._entries.items():
            if oldest is None:
                oldest = k
            if v.pinned:
                continue
            free = int(k) not in protect
            transient = bool(v.prefill_scp_transient)
            cls = (0 if transient else 1) if free else (2 if transient else 3)
            if best[cls] is None:
                best[cls] = k
                if cls == 0:
                    break
        for k in best:
            if k is not None:
                return k
        return oldest

    def put(self, expert_id: int, weights, pinned: bool = False, prefer_hot: bool = False,
            protect_ids: Optional[Set[int]] = None, prefill_scp_transient: bool = False) -> Optional[int]:
        """Insert at the MRU end and evict while over capacity; returns the last evicted id
        (:3748-3797)."""
        if self.capacity <= 0:
            return None
        existing = self._entries.get(expert_id)
        if existing is not None:
            existing.payload = weights
            existing.pinned = existing.pinned or bool(pinned)
            existing.prefill_scp_transient = bool(existing.prefill_scp_transient or prefill_scp_transient)
            self._touch(expert_id)
            return None
        self._entries[expert_id] = CacheEntry(weights, bool(pinned), False, bool(prefill_scp_transient))
        evicted: Optional[int] = None
        was_transient = False
        protect = protect_ids or ()
        while len(self._entries) > self.capacity:
            victim = self._pick_victim(protect)
            was_transient = bool(self._entries[victim].prefill_scp_transient)
            del self._entries[victim]
            evicted = int(victim)
        self._last_evicted_transient = was_transient
        return evicted

    def last_evicted_was_prefill_scp_transient(self) -> bool:
        return self._last_evicted_transient

    def admit_prefetch(self, expert_id: int, weights, *, protect_ids: Optional[Set[int]] = None,
                       preferred_victim: Optional[int] = None) -> bool:
        """Insert a prefetched expert pinned; when full, replace ``preferred_victim`` if it
        is evictable, else the oldest evictable entry; refuse if none (:3803-3841)."""
        if self.capacity <= 0:
            return False
        existing = self._entries.get(expert_id)
        if existing is not None:
            existing.payload = weights
            existing.pinned = True
            self._touch(expert_id)
            return True
        if len(self._entries) >= self.capacity:
            candidates = self.evictable_prefetch_ids(protect_ids or set())
            if not candidates:
                return False
            victim = candidates[0]
            if preferred_victim is not None and int(preferred_victim) in candidates:
                victim = int(preferred_victim)
            self._entries.pop(victim, None)
        self._entries[expert_id] = CacheEntry(weights, True, False)
        return True

    # ---- prefill-transient bookkeeping (:3843-3881) ------------------------------
    def is_prefill_scp_transient(self, expert_id: int) -> bool:
        entry = self._entries.get(int(expert_id))
        return bool(entry.prefill_scp_transient) if entry is not None else False

    def clear_prefill_scp_transient(self, expert_id: int) -> bool:
        entry = self._entries.get(int(expert_id))
        if entry is None or not entry.prefill_scp_transient:
            return False
        entry.prefill_scp_transient = False
        return True

    def prefill_scp_transient_ids(self) -> List[int]:
        return [int(k) for k, v in self._entries.items() if v.prefill_scp_transient]

    def reset_request_metadata(self, *, unpin: bool = True, demote_hot: bool = False) -> None:
        if unpin:
            self.unpin_all()

    def demote_prefill_scp_transients(self) -> int:
        """Move transient entries to the oldest end, keeping their relative order reversed
        as repeated move-to-front does (:3863-3871)."""
        ids = self.prefill_scp_transient_ids()
        if ids:
            moved = {}
            for eid in ids:
                entry = self._entries.pop(eid)
                entry.pinned = False
                moved[eid] = entry
            rebuilt: Dict[int, CacheEntry] = {}
            for eid in reversed(ids):
                rebuilt[eid] = moved[eid]
            rebuilt.update(self._entries)
            self._entries = rebuilt
        return len(ids)

    def occupancy(self) -> Dict[str, int]:
        return {
            "capacity": int(self.capacity),
            "resident": len(self._entries),
            "hot": 0,
            "transient_demand": len(self._entries),
            "transient_prefetch": 0,
            "prefill_scp_transient": len(self.prefill_scp_transient_ids()),
        }


class EpipePrefillExtraCache:
    """Side LRU for payloads staged during prefill; never touches the main cache
    (reference :3884-3950)."""

    def __init__(self, capacity: int) -> None:
        self.capacity = max(0, int(capacity))
        self._entries: Dict[int, Tuple[Any, int]] = {}

    def has(self, expert_id: int) -> bool:
        return int(expert_id) in self._entries

    def get(self, expert_id: int):
        eid = int(expert_id)
        if self.capacity <= 0 or eid not in self._entries:
            return None
        item = self._entries.pop(eid)
        self._entries[eid] = item
        return item[0]

    def peek(self, expert_id: int):
        if self.capacity <= 0:
            return None
        item = self._entries.get(int(expert_id))
        return None if item is None else item[0]

    def put(self, expert_id: int, payload, *, nbytes: int = 0) -> Tuple[bool, bool, Optional[int]]:
        """Returns (stored, was_update, evicted id)."""
        eid = int(expert_id)
        if self.capacity <= 0:
            return False, False, None
        if eid in self._entries:
            self._entries.pop(eid)
            self._entries[eid] = (payload, max(0, int(nbytes)))
            return True, True, None
        evicted = None
        if len(self._entries) >= self.capacity:
            evicted = next(iter(self._entries))
            del self._entries[evicted]
        self._entries[eid] = (payload, max(0, int(nbytes)))
        return True, False, evicted

    def clear(self) -> int:
        n = len(self._entries)
        self._entries.clear()
        return n

    def resident_ids(self) -> List[int]:
        return list(self._entries)

    def resident_count(self) -> int:
        return len(self._entries)

    def resident_nbytes(self) -> int:
        return sum(n for _, n in self._entries.values())


class _Tier:
    """One recency-ordered tier of the tiered cache (oldest first)."""

    def __init__(self) -> None:
        self.entries: Dict[int, CacheEntry] = {}

    def __contains__(self, eid: int) -> bool:
        return eid in self.entries

    def __len__(self) -> int:
        return len(self.entries)

    def get(self, eid: int) -> Optional[CacheEntry]:
        return self.entries.get(eid)

    def to_mru(self, eid: int, entry: Optional[CacheEntry] = None) -> CacheEntry:
        """(Re)insert ``eid`` as the most recently used entry."""
        old = self.entries.pop(eid, None)
        entry = entry if entry is not None else old
        self.entries[eid] = entry
        return entry

    def to_lru(self, eid: int, entry: CacheEntry) -> None:
        rest = self.entries
        rest.pop(eid, None)
        self.entries = {eid: entry}
        self.entries.update(rest)

    def pop(self, eid: int) -> Optional[CacheEntry]:
        return self.entries.pop(eid, None)

    def first(self, ok) -> Optional[int]:
        for eid, entry in self.entries.items():
            if ok(eid, entry):
                return eid
        return None


class TieredExpertWeightCache:
    """Hot / transient-demand / transient-prefetch tiers (reference :3953-4338,
    ``--cache-policy tiered``).  Hot residents are never replaced by speculation; prefetch
    fills its reserved area first, then replaces unpinned speculative residents, then spills
    into the transient-demand tier.  Same methods, recency order and victim choice as the
    reference, so identical operation sequences give identical contents."""

    def __init__(self, capacity: int, hot_capacity: int, prefetch_reserved: int = 1) -> None:
        self.capacity = int(capacity)
        self.hot_capacity = max(0, min(int(hot_capacity), self.capacity))
        self.transient_capacity = max(0, self.capacity - self.hot_capacity)
        self.transient_prefetch_capacity = (
            max(0, min(int(prefetch_reserved), self.transient_capacity)) if self.transient_capacity > 0 else 0)
        self.transient_demand_capacity = max(0, self.transient_capacity - self.transient_prefetch_capacity)
        self._hot, self._demand, self._prefetch = _Tier(), _Tier(), _Tier()
        self._last_evicted_transient = False

    def _tiers(self) -> Tuple[_Tier, _Tier, _Tier]:
        return self._hot, self._demand, self._prefetch

    def _find(self, eid: int) -> Tuple[Optional[_Tier], Optional[CacheEntry]]:
        for tier in self._tiers():
            entry = tier.get(eid)
            if entry is not None:
                return tier, entry
        return None, None

    # ---- eviction -------------------------------------------------------------
    def _shrink(self, tier: _Tier, capacity: int, protect_ids: Optional[Set[int]]) -> Optional[int]:
        """Evict from ``tier`` down to ``capacity``; the four victim classes of the plain
        cache, in the same priority (:3978-4013).  Returns the last evicted id."""
        protect = protect_ids or set()
        evicted: Optional[int] = None
        transient = False
        while len(tier) > int(capacity):
            victim = tier.first(lambda e, v: not v.pinned and int(e) not in protect and v.prefill_scp_transient)
            if victim is None:
                victim = tier.first(lambda e, v: not v.pinned and int(e) not in protect)
            if victim is None:
                victim = tier.first(lambda e, v: not v.pinned and v.prefill_scp_transient)
            if victim is None:
                victim = tier.first(lambda e, v: not v.pinned)
            if victim is None:
                victim = next(iter(tier.entries))
            transient = bool(tier.pop(victim).prefill_scp_transient)
            evicted = int(victim)
        self._last_evicted_transient = transient
        return evicted

    def _insert_hot(self, eid: int, weights, protect_ids: Optional[Set[int]] = None) -> Optional[int]:
        """:4021-4048: enter the hot tier; overflow demotes the oldest unprotected hot entry
        to the transient-demand tier, which may evict in turn."""
        if self.hot_capacity <= 0:
            return self.put(eid, weights, pinned=False, prefer_hot=False, protect_ids=protect_ids)
        self._demand.pop(eid)
        self._prefetch.pop(eid)
        self._hot.to_mru(eid, CacheEntry(weights, pinned=False, hot=True))
        protect = protect_ids or set()
        evicted: Optional[int] = None
        while len(self._hot) > self.hot_capacity:
            demote = self._hot.first(lambda e, v: not v.pinned and int(e) not in protect)
            if demote is None:
                demote = self._hot.first(lambda e, v: not v.pinned)
            if demote is None:
                demote = next(iter(self._hot.entries))
            old = self._hot.pop(demote)
            self._demand.to_mru(demote, CacheEntry(old.payload, pinned=False, hot=False,
                                                   prefill_scp_transient=old.prefill_scp_transient))
            evicted = self._shrink(self._demand, self.transient_demand_capacity, protect_ids)
        return evicted

    # ---- lookups ------------------------------------------------------------------
    def get(self, expert_id: int):
        tier, entry = self._find(expert_id)
        if entry is None:
            return None
        tier.to_mru(expert_id)
        return entry.payload

    def peek(self, expert_id: int):
        _tier, entry = self._find(int(expert_id))
        return entry.payload if entry is not None else None

    def has(self, expert_id: int) -> bool:
        return any(expert_id in tier for tier in self._tiers())

    def resident_ids(self) -> List[int]:
        return [eid for tier in self._tiers() for eid in tier.entries]

    def __len__(self) -> int:
        return sum(len(tier) for tier in self._tiers())

    def discard(self, expert_id: int) -> bool:
        expert_id = int(expert_id)
        return any([tier.pop(expert_id) is not None for tier in self._tiers()])

    def unpin_all(self) -> None:
        for tier in (self._prefetch, self._demand):
            for entry in tier.entries.values():
                entry.pinned = False

    def unpin(self, expert_id: int) -> None:
        for tier in (self._prefetch, self._demand):
            entry = tier.get(expert_id)
            if entry is not None:
                entry.pinned = False

    def clear(self) -> None:
        for tier in self._tiers():
            tier.entries.clear()
        self._last_evicted_transient = False

    def promote_hot(self, expert_id: int) -> None:
        if expert_id in self._hot:
            self._hot.to_mru(expert_id)
            return
        entry = self._demand.get(expert_id) or self._prefetch.get(expert_id)
        if entry is not None:
            self._insert_hot(expert_id, entry.payload)

    def evictable_prefetch_ids(self, protect_ids: Optional[Set[int]] = None) -> List[int]:
        protect = protect_ids or set()
        return [int(e) for tier in (self._prefetch, self._demand) for e, v in tier.entries.items()
                if not v.pinned and e not in protect]

    def prefetch_free_slots(self) -> int:
        """Only the reserved speculative area counts as free (:4145-4150)."""
        return max(0, self.transient_prefetch_capacity - len(self._prefetch))

    # ---- insertion -------------------------------------------------------------------
    def put(self, expert_id: int, weights, pinned: bool = False, prefer_hot: bool = False,
            protect_ids: Optional[Set[int]] = None, prefill_scp_transient: bool = False) -> Optional[int]:
        """:4152-4202.  Pinned insertions go to the speculative tier, others to transient
        demand, ``prefer_hot`` straight to the hot tier."""
        if self.capacity <= 0:
            return None
        if prefer_hot and self.hot_capacity > 0:
            return self._insert_hot(expert_id, weights, protect_ids=protect_ids)
        entry = self._hot.get(expert_id)
        if entry is not None:
            entry.payload = weights
            self._hot.to_mru(expert_id)
            return None
        entry = self._demand.get(expert_id)
        if entry is not None:
            entry.payload = weights
            entry.pinned = entry.pinned or bool(pinned)
            entry.prefill_scp_transient = bool(entry.prefill_scp_transient or prefill_scp_transient)
            self._demand.to_mru(expert_id)
            return None
        entry = self._prefetch.get(expert_id)
        if entry is not None:
            entry.payload = weights
            entry.pinned = entry.pinned or bool(pinned)
            entry.prefill_scp_transient = bool(entry.prefill_scp_transient or prefill_scp_transient)
            self._prefetch.to_mru(expert_id)
            return self._shrink(self._prefetch, self.transient_prefetch_capacity, protect_ids)
        fresh = CacheEntry(weights, pinned=bool(pinned), hot=False, prefill_scp_transient=bool(prefill_scp_transient))
        if pinned:
            self._prefetch.to_mru(expert_id, fresh)
            return self._shrink(self._prefetch, self.transient_prefetch_capacity, protect_ids)
        self._demand.to_mru(expert_id, fresh)
        return self._shrink(self._demand, self.transient_demand_capacity, protect_ids)

    def admit_prefetch(self, expert_id: int, weights, *, protect_ids: Optional[Set[int]] = None,
                       preferred_victim: Optional[int] = None) -> bool:
        """:4204-4270."""
        if self.capacity <= 0:
            return False
        if expert_id in self._hot:
            self._hot.to_mru(expert_id)
            return True
        for tier in (self._demand, self._prefetch):
            entry = tier.get(expert_id)
            if entry is not None:
                entry.payload = weights
                entry.pinned = True
                tier.to_mru(expert_id)
                return True
        protect = protect_ids or set()
        victim_hint = int(preferred_victim) if preferred_victim is not None else None

        def place(tier: _Tier) -> bool:
            tier.to_mru(expert_id, CacheEntry(weights, pinned=True, hot=False))
            return True

        for tier, room in ((self._prefetch, self.transient_prefetch_capacity),
                           (self._demand, self.transient_demand_capacity)):
            if len(tier) < room:
                return place(tier)
            victims = [e for e, v in tier.entries.items() if e not in protect and not v.pinned]
            if victims:
                tier.pop(victim_hint if victim_hint in victims else int(victims[0]))
                return place(tier)
        return False

    # ---- prefill placement transients, request boundaries -----------------------------
    def is_prefill_scp_transient(self, expert_id: int) -> bool:
        _tier, entry = self._find(int(expert_id))
        return bool(entry is not None and entry.prefill_scp_transient)

    def last_evicted_was_prefill_scp_transient(self) -> bool:
        return bool(self._last_evicted_transient)

    def clear_prefill_scp_transient(self, expert_id: int) -> bool:
        _tier, entry = self._find(int(expert_id))
        if entry is not None and entry.prefill_scp_transient:
            entry.prefill_scp_transient = False
            return True
        return False

    def prefill_scp_transient_ids(self) -> List[int]:
        return [int(e) for tier in self._tiers() for e, v in tier.entries.items() if v.prefill_scp_transient]

    def reset_request_metadata(self, *, unpin: bool = True, demote_hot: bool = False) -> None:
        if unpin:
            self.unpin_all()
        if demote_hot and len(self._hot):
            for eid, entry in list(self._hot.entries.items()):
                self._demand.to_mru(int(eid), CacheEntry(entry.payload, pinned=False, hot=False))
            self._hot.entries.clear()
            self._shrink(self._demand, self.transient_demand_capacity, set())

    def demote_prefill_scp_transients(self) -> int:
        ids = self.prefill_scp_transient_ids()
        for eid in ids:
            entry = self._hot.pop(eid) or self._prefetch.pop(eid) or self._demand.get(eid)
            entry.hot = False
            entry.pinned = False
            self._demand.to_lru(eid, entry)
        if ids:
            self._shrink(self._demand, self.transient_demand_capacity, set())
        return len(ids)

    def occupancy(self) -> Dict[str, int]:
        return {"capacity": self.capacity, "resident": len(self), "hot": len(self._hot),
                "transient_demand": len(self._demand), "transient_prefetch": len(self._prefetch),
                "prefill_scp_transient": len(self.prefill_scp_transient_ids())}


def tiered_capacity_split(expert_cache: int, prefetch_enabled: bool, prefetch_reserved: int = 0,
                          prefetch_extra_capacity: int = 0) -> Tuple[int, int, int]:
    """``(total_capacity, hot_capacity, prefetch_reserved)`` of a ``--cache-policy tiered``
    layer (reference :4843-4890).  ``hot_capacity == 0`` means "use the plain LRU"."""
    base = int(expert_cache)
    extra = max(0, int(prefetch_extra_capacity)) if prefetch_enabled else 0
    total = base + extra
    if base <= 1:
        return total, 0, 0
    if base >= 12:
        transient = 4
    elif base >= 8:
        transient = 3
    else:
        transient = max(2, base // 3)
    transient = min(transient, max(1, base - 1))
    reserved = max(0, int(prefetch_reserved)) if prefetch_enabled else 0
    if reserved > 0 and extra <= 0:
        transient = min(max(1, base - 1), transient + reserved)
    reserved = min(reserved, max(0, transient))
    return total, max(1, base - transient), reserved
