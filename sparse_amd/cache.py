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
