"""Per-layer expert residency: HBM slot pool, demand loads, RS prefetch planning and
EPIPE readiness-ordered execution.

Pure Python over a small device ``Backend`` (uploads, events, kernel launches), so the
whole state machine also runs on the CPU with a fake backend.  Behaviour follows the
reference's block methods (utils/eval_core.py): demand path :11388-11435, prefetch cycle
:9619-9665, budget :9754-9810, scoring and planning :10031-10262, admission :10433-10527,
EPIPE upfront scan :11867-12167 and residual scan :12169-12512.  Cache hit / miss events
and the resulting residency are the same as the reference's for the same accesses; what
differs is physical: an expert lives in a numbered HBM slot, experts of one call are run
in batched launches, and a slot is reused only after the launches that read it.

Slots.  ``capacity`` cache slots plus ``staging_slots`` spares.  A spare holds an expert
that the policy has already evicted but an un-launched batch still reads, or an EPIPE
transient.  When no slot is free the pending batch is launched, which releases them.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence, Set, Tuple

from .cache import TieredExpertWeightCache, tiered_capacity_split, EpipePrefillExtraCache, ExpertWeightCache
from .context import Metrics
from .ring import StagingRing

Segment = Tuple[int, int]  # (expert id, routed rows)


def _env_flag(name: str, default: str) -> bool:
    return str(os.environ.get(name, default)).strip().lower() in ("1", "true", "yes", "on")


def _env_int(name: str, default: int) -> int:
    try:
        return int(os.environ.get(name, str(default)) or default)
    except ValueError:
        return int(default)


def _env_float(name: str, default: float) -> float:
    try:
        return float(os.environ.get(name, str(default)) or default)
    except ValueError:
        return float(default)


def normalize_decode_rs_mode(raw: Optional[str]) -> str:
    """Spellings the reference accepts for ``SPARSE_EPIPE_DECODE_RS_MODE`` (:4942-4962)."""
    mode = str(raw or "late_only").strip().lower() or "late_only"
    if mode == "disabled":
        return "off"
    if mode == "late":
        return "late_only"
    if mode == "demand":
        return "demand_only"
    if mode in ("scan", "residual", "residual-scan", "buffered_scan", "buffered-scan"):
        return "residual_scan"
    return mode


@dataclass
class ResidencyConfig:
    """Knobs of the cache / prefetch / EPIPE machinery with the reference's defaults
    (utils/eval_core.py:4939-5075); ``from_env`` reads the same ``SPARSE_*`` variables."""

    capacity: int = 10
    staging_slots: int = 4
    staging_pool_slots: int = 0            # slots reserved for the bounded RS staging engine
    cache_policy: str = "lru"              # lru | tiered (--cache-policy)
    prefetch_reserved: int = 0             # SPARSE_PREFETCH_RESERVED (tiered only)
    prefetch_extra_capacity: int = 0       # SPARSE_PREFETCH_EXTRA_CAPACITY (tiered only)
    planner_mode: str = "none"            # none | rs_prefetch
    prefetch_top_m: int = 4
    pred_topk: Optional[int] = None        # SPARSE_RS_PREFETCH_PRED_TOPK
    rs_policy: str = "default"             # default | cache_safe
    min_candidate_score: float = 0.02
    replace_advantage: float = 0.02
    replace_margin: float = 1.05
    cache_safe_min_score: float = 0.03
    cache_safe_replace_advantage: float = 0.05
    cache_safe_replace_margin: float = 1.10
    allow_active_replace: bool = True
    recent_protect_steps: int = 0
    protect_mode: str = "default"
    wait_before_evict: bool = True
    rs_prefetch_prefill: bool = False
    cache_ttl_steps: int = 0
    # EPIPE
    epipe_enable: bool = False
    epipe_prefill_enable: bool = False
    epipe_mode: str = "upfront_scan"
    epipe_decode_rs_mode: str = "late_only"
    epipe_no_evict: bool = True
    epipe_transient_staging: bool = True
    epipe_max_staged_experts: int = 1
    # Not in the reference, which copies exactly one missing expert per call beside the resident
    # work and the others on the compute lane: with this on, every expert an EPIPE executor finds
    # missing is copied on the EPIPE lane, back to back, and its segment runs behind its own
    # event, after the resident segments.  Cache events, eviction order and final contents are
    # those of the one-staged-expert executors; only lanes and waits change.
    epipe_stream_all: bool = False
    # counting-only variants (reference :4940, :5008-5010): the executors classify ready / missing
    # experts and count what EPIPE could have done, then leave the call to the demand path
    epipe_shadow: bool = False
    epipe_prefill_shadow: bool = False
    epipe_prefill_multistage_shadow: bool = False
    epipe_prefill_multistage_max_n: int = 4
    # prefill: ready experts are read without moving them in the LRU (reference :5018)
    epipe_prefill_no_touch_ready: bool = False
    # the demand stage of the RS executors opens once the exposed demand-copy time seen so far
    # exceeds this many ms (reference :4988, :5880-5893); 0: only `epipe_rs_force_demand_stage` opens it
    epipe_rs_demand_stage_threshold_ms: float = 0.0
    epipe_min_ready_experts: int = 1
    epipe_min_ready_items: int = 1
    epipe_min_missing_experts: int = 1
    epipe_sort_ready_by_work: bool = False
    epipe_prefill_commit: bool = True
    epipe_rs_handle_late_prefetch: bool = True
    epipe_rs_handle_demand_miss: bool = False
    epipe_rs_force_demand_stage: bool = False
    epipe_rs_demand_commit: bool = True
    epipe_deferred_lru_commit: bool = True
    epipe_rs_min_buffer_groups: int = 1
    epipe_rs_min_buffer_items: int = 1
    epipe_rs_rolling_gate: bool = True
    epipe_rs_gate_window: int = 16
    epipe_rs_gate_min_triggers: int = 1
    epipe_rs_gate_skip_steps: int = 8
    epipe_prefill_extra_cache_slots: int = 0
    epipe_prefill_extra_cache_decode_read: bool = True
    epipe_prefill_extra_cache_clear_at_decode: bool = False
    epipe_prefill_extra_cache_persist_requests: bool = False
    epipe_prefill_extra_cache_max_mb: float = 128.0
    epipe_prefill_mark_transient: bool = True     # staged prefill commits are first in line for eviction
    epipe_promote_transient_on_decode_hit: bool = True
    epipe_rs_buffer_max_groups: int = 4
    epipe_rs_buffer_max_items: int = 32
    epipe_lookahead_experts: int = 4
    epipe_lookahead_min_ready_items: int = 64
    epipe_prefill_lookahead_min_ready_items: int = 256
    epipe_decode_rs_commit: bool = True
    epipe_decode_no_rs_commit: bool = True
    # execution order for plain EP: unique_mask | full_mask | sorted_segment (same events)
    plain_ep_exec_mode: str = "unique_mask"
    # The reference's forward reaches the EPIPE executors only through its expert-parallel
    # paths; a single process (world size 1) runs the plain ascending loop whatever the EPIPE
    # switches say (utils/eval_core.py:16520-16526).  This build treats the one GPU as an
    # expert-parallel rank that owns every expert, so EPIPE applies; set this to get the
    # reference's single-process behaviour instead.
    world1_exact: bool = False

    @classmethod
    def from_env(cls, **overrides) -> "ResidencyConfig":
        c = cls()
        c.staging_slots = max(1, _env_int("SPARSE_HIP_STAGING_SLOTS", c.staging_slots))
        c.prefetch_reserved = max(0, _env_int("SPARSE_PREFETCH_RESERVED", 0))
        c.prefetch_extra_capacity = max(0, _env_int("SPARSE_PREFETCH_EXTRA_CAPACITY", 0))
        raw = os.environ.get("SPARSE_RS_PREFETCH_PRED_TOPK", "").strip()
        c.pred_topk = int(raw) if raw else None
        c.rs_policy = str(os.environ.get("SPARSE_RS_PREFETCH_POLICY", "default") or "default").strip().lower()
        c.min_candidate_score = _env_float("SPARSE_PREFETCH_MIN_CAND_SCORE", 0.02)
        c.replace_advantage = _env_float("SPARSE_PREFETCH_REPLACE_ADVANTAGE", 0.02)
        c.replace_margin = _env_float("SPARSE_PREFETCH_REPLACE_MARGIN", 1.05)
        c.cache_safe_min_score = _env_float("SPARSE_RS_CACHE_SAFE_MIN_SCORE", 0.03)
        c.cache_safe_replace_advantage = _env_float("SPARSE_RS_CACHE_SAFE_REPLACE_ADVANTAGE", 0.05)
        c.cache_safe_replace_margin = _env_float("SPARSE_RS_CACHE_SAFE_REPLACE_MARGIN", 1.10)
        c.allow_active_replace = _env_flag("SPARSE_PREFETCH_ALLOW_ACTIVE_REPLACE", "1")
        c.recent_protect_steps = _env_int("SPARSE_RS_PREFETCH_RECENT_PROTECT_STEPS", 0)
        c.protect_mode = str(os.environ.get("SPARSE_PREFETCH_PROTECT_MODE", "default") or "default").strip().lower()
        c.wait_before_evict = _env_flag("SPARSE_PREFETCH_WAIT_BEFORE_EVICT", "1")
        c.rs_prefetch_prefill = _env_flag("SPARSE_RS_PREFETCH_PREFILL", "0")
        c.cache_ttl_steps = _env_int("SPARSE_CACHE_TTL_STEPS", 0)
        c.epipe_enable = _env_flag("SPARSE_EPIPE_ENABLE", "0")
        c.epipe_prefill_enable = _env_flag("SPARSE_EPIPE_PREFILL_ENABLE", "0")
        c.epipe_mode = str(os.environ.get("SPARSE_EPIPE_MODE", "upfront_scan") or "upfront_scan").strip().lower()
        c.epipe_decode_rs_mode = normalize_decode_rs_mode(os.environ.get(
            "SPARSE_EPIPE_DECODE_RS_MODE", os.environ.get("SPARSE_EPIPE_DECODE_WITH_RS_MODE", "late_only")))
        c.epipe_no_evict = _env_flag("SPARSE_EPIPE_NO_EVICT", "1")
        c.epipe_transient_staging = _env_flag("SPARSE_EPIPE_TRANSIENT_STAGING", "1")
        c.epipe_max_staged_experts = _env_int("SPARSE_EPIPE_MAX_STAGED_EXPERTS", 1)
        c.epipe_stream_all = _env_flag("SPARSE_HIP_EPIPE_STREAM_ALL", "0")
        c.epipe_shadow = _env_flag("SPARSE_EPIPE_SHADOW", "0")
        c.epipe_prefill_shadow = _env_flag("SPARSE_EPIPE_PREFILL_SHADOW", "0")
        c.epipe_prefill_multistage_shadow = _env_flag("SPARSE_EPIPE_PREFILL_MULTI_STAGE_SHADOW", "0")
        c.epipe_prefill_multistage_max_n = max(1, _env_int("SPARSE_EPIPE_PREFILL_MULTI_STAGE_MAX_N", 4))
        c.epipe_prefill_no_touch_ready = _env_flag("SPARSE_EPIPE_PREFILL_NO_TOUCH_READY", "0")
        c.epipe_rs_demand_stage_threshold_ms = max(0.0, _env_float("SPARSE_EPIPE_RS_DEMAND_STAGE_THRESHOLD_MS", 0.0))
        c.epipe_sort_ready_by_work = _env_flag("SPARSE_EPIPE_SORT_READY_BY_WORK", "0")
        # the prefill policy sets the defaults of commit and transient mark (reference :5007-5016)
        policy = str(os.environ.get("SPARSE_EPIPE_PREFILL_POLICY", "deferred_lru_commit")
                     or "deferred_lru_commit").strip().lower()
        commit_default = "1" if policy in ("deferred_lru_commit", "commit", "lru_commit") else "0"
        c.epipe_prefill_commit = _env_flag("SPARSE_EPIPE_PREFILL_COMMIT", commit_default)
        c.epipe_prefill_mark_transient = _env_flag("SPARSE_EPIPE_PREFILL_MARK_TRANSIENT", commit_default)
        c.epipe_promote_transient_on_decode_hit = _env_flag("SPARSE_EPIPE_PROMOTE_TRANSIENT_ON_DECODE_HIT", "1")
        c.epipe_rs_buffer_max_groups = max(1, _env_int("SPARSE_EPIPE_RS_BUFFER_MAX_GROUPS", 4))
        c.epipe_rs_buffer_max_items = max(1, _env_int("SPARSE_EPIPE_RS_BUFFER_MAX_ITEMS", 32))
        c.epipe_lookahead_experts = max(0, _env_int("SPARSE_EPIPE_LOOKAHEAD_EXPERTS", 4))
        c.epipe_lookahead_min_ready_items = max(0, _env_int("SPARSE_EPIPE_LOOKAHEAD_MIN_READY_ITEMS", 64))
        c.epipe_prefill_lookahead_min_ready_items = max(
            0, _env_int("SPARSE_EPIPE_PREFILL_LOOKAHEAD_MIN_READY_ITEMS", 256))
        c.epipe_decode_rs_commit = _env_flag("SPARSE_EPIPE_DECODE_RS_COMMIT", "1")
        c.epipe_decode_no_rs_commit = _env_flag("SPARSE_EPIPE_DECODE_NO_RS_COMMIT", "1")
        c.epipe_rs_handle_late_prefetch = _env_flag("SPARSE_EPIPE_RS_HANDLE_LATE_PREFETCH", "1")
        c.epipe_rs_handle_demand_miss = _env_flag("SPARSE_EPIPE_RS_HANDLE_DEMAND_MISS", "0")
        c.epipe_rs_force_demand_stage = _env_flag("SPARSE_EPIPE_RS_FORCE_DEMAND_STAGE", "0")
        c.epipe_rs_min_buffer_groups = _env_int("SPARSE_EPIPE_RS_MIN_BUFFER_GROUPS", 1)
        c.epipe_rs_min_buffer_items = _env_int("SPARSE_EPIPE_RS_MIN_BUFFER_ITEMS", 1)
        c.epipe_rs_rolling_gate = _env_flag("SPARSE_EPIPE_RS_ROLLING_GATE", "1")
        c.epipe_rs_gate_window = _env_int("SPARSE_EPIPE_RS_GATE_WINDOW", 16)
        c.epipe_rs_gate_min_triggers = _env_int("SPARSE_EPIPE_RS_GATE_MIN_TRIGGERS", 1)
        c.epipe_rs_gate_skip_steps = _env_int("SPARSE_EPIPE_RS_GATE_SKIP_STEPS", 8)
        c.epipe_prefill_extra_cache_slots = _env_int("SPARSE_EPIPE_PREFILL_EXTRA_CACHE_SLOTS", 0)
        c.epipe_prefill_extra_cache_decode_read = _env_flag("SPARSE_EPIPE_PREFILL_EXTRA_CACHE_DECODE_READ", "1")
        c.epipe_prefill_extra_cache_clear_at_decode = _env_flag("SPARSE_EPIPE_PREFILL_EXTRA_CACHE_CLEAR_AT_DECODE", "0")
        c.epipe_prefill_extra_cache_persist_requests = _env_flag(
            "SPARSE_EPIPE_PREFILL_EXTRA_CACHE_PERSIST_REQUESTS", "0")
        c.epipe_prefill_extra_cache_max_mb = max(0.0, _env_float("SPARSE_EPIPE_PREFILL_EXTRA_CACHE_MAX_MB", 128.0))
        c.plain_ep_exec_mode = str(
            os.environ.get("SPARSE_PLAIN_EP_EXEC_MODE", "unique_mask") or "unique_mask").strip().lower()
        c.world1_exact = _env_flag("SPARSE_HIP_WORLD1_EXACT", "0")
        for k, v in overrides.items():
            if not hasattr(c, k):
                raise ValueError(f"unknown residency option {k}")
            setattr(c, k, v)
        return c


@dataclass
class StagedExpert:
    """An expert readable from a slot of the staging ring during one layer call."""

    pos: int                  # ring position that lent the slot
    slot: int
    event: Any                # recorded behind the copy
    touched: bool = False     # a lookup used it
    kept: bool = False        # the LRU took it, and its slot, at the call's end
    recycled: bool = False    # ... and the ring got the slot of the resident it pushed out
    ring_slot: Optional[int] = None   # what the ring position holds afterwards, when kept


class Backend:
    """Device services the policy needs.  Lanes: ``compute`` (the stream the layer's
    kernels run on), ``prefetch`` and ``epipe`` (side streams for uploads)."""

    def upload(self, eid: int, slot: int, lane: str) -> Any:
        """Enqueue the H2D copy of expert ``eid`` into ``slot`` on ``lane``; return an event
        recorded behind the copy."""
        raise NotImplementedError

    def event_done(self, event: Any) -> bool:
        raise NotImplementedError

    def wait_event(self, event: Any, lane: str, ordering: bool = False) -> None:
        """Make ``lane`` wait for ``event`` (never blocks the host).  ``ordering`` marks waits
        that only protect the reuse of a slot, as opposed to waits the policy itself asks for."""
        raise NotImplementedError

    def run_segments(self, segments: Sequence[Tuple[int, int]]) -> None:
        """Launch the expert FFN for ``(expert id, slot)`` pairs, in this order."""
        raise NotImplementedError

    def fence(self) -> Any:
        """Event recorded on the compute lane now."""
        raise NotImplementedError

    def free_device_bytes(self) -> Optional[int]:
        return None


class LayerResidency:
    """Residency state of one layer's routed experts."""

    def __init__(self, layer_idx: int, num_experts: int, top_k: int, config: ResidencyConfig,
                 backend: Backend, metrics: Optional[Metrics] = None, expert_bytes: int = 0) -> None:
        self.layer_idx = int(layer_idx)
        self.num_experts = int(num_experts)
        self.top_k = int(top_k)
        self.cfg = config
        self.backend = backend
        self.metrics = metrics if metrics is not None else Metrics()
        self.expert_bytes = int(expert_bytes)
        total_capacity = int(config.capacity)
        self.cache: Any = None
        if str(config.cache_policy) == "tiered":
            # hot / transient-demand / transient-prefetch split of the constructor (reference :4843-4899)
            total_capacity, hot, reserved = tiered_capacity_split(
                int(config.capacity), config.planner_mode == "rs_prefetch", int(config.prefetch_reserved),
                int(config.prefetch_extra_capacity))
            if hot > 0:
                self.cache = TieredExpertWeightCache(total_capacity, hot_capacity=hot, prefetch_reserved=reserved)
        elif str(config.cache_policy) not in ("lru", "lfu"):
            # lfu shares the plain cache with lru (reference :4840-4841); it only lowers the
            # prefer-hot threshold, which the plain cache ignores
            raise ValueError(f"cache_policy must be lru|lfu|tiered, got {config.cache_policy}")
        if self.cache is None:
            self.cache = ExpertWeightCache(total_capacity)
        self.extra_cache = EpipePrefillExtraCache(int(config.epipe_prefill_extra_cache_slots))
        self.num_slots = max(0, total_capacity) + max(1, int(config.staging_slots)) + \
            max(0, int(config.epipe_prefill_extra_cache_slots))
        self._free_slots: List[int] = list(range(self.num_slots - 1, -1, -1))
        # the staging ring's slots sit after the ordinary ones and never enter the free list
        ring_slots = max(0, int(config.staging_pool_slots))
        self.ring: Optional[StagingRing] = \
            StagingRing(range(self.num_slots, self.num_slots + ring_slots)) if ring_slots else None
        self.num_slots += ring_slots
        self.staged: Dict[int, StagedExpert] = {}   # experts readable from ring slots during this call
        self.staged_touched: List[int] = []         # those a lookup really used, in first-use order
        self.staged_unconfirmed = 0                 # unused copies whose completion nobody has counted yet
        self.staging: Any = None   # the forecast engine (sparse_amd.staging) while it serves this layer's calls
        self.light_policy: Optional[Any] = None     # sparse_amd.local_policy.LocalPolicy, when installed
        self._retired: List[int] = []           # evicted, still read by the pending batch
        self._pending: List[Tuple[int, int]] = []  # (eid, slot) not launched yet
        self._pending_slots: Set[int] = set()
        self._slot_fence: Dict[int, Any] = {}    # compute-lane event after the last read
        self._slot_upload: Dict[int, Tuple[Any, str]] = {}  # last upload (event, lane)
        self._slot_of: Dict[int, int] = {}       # resident expert -> slot (mirrors the cache)
        self._miss_lane = "compute"              # where a demand miss is copied ("epipe": stream-all EPIPE)
        self._slot_ready: Dict[int, Any] = {}    # slot -> event of a side-lane demand copy nobody has waited yet
        # prefetch cycle state (reference :5056-5083)
        self.prefetched_ids: Set[int] = set()
        self.prefetch_used_ids: Set[int] = set()
        self.prefetch_events: Dict[int, Any] = {}
        self.cycle_key: Optional[Tuple[Any, ...]] = None
        self.access_freq: Dict[int, int] = {}
        self.last_used_decode_step: Dict[int, int] = {}
        # rolling gate of the residual scan (reference :4989-4998)
        self._gate_calls = 0
        self._gate_triggers = 0
        self._gate_skip_remaining = 0
        # harness state, set by the block before each call
        self.phase = "none"
        self.call_id = -1
        self.stage = "decode"

    # ------------------------------------------------------------------ events / counters
    def _event(self, kind: str, eid: int) -> None:
        m = self.metrics
        if kind == "hit":
            m.cache_hit_count += 1
        elif kind == "prefetch_hit":
            m.prefetch_hit_count += 1
        else:
            m.cache_miss_count += 1
            if self.staging is not None and self.stage == "decode":
                self.staging.demand_miss(self.layer_idx)
        if m.events is not None:
            m.events.append((kind, self.layer_idx, int(eid)))

    # ------------------------------------------------------------------ slot pool
    def _release_slot(self, slot: int) -> None:
        if slot in self._pending_slots:
            self._retired.append(slot)
        else:
            self._free_slots.append(slot)

    def _acquire_slot(self) -> int:
        if not self._free_slots:
            self.flush()
        if not self._free_slots:
            raise RuntimeError(
                f"Insufficient HBM slots before expert H2D: layer={self.layer_idx} "
                f"slots={self.num_slots} capacity={self.cache.capacity}")
        return self._free_slots.pop()

    def _upload(self, eid: int, slot: int, lane: str) -> Any:
        fence = self._slot_fence.pop(slot, None)
        if fence is not None and lane != "compute":
            self.backend.wait_event(fence, lane, True)
        prev = self._slot_upload.get(slot)
        if prev is not None and prev[1] != lane:
            self.backend.wait_event(prev[0], lane, True)
        ev = self.backend.upload(int(eid), int(slot), lane)
        self._slot_upload[slot] = (ev, lane)
        return ev

    def _enqueue(self, eid: int, slot: int) -> None:
        ready = self._slot_ready.pop(int(slot), None)
        if ready is not None:
            # weights still travelling on a side lane: what is queued goes first, then the
            # compute lane waits this copy and this segment opens the next batch
            self.flush()
            self.backend.wait_event(ready, "compute")
        self._pending.append((int(eid), int(slot)))
        self._pending_slots.add(int(slot))

    def flush(self) -> None:
        """Launch the pending batch; slots it alone kept alive become free."""
        if self._pending:
            self.backend.run_segments(self._pending)
            fence = self.backend.fence()
            for _eid, slot in self._pending:
                self._slot_fence[slot] = fence
            self._pending = []
            self._pending_slots = set()
        if self._retired:
            self._free_slots.extend(self._retired)
            self._retired = []

    # ------------------------------------------------------------------ demand path
    def _cache_protect_ids(self) -> Set[int]:
        """TTL protection (reference :5929-5938); off by default."""
        protect: Set[int] = set()
        ttl = int(self.cfg.cache_ttl_steps)
        if ttl > 0 and self.phase == "decode" and self.call_id >= 0:
            for eid, last in self.last_used_decode_step.items():
                if self.call_id - int(last) <= ttl:
                    protect.add(int(eid))
        return protect

    def _protect_with_fallback(self, new_eid: int) -> Set[int]:
        protect = self._cache_protect_ids()
        protect.discard(int(new_eid))
        resident = set(self.cache.resident_ids())
        if resident and resident.issubset(protect):
            self.metrics.bump("cache_eviction_fallback_all_protected")
            return set()
        return protect

    def _on_demand_access(self, eid: int) -> None:
        """Reference :11213-11221."""
        self.access_freq[eid] = int(self.access_freq.get(eid, 0)) + 1
        if self.phase == "decode":
            self.last_used_decode_step[int(eid)] = int(self.call_id)
        if self.access_freq[eid] >= 2:
            self.cache.promote_hot(eid)
            self._sync_slots()   # entering the hot tier of a tiered cache may push another expert out

    def _sync_slots(self) -> None:
        """Release the slot of every expert the cache no longer holds."""
        if len(self._slot_of) == len(self.cache):
            return
        for eid in [e for e in self._slot_of if not self.cache.has(e)]:
            self.prefetch_events.pop(eid, None)
            self._release_slot(self._slot_of.pop(eid))

    def _cache_put(self, eid: int, slot: int, transient: bool = False) -> None:
        """``_cache_put_guarded`` (reference :5985-6022) plus slot bookkeeping.  ``transient``
        is the entry's ``prefill_scp_transient`` mark: such entries are evicted first."""
        if self.cache.capacity <= 0:
            # nothing is ever stored: the slot only lives until the batch is launched
            self._pending_slots.add(slot)
            self._retired.append(slot)
            return
        protect = self._protect_with_fallback(eid)
        # a repeatedly used expert enters the hot tier of a tiered cache (reference :11223-11232)
        prefer_hot = int(self.access_freq.get(int(eid), 0)) >= 2
        self.cache.put(int(eid), slot, pinned=False, prefer_hot=prefer_hot, protect_ids=protect,
                       prefill_scp_transient=bool(transient))
        if transient:
            self.metrics.bump("prefill_scp_transient_load_count")
        if self.cache.has(int(eid)):
            self._slot_of[int(eid)] = slot
        else:
            # a full tier whose other entries are all pinned or protected gives the newcomer up at
            # once: its slot then only lives until the batch that uses it is launched
            self._pending_slots.add(slot)
            self._retired.append(slot)
        self._sync_slots()

    def _record_cached_use(self, eid: int, wait_prefetch: bool) -> None:
        """Hit accounting shared by the demand path and EPIPE (reference :11395-11412,
        :11652-11670).  A decode hit on an entry staged during prefill makes it an ordinary
        entry again (:11324-11336)."""
        if (self.stage == "decode" and self.cfg.epipe_promote_transient_on_decode_hit
                and self.cache.is_prefill_scp_transient(eid)):
            self.metrics.bump("prefill_scp_transient_hit_count")
            if self.cache.clear_prefill_scp_transient(eid):
                self.metrics.bump("prefill_scp_transient_promote_count")
        if eid in self.prefetched_ids:
            self._event("prefetch_hit", eid)
            self.prefetch_used_ids.add(eid)
            self.cache.unpin(eid)
            self.cache.promote_hot(eid)
            self._sync_slots()
        else:
            self._event("hit", eid)
        if wait_prefetch:
            self._maybe_wait_prefetch(eid)

    def _maybe_wait_prefetch(self, eid: int) -> None:
        """Reference :11176-11210: the compute lane waits the copy event, the host never."""
        ev = self.prefetch_events.pop(eid, None)
        if ev is None:
            return
        if self.backend.event_done(ev):
            self.metrics.prefetch_complete_before_use_count += 1
        self.backend.wait_event(ev, "compute")
        self.metrics.prefetch_completed_count += 1

    def _demand(self, eid: int) -> int:
        """``_get_local_module_weights`` (reference :11388-11435): returns the slot."""
        slot = self.find(eid)
        if slot is not None:
            self._record_cached_use(eid, wait_prefetch=True)
            return slot
        extra = self._extra_get(eid)
        if extra is not None:
            return extra
        self._event("miss", eid)
        slot = self._acquire_slot()
        if self._miss_lane == "compute":
            self._upload(eid, slot, "compute")
        else:
            # stream-all EPIPE: the copy travels on the side lane; the segment is launched behind
            # its event (see _enqueue), whatever was queued before it runs meanwhile
            self._slot_ready[slot] = self._upload(eid, slot, self._miss_lane)
            self.metrics.bump("epipe_stream_all_copies")
        self.metrics.demand_h2d_bytes += self.expert_bytes
        self._on_demand_access(eid)
        self._cache_put(eid, slot)
        return slot

    # ---- prefill side cache (reference :5637-5720) ------------------------------------
    def _extra_enabled(self) -> bool:
        cfg = self.cfg   # reference :5636-5644
        return self.extra_cache.capacity > 0 and bool(
            cfg.epipe_prefill_enable or cfg.epipe_prefill_shadow or cfg.epipe_prefill_multistage_shadow)

    def _extra_readable(self) -> bool:
        return self._extra_enabled() and not (self.stage == "decode"
                                              and not self.cfg.epipe_prefill_extra_cache_decode_read)

    def _extra_get(self, eid: int, touch: bool = True) -> Optional[int]:
        """Slot of an expert staged during prefill; finding it counts as an ordinary hit."""
        if not self._extra_readable():
            return None
        slot = self.extra_cache.get(eid) if touch else self.extra_cache.peek(eid)
        if slot is not None:
            self._event("hit", eid)
            self.metrics.bump("epipe_prefill_extra_cache_hit_count")
        return slot

    def _extra_store(self, eid: int, slot: int) -> bool:
        """Keep a staged payload for later prefill / decode calls: prefill only, bounded by
        slots and by bytes (reference :5647-5685).  Slots of entries it pushes out return to
        the pool."""
        if self.stage != "prefill" or not self._extra_enabled():
            return False
        max_bytes = int(float(self.cfg.epipe_prefill_extra_cache_max_mb) * 1024.0 * 1024.0)
        if (max_bytes > 0 and not self.extra_cache.has(eid)
                and self.extra_cache.resident_nbytes() + self.expert_bytes > max_bytes):
            self.metrics.bump("epipe_prefill_extra_cache_no_room_count")
            return False
        before = {e: self.extra_cache.peek(e) for e in self.extra_cache.resident_ids()}
        kept, _updated, _evicted = self.extra_cache.put(eid, slot, nbytes=self.expert_bytes)
        for e, s_old in before.items():
            if not self.extra_cache.has(e) or (e == eid and s_old != slot):
                self._release_slot(s_old)
        return bool(kept)

    def clear_extra_cache(self) -> int:
        for eid in self.extra_cache.resident_ids():
            self._release_slot(self.extra_cache.peek(eid))
        return self.extra_cache.clear()

    def _compute(self, eid: int, slot: Optional[int] = None) -> None:
        """Queue expert ``eid`` for execution, loading it on demand when no slot is given."""
        if slot is None:
            slot = self._demand(eid)
        self._enqueue(eid, slot)

    # ------------------------------------------------------------------ executors
    def execute(self, segments: Sequence[Segment]) -> str:
        """Run the routed experts of one call; ``segments`` is ``(eid, rows)`` ascending by
        expert id.  Picks the executor like ``_execute_local_recv_groups`` (reference
        :13264-13357) and returns its name."""
        if not segments:
            return "empty"
        name = None
        epipe = self._epipe_stage_enabled() and self.cfg.epipe_mode != "off" and not self.cfg.world1_exact
        self._miss_lane = "epipe" if (epipe and self.cfg.epipe_stream_all) else "compute"
        try:
            name = self._execute(segments, epipe)
        finally:
            self._miss_lane = "compute"
        return name

    def _execute(self, segments: Sequence[Segment], epipe: bool) -> str:
        name = None
        if epipe:
            rs_active = self.cfg.planner_mode == "rs_prefetch"
            mode = self.cfg.epipe_decode_rs_mode
            if self.stage == "decode" and rs_active and mode == "off":
                name = None
            elif self.stage == "decode" and rs_active and mode == "residual_scan":
                if self.staging is not None:
                    # staged experts are classified like cached ones by the upfront scan
                    # (utils/rs_overlap.py:474-479)
                    self.staging.count("unified_epipe_calls")
                    name = self._epipe_upfront_scan(segments)
                else:
                    name = self._epipe_rs_residual_scan(segments)
            elif self.stage == "decode" and rs_active and mode in ("buffered", "late_only", "demand_only"):
                name = self._epipe_rs_buffered(segments)
            elif self.stage == "decode" and not rs_active and self.cfg.epipe_mode != "miss_triggered":
                name = self._epipe_upfront_scan(segments)
            elif self.cfg.epipe_mode == "upfront_scan":
                name = self._epipe_upfront_scan(segments)
            else:
                name = self._epipe_miss_triggered(segments)
        if name is None:
            for eid, _rows in segments:
                self._compute(eid)
            name = "plain"
        self.flush()
        return name

    def _epipe_stage_enabled(self) -> bool:
        """Reference :5585-5598."""
        cfg = self.cfg
        if self.stage == "prefill":
            return bool(cfg.epipe_prefill_enable or cfg.epipe_prefill_shadow or cfg.epipe_prefill_multistage_shadow)
        if self.stage == "decode":
            if cfg.planner_mode == "rs_prefetch":
                return bool(cfg.epipe_enable and cfg.epipe_decode_rs_mode not in ("off", "disabled"))
            return bool(cfg.epipe_enable or cfg.epipe_shadow)
        return False

    def _shadow_for_stage(self) -> bool:
        cfg = self.cfg
        if self.stage == "decode":
            return bool(cfg.epipe_shadow)
        return bool(cfg.epipe_prefill_shadow or cfg.epipe_prefill_multistage_shadow)

    def _record_multistage_shadow(self, ready: Sequence[Segment], missing: Sequence[Segment]) -> None:
        """What staging the n largest missing experts of a prefill call at once would have moved and
        hidden (reference :5738-5778); counters only."""
        cfg, m = self.cfg, self.metrics
        if self.stage != "prefill" or not cfg.epipe_prefill_multistage_shadow:
            return
        ready_items = sum(r for _, r in ready)
        m.bump("epipe_prefill_multistage_shadow_count")
        m.bump("epipe_prefill_multistage_ready_expert_count", len(ready))
        m.bump("epipe_prefill_multistage_missing_expert_count", len(missing))
        m.bump("epipe_prefill_multistage_ready_item_count", ready_items)
        m.bump("epipe_prefill_multistage_missing_item_count", sum(r for _, r in missing))
        if not missing:
            return
        ranked = sorted((int(r) for _, r in missing), reverse=True)   # stable: equal sizes keep segment order
        max_n = max(1, int(cfg.epipe_prefill_multistage_max_n))
        top = ranked[:min(max_n, len(ranked))]
        m.bump("epipe_prefill_multistage_top_missing_item_count_sum", sum(top))
        m.bump("epipe_prefill_multistage_est_expert_h2d_bytes", len(top) * self.expert_bytes)
        m.bump("epipe_prefill_multistage_est_ready_compute_items", ready_items)
        for n in (1, 2, 4):
            if max_n >= n:
                m.bump(f"epipe_prefill_multistage_est_hidden_h2d_items_n{n}", sum(ranked[:min(n, len(ranked))]))

    def _contains_no_touch(self, eid: int) -> bool:
        """Reference :5815-5851."""
        return (self._extra_readable() and self.extra_cache.has(eid)) or self.holds(eid)

    def _headroom_ok(self) -> bool:
        """A transient needs a slot that no cache entry owns."""
        return bool(self._free_slots) or bool(self._retired) or bool(self._pending)

    def _fallback(self, reason: str) -> None:
        self.metrics.bump("epipe_fallback_count")
        if reason:
            self.metrics.bump(reason)

    # ---- EPIPE without RS, and prefill: upfront scan (reference :11867-12167) ----------
    def _epipe_upfront_scan(self, segments: Sequence[Segment]) -> Optional[str]:
        cfg, m = self.cfg, self.metrics
        stage = self.stage
        enabled = bool(cfg.epipe_enable if stage == "decode" else cfg.epipe_prefill_enable)
        shadow = self._shadow_for_stage()
        if not (enabled or shadow):
            return None
        ready = [s for s in segments if self._contains_no_touch(s[0])]
        missing = [s for s in segments if not self._contains_no_touch(s[0])]
        ready_items = sum(r for _, r in ready)
        free_cache_slots = max(0, self.cache.capacity - len(self.cache))
        self._record_multistage_shadow(ready, missing)
        if shadow and not enabled:      # reference :11919-11932: count the opportunity, execute nothing
            m.bump("epipe_shadow_count")
            m.bump("epipe_ready_expert_count", len(ready))
            m.bump("epipe_missing_expert_count", len(missing))
            m.bump("epipe_ready_item_count", ready_items)
            m.bump("epipe_missing_item_count", sum(r for _, r in missing))
            m.bump("epipe_missing_h2d_bytes_est", len(missing) * self.expert_bytes)
            if free_cache_slots > 0:
                m.bump("epipe_cache_free_slot_count", free_cache_slots)
            elif missing and cfg.epipe_transient_staging:
                m.bump("epipe_cache_full_staged_count")
            return None
        if not cfg.epipe_no_evict:
            raise NotImplementedError("SPARSE_EPIPE_NO_EVICT=0 is not implemented in EPIPE-Lite.")
        if cfg.epipe_max_staged_experts != 1:
            raise NotImplementedError("EPIPE-Lite currently supports only one staged missing expert.")
        if len(ready) < cfg.epipe_min_ready_experts or ready_items < cfg.epipe_min_ready_items:
            self._fallback("epipe_fallback_no_ready")
            return None
        if len(missing) < cfg.epipe_min_missing_experts:
            self._fallback("epipe_fallback_no_missing")
            return None
        staged_eid = missing[0][0]
        can_insert = (free_cache_slots > 0 and cfg.cache_policy != "tiered"
                      and not (stage == "prefill" and not cfg.epipe_prefill_commit))
        use_transient = not can_insert
        if use_transient:
            if not cfg.epipe_transient_staging:
                self._fallback("epipe_fallback_cache_full_no_temp")
                return None
            if not self._headroom_ok():
                self._fallback("epipe_fallback_no_memory_headroom")
                return None
        # stage the first missing expert on the EPIPE lane
        slot = self._acquire_slot()
        stage_event = self._upload(staged_eid, slot, "epipe")
        ready_order = list(ready)
        if cfg.epipe_sort_ready_by_work:
            ready_order.sort(key=lambda s: s[1], reverse=True)
        for eid, _rows in ready_order:
            # prefill with `epipe_prefill_no_touch_ready`: the ready expert is read where it lies, its
            # place in the LRU unchanged (reference :12020-12021, :11672-11698)
            ready_slot = (self._ready_slot_for_compute(eid)
                          if stage == "prefill" and cfg.epipe_prefill_no_touch_ready else None)
            self._compute(eid, ready_slot)
        # the ready batch must be on the device before the compute lane waits the copy
        self.flush()
        self.backend.wait_event(stage_event, "compute")
        self._event("miss", staged_eid)
        if stage != "prefill":
            self._on_demand_access(staged_eid)
        m.demand_h2d_bytes += self.expert_bytes
        m.bump("epipe_staged_missing_count")
        m.bump("epipe_enabled_count")
        m.bump("epipe_staged_expert_count")
        m.bump("epipe_no_evict_count")
        m.bump("epipe_ready_expert_count", len(ready))
        m.bump("epipe_missing_expert_count", len(missing))
        m.bump("epipe_ready_item_count", ready_items)
        m.bump("epipe_missing_item_count", sum(r for _, r in missing))
        m.bump("epipe_missing_h2d_bytes_est", len(missing) * self.expert_bytes)
        if free_cache_slots > 0:
            m.bump("epipe_cache_free_slot_count", free_cache_slots)
        kept = False  # does some cache keep the staged slot alive after this call?
        if can_insert:
            if len(self.cache) < self.cache.capacity:
                if stage == "prefill":
                    self._on_demand_access(staged_eid)
                self._enqueue(staged_eid, slot)
                self._cache_put(staged_eid, slot,
                                transient=stage == "prefill" and cfg.epipe_prefill_mark_transient)
                m.bump("epipe_cache_insert_count")
                kept = True
            else:
                use_transient = True
        if not kept:
            self._enqueue(staged_eid, slot)
            if use_transient and stage == "prefill":
                kept = self._extra_store(staged_eid, slot)
            if not kept:
                if use_transient:
                    m.bump("epipe_cache_full_staged_count")
                m.bump("epipe_transient_payload_count")
                self._retired.append(slot)  # back to the pool once this batch is launched
        for eid, _rows in missing[1:]:
            self._compute(eid)
        return "epipe_upfront"

    # ---- EPIPE on top of RS prefetch: residual scan (reference :12169-12512) -----------
    def _pending_prefetch_event(self, eid: int):
        """Reference :11636-11650: an event that is still in flight, else None."""
        ev = self.prefetch_events.get(eid)
        if ev is None:
            return None
        if self.backend.event_done(ev):
            self.prefetch_events.pop(eid, None)
            self.metrics.prefetch_complete_before_use_count += 1
            self.metrics.prefetch_completed_count += 1
            return None
        return ev

    def _demand_gate_can_open(self) -> bool:
        """Reference :5880-5893: forced open, or open once the exposed demand-copy time of the decode
        phase (as far as the metrics have it: sampled or measured, whichever is larger) exceeds the
        threshold."""
        if not self._handle_demand():
            return False
        if self.cfg.epipe_rs_force_demand_stage:
            return True
        threshold = float(self.cfg.epipe_rs_demand_stage_threshold_ms)
        if threshold <= 0.0:
            return False
        observed = max(float(getattr(self.metrics, "sampled_demand_h2d_exposed_decode_ms", 0.0)),
                       float(getattr(self.metrics, "demand_h2d_exposed_decode_ms", 0.0)))
        return observed > threshold

    def _handle_late(self) -> bool:
        """``demand_only`` switches the handling of late prefetches off (reference :4975-4984)."""
        return bool(self.cfg.epipe_rs_handle_late_prefetch) and self.cfg.epipe_decode_rs_mode != "demand_only"

    def _handle_demand(self) -> bool:
        """``late_only`` switches the staging of demand misses off."""
        return bool(self.cfg.epipe_rs_handle_demand_miss) and self.cfg.epipe_decode_rs_mode != "late_only"

    def _residual_present(self, segments: Sequence[Segment]) -> bool:
        for eid, _rows in segments:
            ev = self.prefetch_events.get(eid)
            if ev is not None and self._handle_late() and not self.backend.event_done(ev):
                return True
            if self._demand_gate_can_open() and not self._contains_no_touch(eid):
                return True
        return False

    def _maybe_skip_gate(self, segments: Sequence[Segment]) -> bool:
        cfg = self.cfg
        if not cfg.epipe_rs_rolling_gate:
            return False
        if self._gate_skip_remaining > 0:
            if self._residual_present(segments):
                self._gate_skip_remaining = 0
                self.metrics.bump("epipe_rs_gate_reenable_count")
                return False
            self._gate_skip_remaining -= 1
            self.metrics.bump("epipe_rs_gate_skip_count")
            return True
        self._gate_calls += 1
        if self._gate_calls >= cfg.epipe_rs_gate_window and self._gate_triggers < cfg.epipe_rs_gate_min_triggers:
            self._gate_calls = 0
            self._gate_triggers = 0
            self._gate_skip_remaining = int(cfg.epipe_rs_gate_skip_steps)
            if self._gate_skip_remaining > 0:
                self.metrics.bump("epipe_rs_gate_skip_count")
                self._gate_skip_remaining -= 1
                return True
        if self._gate_calls >= cfg.epipe_rs_gate_window:
            self._gate_calls = 0
            self._gate_triggers = 0
        return False

    def _epipe_rs_residual_scan(self, segments: Sequence[Segment]) -> Optional[str]:
        cfg, m = self.cfg, self.metrics
        if self.stage != "decode" or cfg.planner_mode != "rs_prefetch" or not cfg.epipe_enable:
            return None
        m.bump("epipe_rs_residual_scan_calls")
        if self._maybe_skip_gate(segments):
            return None
        ready_idx: List[int] = []
        late_idx: List[int] = []
        demand_idx: List[int] = []
        for i, (eid, _rows) in enumerate(segments):
            pending_ev = self._pending_prefetch_event(eid)
            cached = self._contains_no_touch(eid)
            if cached and pending_ev is None:
                ready_idx.append(i)
            elif cached and pending_ev is not None and cfg.epipe_rs_handle_late_prefetch:
                late_idx.append(i)
            elif (not cached) and cfg.epipe_rs_handle_demand_miss and self._demand_gate_can_open():
                demand_idx.append(i)
        ready_items = sum(segments[i][1] for i in ready_idx)
        policy = self.light_policy
        if policy is not None:
            policy.observe_ready(len(ready_idx), ready_items)
        if len(ready_idx) < cfg.epipe_rs_min_buffer_groups or ready_items < cfg.epipe_rs_min_buffer_items:
            m.bump("epipe_rs_residual_scan_no_ready_count")
            return None
        residual: Optional[int] = None
        kind = ""
        if late_idx:
            residual, kind = late_idx[0], "late"
        elif demand_idx and self._demand_gate_open(ready_items):
            residual, kind = demand_idx[0], "demand"
        if policy is not None and policy.feedback:
            # cost-aware choice among all candidates, late ones first (reference :12342-12348)
            stageable = demand_idx if self._demand_gate_open(ready_items) else []
            candidates = [(i, segments[i][0], "late") for i in late_idx]
            candidates.extend((i, segments[i][0], "demand") for i in stageable)
            chosen = policy.residual(len(ready_idx), ready_items, candidates)
            residual, kind = chosen if chosen is not None else (None, "")
        if residual is None:
            m.bump("epipe_fallback_no_miss_trigger")
            return None
        residual_eid = segments[residual][0]
        cover = [i for i in ready_idx if i != residual]
        if len(cover) < cfg.epipe_rs_min_buffer_groups:
            m.bump("epipe_rs_residual_scan_no_ready_count")
            return None
        m.bump("epipe_rs_trigger_count")
        m.bump("epipe_rs_residual_scan_late_count" if kind == "late" else "epipe_rs_residual_scan_demand_count")
        if cfg.epipe_rs_rolling_gate:
            self._gate_triggers += 1

        def compute_ready(indices: Sequence[int]) -> None:
            for i in indices:
                eid = segments[i][0]
                slot = self.cache.get(eid)
                if slot is None:
                    self._compute(eid)
                else:
                    self._record_cached_use(eid, wait_prefetch=False)
                    self._compute(eid, slot)

        done: Set[int] = set()
        if kind == "late":
            slot = self.cache.get(residual_eid)
            if slot is None:
                return None
            compute_ready(cover)
            done.update(cover)
            self.flush()  # resident experts run while the late copy lands
            self._maybe_wait_prefetch(residual_eid)
            self._record_cached_use(residual_eid, wait_prefetch=False)
            m.bump("epipe_enabled_count")
            m.bump("epipe_rs_late_prefetch_overlap_count")
            self._compute(residual_eid, slot)
            done.add(residual)
        else:
            if not self._headroom_ok():
                self._fallback("epipe_fallback_memory")
                return None
            slot = self._acquire_slot()
            stage_event = self._upload(residual_eid, slot, "epipe")
            compute_ready(cover)
            done.update(cover)
            self.flush()
            self.backend.wait_event(stage_event, "compute")
            self._event("miss", residual_eid)
            self._on_demand_access(residual_eid)
            m.demand_h2d_bytes += self.expert_bytes
            free_cache_slots = max(0, self.cache.capacity - len(self.cache))
            commit = bool(cfg.epipe_rs_demand_commit and cfg.epipe_deferred_lru_commit
                          and (free_cache_slots > 0 or not cfg.epipe_no_evict))
            self._enqueue(residual_eid, slot)
            if commit and self.cache.capacity > 0:
                self._cache_put(residual_eid, slot)
                m.bump("epipe_cache_insert_count")
            else:
                self._retired.append(slot)
                m.bump("epipe_transient_payload_count")
            m.bump("epipe_enabled_count")
            m.bump("epipe_staged_missing_count")
            done.add(residual)
        for i, (eid, _rows) in enumerate(segments):
            if i not in done:
                self._compute(eid)
        if cfg.epipe_rs_rolling_gate and self._gate_skip_remaining > 0:
            self._gate_skip_remaining = 0
            m.bump("epipe_rs_gate_reenable_count")
        return "epipe_rs_residual_scan"

    def _demand_gate_open(self, ready_items: int) -> bool:
        """Reference :5895-5907."""
        if not self._handle_demand():
            return False
        if ready_items < self.cfg.epipe_rs_min_buffer_items:
            return False
        return self._demand_gate_can_open()

    def _stage_on_epipe_lane(self, eid: int) -> Tuple[int, Any]:
        slot = self._acquire_slot()
        return slot, self._upload(eid, slot, "epipe")

    def _finish_staged(self, eid: int, slot: int, stage_event: Any, commit: bool, transient: bool = False,
                       to_extra: bool = False) -> bool:
        """Wait a staged copy on the compute lane, queue the expert, and either commit its
        slot to the cache, hand it to the prefill side cache, or let it go after the batch."""
        m = self.metrics
        self.backend.wait_event(stage_event, "compute")
        m.demand_h2d_bytes += self.expert_bytes
        self._enqueue(eid, slot)
        kept = False
        if commit and self.cache.capacity > 0:
            self._cache_put(eid, slot, transient=transient)
            m.bump("epipe_cache_insert_count")
            kept = True
        elif to_extra:
            kept = self._extra_store(eid, slot)
        if not kept:
            m.bump("epipe_transient_payload_count")
            self._retired.append(slot)
        m.bump("epipe_enabled_count")
        m.bump("epipe_staged_missing_count")
        return kept

    # ---- EPIPE on top of RS prefetch: bounded ready buffer (reference :12514-12843) -----
    def _epipe_rs_buffered(self, segments: Sequence[Segment]) -> Optional[str]:
        """One pass in ascending expert id.  Resident experts are counted as hits when seen
        and queued; the queue is launched before any segment that has to wait (a prefetch in
        flight, a staged copy), so the wait only starts once the resident work is on the
        device.  The reference also drains its buffer every ``max_groups`` / ``max_items``;
        here that only closes a batch, which changes no order."""
        cfg, m = self.cfg, self.metrics
        if self.stage != "decode" or cfg.planner_mode != "rs_prefetch" or not cfg.epipe_enable:
            return None
        m.bump("epipe_rs_buffered_calls")
        if self._maybe_skip_gate(segments):
            return None
        handle_late, handle_demand = self._handle_late(), self._handle_demand()
        groups = items = 0
        trigger_seen = False

        def drain() -> None:
            nonlocal groups, items
            self.flush()
            if groups:
                m.bump("epipe_rs_buffer_flush_count")
            groups = items = 0

        def sufficient() -> bool:
            return groups >= cfg.epipe_rs_min_buffer_groups and items >= cfg.epipe_rs_min_buffer_items

        def trigger(kind: str) -> None:
            nonlocal trigger_seen
            m.bump("epipe_rs_trigger_count")
            m.bump(kind)
            if cfg.epipe_rs_rolling_gate:
                self._gate_triggers += 1
            trigger_seen = True

        for eid, rows in segments:
            pending = self._pending_prefetch_event(eid)
            slot = self.cache.get(eid)
            if slot is not None:
                if pending is None:
                    self._record_cached_use(eid, wait_prefetch=False)
                    self._enqueue(eid, slot)
                    groups += 1
                    items += rows
                    if groups >= cfg.epipe_rs_buffer_max_groups or items >= cfg.epipe_rs_buffer_max_items:
                        groups = items = 0      # the reference's buffer starts over here
                    continue
                if not handle_late:
                    drain()
                    self._record_cached_use(eid, wait_prefetch=True)
                    self._enqueue(eid, slot)
                    continue
                trigger("epipe_rs_late_prefetch_trigger_count")
                if not sufficient():
                    m.bump("epipe_rs_buffer_too_small_count")
                    drain()
                    self._record_cached_use(eid, wait_prefetch=True)
                    self._enqueue(eid, slot)
                    continue
                drain()
                self._maybe_wait_prefetch(eid)
                self._record_cached_use(eid, wait_prefetch=False)
                m.bump("epipe_enabled_count")
                m.bump("epipe_rs_late_prefetch_overlap_count")
                self._enqueue(eid, slot)
                continue
            if not handle_demand:
                drain()
                self._compute(eid)
                continue
            trigger("epipe_rs_demand_miss_trigger_count")
            if not sufficient() or not self._demand_gate_open(items):
                if not sufficient():
                    m.bump("epipe_rs_buffer_too_small_count")
                drain()
                self._compute(eid)
                continue
            if not self._headroom_ok():
                self._fallback("epipe_fallback_memory")
                drain()
                self._compute(eid)
                continue
            slot, stage_event = self._stage_on_epipe_lane(eid)
            drain()
            self._event("miss", eid)
            self._on_demand_access(eid)
            free_cache_slots = max(0, self.cache.capacity - len(self.cache))
            commit = bool(cfg.epipe_rs_demand_commit and cfg.epipe_deferred_lru_commit
                          and (free_cache_slots > 0 or not cfg.epipe_no_evict))
            self._finish_staged(eid, slot, stage_event, commit)
            m.bump("epipe_rs_demand_stage_count")
        if trigger_seen and cfg.epipe_rs_rolling_gate and self._gate_skip_remaining > 0:
            self._gate_skip_remaining = 0
            m.bump("epipe_rs_gate_reenable_count")
        if not trigger_seen:
            m.bump("epipe_fallback_no_miss_trigger")
        return "epipe_rs_buffered"

    # ---- EPIPE, miss-triggered look-ahead (reference :12845-13154) -----------------------
    def _ready_slot_for_compute(self, eid: int) -> Optional[int]:
        """Reference :11672-11698: the cache first (touched, counted as a hit, a pending copy
        waited for), then the prefill side cache (touched, not counted)."""
        no_touch = self.stage == "prefill" and self.cfg.epipe_prefill_no_touch_ready
        slot = self.cache.peek(eid) if no_touch else self.cache.get(eid)
        if slot is not None:
            self._record_cached_use(eid, wait_prefetch=True)
            return slot
        return self._extra_get(eid, touch=not no_touch)

    def _epipe_miss_triggered(self, segments: Sequence[Segment]) -> Optional[str]:
        """Walk the segments in ascending expert id; at the first miss look a few segments
        ahead for resident experts, stage the missing expert on the EPIPE lane, run those
        resident experts meanwhile, then wait, count the miss and run it.  Later misses of
        the call take the ordinary demand path."""
        cfg, m = self.cfg, self.metrics
        stage, rs_active = self.stage, cfg.planner_mode == "rs_prefetch"
        enabled = bool(cfg.epipe_prefill_enable if stage == "prefill" else cfg.epipe_enable)
        shadow = self._shadow_for_stage()
        if not (enabled or shadow):
            return None
        mode = cfg.epipe_decode_rs_mode
        if stage == "decode" and rs_active and mode == "off":
            return None
        if stage == "decode" and rs_active and mode == "buffered":
            return self._epipe_rs_buffered(segments)
        if stage == "decode" and rs_active and mode == "upfront_scan":
            return self._epipe_upfront_scan(segments)
        min_ready_items = (cfg.epipe_prefill_lookahead_min_ready_items if stage == "prefill"
                           else cfg.epipe_lookahead_min_ready_items)
        done: Set[int] = set()
        staged_once = False
        for i, (eid, _rows) in enumerate(segments):
            if i in done:
                continue
            slot = self._ready_slot_for_compute(eid)
            if slot is not None:
                self._enqueue(eid, slot)
                continue
            if staged_once:
                self._compute(eid)
                continue
            ahead = [j for j in range(i + 1, min(len(segments), i + 1 + int(cfg.epipe_lookahead_experts)))
                     if j not in done and self._contains_no_touch(segments[j][0])]
            ready_items = sum(segments[j][1] for j in ahead)
            if shadow and not enabled:   # reference :12982-12991: count the opportunity, take the demand path
                if ahead:
                    m.bump("epipe_prefill_shadow_opportunity_count" if stage == "prefill" else "epipe_shadow_count")
                m.bump("epipe_lookahead_ready_group_count", len(ahead))
                m.bump("epipe_lookahead_ready_item_count", ready_items)
                self._compute(eid)
                continue
            if not ahead:
                self._fallback("epipe_fallback_no_ready_lookahead")
                self._compute(eid)
                continue
            if ready_items < min_ready_items:
                self._fallback("epipe_fallback_low_ready_items")
                self._compute(eid)
                continue
            if not self._headroom_ok():
                self._fallback("epipe_fallback_memory")
                self._compute(eid)
                continue
            slot, stage_event = self._stage_on_epipe_lane(eid)
            for j in ahead:
                self._compute(segments[j][0])
                done.add(j)
            self.flush()   # everything queued so far runs while the copy lands
            self._event("miss", eid)
            if stage != "prefill":
                self._on_demand_access(eid)
            free_cache_slots = max(0, self.cache.capacity - len(self.cache))
            if free_cache_slots > 0:
                m.bump("epipe_cache_free_slot_count", free_cache_slots)
            if stage == "prefill":
                commit_allowed, mark = bool(cfg.epipe_prefill_commit), bool(cfg.epipe_prefill_mark_transient)
            elif rs_active:
                commit_allowed, mark = bool(cfg.epipe_decode_rs_commit) or free_cache_slots > 0, False
            else:
                commit_allowed, mark = bool(cfg.epipe_decode_no_rs_commit), False
            insert = bool(commit_allowed and cfg.epipe_deferred_lru_commit
                          and (free_cache_slots > 0 or not cfg.epipe_no_evict))
            if stage == "prefill" and insert:
                self._on_demand_access(eid)
            kept = self._finish_staged(eid, slot, stage_event, insert, transient=mark, to_extra=stage == "prefill")
            if not kept and free_cache_slots <= 0:
                m.bump("epipe_cache_full_staged_count")
            # reference :13132-13142
            m.bump("epipe_staged_expert_count")
            m.bump("epipe_ready_expert_count", len(ahead))
            m.bump("epipe_ready_item_count", ready_items)
            m.bump("epipe_lookahead_ready_group_count", len(ahead))
            m.bump("epipe_lookahead_ready_item_count", ready_items)
            m.bump("epipe_missing_expert_count")
            m.bump("epipe_missing_item_count", _rows)
            m.bump("epipe_missing_h2d_bytes_est", self.expert_bytes)
            staged_once = True
        return "epipe_miss_triggered"

    # ------------------------------------------------------------------ RS prefetch
    # ---- staged experts: a third state of the slot table ---------------------------------
    # Besides *resident* (the LRU owns the slot) and *transient* (the slot lives for one batch)
    # an expert can be *staged*: a forecast copied it into a slot of the layer's ring, this
    # call's lookups may read it there, and the LRU learns of it only at the call's end and
    # only if a lookup really used it.  A wrong forecast therefore never evicts and never
    # moves recency (the ownership rule of utils/rs_staging.py:52-94).
    @property
    def _pool_slots(self) -> List[int]:
        return self.ring.slots if self.ring is not None else []

    def staging_ring(self, positions: int) -> StagingRing:
        """The layer's ring, which must have at least ``positions`` slots."""
        have = len(self.ring) if self.ring is not None else 0
        if positions > have:
            raise ValueError(
                f"layer {self.layer_idx}: {positions} staging slots asked, {have} reserved "
                "(set ResidencyConfig.staging_pool_slots before the block is built)")
        return self.ring

    def find(self, eid: int, touch: bool = True) -> Optional[int]:
        """Slot that holds ``eid`` for this call, or None.  A resident copy wins over a staged
        one; ``touch`` moves the LRU's recency for the former and records first use of the
        latter."""
        slot = self.cache.get(eid) if touch else self.cache.peek(eid)
        if slot is not None:
            return slot
        rec = self.staged.get(int(eid))
        if rec is None:
            return None
        if touch and not rec.touched:
            rec.touched = True
            self.staged_touched.append(int(eid))
        return rec.slot

    def holds(self, eid: int) -> bool:
        return bool(self.cache.has(eid)) or int(eid) in self.staged

    def expose_staged(self, filled: Sequence[Tuple[int, int, Any]]) -> None:
        """Make the copies of a sealed ring window readable: ``(expert, ring position, copy
        event)``.  They count as issued prefetches; the compute lane waits a copy's event on
        first use like that of any prefetch (utils/rs_overlap.py:326-340)."""
        assert not self.staged and not self.staged_touched, "the last call's staged experts were not settled"
        for eid, pos, event in filled:
            self.staged[int(eid)] = StagedExpert(pos, self.ring.slots[pos], event)
            self.prefetched_ids.add(int(eid))
            self.prefetch_events[int(eid)] = event
            self.metrics.prefetch_h2d_bytes += self.expert_bytes
            self.metrics.prefetch_issued_count += 1
            self.metrics.prefetch_admitted_count += 1

    def _keep_staged(self, eid: int, rec: StagedExpert) -> None:
        """Admit a staged expert that was used to the LRU where its bytes are: its slot becomes
        the cache's; the ring gets the slot of the resident it pushed out, or a free one while
        the cache is not full (utils/rs_overlap.py:352-381 exchanges payload objects)."""
        if self.cache.capacity <= 0:
            return
        self._on_demand_access(eid)
        self.cache.put(int(eid), rec.slot, pinned=False, protect_ids=self._protect_with_fallback(eid))
        if not self.cache.has(eid):
            return
        self._slot_of[int(eid)] = rec.slot
        self._slot_upload[rec.slot] = (rec.event, "staging")
        pushed_out = [e for e in self._slot_of if not self.cache.has(e)]
        assert len(pushed_out) <= 1, "staging needs the plain per-layer LRU"
        if pushed_out:
            self.prefetch_events.pop(pushed_out[0], None)
            rec.ring_slot, rec.recycled = self._slot_of.pop(pushed_out[0]), True
        else:
            rec.ring_slot = self._acquire_slot()
        rec.kept = True

    def settle_staged(self) -> List[Tuple[int, StagedExpert]]:
        """End of the layer call: keep what was used (first-use order), give every ring position
        back -- a used one behind a fence on the compute lane, an unused one behind its own
        copy -- and forget the staged state (utils/rs_overlap.py:383-408).  Returns the settled
        records, used ones first."""
        if not self.staged:
            return []
        fence = self.backend.fence() if self.staged_touched else None   # after every reader of this call
        for eid in self.staged_touched:
            self._keep_staged(eid, self.staged[eid])
        order = self.staged_touched + [e for e in self.staged if not self.staged[e].touched]
        settled = [(e, self.staged[e]) for e in order]
        for eid, rec in settled:
            self.ring.give_back(rec.pos, fence if rec.touched else rec.event, rec.ring_slot if rec.kept else None)
            if not rec.touched:
                self.metrics.prefetch_wasted_count += 1
                self.staged_unconfirmed += 1
            self.prefetch_events.pop(eid, None)
            self.prefetched_ids.discard(eid)
            self.prefetch_used_ids.discard(eid)
        self.staged, self.staged_touched = {}, []
        return settled

    def confirm_staged_copies(self) -> None:
        """After the copy lane has drained: the unused copies have completed too."""
        self.metrics.prefetch_completed_count += self.staged_unconfirmed
        self.staged_unconfirmed = 0

    def min_candidate_score(self) -> float:
        """``_prefetch_min_candidate_score`` with the cache-safe floor (reference :4954-4972)."""
        score = float(self.cfg.min_candidate_score)
        if self.cfg.rs_policy in ("cache_safe", "cache-safe", "benefit_gate", "benefit-gate"):
            score = max(score, float(self.cfg.cache_safe_min_score))
        return score

    def effective_top_m(self) -> int:
        return max(0, int(self.cfg.prefetch_top_m))

    def predict_topk(self) -> int:
        """Reference :10888-10901."""
        if self.cfg.pred_topk is not None:
            return max(1, min(int(self.cfg.pred_topk), self.num_experts))
        return max(self.top_k, min(self.num_experts, self.effective_top_m()))

    def finalize_prev_group_prefetch(self) -> None:
        """Reference :9619-9635."""
        for eid, ev in list(self.prefetch_events.items()):
            if self.backend.event_done(ev):
                self.metrics.prefetch_completed_count += 1
                self.prefetch_events.pop(eid, None)
        self.metrics.prefetch_wasted_count += len(self.prefetched_ids - self.prefetch_used_ids)
        self.cache.unpin_all()
        self.prefetched_ids.clear()
        self.prefetch_used_ids.clear()
        self.cycle_key = None

    def _begin_cycle(self, key: Tuple[Any, ...]) -> None:
        if self.cycle_key == key:
            return
        self.finalize_prev_group_prefetch()
        self.cycle_key = key

    def prefetch_protect_ids(self) -> Set[int]:
        """Reference :9651-9665."""
        if self.cfg.protect_mode in ("minimal", "current_next", "current-next"):
            protect = set(self.prefetch_used_ids)
        else:
            protect = set(self.prefetched_ids) | set(self.prefetch_used_ids)
        protect.update(self._cache_protect_ids())
        recent = int(self.cfg.recent_protect_steps)
        if recent > 0 and self.phase == "decode" and self.call_id >= 0:
            for eid, last in self.last_used_decode_step.items():
                if self.call_id - int(last) <= recent:
                    protect.add(int(eid))
        return protect

    def prefetch_budget(self, cycle_key: Tuple[Any, ...]) -> int:
        """``_prefetch_target_budget`` (reference :9785-9810)."""
        top_m = self.effective_top_m()
        if self.cfg.planner_mode != "rs_prefetch" or top_m <= 0 or self.num_experts == 0:
            return 0
        self._begin_cycle(cycle_key)
        protect = self.prefetch_protect_ids()
        room = self.cache.prefetch_free_slots()
        if self.cfg.allow_active_replace:
            room += len(self.cache.evictable_prefetch_ids(protect))
        budget = max(0, min(max(0, top_m - len(self.prefetched_ids)), room))
        if budget <= 0:
            self.metrics.prefetch_budget_zero_count += 1
        else:
            self.metrics.prefetch_budget_positive_count += 1
        return budget

    @staticmethod
    def score_map(flat_ids: Sequence[int], flat_probs: Sequence[float]) -> Dict[int, float]:
        """Aggregate predicted probabilities per expert (reference :10040-10107):
        ``sum * (1 + 0.15*(count-1)) + 0.05*max``, keyed in first-seen order."""
        total: Dict[int, float] = {}
        count: Dict[int, int] = {}
        peak: Dict[int, float] = {}
        for eid, p in zip(flat_ids, flat_probs):
            eid, p = int(eid), float(p)
            total[eid] = total.get(eid, 0.0) + p
            count[eid] = count.get(eid, 0) + 1
            peak[eid] = max(peak.get(eid, 0.0), p)
        return {eid: total[eid] * (1.0 + 0.15 * float(max(count[eid] - 1, 0))) + 0.05 * peak[eid]
                for eid in total}

    def _keep_bias(self, eid: int) -> float:
        """Reference :10031-10038 (no hot tier in the plain LRU)."""
        bias = 0.02 * float(min(self.access_freq.get(int(eid), 0), 16))
        if int(eid) in self.prefetched_ids:
            bias += 0.10
        return bias

    def build_plan(self, scores: Dict[int, float], protect: Set[int],
                   budget: int) -> List[Tuple[int, Optional[int]]]:
        """``_build_prefetch_plan_from_score_map`` (reference :10144-10262)."""
        cfg, m = self.cfg, self.metrics
        if budget <= 0 or not scores:
            return []
        min_score, adv, margin = cfg.min_candidate_score, cfg.replace_advantage, cfg.replace_margin
        if cfg.rs_policy in ("cache_safe", "cache-safe", "benefit_gate", "benefit-gate"):
            min_score = max(min_score, cfg.cache_safe_min_score)
            adv = max(adv, cfg.cache_safe_replace_advantage)
            margin = max(margin, cfg.cache_safe_replace_margin)
        candidates: List[Tuple[float, int]] = []
        for eid, score in scores.items():
            if self.cache.has(eid):
                m.bump("rs_candidate_filter_out_cached_count")
                continue
            if float(score) < min_score:
                m.bump("prefetch_rejected_low_score")
                continue
            candidates.append((float(score), int(eid)))
        if not candidates:
            return []
        candidates.sort(key=lambda c: c[0], reverse=True)
        free = self.cache.prefetch_free_slots()
        ranked = []
        for order, eid in enumerate(self.cache.evictable_prefetch_ids(protect)):
            ranked.append((float(scores.get(eid, 0.0)) + self._keep_bias(eid), order, eid))
        ranked.sort(key=lambda v: (v[0], v[1]))
        victims = [eid for _, _, eid in ranked]
        plan: List[Tuple[int, Optional[int]]] = []
        pos = 0
        for _ in range(min(free, budget, len(candidates))):
            plan.append((candidates[pos][1], None))
            pos += 1
        remaining = budget - len(plan)
        if remaining <= 0:
            return plan
        if not cfg.allow_active_replace:
            m.bump("prefetch_rejected_active_replace", min(remaining, max(0, len(candidates) - pos)))
            return plan
        vpos = 0
        while pos < len(candidates) and vpos < len(victims) and remaining > 0:
            cand_score, cand = candidates[pos]
            victim = victims[vpos]
            victim_score = float(scores.get(victim, 0.0)) + self._keep_bias(victim)
            if cand_score >= victim_score * margin or (cand_score - victim_score) >= adv:
                plan.append((cand, victim))
                remaining -= 1
                pos += 1
                vpos += 1
            else:
                m.bump("prefetch_rejected_margin", max(1, len(candidates) - pos))
                break
        if remaining > 0 and pos < len(candidates) and vpos >= len(victims):
            m.bump("prefetch_rejected_cache_full", min(remaining, len(candidates) - pos))
        return plan

    def admit_plan(self, plan: Sequence[Tuple[int, Optional[int]]]) -> None:
        """``_admit_prefetch_plan`` (reference :10433-10527): uploads ride the prefetch lane."""
        if not plan:
            return
        m = self.metrics
        m.prefetch_issued_count += len(plan)
        protect = self.prefetch_protect_ids()
        for eid, victim in plan:
            eid = int(eid)
            if self.cache.has(eid):
                slot = self.cache.get(eid)
                if not self.cache.admit_prefetch(eid, slot, protect_ids=protect, preferred_victim=victim):
                    continue
                self.prefetched_ids.add(eid)
                protect.add(eid)
                m.prefetch_admitted_count += 1
                continue
            if victim is not None:
                self._discard_before_prefetch(int(victim))
            if not self._free_slots and not self._retired and not self._pending:
                # every slot is owned by a resident that may not go: skip, demand loads it later
                m.bump("prefetch_oom_skip_count")
                continue
            slot = self._acquire_slot()
            ev = self._upload(eid, slot, "prefetch")
            m.prefetch_h2d_bytes += self.expert_bytes
            ok = self.cache.admit_prefetch(eid, slot, protect_ids=protect, preferred_victim=victim)
            if not ok:
                self._free_slots.append(slot)
                continue
            self._slot_of[eid] = slot
            self._sync_slots()
            self.prefetch_events[eid] = ev
            self.prefetched_ids.add(eid)
            protect.add(eid)
            if self.cfg.protect_mode in ("minimal", "current_next", "current-next"):
                self.cache.unpin(eid)
            m.prefetch_admitted_count += 1

    def _discard_before_prefetch(self, eid: int) -> None:
        """Reference :10011-10026."""
        ev = self.prefetch_events.pop(eid, None)
        if ev is not None and self.cfg.wait_before_evict:
            self.backend.wait_event(ev, "prefetch")
        if self.cache.discard(eid):
            self._release_slot(self._slot_of.pop(eid))
        self.prefetched_ids.discard(eid)
        self.prefetch_used_ids.discard(eid)

    def schedule_prefetch(self, flat_ids: Sequence[int], flat_probs: Sequence[float], budget: int) -> \
            List[Tuple[int, Optional[int]]]:
        """Plan and admit from the predictor's flattened ``[T, pred_k]`` top-k
        (reference :10996-11010, :10413-10431)."""
        protect = self.prefetch_protect_ids()
        scores = self.score_map(flat_ids, flat_probs)
        if self.light_policy is not None and self.phase == "decode":     # reference :10428-10430
            scores = self.light_policy.scores(scores, set(self.cache.resident_ids()))
        plan = self.build_plan(scores, protect, int(budget))
        self.admit_plan(plan)
        return plan

    # ------------------------------------------------------------------ lifecycle
    def reset_for_new_request(self, *, clear_expert_cache: bool = False, clear_cache_metadata: bool = True) -> None:
        """Reference :6097-6147."""
        if self.light_policy is not None:
            self.light_policy.reset()
        self.metrics.prefetch_completed_count += len(self.prefetch_events)
        for ev in self.prefetch_events.values():
            self.backend.wait_event(ev, "compute", True)  # nothing may read a slot before its copy lands
        self.prefetch_events.clear()
        self.prefetched_ids.clear()
        self.prefetch_used_ids.clear()
        self.access_freq.clear()
        self.last_used_decode_step.clear()
        self.cycle_key = None
        if clear_expert_cache:
            self.clear()
        elif clear_cache_metadata:
            self.cache.reset_request_metadata(unpin=True)
        if not clear_expert_cache and not self.cfg.epipe_prefill_extra_cache_persist_requests:
            self.flush()
            self.clear_extra_cache()       # reference :6146-6147

    def clear(self) -> None:
        """Drop every resident expert; all slots return to the pool."""
        self.flush()
        self.cache.clear()
        self.extra_cache.clear()
        self._slot_of.clear()
        ring = set(self._pool_slots)
        self._free_slots = [s for s in range(self.num_slots - 1, -1, -1) if s not in ring]
        self._retired = []
