"""CPU oracle of one layer's cache / prefetch / EPIPE state machine.  TEST INFRASTRUCTURE
ONLY: only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg
may import this.

``RefLayer`` restates, method by method, the parts of the reference's
``DistributedSparseMoeBlock`` that decide residency and execution order on one GPU
(world size 1, ``cache_policy=lru``, ``expert_offload=cpu``), without any device work.
Every method names the reference lines it follows (utils/eval_core.py).  Device effects
are recorded in ``trace`` as tuples:

    ("hit" | "prefetch_hit" | "miss", eid)       cache events (:5400-5418)
    ("h2d", lane, eid)                           a copy enqueued on compute/prefetch/epipe
    ("wait", eid)                                the compute stream waits a copy event
    ("compute", eid)                             the expert's segment is executed
    ("plan", ((eid, victim), ...))               an admitted prefetch plan

Copy completion is not modelled by time: ``copy_done(eid)`` (a callable given by the
test, default "always complete") answers ``event.query()``.

Pinned by (tests/test_residency.py and tests/golden/):
  score map          the reference's known-answer tests of the same formula through
                     ``select_candidates`` (tests/test_rs_staging.py:147-150, :308-312)
                     and golden vectors from the reference's own
                     ``_build_target_layer_prob_score_map``.
  plan / victims     golden vectors from the reference's own
                     ``_build_prefetch_plan_from_score_map`` and
                     ``_pick_victims_by_low_value`` on random states; invariants (plan
                     never exceeds the budget, never names a cached expert, victims are
                     evictable and unprotected).
  demand path        reference test tests/test_rs_staging.py:74-92 (in-flight prefetch hit:
                     exactly one wait, ``is_prefetch_hit``, no second load) restated;
                     textbook LRU replay.
  EPIPE executors    (upfront scan, RS residual scan, bounded ready buffer, miss-triggered
  and the whole      look-ahead) golden traces recorded from the reference's own methods
  state machine      (tests/golden/make_layer_golden.py -> layer_traces.json): the methods are
                     taken out of the reference source with ``ast`` and run as written
                     against recording stand-ins for streams, events and weights, because
                     they refuse to run without a CUDA device (:11881, :12184, :12530,
                     :12860).  55 cases cover every method switch, late prefetch copies,
                     prefill commits / side cache / transient marks, the tiered cache,
                     request resets and the local policy; tests/test_layer_golden.py
                     replays them through this oracle and through the product.  Hand-made
                     walk-throughs and invariants (every segment computed exactly once, the
                     staged expert counts exactly one miss, resident experts run before the
                     wait) stay in tests/test_residency.py.
"""
from __future__ import annotations

from typing import Any, Callable, Dict, List, Optional, Sequence, Set, Tuple

from . import ref_policy
from .ref_cache import (RefEpipePrefillExtraCache, RefExpertWeightCache, RefTieredExpertWeightCache,
                        ref_tiered_capacity_split)

Segment = Tuple[int, int]  # (expert id, rows)


class RefConfig:
    """Reference defaults (:4939-5075, :5066-5075, :10162-10183)."""

    def __init__(self, **kw: Any) -> None:
        self.capacity = 10
        self.cache_policy = "lru"            # lru | tiered (:4843-4899)
        self.prefetch_reserved = 0
        self.prefetch_extra_capacity = 0
        self.planner_mode = "none"
        self.prefetch_top_m = 4
        self.pred_topk: Optional[int] = None
        self.rs_policy = "default"
        self.min_candidate_score = 0.02
        self.replace_advantage = 0.02
        self.replace_margin = 1.05
        self.cache_safe_min_score = 0.03
        self.cache_safe_replace_advantage = 0.05
        self.cache_safe_replace_margin = 1.10
        self.allow_active_replace = True
        self.recent_protect_steps = 0
        self.protect_mode = "default"
        self.wait_before_evict = True
        self.cache_ttl_steps = 0
        self.epipe_enable = False
        self.epipe_prefill_enable = False
        self.epipe_mode = "upfront_scan"
        self.epipe_decode_rs_mode = "late_only"
        self.epipe_no_evict = True
        self.epipe_transient_staging = True
        self.epipe_min_ready_experts = 1
        self.epipe_min_ready_items = 1
        self.epipe_min_missing_experts = 1
        self.epipe_sort_ready_by_work = False
        self.epipe_prefill_commit = True
        self.epipe_rs_handle_late_prefetch = True
        self.epipe_rs_handle_demand_miss = False
        self.epipe_rs_force_demand_stage = False
        self.epipe_rs_demand_commit = True
        self.epipe_deferred_lru_commit = True
        self.epipe_rs_min_buffer_groups = 1
        self.epipe_rs_min_buffer_items = 1
        self.epipe_rs_rolling_gate = True
        self.epipe_rs_gate_window = 16
        self.epipe_rs_gate_min_triggers = 1
        self.epipe_rs_gate_skip_steps = 8
        self.epipe_prefill_extra_cache_slots = 0
        self.epipe_prefill_extra_cache_decode_read = True
        self.epipe_prefill_extra_cache_clear_at_decode = False
        self.epipe_prefill_extra_cache_persist_requests = False
        self.epipe_prefill_extra_cache_max_mb = 128.0
        self.epipe_prefill_mark_transient = True      # default follows the default prefill policy (:5012-5016)
        self.epipe_promote_transient_on_decode_hit = True
        self.epipe_rs_buffer_max_groups = 4
        self.epipe_rs_buffer_max_items = 32
        self.epipe_lookahead_experts = 4
        self.epipe_lookahead_min_ready_items = 64
        self.epipe_prefill_lookahead_min_ready_items = 256
        self.epipe_decode_rs_commit = True
        self.epipe_decode_no_rs_commit = True
        self.epipe_stream_all = False                 # this build's addition, see RefLayer.execute
        self.epipe_shadow = False                     # :4940
        self.epipe_prefill_shadow = False             # :5008
        self.epipe_prefill_multistage_shadow = False  # :5009
        self.epipe_prefill_multistage_max_n = 4       # :5010
        self.epipe_prefill_no_touch_ready = False     # :5018
        self.epipe_rs_demand_stage_threshold_ms = 0.0  # :4988
        for k, v in kw.items():
            if not hasattr(self, k):
                raise ValueError(f"unknown option {k}")
            setattr(self, k, v)


class RefLayer:
    def __init__(self, layer_idx: int, num_experts: int, top_k: int, cfg: RefConfig,
                 copy_done: Optional[Callable[[int], bool]] = None) -> None:
        self.layer_idx, self.num_experts, self.top_k, self.cfg = layer_idx, num_experts, top_k, cfg
        self.cache = None
        if cfg.cache_policy == "tiered":
            total, hot, reserved = ref_tiered_capacity_split(cfg.capacity, cfg.planner_mode == "rs_prefetch",
                                                              cfg.prefetch_reserved, cfg.prefetch_extra_capacity)
            self.cache = RefTieredExpertWeightCache(total, hot, reserved) if hot > 0 else RefExpertWeightCache(total)
        else:
            self.cache = RefExpertWeightCache(cfg.capacity)
        self.extra = RefEpipePrefillExtraCache(cfg.epipe_prefill_extra_cache_slots)
        self.expert_bytes = 0                    # size of one expert for the side cache's byte guard
        self.copy_done = copy_done or (lambda eid: True)
        self.miss_lane = "compute"
        self.prefetched: Set[int] = set()        # _prefetched_ids_this_group
        self.used: Set[int] = set()              # _prefetch_used_ids_this_group
        self.events: Dict[int, int] = {}         # _prefetch_events: eid -> token
        self.cycle_key = None
        self.freq: Dict[int, int] = {}           # _expert_access_freq
        self.last_used: Dict[int, int] = {}      # _last_used_decode_step
        self.gate_calls = self.gate_triggers = self.gate_skip = 0
        self.phase, self.call_id, self.stage = "none", -1, "decode"
        self.trace: List[Tuple] = []
        self.counters: Dict[str, int] = {}
        self.observed_exposed_ms = 0.0   # what the reference's metrics would hold; the caller sets it
        # cost-aware local policy (utils/lightweight_policy.py), off unless a test sets it:
        # dict(costs=..., expert_bytes=..., window_ms=0.0, ready_ms=0.0, feedback=True, prefetch=True)
        self.policy: Optional[Dict[str, Any]] = None

    def _count(self, name: str, n: int = 1) -> None:
        self.counters[name] = self.counters.get(name, 0) + n

    # ------------------------------------------------------------ demand path
    def _protect_ttl(self) -> Set[int]:
        """:5929-5938."""
        out: Set[int] = set()
        if self.cfg.cache_ttl_steps > 0 and self.phase == "decode" and self.call_id >= 0:
            for eid, last in self.last_used.items():
                if self.call_id - last <= self.cfg.cache_ttl_steps:
                    out.add(eid)
        return out

    def on_demand_access(self, eid: int) -> None:
        """:11213-11221."""
        self.freq[eid] = self.freq.get(eid, 0) + 1
        if self.phase == "decode":
            self.last_used[eid] = self.call_id
        if self.freq[eid] >= 2:
            self.cache.promote_hot(eid)

    def cache_put_guarded(self, eid: int, transient: bool = False) -> None:
        """:5985-6022 with :5940-5951.  ``transient`` is the ``prefill_scp_transient`` mark; at
        world size 1 only EPIPE prefill commits set it (:12083-12089, :13103-13109)."""
        protect = self._protect_ttl()
        protect.discard(eid)
        resident = set(self.cache.resident_ids())
        if resident and resident.issubset(protect):
            protect = set()
        prefer_hot = int(self.freq.get(eid, 0)) >= 2   # _should_prefer_hot, :11223-11232
        self.cache.put(eid, ("w", eid), pinned=False, prefer_hot=prefer_hot, protect_ids=protect,
                       prefill_scp_transient=bool(transient))
        if transient:
            self._count("prefill_scp_transient_load_count")

    def maybe_wait_prefetch(self, eid: int) -> None:
        """:11176-11210."""
        if eid in self.events:
            del self.events[eid]
            if self.copy_done(eid):
                self._count("prefetch_complete_before_use")
            self.trace.append(("wait", eid))
            self._count("prefetch_completed")

    def record_cached_use(self, eid: int, wait: bool) -> None:
        """:11395-11412 and :11652-11670; first the transient upgrade of :11324-11336."""
        if (self.stage == "decode" and self.cfg.epipe_promote_transient_on_decode_hit
                and self.cache.is_prefill_scp_transient(eid)):
            self._count("prefill_scp_transient_hit_count")
            if self.cache.clear_prefill_scp_transient(eid):
                self._count("prefill_scp_transient_promote_count")
        if eid in self.prefetched:
            self.trace.append(("prefetch_hit", eid))
            self.used.add(eid)
            self.cache.unpin(eid)
            self.cache.promote_hot(eid)
        else:
            self.trace.append(("hit", eid))
        if wait:
            self.maybe_wait_prefetch(eid)

    def demand(self, eid: int) -> None:
        """``_get_local_module_weights`` :11388-11435."""
        if self.cache.get(eid) is not None:
            self.record_cached_use(eid, wait=True)
            return
        if self.extra_get(eid):
            return
        self.trace.append(("miss", eid))
        self.trace.append(("h2d", self.miss_lane, eid))
        self.on_demand_access(eid)
        self.cache_put_guarded(eid)
        if self.miss_lane != "compute":     # stream-all EPIPE (not in the reference): the compute lane waits this copy
            self.trace.append(("wait", eid))

    # ---- prefill side cache (:5637-5720) -----------------------------------------------
    def extra_enabled(self) -> bool:
        """:5636-5644."""
        c = self.cfg
        return self.extra.capacity > 0 and bool(
            c.epipe_prefill_enable or c.epipe_prefill_shadow or c.epipe_prefill_multistage_shadow)

    def _extra_readable(self) -> bool:
        return self.extra_enabled() and not (self.stage == "decode"
                                             and not self.cfg.epipe_prefill_extra_cache_decode_read)

    def extra_get(self, eid: int, touch: bool = True) -> bool:
        """A payload found in the side cache counts as an ordinary hit (:5687-5704)."""
        if not self._extra_readable():
            return False
        if (self.extra.get(eid) if touch else self.extra.peek(eid)) is None:
            return False
        self.trace.append(("hit", eid))
        self._count("epipe_prefill_extra_cache_hit_count")
        return True

    def extra_store(self, eid: int) -> bool:
        """:5647-5685: prefill only, bounded by slots and by bytes."""
        if self.stage != "prefill" or not self.extra_enabled():
            return False
        max_bytes = int(float(self.cfg.epipe_prefill_extra_cache_max_mb) * 1024.0 * 1024.0)
        if max_bytes > 0 and not self.extra.has(eid) and self.extra.resident_nbytes() + self.expert_bytes > max_bytes:
            self._count("epipe_prefill_extra_cache_no_room_count")
            return False
        ok, _updated, _evicted = self.extra.put(eid, ("w", eid), nbytes=self.expert_bytes)
        return bool(ok)

    def decode_boundary(self) -> int:
        """Per-layer part of the prefill -> decode hooks (:16565-16640): transients to the LRU
        end, the side cache dropped only when asked to.  Returns the demoted count."""
        demoted = self.cache.demote_prefill_scp_transients()
        if self.cfg.epipe_prefill_extra_cache_clear_at_decode:
            self.extra.clear()
        return demoted

    def compute(self, eid: int, have_payload: bool = False) -> None:
        if not have_payload:
            self.demand(eid)
        self.trace.append(("compute", eid))

    # ------------------------------------------------------------ executors
    def epipe_stage_enabled(self) -> bool:
        """:5585-5598."""
        c = self.cfg
        if self.stage == "prefill":
            return bool(c.epipe_prefill_enable or c.epipe_prefill_shadow or c.epipe_prefill_multistage_shadow)
        if self.stage == "decode":
            if c.planner_mode == "rs_prefetch":
                return bool(c.epipe_enable and c.epipe_decode_rs_mode not in ("off", "disabled"))
            return bool(c.epipe_enable or c.epipe_shadow)
        return False

    def shadow_for_stage(self) -> bool:
        """:11890-11894, :12906-12910."""
        c = self.cfg
        return bool(c.epipe_shadow if self.stage == "decode"
                    else (c.epipe_prefill_shadow or c.epipe_prefill_multistage_shadow))

    def record_multistage_shadow(self, ready: Sequence[Segment], missing: Sequence[Segment]) -> None:
        """:5738-5778."""
        c = self.cfg
        if self.stage != "prefill" or not c.epipe_prefill_multistage_shadow:
            return
        ready_items = sum(n for _, n in ready)
        self._count("epipe_prefill_multistage_shadow_count")
        self._count("epipe_prefill_multistage_ready_expert_count", len(ready))
        self._count("epipe_prefill_multistage_missing_expert_count", len(missing))
        self._count("epipe_prefill_multistage_ready_item_count", ready_items)
        self._count("epipe_prefill_multistage_missing_item_count", sum(n for _, n in missing))
        if not missing:
            return
        ranked = sorted(((n, self.expert_bytes) for _, n in missing), key=lambda x: x[0], reverse=True)
        top = ranked[:min(max(1, int(c.epipe_prefill_multistage_max_n)), len(ranked))]
        self._count("epipe_prefill_multistage_top_missing_item_count_sum", sum(x[0] for x in top))
        self._count("epipe_prefill_multistage_est_expert_h2d_bytes", sum(x[1] for x in top))
        self._count("epipe_prefill_multistage_est_ready_compute_items", ready_items)
        for n in (1, 2, 4):
            if int(c.epipe_prefill_multistage_max_n) >= n:
                self._count(f"epipe_prefill_multistage_est_hidden_h2d_items_n{n}",
                            sum(x[0] for x in ranked[:min(n, len(ranked))]))

    def execute(self, segments: Sequence[Segment]) -> str:
        """Executor choice of ``_execute_local_recv_groups`` :13264-13357."""
        if not segments:
            return "empty"
        c = self.cfg
        epipe = self.epipe_stage_enabled() and c.epipe_mode != "off"
        # stream-all EPIPE, an addition of this build: every miss inside an EPIPE call is copied
        # on the EPIPE lane and awaited by the compute lane; events and cache state are unchanged
        self.miss_lane = "epipe" if (epipe and getattr(c, "epipe_stream_all", False)) else "compute"
        try:
            return self._execute(segments, epipe)
        finally:
            self.miss_lane = "compute"

    def _execute(self, segments: Sequence[Segment], epipe: bool) -> str:
        c = self.cfg
        result = None
        if epipe:
            rs_active = c.planner_mode == "rs_prefetch"
            if self.stage == "decode" and rs_active and c.epipe_decode_rs_mode == "off":
                result = None
            elif self.stage == "decode" and rs_active and c.epipe_decode_rs_mode == "residual_scan":
                result = self.epipe_rs_residual_scan(segments)
            elif self.stage == "decode" and rs_active and c.epipe_decode_rs_mode in (
                    "buffered", "late_only", "demand_only"):
                result = self.epipe_rs_buffered(segments)
            elif self.stage == "decode" and not rs_active and c.epipe_mode != "miss_triggered":
                result = self.epipe_upfront_scan(segments)
            elif c.epipe_mode == "upfront_scan":
                result = self.epipe_upfront_scan(segments)
            else:
                result = self.epipe_miss_triggered(segments)
        if result is None:
            for eid, _ in segments:  # ascending expert id, :13340-13357
                self.compute(eid)
            result = "plain"
        return result

    def contains_no_touch(self, eid: int) -> bool:
        """:5815-5851."""
        return (self._extra_readable() and self.extra.has(eid)) or self.cache.has(eid)

    def epipe_upfront_scan(self, segments: Sequence[Segment]) -> Optional[str]:
        """:11867-12167."""
        c = self.cfg
        enabled = bool(c.epipe_enable if self.stage == "decode" else c.epipe_prefill_enable)
        shadow = self.shadow_for_stage()
        if not (enabled or shadow):
            return None
        ready = [s for s in segments if self.contains_no_touch(s[0])]
        missing = [s for s in segments if not self.contains_no_touch(s[0])]
        ready_items = sum(n for _, n in ready)
        free = max(0, self.cache.capacity - len(self.cache.resident_ids()))
        self.record_multistage_shadow(ready, missing)
        if shadow and not enabled:   # :11919-11932
            self._count("epipe_shadow_count")
            self._count("epipe_ready_expert_count", len(ready))
            self._count("epipe_missing_expert_count", len(missing))
            self._count("epipe_ready_item_count", ready_items)
            self._count("epipe_missing_item_count", sum(n for _, n in missing))
            self._count("epipe_missing_h2d_bytes_est", len(missing) * self.expert_bytes)
            if free > 0:
                self._count("epipe_cache_free_slot_count", free)
            elif missing and c.epipe_transient_staging:
                self._count("epipe_cache_full_staged_count")
            return None
        if len(ready) < c.epipe_min_ready_experts or ready_items < c.epipe_min_ready_items:
            self._count("epipe_fallback_no_ready")
            return None
        if len(missing) < c.epipe_min_missing_experts:
            self._count("epipe_fallback_no_missing")
            return None
        staged = missing[0][0]
        can_insert = (free > 0 and c.cache_policy != "tiered"
                      and not (self.stage == "prefill" and not c.epipe_prefill_commit))   # :11964-11969
        use_transient = not can_insert
        if use_transient and not c.epipe_transient_staging:
            self._count("epipe_fallback_cache_full_no_temp")
            return None
        self.trace.append(("h2d", "epipe", staged))
        order = list(ready)
        if c.epipe_sort_ready_by_work:
            order.sort(key=lambda s: s[1], reverse=True)
        for eid, _ in order:
            # :12020-12031: with the no-touch switch a prefill call reads the ready payload itself
            have = (self.stage == "prefill" and c.epipe_prefill_no_touch_ready
                    and self.ready_payload_for_compute(eid))
            self.compute(eid, have_payload=bool(have))
        self.trace.append(("wait", staged))
        self.trace.append(("miss", staged))
        if self.stage != "prefill":
            self.on_demand_access(staged)
        for name, n in (("epipe_staged_missing_count", 1), ("epipe_enabled_count", 1), ("epipe_staged_expert_count", 1),
                        ("epipe_no_evict_count", 1), ("epipe_ready_expert_count", len(ready)),
                        ("epipe_missing_expert_count", len(missing)), ("epipe_ready_item_count", ready_items),
                        ("epipe_missing_item_count", sum(n for _, n in missing)),
                        ("epipe_missing_h2d_bytes_est", len(missing) * self.expert_bytes)):   # :12065-12074
            self._count(name, n)
        if free > 0:
            self._count("epipe_cache_free_slot_count", free)
        if can_insert:
            if len(self.cache.resident_ids()) < self.cache.capacity:
                if self.stage == "prefill":
                    self.on_demand_access(staged)
                self.cache_put_guarded(staged, transient=self.stage == "prefill" and c.epipe_prefill_mark_transient)
            else:
                use_transient = True
        if use_transient and not (self.stage == "prefill" and self.extra_store(staged)):   # :12101-12108
            self._count("epipe_cache_full_staged_count")
            self._count("epipe_transient_payload_count")
        self.compute(staged, have_payload=True)
        for eid, _ in missing[1:]:
            self.compute(eid)
        return "epipe_upfront"

    def pending_prefetch_event(self, eid: int) -> bool:
        """:11636-11650: True while the copy is in flight; a finished one is retired."""
        if eid not in self.events:
            return False
        if self.copy_done(eid):
            del self.events[eid]
            self._count("prefetch_complete_before_use")
            self._count("prefetch_completed")
            return False
        return True

    def demand_gate_can_open(self) -> bool:
        """:5880-5893.  ``observed_exposed_ms`` stands for max(sampled, measured) exposed demand-copy ms
        of the decode phase, which the reference reads from its metrics."""
        if not self._handle_demand():
            return False
        if self.cfg.epipe_rs_force_demand_stage:
            return True
        threshold = float(self.cfg.epipe_rs_demand_stage_threshold_ms)
        if threshold <= 0.0:
            return False
        return float(self.observed_exposed_ms) > threshold

    def _residual_present(self, segments: Sequence[Segment]) -> bool:
        for eid, _ in segments:
            if eid in self.events and self._handle_late() and not self.copy_done(eid):
                return True
            if self.demand_gate_can_open() and not self.contains_no_touch(eid):
                return True
        return False

    def _maybe_skip_gate(self, segments: Sequence[Segment]) -> bool:
        """:12228-12254."""
        c = self.cfg
        if not c.epipe_rs_rolling_gate:
            return False
        if self.gate_skip > 0:
            if self._residual_present(segments):
                self.gate_skip = 0
                return False
            self.gate_skip -= 1
            return True
        self.gate_calls += 1
        if self.gate_calls >= c.epipe_rs_gate_window and self.gate_triggers < c.epipe_rs_gate_min_triggers:
            self.gate_calls = self.gate_triggers = 0
            self.gate_skip = int(c.epipe_rs_gate_skip_steps)
            if self.gate_skip > 0:
                self.gate_skip -= 1
                return True
        if self.gate_calls >= c.epipe_rs_gate_window:
            self.gate_calls = self.gate_triggers = 0
        return False

    def epipe_rs_residual_scan(self, segments: Sequence[Segment]) -> Optional[str]:
        """:12169-12512."""
        c = self.cfg
        if self.stage != "decode" or c.planner_mode != "rs_prefetch" or not c.epipe_enable:
            return None
        if self._maybe_skip_gate(segments):
            return None
        ready: List[int] = []
        late: List[int] = []
        dem: List[int] = []
        for i, (eid, _) in enumerate(segments):
            pending = self.pending_prefetch_event(eid)
            cached = self.contains_no_touch(eid)
            if cached and not pending:
                ready.append(i)
            elif cached and pending and c.epipe_rs_handle_late_prefetch:
                late.append(i)
            elif not cached and c.epipe_rs_handle_demand_miss and self.demand_gate_can_open():
                dem.append(i)
        ready_items = sum(segments[i][1] for i in ready)
        pol = self.policy
        if pol is not None and pol["feedback"]:                                  # :12322-12324
            pol["ready_ms"] = ref_policy.compute_ms(pol["costs"], len(ready), ready_items)
        if len(ready) < c.epipe_rs_min_buffer_groups or ready_items < c.epipe_rs_min_buffer_items:
            return None
        residual, kind = None, ""
        if late:
            residual, kind = late[0], "late"
        elif dem and self.demand_gate_open(ready_items):
            residual, kind = dem[0], "demand"
        if pol is not None and pol["feedback"]:                                  # :12342-12348
            stageable = dem if self.demand_gate_open(ready_items) else []
            cands = [(i, segments[i][0], "late") for i in late] + [(i, segments[i][0], "demand") for i in stageable]
            chosen = ref_policy.choose_residual(pol["costs"], pol["expert_bytes"], len(ready), ready_items, cands)
            residual, kind = chosen if chosen is not None else (None, "")
        if residual is None:
            return None
        reid = segments[residual][0]
        cover = [i for i in ready if i != residual]
        if len(cover) < c.epipe_rs_min_buffer_groups:
            return None
        if c.epipe_rs_rolling_gate:
            self.gate_triggers += 1

        def compute_ready(indices: Sequence[int]) -> None:
            for i in indices:
                eid = segments[i][0]
                if self.cache.get(eid) is None:
                    self.compute(eid)
                else:
                    self.record_cached_use(eid, wait=False)
                    self.compute(eid, have_payload=True)

        done = set()
        if kind == "late":
            if self.cache.get(reid) is None:
                return None
            compute_ready(cover)
            done.update(cover)
            self.maybe_wait_prefetch(reid)
            self.record_cached_use(reid, wait=False)
            self.compute(reid, have_payload=True)
            done.add(residual)
        else:
            self.trace.append(("h2d", "epipe", reid))
            compute_ready(cover)
            done.update(cover)
            self.trace.append(("wait", reid))
            self.trace.append(("miss", reid))
            self.on_demand_access(reid)
            free = max(0, self.cache.capacity - len(self.cache.resident_ids()))
            if c.epipe_rs_demand_commit and c.epipe_deferred_lru_commit and (free > 0 or not c.epipe_no_evict):
                self.cache_put_guarded(reid)
            self.compute(reid, have_payload=True)
            done.add(residual)
        for i, (eid, _) in enumerate(segments):
            if i not in done:
                self.compute(eid)
        if c.epipe_rs_rolling_gate and self.gate_skip > 0:
            self.gate_skip = 0
        return "epipe_rs_residual_scan"

    def _handle_late(self) -> bool:
        """:4975-4984: ``demand_only`` switches the late-prefetch handling off."""
        return bool(self.cfg.epipe_rs_handle_late_prefetch) and self.cfg.epipe_decode_rs_mode != "demand_only"

    def _handle_demand(self) -> bool:
        """``late_only`` switches the demand-miss handling off."""
        return bool(self.cfg.epipe_rs_handle_demand_miss) and self.cfg.epipe_decode_rs_mode != "late_only"

    def demand_gate_open(self, ready_items: int) -> bool:
        """:5895-5907."""
        if not self._handle_demand() or ready_items < self.cfg.epipe_rs_min_buffer_items:
            return False
        return self.demand_gate_can_open()

    def epipe_rs_buffered(self, segments: Sequence[Segment]) -> Optional[str]:
        """:12514-12843.  One pass in ascending expert id: resident experts collect in a
        bounded buffer (their hits counted as they are seen), which is executed when it is
        full and in any case before a segment that has to wait; a prefetch still in flight
        is waited for only after the buffer ran; a miss is staged beside the buffer only in
        the modes that handle demand misses."""
        c = self.cfg
        if self.stage != "decode" or c.planner_mode != "rs_prefetch" or not c.epipe_enable:
            return None
        handle_late, handle_demand = self._handle_late(), self._handle_demand()
        if self._maybe_skip_gate(segments):
            return None
        buffered: List[int] = []
        items = [0]
        trigger_seen = False

        def flush() -> None:
            for e in buffered:
                self.compute(e, have_payload=True)
            buffered.clear()
            items[0] = 0

        def sufficient() -> bool:
            return len(buffered) >= c.epipe_rs_min_buffer_groups and items[0] >= c.epipe_rs_min_buffer_items

        for eid, rows in segments:
            pending = self.pending_prefetch_event(eid)
            if self.cache.get(eid) is not None:
                if not pending:
                    self.record_cached_use(eid, wait=False)
                    buffered.append(eid)
                    items[0] += rows
                    if len(buffered) >= c.epipe_rs_buffer_max_groups or items[0] >= c.epipe_rs_buffer_max_items:
                        flush()
                    continue
                if not handle_late:
                    flush()
                    self.record_cached_use(eid, wait=True)
                    self.compute(eid, have_payload=True)
                    continue
                if c.epipe_rs_rolling_gate:
                    self.gate_triggers += 1
                trigger_seen = True
                if not sufficient():
                    flush()
                    self.record_cached_use(eid, wait=True)
                    self.compute(eid, have_payload=True)
                    continue
                flush()
                self.maybe_wait_prefetch(eid)
                self.record_cached_use(eid, wait=False)
                self.compute(eid, have_payload=True)
                continue
            if not handle_demand:
                flush()
                self.compute(eid)
                continue
            if c.epipe_rs_rolling_gate:
                self.gate_triggers += 1
            trigger_seen = True
            if not sufficient() or not self.demand_gate_open(items[0]):
                flush()
                self.compute(eid)
                continue
            self.trace.append(("h2d", "epipe", eid))
            flush()
            self.trace.append(("wait", eid))
            self.trace.append(("miss", eid))
            self.on_demand_access(eid)
            free = max(0, self.cache.capacity - len(self.cache.resident_ids()))
            if c.epipe_rs_demand_commit and c.epipe_deferred_lru_commit and (free > 0 or not c.epipe_no_evict):
                self.cache_put_guarded(eid)
            self.compute(eid, have_payload=True)
        flush()
        if trigger_seen and c.epipe_rs_rolling_gate and self.gate_skip > 0:
            self.gate_skip = 0
        return "epipe_rs_buffered"

    def ready_payload_for_compute(self, eid: int) -> bool:
        """:11672-11698: cache first (touching, counted as a hit, waiting a pending copy),
        then the prefill side cache (touching, not counted)."""
        no_touch = self.stage == "prefill" and bool(self.cfg.epipe_prefill_no_touch_ready)
        if (self.cache.peek(eid) if no_touch else self.cache.get(eid)) is not None:
            self.record_cached_use(eid, wait=True)
            return True
        return self.extra_get(eid, touch=not no_touch)

    def epipe_miss_triggered(self, segments: Sequence[Segment]) -> Optional[str]:
        """:12845-13154.  Walk the segments in ascending expert id; at the first miss look
        ahead a few segments for resident experts, stage the missing expert on the side
        lane, run those resident experts meanwhile, then wait, count the miss and run it.
        Later misses of the same call take the ordinary demand path."""
        c = self.cfg
        stage, rs_active = self.stage, c.planner_mode == "rs_prefetch"
        enabled = bool(c.epipe_prefill_enable if stage == "prefill" else c.epipe_enable)
        shadow = self.shadow_for_stage()
        if not (enabled or shadow):
            return None
        if stage == "decode" and rs_active and c.epipe_decode_rs_mode == "off":
            return None
        if stage == "decode" and rs_active and c.epipe_decode_rs_mode == "buffered":
            return self.epipe_rs_buffered(segments)
        if stage == "decode" and rs_active and c.epipe_decode_rs_mode == "upfront_scan":
            return self.epipe_upfront_scan(segments)
        min_ready_items = (c.epipe_prefill_lookahead_min_ready_items if stage == "prefill"
                           else c.epipe_lookahead_min_ready_items)
        done: Set[int] = set()
        staged_once = False
        for i, (eid, _rows) in enumerate(segments):
            if i in done:
                continue
            if self.ready_payload_for_compute(eid):
                self.compute(eid, have_payload=True)
                continue
            if staged_once:
                self.compute(eid)
                continue
            ahead = [j for j in range(i + 1, min(len(segments), i + 1 + int(c.epipe_lookahead_experts)))
                     if j not in done and self.contains_no_touch(segments[j][0])]
            ready_items = sum(segments[j][1] for j in ahead)
            if shadow and not enabled:   # :12982-12991
                if ahead:
                    self._count("epipe_prefill_shadow_opportunity_count" if stage == "prefill" else "epipe_shadow_count")
                self._count("epipe_lookahead_ready_group_count", len(ahead))
                self._count("epipe_lookahead_ready_item_count", ready_items)
                self.compute(eid)
                continue
            if not ahead:
                self._count("epipe_fallback_no_ready_lookahead")
                self.compute(eid)
                continue
            if ready_items < min_ready_items:
                self._count("epipe_fallback_low_ready_items")
                self.compute(eid)
                continue
            self.trace.append(("h2d", "epipe", eid))
            for j in ahead:
                self.compute(segments[j][0])
                done.add(j)
            self.trace.append(("wait", eid))
            self.trace.append(("miss", eid))
            if stage != "prefill":
                self.on_demand_access(eid)
            free = max(0, self.cache.capacity - len(self.cache.resident_ids()))
            if free > 0:
                self._count("epipe_cache_free_slot_count", free)
            if stage == "prefill":
                commit_allowed, mark = bool(c.epipe_prefill_commit), bool(c.epipe_prefill_mark_transient)
            elif rs_active:
                commit_allowed, mark = bool(c.epipe_decode_rs_commit) or free > 0, False
            else:
                commit_allowed, mark = bool(c.epipe_decode_no_rs_commit), False
            insert = commit_allowed and c.epipe_deferred_lru_commit and (free > 0 or not c.epipe_no_evict)
            if stage == "prefill" and insert:
                self.on_demand_access(eid)
            if insert:
                self.cache_put_guarded(eid, transient=mark)
            elif not (stage == "prefill" and self.extra_store(eid)):   # :13121-13130
                if free <= 0:
                    self._count("epipe_cache_full_staged_count")
                self._count("epipe_transient_payload_count")
            for name, n in (("epipe_enabled_count", 1), ("epipe_staged_missing_count", 1), ("epipe_staged_expert_count", 1),
                            ("epipe_ready_expert_count", len(ahead)), ("epipe_ready_item_count", ready_items),
                            ("epipe_lookahead_ready_group_count", len(ahead)),
                            ("epipe_lookahead_ready_item_count", ready_items), ("epipe_missing_expert_count", 1),
                            ("epipe_missing_item_count", _rows), ("epipe_missing_h2d_bytes_est", self.expert_bytes)):
                self._count(name, n)   # :13132-13142
            self.compute(eid, have_payload=True)
            staged_once = True
        return "epipe_miss_triggered"

    # ------------------------------------------------------------ RS prefetch
    def effective_top_m(self) -> int:
        return max(0, int(self.cfg.prefetch_top_m))

    def predict_topk(self) -> int:
        """:10888-10901."""
        if self.cfg.pred_topk is not None:
            return max(1, min(int(self.cfg.pred_topk), self.num_experts))
        return max(self.top_k, min(self.num_experts, self.effective_top_m()))

    def finalize_prev_group_prefetch(self) -> None:
        """:9598-9635."""
        for eid in list(self.events):
            if self.copy_done(eid):
                self._count("prefetch_completed")
                del self.events[eid]
        self._count("prefetch_wasted", len(self.prefetched - self.used))
        self.cache.unpin_all()
        self.prefetched.clear()
        self.used.clear()
        self.cycle_key = None

    def begin_cycle(self, key) -> None:
        """:9637-9649."""
        if self.cycle_key == key:
            return
        self.finalize_prev_group_prefetch()
        self.cycle_key = key

    def prefetch_protect_ids(self) -> Set[int]:
        """:9651-9665."""
        if self.cfg.protect_mode in ("minimal", "current_next", "current-next"):
            protect = set(self.used)
        else:
            protect = set(self.prefetched) | set(self.used)
        protect |= self._protect_ttl()
        r = int(self.cfg.recent_protect_steps)
        if r > 0 and self.phase == "decode" and self.call_id >= 0:
            for eid, last in self.last_used.items():
                if self.call_id - last <= r:
                    protect.add(eid)
        return protect

    def prefetch_budget(self, key) -> int:
        """:9785-9810 with :9754-9771."""
        top_m = self.effective_top_m()
        if self.cfg.planner_mode != "rs_prefetch" or top_m <= 0:
            return 0
        self.begin_cycle(key)
        protect = self.prefetch_protect_ids()
        room = self.cache.prefetch_free_slots()
        if self.cfg.allow_active_replace:
            room += len(self.cache.evictable_prefetch_ids(protect))
        return max(0, min(max(0, top_m - len(self.prefetched)), room))

    @staticmethod
    def score_map(flat_ids: Sequence[int], flat_probs: Sequence[float]) -> Dict[int, float]:
        """:10040-10107 at world size 1 (every expert is local)."""
        raw: Dict[int, float] = {}
        occ: Dict[int, int] = {}
        top: Dict[int, float] = {}
        for eid, w in zip(flat_ids, flat_probs):
            eid, w = int(eid), float(w)
            raw[eid] = raw.get(eid, 0.0) + w
            occ[eid] = occ.get(eid, 0) + 1
            top[eid] = max(top.get(eid, 0.0), w)
        out: Dict[int, float] = {}
        for eid, s in raw.items():
            out[eid] = float(s)
        for eid in list(out):
            boost = 1.0 + 0.15 * float(max(occ.get(eid, 1) - 1, 0))
            out[eid] = out[eid] * boost + 0.05 * float(top.get(eid, 0.0))
        return out

    def resident_keep_bias(self, eid: int) -> float:
        """:10031-10038 (plain LRU has no hot tier)."""
        bias = 0.02 * float(min(self.freq.get(int(eid), 0), 16))
        if int(eid) in self.prefetched:
            bias += 0.10
        return float(bias)

    def pick_victims_by_low_value(self, scores: Dict[int, float], protect: Set[int]) -> List[int]:
        """:10135-10142."""
        ranked = []
        for pos, eid in enumerate(self.cache.evictable_prefetch_ids(protect)):
            ranked.append((float(scores.get(int(eid), 0.0)) + self.resident_keep_bias(int(eid)), pos, int(eid)))
        ranked.sort(key=lambda x: (x[0], x[1]))
        return [e for _, _, e in ranked]

    def build_plan(self, scores: Dict[int, float], protect: Set[int], budget: int):
        """:10144-10262."""
        c = self.cfg
        if budget <= 0 or len(scores) == 0:
            return []
        min_score, adv, margin = c.min_candidate_score, c.replace_advantage, c.replace_margin
        if c.rs_policy in ("cache_safe", "cache-safe", "benefit_gate", "benefit-gate"):
            min_score = max(min_score, c.cache_safe_min_score)
            adv = max(adv, c.cache_safe_replace_advantage)
            margin = max(margin, c.cache_safe_replace_margin)
        cands = []
        for eid, sc in scores.items():
            if self.cache.has(int(eid)):
                continue
            if float(sc) < min_score:
                continue
            cands.append((float(sc), int(eid)))
        if not cands:
            return []
        cands.sort(key=lambda x: x[0], reverse=True)
        free = self.cache.prefetch_free_slots()
        victims = self.pick_victims_by_low_value(scores, protect)
        plan = []
        cpos = 0
        for _ in range(min(int(free), int(budget), len(cands))):
            plan.append((cands[cpos][1], None))
            cpos += 1
        remaining = int(budget) - len(plan)
        if remaining <= 0 or not c.allow_active_replace:
            return plan
        vpos = 0
        while cpos < len(cands) and vpos < len(victims) and remaining > 0:
            cs, ce = cands[cpos]
            v = victims[vpos]
            vs = float(scores.get(v, 0.0)) + self.resident_keep_bias(v)
            if cs >= vs * margin or (cs - vs) >= adv:
                plan.append((ce, v))
                remaining -= 1
                cpos += 1
                vpos += 1
            else:
                break
        return plan

    def admit_plan(self, plan) -> None:
        """:10433-10527."""
        if not plan:
            return
        self._count("prefetch_issued", len(plan))
        protect = self.prefetch_protect_ids()
        for eid, victim in plan:
            eid = int(eid)
            if self.cache.has(eid):
                payload = self.cache.get(eid)
                if not self.cache.admit_prefetch(eid, payload, protect_ids=protect, preferred_victim=victim):
                    continue
                self.prefetched.add(eid)
                protect.add(eid)
                self._count("prefetch_admitted")
                continue
            if victim is not None:  # :10011-10026
                if victim in self.events:
                    del self.events[victim]
                    if self.cfg.wait_before_evict:
                        self.trace.append(("wait_prefetch_lane", victim))
                self.cache.discard(victim)
                self.prefetched.discard(victim)
                self.used.discard(victim)
            self.trace.append(("h2d", "prefetch", eid))
            if not self.cache.admit_prefetch(eid, ("w", eid), protect_ids=protect, preferred_victim=victim):
                continue
            self.events[eid] = 1
            self.prefetched.add(eid)
            protect.add(eid)
            if self.cfg.protect_mode in ("minimal", "current_next", "current-next"):
                self.cache.unpin(eid)
            self._count("prefetch_admitted")

    def schedule_prefetch(self, flat_ids, flat_probs, budget: int):
        """:10996-11010 with :10413-10431."""
        protect = self.prefetch_protect_ids()
        scores = self.score_map(flat_ids, flat_probs)
        pol = self.policy
        if pol is not None and pol["prefetch"] and self.phase == "decode":      # :10428-10430
            scores = ref_policy.adjusted_scores(pol["costs"], pol["expert_bytes"], scores,
                                                set(self.cache.resident_ids()), pol["window_ms"], pol["ready_ms"],
                                                pol["feedback"])
        plan = self.build_plan(scores, protect, budget)
        if plan:
            self.trace.append(("plan", tuple(plan)))
        self.admit_plan(plan)
        return plan

    def reset_for_new_request(self, clear_expert_cache: bool = False, clear_cache_metadata: bool = True) -> None:
        """:6097-6147."""
        if self.policy is not None:
            self.policy["ready_ms"] = self.policy["window_ms"] = 0.0
        self.events.clear()
        self.prefetched.clear()
        self.used.clear()
        self.freq.clear()
        self.last_used.clear()
        self.cycle_key = None
        if clear_expert_cache:
            self.cache.clear()
        elif clear_cache_metadata:
            self.cache.reset_request_metadata(unpin=True)
        if clear_expert_cache or not self.cfg.epipe_prefill_extra_cache_persist_requests:     # :6146-6147
            self.extra.clear()
