"""Forecast staging for decode: while layer l computes, a predictor names the experts layer
l+1 will probably route to, and their weights are copied into l+1's staging ring before l+1
asks for them -- without ever touching l+1's resident cache on a guess.

This is the build's counterpart of the reference's bounded staging adapter
(utils/rs_overlap.py:58-433, ownership rules utils/rs_staging.py:12-118); the harness-facing
surface keeps its names (``BoundedRS``: ``configure``, ``prepare``, ``begin``, ``finish``,
``install``, ``restore``, ``enabled``; ``select_candidates``), the machinery is this build's:

  * a staged expert is a state of the target layer's slot table
    (``LayerResidency.staged`` / ``find`` / ``holds``), not a cache wrapper: the layer's
    lookups read ring slots directly, and ``settle_staged`` hands a used expert to the LRU
    by exchanging slot indices with the ring;
  * publication goes through ``StagingRing`` (sparse_amd/ring.py): ``open`` at the source
    layer, ``publish`` from the scoring thread, ``seal`` at the target's executor, all under
    the ring's lock, so a forecast is never joined -- late copies are simply declined;
  * candidates are scored by ``LayerResidency.score_map``, the in-line planner's own
    aggregate, after the entries that need no copy are filtered out;
  * the forecast itself -- predictor, top-k, renormalisation, rounding -- is
    ``rs.topk_for_planning`` captured once per source layer in a HIP graph, so both planners
    see the same candidates for the same hidden state.

One engine serves a whole stack.  Timeline of a decode step at layer l:
``forecast_next`` (graph launch on the forecast stream, asynchronous read-back into pinned
memory, scoring task queued; nothing waits) -> router, permutation -> ``seal`` (l's own ring
window ends, its copies become readable) -> executor -> ``settle`` (admission, ring slots
returned behind fences).
"""
from __future__ import annotations

import threading
from concurrent.futures import ThreadPoolExecutor
from contextlib import contextmanager
from time import perf_counter
from typing import Any, Dict, Iterable, List, Optional

import torch

from .residency import LayerResidency
from .ring import StagingRing


def select_candidates(ids: Iterable[int], weights: Iterable[float], *, allowed, resident, minimum: float,
                      budget: int, diagnostics: Optional[dict] = None) -> List[int]:
    """Which forecast experts are worth a copy: drop entries this rank does not own or already
    holds, score the rest with the planner's aggregate, keep those at or above ``minimum``, best
    first, at most ``budget`` (utils/rs_staging.py:97-118).  No victim is chosen: a staged
    copy displaces nothing."""
    foreign = held = 0
    keep_ids: List[int] = []
    keep_w: List[float] = []
    for eid, w in zip(ids, weights):
        eid = int(eid)
        if eid not in allowed:
            foreign += 1
        elif eid in resident:
            held += 1
        else:
            keep_ids.append(eid)
            keep_w.append(float(w))
    score = LayerResidency.score_map(keep_ids, keep_w)
    good = [eid for eid in score if score[eid] >= minimum]
    if diagnostics is not None:
        diagnostics.update(nonlocal_entries=foreign, resident_entries=held, scored=len(score),
                           below_threshold=len(score) - len(good))
    good.sort(key=score.get, reverse=True)     # stable: equal scores stay in first-seen order
    return good[:budget]


class ForecastPause:
    """Empty-forecast cool-down (utils/rs_overlap.py:87-109).  A forecast that named nothing
    worth copying is not repeated for ``steps`` decode steps of that layer, unless a demand
    miss there or a change of the cache's membership says the situation moved; a change of
    recency alone does not."""

    def __init__(self, steps: int = 0) -> None:
        self.steps = int(steps)
        self.until: Dict[int, int] = {}            # layer -> first step that forecasts again
        self.members: Dict[int, frozenset] = {}    # layer -> cache membership when the pause began

    def arm(self, layer: int, step: int, members: Iterable[int]) -> None:
        self.until[layer] = int(step) + self.steps + 1
        self.members[layer] = frozenset(members)

    def wake(self, layer: int) -> bool:
        self.members.pop(layer, None)
        return self.until.pop(layer, None) is not None

    def verdict(self, layer: int, step: int, members: Iterable[int]) -> str:
        """``"run"`` (no pause, or it ran out), ``"moved"`` (membership changed: pause dropped)
        or ``"hold"``."""
        if step >= self.until.get(layer, 0):
            self.wake(layer)
            return "run"
        if frozenset(members) != self.members[layer]:
            self.wake(layer)
            return "moved"
        return "hold"

    def clear(self) -> None:
        self.until.clear()
        self.members.clear()


class CapturedForecast:
    """Predictor and planner top-k of one source layer as a replayable HIP graph
    (utils/rs_overlap.py:21-55), with the pinned read-back buffers that belong to it."""

    def __init__(self, predictor, rows: int, width: int, k: int, dtype, renorm: bool, device) -> None:
        from .rs import topk_for_planning
        self.k = int(k)
        self._plan = lambda x: topk_for_planning(predictor(x), self.k, bool(renorm), dtype)
        self.x = torch.zeros((rows, width), dtype=torch.float32, device=device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.inference_mode():
            for _ in range(3):                      # lazy initialisation happens outside the capture
                self._plan(self.x)
            torch.cuda.synchronize(device)
            with torch.cuda.graph(self.graph):      # captures on a stream of its own and rejoins
                self.ids, self.probs = self._plan(self.x)
        self.host_ids = torch.empty((rows, self.k), dtype=torch.long, pin_memory=True)
        self.host_probs = torch.empty((rows, self.k), dtype=torch.float32, pin_memory=True)
        self.landed = torch.cuda.Event(blocking=False)
        self.task = None          # scoring task that reads the host buffers, until it is done
        self.checked = 0

    def launch(self, x, stream) -> None:
        """Replay for hidden state ``x`` on ``stream`` and start the read-back behind it."""
        with torch.inference_mode(), torch.cuda.stream(stream):
            self.x.copy_(x)
            self.graph.replay()
            for host, dev in ((self.host_ids, self.ids), (self.host_probs, self.probs)):
                host.copy_(dev, non_blocking=True)
            self.landed.record(stream)

    def check_against_eager(self, x) -> None:
        """A replay must give the eager result bit for bit."""
        with torch.inference_mode():
            want_ids, want_probs = self._plan(x.float())
            self.x.copy_(x)
            self.graph.replay()
        assert torch.equal(self.ids, want_ids) and torch.equal(self.probs, want_probs)
        self.checked += 1


_COUNTERS = ("predictions", "plans", "issued", "used", "wasted", "closed_before_publish", "skipped_slots",
             "skipped_cooldown", "unified_epipe_calls", "demand_deadline_activations", "empty_plan_closes",
             "unplanned_closes", "planned_no_publish_closes", "observed_decode_misses",
             "cooldown_miss_invalidations", "cooldown_cache_invalidations", "candidate_nonlocal_entries",
             "candidate_resident_entries", "candidate_scored", "candidate_below_threshold", "retained",
             "recycled_payloads", "allocated_replacements")
_TIMERS = ("worker_ms", "readback_wait_ms", "main_submission_ms", "target_close_ms", "request_drain_ms")


class BoundedRS:
    """The staging engine of a layer stack.  ``slots`` ring positions per layer, of which one
    window uses at most half, so the copies of step s+1 never wait for the readers of step s."""

    def __init__(self, *, slots: int = 4, empty_steps: int = 0) -> None:
        if int(slots) < 2:
            raise ValueError("the staging ring needs at least two slots per layer")
        self.enabled = False
        self.positions = int(slots)
        self.pause = ForecastPause(empty_steps)
        if self.pause.steps < 0:
            raise ValueError("empty_steps must be a nonnegative integer")
        self.scorer = ThreadPoolExecutor(max_workers=1, thread_name_prefix="forecast-scorer")
        self.layers: Dict[int, Any] = {}                    # layer -> block
        self.forecasts: Dict[int, CapturedForecast] = {}    # source layer -> its captured predictor
        self.copy_events: Dict[int, List[Any]] = {}         # layer -> one event per ring position
        self.owned: Dict[int, frozenset] = {}               # layer -> experts this rank holds in host memory
        self.forecast_stream = None
        self.copy_lane = None
        self.epoch = 0
        self.case = None
        self.stats: Dict[str, Any] = {}
        self.home_thread = threading.get_ident()

    # ---- harness surface --------------------------------------------------------------
    @property
    def empty_steps(self) -> int:
        return self.pause.steps

    def _quiet(self) -> bool:
        return all(b.residency.ring.all_idle() and not b.residency.staged for b in self.layers.values()) \
            and all(f.task is None for f in self.forecasts.values())

    def configure(self, *, empty_steps) -> None:
        """Change the cool-down length; only between drained requests (utils/rs_overlap.py:76-83)."""
        if type(empty_steps) is not int or empty_steps < 0:
            raise ValueError("empty_steps must be a nonnegative integer")
        assert self._quiet(), "configure() between requests only"
        self.pause.steps = empty_steps
        self.pause.clear()

    def prepare(self, blocks: Dict[int, Any], rs_bank, *, batch: int, dtype, k: Optional[int] = None) -> None:
        """Bind the stack: check every layer's ring, create the copy events, capture one
        forecast graph per layer that has a successor (``prepare_graphs``,
        utils/rs_overlap.py:113-157).  Once, before the first ``begin``."""
        from . import ops
        assert not self.layers, "prepare() once per engine"
        self.layers = dict(sorted(blocks.items()))
        for layer, block in self.layers.items():
            if block.residency is None or block.expert_offload != "cpu" or block.cache_policy != "lru":
                raise ValueError("forecast staging needs offloaded layers with the plain LRU cache")
            ring = block.residency.staging_ring(self.positions)
            self.copy_events[layer] = [ops.Event() for _ in range(len(ring))]
            self.owned[layer] = frozenset(block._local_eid_set)
        for layer, block in self.layers.items():
            nxt = self.layers.get(layer + 1)
            if nxt is None:
                continue
            # a captured forecast can only read what exists before the layer's router has run
            if str(getattr(rs_bank[layer + 1], "rs_feature_mode", "hidden")) != "hidden":
                raise ValueError("the bounded staging engine needs predictors with feature_mode='hidden'")
            kk = int(k) if k is not None else min(block.num_experts, nxt.residency.predict_topk())
            fc = CapturedForecast(rs_bank[layer + 1], batch, block.hidden_size, kk, dtype, block.norm_topk_prob,
                                  block.device)
            ramp = torch.arange(batch * block.hidden_size, device=block.device, dtype=torch.float32)
            for modulus in (97, 98, 99):
                fc.check_against_eager(((ramp % modulus) - 48).reshape(batch, -1) / 30)
            self.forecasts[layer] = fc
        device = next(iter(self.layers.values())).device
        self.forecast_stream = torch.cuda.Stream(device=device)     # default priority
        self.copy_lane = ops.SideStream()
        torch.cuda.synchronize()

    def begin(self, case=None) -> None:
        """Start a request (utils/rs_overlap.py:159-195)."""
        assert self._quiet(), "the previous request was not finished"
        self.epoch += 1
        self.case = case
        self.pause.clear()
        self.stats = {key: 0 for key in _COUNTERS}
        self.stats.update({key: 0.0 for key in _TIMERS})
        self.stats.update(effective_empty_steps=self.pause.steps,
                          staging_bytes=sum(len(b.residency.ring) * int(b.residency.expert_bytes)
                                            for b in self.layers.values()))
        if self.enabled:
            for block in self.layers.values():
                assert block.expert_source == "router" and block.exec_routing_mode == "router"

    def install(self) -> None:
        """Route the blocks' hooks to this engine (the reference patches seven methods of its
        block class at this point, utils/rs_overlap.py:436-489)."""
        from .context import SparseContext
        SparseContext.staging = self
        self.enabled = True

    def restore(self) -> None:
        from .context import SparseContext
        if SparseContext.staging is self:
            SparseContext.staging = None
        self.enabled = False

    def count(self, key: str, n: int = 1) -> None:
        self.stats[key] += n

    @contextmanager
    def _timed(self, key: str):
        """Add the host time of the enclosed block to ``stats[key]``, in ms."""
        t0 = perf_counter()
        try:
            yield
        finally:
            self.stats[key] += (perf_counter() - t0) * 1e3

    # ---- hooks called by the blocks ---------------------------------------------------------
    def handles(self, block, seq_len: int) -> bool:
        """Decode calls of layers whose planner is the RS prefetch."""
        return bool(self.enabled and int(seq_len) == 1 and block.planner_mode == "rs_prefetch")

    def demand_miss(self, layer: int) -> None:
        """A decode miss at ``layer``: whatever paused its forecasts is out of date."""
        self.count("observed_decode_misses")
        if self.pause.wake(int(layer)):
            self.count("cooldown_miss_invalidations")

    def _paused(self, layer: int, step: int) -> bool:
        verdict = self.pause.verdict(layer, step, self.layers[layer].residency.cache.resident_ids())
        if verdict == "moved":
            self.count("cooldown_cache_invalidations")
        elif verdict == "hold":
            self.count("skipped_cooldown")
        return verdict == "hold"

    def _absorb(self, fc: CapturedForecast) -> None:
        """Fold a finished scoring task's timings and counts into the request's statistics."""
        if fc.task is None or not fc.task.done():
            return
        row, fc.task = fc.task.result(), None       # done: this does not wait
        self.stats["worker_ms"] += row["ms"]
        self.stats["readback_wait_ms"] += row["waited_ms"]
        for key, value in row["seen"].items():
            self.stats["candidate_" + key] += value

    def forecast_next(self, block, x, step: int) -> None:
        """At source layer l: open l+1's ring window, launch the forecast, queue the scoring
        task (utils/rs_overlap.py:255-301).  Waits for nothing."""
        src = int(block.layer_idx)
        fc = self.forecasts.get(src)
        if fc is None:
            return
        assert threading.get_ident() == self.home_thread, "hooks run on the thread that built the engine"
        dst, step = src + 1, int(step)
        target = self.layers[dst]
        res: LayerResidency = target.residency
        if self.pause.steps and self._paused(dst, step):
            return
        self._absorb(fc)
        want = min(int(res.effective_top_m()), self.positions // 2)
        if want <= 0:
            return
        # the graph's buffers belong to the last task until it is done, a layer has one window at
        # a time, and a window needs at least one ring position whose last readers have finished
        ticket = (self.epoch, step, dst)
        with self._timed("main_submission_ms"):
            room = 0 if (fc.task is not None or res.ring.is_open()) else \
                res.ring.open(ticket, want, res.backend.event_done)
            if room == 0:
                self.count("skipped_slots")
                return
            assert x.shape == fc.x.shape, "forecast graphs are captured for one batch size"
            self.forecast_stream.wait_stream(torch.cuda.current_stream(block.device))
            x.record_stream(self.forecast_stream)
            fc.launch(x, self.forecast_stream)
            snapshot = dict(ticket=ticket, room=room, members=frozenset(res.cache.resident_ids()),
                            minimum=float(res.min_candidate_score()))
            fc.task = res.ring.worker = self.scorer.submit(self._score_and_publish, fc, target, **snapshot)
        block.metrics.rs_next_layer_pred_calls += 1
        self.count("predictions")

    def _score_and_publish(self, fc: CapturedForecast, target, *, ticket, room: int, members: frozenset,
                           minimum: float) -> dict:
        """Scoring thread: wait for the read-back, choose, publish copies until the ring declines
        (utils/rs_overlap.py:227-253).  Reads snapshots only; the ring's lock is the single
        point of contact with the layer's thread."""
        from . import ops
        t0 = perf_counter()
        fc.landed.synchronize()
        t1 = perf_counter()
        ring: StagingRing = target.residency.ring
        layer = int(target.layer_idx)
        events, lane, arena = self.copy_events[layer], self.copy_lane.handle, target.arena
        seen: Dict[str, int] = {}

        def copy_of(eid: int):
            def enqueue(slot: int, pos: int):
                ops.expert_upload_async(target.slab.slot_ptr(slot), arena.host_ptr(eid), arena.expert_bytes, lane,
                                        events[pos])
                return events[pos]
            return enqueue

        if ring.ticket == ticket:       # a stale read only costs a scoring pass; publish() decides
            chosen = select_candidates(fc.host_ids.flatten().tolist(), fc.host_probs.flatten().tolist(),
                                       allowed=self.owned[layer], resident=members, minimum=minimum, budget=room,
                                       diagnostics=seen)
            ring.note_chosen(ticket, len(chosen))
            for eid in chosen:
                if not ring.publish(ticket, eid, copy_of(eid)):
                    break           # sealed, or full: nothing later can get in either
        return dict(ms=(perf_counter() - t0) * 1e3, waited_ms=(t1 - t0) * 1e3, seen=seen)

    def seal(self, block, step: int) -> None:
        """At the target's executor, after router and permutation: end the window and make its
        copies readable (utils/rs_overlap.py:303-346).  A scoring task that has not published
        yet has lost its chance for this step; it is not waited for."""
        layer, res = int(block.layer_idx), block.residency
        self.count("demand_deadline_activations")
        with self._timed("target_close_ms"):
            ticket, filled, chosen = res.ring.seal()
        if ticket is None:
            return
        assert ticket == (self.epoch, int(step), layer), "a forecast crossed a request or step boundary"
        if chosen == 0 and self.pause.steps:
            self.pause.arm(layer, int(step), res.cache.resident_ids())
        if filled:
            res.expose_staged(filled)
            self.count("plans")
            self.count("issued", len(filled))
        else:
            self.count("closed_before_publish")
            self.count("unplanned_closes" if chosen is None else
                       "empty_plan_closes" if chosen == 0 else "planned_no_publish_closes")

    def settle(self, block) -> list:
        """Layer exit: the residency admits what was used and returns the ring's positions; the
        engine only keeps count.  Returns the settled ``(expert, record)`` pairs."""
        settled = block.residency.settle_staged()
        for _eid, rec in settled:
            self.count("used" if rec.touched else "wasted")
            if rec.kept:
                self.count("retained")
                self.count("recycled_payloads" if rec.recycled else "allocated_replacements")
        return settled

    # ---- end of request ------------------------------------------------------------------------
    def finish(self) -> dict:
        """Drain: seal what is still open, let the scoring tasks and both streams run out, settle
        (utils/rs_overlap.py:406-432).  Returns the request's statistics."""
        t0 = perf_counter()
        for block in self.layers.values():
            ring = block.residency.ring
            _ticket, filled, _chosen = ring.seal()
            for _eid, pos, event in filled:         # copied for a step that never came
                ring.give_back(pos, event)
        for fc in self.forecasts.values():
            if fc.task is not None:
                fc.task.result(timeout=30)
                self._absorb(fc)
        if self.copy_lane is not None:      # None: the engine was never bound to a device
            self.forecast_stream.synchronize()
            self.copy_lane.synchronize()
        for block in self.layers.values():
            self.settle(block)
            block.residency.confirm_staged_copies()
            block.residency.ring.worker = None
        self.stats["request_drain_ms"] = (perf_counter() - t0) * 1e3
        return {"case": self.case, **self.stats}

    def shutdown(self) -> None:
        assert self._quiet(), "finish() the request first"
        self.scorer.shutdown(wait=True)
