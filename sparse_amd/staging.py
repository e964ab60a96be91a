"""Bounded next-layer RS staging: the opt-in alternative to the in-line prefetch planner.

Mirrors the reference's ownership rules (utils/rs_staging.py:12-118) and pipeline
(utils/rs_overlap.py:58-497) on this build's slot model:

  * speculation never writes the resident LRU; a staged expert sits in a slot of the
    target layer's *staging pool* and is visible to demand lookups through
    ``DemandCacheView`` only;
  * the predictor's top-k is captured in a graph on a side stream, read back
    asynchronously into pinned memory, and scored by one worker thread, which publishes
    copies under the target's lock; the target closes publication when its executor starts
    (``activate_at_demand``) -- a prediction is never joined;
  * at the target layer's exit (``release``) the experts that were actually used are
    admitted to the LRU in first-use order by exchanging slot ownership, not bytes: the
    evicted resident's slot becomes the pool's next scratch slot.

Where the reference's pool is four free-standing payloads shared by all layers, a payload
here is a slot index of the target layer's own HBM slab (a kernel addresses weights as
slab base + slot * stride), so every offloaded layer carries ``pool_slots`` extra slots
(``ResidencyConfig.staging_pool_slots``).  The engine is wired into the block through
``SparseContext.staging`` instead of patching methods at run time
(utils/rs_overlap.py:434-486 lists the seven patch points; the hooks sit at the same
places).
"""
from __future__ import annotations

import threading
import time
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass
from typing import Any, Callable, Dict, Iterable, List, Optional


# --------------------------------------------------------------------------- ownership rules
@dataclass
class Transfer:
    """One issued copy (utils/rs_staging.py:12-20)."""

    expert: int
    payload: Any
    event: Any
    slot: Any
    nbytes: int
    used: bool = False
    retained: bool = False


class TargetJob:
    """Copies predicted for one (epoch, step, target layer) (utils/rs_staging.py:23-49)."""

    def __init__(self, ticket, slots) -> None:
        self.ticket = ticket
        self.slots = slots
        self.transfers: Dict[int, Transfer] = {}
        self.closed = False
        self.lock = threading.Lock()
        self.future = None
        self.plan_count: Optional[int] = None

    def publish(self, expert: int, submit: Callable[[], Transfer]) -> bool:
        """Submit and publish one transfer atomically, or decline once the target has closed.
        ``submit`` may only enqueue on preallocated storage."""
        with self.lock:
            if self.closed:
                return False
            transfer = submit()
            assert transfer.expert == expert and expert not in self.transfers
            self.transfers[expert] = transfer
            return True

    def close(self) -> Dict[int, Transfer]:
        with self.lock:
            self.closed = True
            return dict(self.transfers)


class DemandCacheView:
    """The resident cache plus the copies issued for this layer call; only the resident part
    has capacity, recency and eviction (utils/rs_staging.py:52-94)."""

    def __init__(self, resident) -> None:
        self.resident = resident
        self.staged: Dict[int, Transfer] = {}
        self.used_in_order: List[Transfer] = []

    def __getattr__(self, name):
        return getattr(self.resident, name)

    def __len__(self) -> int:
        return len(self.resident)

    def has(self, expert) -> bool:
        return self.resident.has(expert) or int(expert) in self.staged

    def get(self, expert):
        payload = self.resident.get(expert)
        if payload is not None:
            return payload
        transfer = self.staged.get(int(expert))
        if transfer is None:
            return None
        if not transfer.used:
            transfer.used = True
            self.used_in_order.append(transfer)
        return transfer.payload

    def peek(self, expert):
        payload = self.resident.peek(expert)
        if payload is not None:
            return payload
        transfer = self.staged.get(int(expert))
        return None if transfer is None else transfer.payload

    def resident_ids(self):
        return self.resident.resident_ids()


def select_candidates(ids: Iterable[int], weights: Iterable[float], *, allowed, resident, minimum: float,
                      budget: int, diagnostics: Optional[dict] = None) -> List[int]:
    """Aggregate probability / reuse score without victim selection
    (utils/rs_staging.py:97-118; the formula of utils/eval_core.py:10104-10106)."""
    total: Dict[int, float] = {}
    hits: Dict[int, int] = {}
    peak: Dict[int, float] = {}
    skipped_owner = skipped_resident = 0
    for eid, weight in zip(ids, weights):
        eid, weight = int(eid), float(weight)
        if eid not in allowed:
            skipped_owner += 1
        elif eid in resident:
            skipped_resident += 1
        else:
            total[eid] = total.get(eid, 0.0) + weight
            hits[eid] = hits.get(eid, 0) + 1
            peak[eid] = max(peak.get(eid, 0.0), weight)
    score = {eid: s * (1 + .15 * (hits[eid] - 1)) + .05 * peak[eid] for eid, s in total.items()}
    if diagnostics is not None:
        diagnostics.update(nonlocal_entries=skipped_owner, resident_entries=skipped_resident, scored=len(score),
                           below_threshold=sum(v < minimum for v in score.values()))
    ranked = sorted(score, key=score.get, reverse=True)
    return [eid for eid in ranked if score[eid] >= minimum][:budget]


# --------------------------------------------------------------------------- predictor
class GraphPrediction:
    """Predictor + top-k of one source layer, captured once and replayed
    (utils/rs_overlap.py:21-55)."""

    def __init__(self, model, batch: int, width: int, k: int, dtype, normalize: bool, device) -> None:
        import torch
        self.torch, self.model = torch, model
        self.k, self.dtype, self.normalize = int(k), dtype, bool(normalize)
        self.input = torch.zeros((batch, width), device=device, dtype=torch.float32)
        stream = torch.cuda.Stream(device=device)
        stream.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(stream), torch.inference_mode():
            for _ in range(3):
                self.compute(self.input)
        stream.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=stream), torch.inference_mode():
            self.ids, self.values = self.compute(self.input)
        torch.cuda.current_stream(device).wait_stream(stream)
        self.validations = 0

    def compute(self, x):
        t = self.torch
        values, ids = t.topk(self.model(x).to(t.float32), k=self.k, dim=-1)
        if self.normalize:
            values = values / values.sum(-1, keepdim=True).clamp_min(1e-12)
        return ids.to(t.long), values.to(self.dtype)

    def __call__(self, x):
        self.input.copy_(x)
        self.graph.replay()
        return self.ids, self.values

    def verify(self, x) -> None:
        want_ids, want_values = self.compute(x.float())
        ids, values = self(x.float())
        assert self.torch.equal(ids, want_ids) and self.torch.equal(values, want_values)
        self.validations += 1


_STAT_KEYS = ("predictions", "plans", "issued", "used", "wasted", "closed_before_publish", "skipped_slots",
              "skipped_cooldown", "unified_epipe_calls", "demand_deadline_activations", "empty_plan_closes",
              "unplanned_closes", "planned_no_publish_closes", "observed_decode_misses",
              "cooldown_miss_invalidations", "cooldown_cache_invalidations", "candidate_nonlocal_entries",
              "candidate_resident_entries", "candidate_scored", "candidate_below_threshold", "retained",
              "recycled_payloads", "allocated_replacements")


class BoundedRS:
    """The staging controller (utils/rs_overlap.py:58-433).  One instance serves the whole
    layer stack; ``SparseContext.staging`` points at it while it is installed."""

    def __init__(self, *, slots: int = 4, empty_steps: int = 0) -> None:
        self.enabled = False
        self.slot_count, self.empty_steps = int(slots), int(empty_steps)
        assert self.slot_count >= 2 and self.empty_steps >= 0
        self.pool = ThreadPoolExecutor(max_workers=1, thread_name_prefix="rs-staging")
        self.graphs: Dict[Any, GraphPrediction] = {}
        self.buffers: Dict[Any, Any] = {}
        self.jobs: Dict[int, TargetJob] = {}
        self.retired: List[Any] = []
        self.slots: Dict[int, List[dict]] = {}      # layer -> pool slot records
        self.views: Dict[int, DemandCacheView] = {}
        self.next_probe: Dict[int, int] = {}
        self.allowed: Dict[int, frozenset] = {}
        self.cooldown_residents: Dict[int, frozenset] = {}
        self.pending_completion_metrics: List[Any] = []
        self.epoch = 0
        self.stream = None
        self.copy_stream = None
        self.owner = threading.get_ident()
        self.case = None
        self.stats: Dict[str, Any] = {}
        self.blocks: Dict[int, Any] = {}

    # ---- configuration ------------------------------------------------------------
    def configure(self, *, empty_steps) -> None:
        """Set the empty-forecast cool-down, only between drained requests
        (utils/rs_overlap.py:78-85)."""
        if type(empty_steps) is not int or empty_steps < 0:
            raise ValueError("empty_steps must be a nonnegative integer")
        assert not self.jobs and not self.retired and not self.views
        self.empty_steps = empty_steps
        self.next_probe.clear()
        self.cooldown_residents.clear()

    def note_demand_miss(self, block) -> None:
        """A new miss invalidates the target's stale empty forecast (utils/rs_overlap.py:87-93)."""
        layer = int(block.layer_idx)
        self.stats["observed_decode_misses"] += 1
        if self.next_probe.pop(layer, None) is not None:
            self.cooldown_residents.pop(layer, None)
            self.stats["cooldown_miss_invalidations"] += 1

    def _skip_cooldown(self, layer: int, step: int) -> bool:
        """utils/rs_overlap.py:95-109."""
        deadline = self.next_probe.get(layer, 0)
        if step >= deadline:
            self.next_probe.pop(layer, None)
            self.cooldown_residents.pop(layer, None)
            return False
        resident = frozenset(self.views[layer].resident_ids())
        if resident != self.cooldown_residents[layer]:
            self.next_probe.pop(layer, None)
            self.cooldown_residents.pop(layer, None)
            self.stats["cooldown_cache_invalidations"] += 1
            return False
        self.stats["skipped_cooldown"] += 1
        return True

    # ---- set-up ---------------------------------------------------------------------
    def prepare(self, blocks: Dict[int, Any], rs_bank, *, batch: int, dtype, k: Optional[int] = None) -> None:
        """Capture the predictors and claim every layer's pool slots
        (``prepare_graphs``, utils/rs_overlap.py:116-166).  Call once, before ``begin``."""
        import torch
        from . import ops
        assert not self.jobs and not self.retired
        self.blocks = dict(blocks)
        for layer, block in sorted(self.blocks.items()):
            res = block.residency
            assert res is not None and block.expert_offload == "cpu" and block.cache_policy == "lru"
            pool = res.claim_staging_pool(self.slot_count)
            self.slots[layer] = [dict(payload=s, event=ops.Event(), retire=None, busy=False,
                                      nbytes=int(res.expert_bytes), layer=layer) for s in pool]
            if layer + 1 >= block.num_layers or layer + 1 not in self.blocks:
                continue
            target = self.blocks[layer + 1].residency
            kk = int(k) if k is not None else min(block.num_experts, target.predict_topk())
            # the captured prediction reads the hidden state only (utils/rs_overlap.py:124)
            if str(getattr(rs_bank[layer + 1], "rs_feature_mode", "hidden")) != "hidden":
                raise ValueError("the bounded staging engine needs predictors with feature_mode='hidden'")
            graph = GraphPrediction(rs_bank[layer + 1], batch, block.hidden_size, kk, dtype,
                                    block.norm_topk_prob, block.device)
            for seed in range(3):
                x = torch.arange(batch * block.hidden_size, device=block.device,
                                 dtype=torch.float32).reshape(batch, -1)
                graph.verify(((x % (97 + seed)) - 48) / 30)
            self.graphs[layer, kk] = graph
            self.buffers[layer, kk] = (torch.empty((batch, kk), dtype=torch.long, pin_memory=True),
                                       torch.empty((batch, kk), dtype=dtype, pin_memory=True),
                                       torch.cuda.Event(blocking=False))
        device = next(iter(self.blocks.values())).device
        self.stream = torch.cuda.Stream(device=device, priority=0)
        self.copy_stream = ops.SideStream()
        torch.cuda.synchronize()

    def begin(self, case=None) -> None:
        """Start a request (utils/rs_overlap.py:168-205)."""
        assert not self.jobs and not self.retired and not self.views
        self.epoch += 1
        self.case, self.next_probe, self.cooldown_residents = case, {}, {}
        assert not self.pending_completion_metrics
        self.stats = {key: 0 for key in _STAT_KEYS}
        self.stats.update(worker_ms=0.0, readback_wait_ms=0.0, main_submission_ms=0.0, target_close_ms=0.0,
                          request_drain_ms=0.0, effective_empty_steps=self.empty_steps,
                          staging_bytes=sum(s["nbytes"] for pool in self.slots.values() for s in pool))
        if not self.enabled:
            return
        for layer, block in self.blocks.items():
            assert block.expert_source == "router" and block.exec_routing_mode == "router"
            res = block.residency
            view = DemandCacheView(res.cache)
            self.views[layer] = view
            res.cache = view
            block._cache = view
            self.allowed[layer] = frozenset(block._local_eid_set)   # one GPU owns every expert

    # ---- slot pool ---------------------------------------------------------------------
    def _retire(self, slot: dict, event) -> None:
        assert slot["busy"]
        slot["busy"], slot["retire"] = False, event

    def _collect(self) -> None:
        keep = []
        for job, transferred in self.retired:
            if not job.future.done():
                keep.append((job, transferred))
                continue
            row = job.future.result()   # already complete: never a layer join
            self.stats["worker_ms"] += row["worker_ms"]
            self.stats["readback_wait_ms"] += row["readback_wait_ms"]
            for key, value in row.get("candidate_counts", {}).items():
                self.stats["candidate_" + key] += value
            used = {id(x.slot) for x in transferred.values()}
            for slot in job.slots:
                if id(slot) not in used:
                    self._retire(slot, None)
        self.retired = keep

    def _reserve(self, layer: int, budget: int) -> List[dict]:
        self._collect()
        free = [s for s in self.slots[layer] if not s["busy"] and (s["retire"] is None or s["retire"].query())]
        chosen = free[:budget]
        for slot in chosen:
            slot["busy"], slot["retire"] = True, None
        return chosen

    # ---- worker thread --------------------------------------------------------------
    def _work(self, job: TargetJob, target, ids, weights, readback, resident, minimum: float) -> dict:
        """Wait for the read-back, score, publish copies (utils/rs_overlap.py:230-263).
        Works on snapshots only; the single mutation is ``job.publish`` under its lock."""
        from . import ops
        started = time.perf_counter()
        counts: Dict[str, int] = {}
        stamp = time.perf_counter()
        readback.synchronize()
        waited = (time.perf_counter() - stamp) * 1000
        if not job.closed:
            chosen = select_candidates(ids.reshape(-1).tolist(), weights.float().reshape(-1).tolist(),
                                       allowed=self.allowed[target.layer_idx], resident=resident, minimum=minimum,
                                       budget=len(job.slots), diagnostics=counts)
            job.plan_count = len(chosen)
            for eid, slot in zip(chosen, job.slots):
                def submit(eid=eid, slot=slot):
                    ops.expert_upload_async(target.slab.slot_ptr(slot["payload"]), target.arena.host_ptr(eid),
                                            target.arena.expert_bytes, self.copy_stream.handle, slot["event"])
                    return Transfer(eid, slot["payload"], slot["event"], slot, slot["nbytes"])
                if not job.publish(eid, submit):
                    break
        return dict(worker_ms=(time.perf_counter() - started) * 1000, readback_wait_ms=waited,
                    candidate_counts=counts)

    # ---- source layer: predict ---------------------------------------------------------
    def handles(self, block, seq_len: int) -> bool:
        return bool(self.enabled and int(seq_len) == 1 and block.planner_mode == "rs_prefetch")

    def predict(self, block, x, step: int) -> None:
        """Launch the prediction for layer l+1 and hand it to the worker
        (utils/rs_overlap.py:255-303).  Never waits for anything."""
        import torch
        target_layer = int(block.layer_idx) + 1
        if target_layer >= block.num_layers or target_layer not in self.blocks:
            return
        assert threading.get_ident() == self.owner
        target = self.blocks[target_layer]
        if self.empty_steps and self._skip_cooldown(target_layer, step):
            return
        self._collect()   # graph and host buffers must not be reused while an old worker may read them
        if target_layer in self.jobs or any(j.ticket[2] == target_layer for j, _ in self.retired):
            self.stats["skipped_slots"] += 1
            return
        tres = target.residency
        budget = min(int(tres.effective_top_m()), self.slot_count // 2)
        if budget <= 0:
            return
        slots = self._reserve(target_layer, budget)
        if not slots:
            self.stats["skipped_slots"] += 1
            return
        stamp = time.perf_counter()
        k = min(block.num_experts, tres.predict_topk())
        graph = self.graphs[block.layer_idx, k]
        host_ids, host_weights, event = self.buffers[block.layer_idx, k]
        assert tuple(x.shape) == tuple(graph.input.shape)
        self.stream.wait_stream(torch.cuda.current_stream(block.device))
        x.record_stream(self.stream)
        with torch.cuda.stream(self.stream), torch.inference_mode():
            ids, weights = graph(x)
            host_ids.copy_(ids, non_blocking=True)
            host_weights.copy_(weights, non_blocking=True)
            event.record(self.stream)
        job = TargetJob((self.epoch, int(step), target_layer), slots)
        self.jobs[target_layer] = job
        resident = frozenset(self.views[target_layer].resident_ids())
        job.future = self.pool.submit(self._work, job, target, host_ids, host_weights, event, resident,
                                      float(tres.min_candidate_score()))
        block.metrics.rs_next_layer_pred_calls += 1
        self.stats["predictions"] += 1
        self.stats["main_submission_ms"] += (time.perf_counter() - stamp) * 1000

    # ---- target layer: close, use, release ----------------------------------------------
    def activate(self, block, step: int) -> None:
        """Close publication for this layer and expose what was issued
        (utils/rs_overlap.py:305-340)."""
        layer = int(block.layer_idx)
        view = self.views[layer]
        assert not view.staged and not view.used_in_order
        job = self.jobs.pop(layer, None)
        if job is None:
            return
        stamp = time.perf_counter()
        transfers = job.close()
        self.stats["target_close_ms"] += (time.perf_counter() - stamp) * 1000
        ticket = (self.epoch, int(step), layer)
        assert job.ticket == ticket, "Stale prediction crossed a request/step boundary"
        self.retired.append((job, transfers))
        if job.plan_count == 0 and self.empty_steps:
            self.next_probe[layer] = ticket[1] + self.empty_steps + 1
            self.cooldown_residents[layer] = frozenset(view.resident_ids())
        if not transfers:
            self.stats["closed_before_publish"] += 1
            if job.plan_count is None:
                self.stats["unplanned_closes"] += 1
            elif job.plan_count == 0:
                self.stats["empty_plan_closes"] += 1
            else:
                self.stats["planned_no_publish_closes"] += 1
        view.staged = transfers
        res = block.residency
        self.stats["plans"] += bool(transfers)
        for eid, transfer in transfers.items():
            res.prefetched_ids.add(eid)
            res.prefetch_events[eid] = transfer.event
            res.metrics.prefetch_h2d_bytes += transfer.nbytes
            res.metrics.prefetch_issued_count += 1
            res.metrics.prefetch_admitted_count += 1
            self.stats["issued"] += 1

    def activate_at_demand(self, block, step: int) -> None:
        """Publication stays open through router and permutation; it closes here, at the
        executor's entry (utils/rs_overlap.py:342-350)."""
        self.activate(block, step)
        self.stats["demand_deadline_activations"] += 1

    def _retain_used(self, block, transfer: Transfer) -> None:
        """Admit an expert that was really used, after the layer: exchange slot ownership
        with the evicted resident instead of moving bytes (utils/rs_overlap.py:352-381)."""
        assert transfer.used and not transfer.retained
        replacement, recycled = block.residency.adopt_staged(transfer.expert, transfer.payload, transfer.event)
        if replacement is None:
            return
        self.stats["recycled_payloads" if recycled else "allocated_replacements"] += 1
        transfer.slot["payload"] = replacement
        transfer.retained = True
        self.stats["retained"] += 1

    def release(self, block) -> None:
        """Layer exit (utils/rs_overlap.py:383-408)."""
        view = self.views[int(block.layer_idx)]
        res = block.residency
        used = [x for x in view.staged.values() if x.used]
        done = res.backend.fence() if used else None   # after every consumer on the compute lane
        for transfer in view.used_in_order:
            self._retain_used(block, transfer)
        for eid, transfer in view.staged.items():
            self._retire(transfer.slot, done if transfer.used else transfer.event)
            self.stats["used" if transfer.used else "wasted"] += 1
            if not transfer.used:
                res.metrics.prefetch_wasted_count += 1
                self.pending_completion_metrics.append(res)
            res.prefetch_events.pop(eid, None)
            res.prefetched_ids.discard(eid)
            res.prefetch_used_ids.discard(eid)
        view.staged = {}
        view.used_in_order = []

    def finish(self) -> dict:
        """Drain the request (utils/rs_overlap.py:410-432)."""
        stamp = time.perf_counter()
        for layer, job in list(self.jobs.items()):
            transfers = job.close()
            self.retired.append((job, transfers))
            for transfer in transfers.values():
                self._retire(transfer.slot, transfer.event)
        self.jobs.clear()
        for job, _ in self.retired:
            job.future.result(timeout=30)
        self._collect()
        if self.stream is not None:
            self.stream.synchronize()
            self.copy_stream.synchronize()
        for layer, view in self.views.items():
            block = self.blocks[layer]
            if view.staged:
                self.release(block)
            assert block.residency.cache is view
            block.residency.cache = view.resident
            block._cache = view.resident
        self.views = {}
        for res in self.pending_completion_metrics:
            res.metrics.prefetch_completed_count += 1
        self.pending_completion_metrics = []
        self.stats["request_drain_ms"] = (time.perf_counter() - stamp) * 1000
        return dict(case=self.case, **self.stats)

    def shutdown(self) -> None:
        assert not self.jobs and not self.retired and not self.views
        self.pool.shutdown(wait=True)
