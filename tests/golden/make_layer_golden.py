#!/usr/bin/env python3
"""Write golden traces of one layer's residency state machine from the reference's own code.

Runs ONLY in the build container, where the reference checkout is mounted at
/root/reference; the fixture it writes (``layer_traces.json``) is what the tests read, so
nothing at test time touches the reference.

The reference's executors refuse to run without a CUDA device
(utils/eval_core.py:11881, :12184, :12530, :12860), and the reference package cannot be
imported here (it needs transformers and a GPU at import time).  As in the reference's own
tests (tests/test_rs_staging.py:18-34, tests/test_lightweight_policy.py:63-71), the methods
are therefore taken out of ``utils/eval_core.py`` by name with ``ast`` and executed against
a stub block: the demand path, the four EPIPE executors, the prefetch cycle / budget / plan /
admission methods, the prefill side cache helpers and the cache classes all run as written.
Only device services are replaced: streams and events are recording stand-ins, weight
tensors are tagged placeholders, and the expert FFN returns zeros.  What the stand-ins
record is exactly what the oracle's trace records:

    cache events (hit / prefetch_hit / miss, in order), copies (lane, expert), waits of the
    compute stream on a copy (and of a side stream on a copy it is about to overwrite), the
    order experts are executed in, admitted prefetch plans, the executor chosen per call, and
    the contents of cache and side cache at the end.

Inputs (routing per step and layer, predictor top-k lists, which prefetch copies are still
in flight when first looked at) are generated here from a seed and stored in the fixture
next to the expected traces, so the tests replay exactly the same calls.
"""
from __future__ import annotations

import ast
import json
import os
import random
import sys
from collections import OrderedDict
from contextlib import nullcontext
from dataclasses import dataclass
from pathlib import Path
from types import SimpleNamespace as NS
from typing import Any, Dict, List, Optional, Sequence, Set, Tuple

ROOT = Path(__file__).resolve().parents[2]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

from tests.helpers import copy_is_late, seeded_prediction  # noqa: E402  (shared with the tests that replay the fixture)

REF = Path("/root/reference/utils/eval_core.py")
OUT = Path(__file__).resolve().parent

CLASSES = ("CacheEntry", "ExpertWeightCache", "EpipePrefillExtraCache", "TieredExpertWeightCache")
METHODS = (
    # demand path
    "_get_local_module_weights", "_maybe_wait_prefetch", "_on_demand_access", "_should_prefer_hot",
    "_cache_put_guarded", "_cache_protect_ids", "_cache_protect_ids_with_fallback",
    "_record_protected_eviction_effect", "_should_mark_prefill_scp_transient",
    "_maybe_upgrade_prefill_scp_transient_on_decode", "_current_stage",
    # segment execution
    "_plain_ep_compute_segment", "_epipe_compute_segment",
    # EPIPE helpers and executors
    "_epipe_stage_enabled", "_cache_contains_no_touch", "_epipe_get_prefetch_pending_event",
    "_epipe_record_cached_payload_use", "_epipe_get_ready_payload_for_compute",
    "_epipe_rs_demand_stage_gate_can_open", "_epipe_rs_demand_stage_gate_open",
    "_epipe_prefill_extra_cache_enabled", "_epipe_prefill_extra_cache_store", "_epipe_prefill_extra_cache_get",
    "_epipe_prefill_extra_cache_contains", "_epipe_prefill_extra_cache_resident_count",
    "_epipe_prefill_extra_cache_clear", "_epipe_record_prefill_multistage_shadow",
    "_try_execute_local_recv_groups_epipe", "_try_execute_local_recv_groups_epipe_rs_residual_scan",
    "_try_execute_local_recv_groups_epipe_rs_buffered", "_try_execute_local_recv_groups_epipe_miss_triggered",
    # RS prefetch cycle, budget, plan, admission
    "_prefetch_target_budget", "_begin_group_prefetch_cycle", "_finalize_prev_group_prefetch",
    "_finalize_completed_prefetch_events", "_prefetch_protect_ids", "_prefetch_total_insert_capacity",
    "_prefetch_evictable_ids", "_prefetch_free_slots", "_effective_rs_prefetch_top_m", "_rs_prefetch_predict_topk",
    "_build_prefetch_plan_from_prob_predictions", "_build_target_layer_prob_score_map",
    "_build_prefetch_plan_from_score_map", "_resident_keep_bias", "_pick_victims_by_low_value",
    "_admit_prefetch_plan", "_discard_cache_entry_before_prefetch", "_record_prefetch_event",
    "_compute_and_schedule_next_layer_rs", "_run_rs_mlp_timed", "_next_layer_rs_feature_mode",
    # environment readers
    "_rank_env_value", "_rank_env_int", "_rank_env_float", "_rs_env_int", "_rs_env_float",
    # lifecycle
    "reset_runtime_state_for_new_request",
)


# ------------------------------------------------------------------------------------ device stand-ins
class Recorder:
    def __init__(self) -> None:
        self.trace: List[Tuple] = []
        self.lane = "compute"
        self.step = 0


class FakeStream:
    def __init__(self, rec: Recorder, lane: str) -> None:
        self.rec, self.lane = rec, lane

    def wait_event(self, event: "FakeEvent") -> None:
        if event.copy_of is not None:
            self.rec.trace.append(("wait" if self.lane == "compute" else f"wait_{self.lane}_lane", event.copy_of))

    def synchronize(self) -> None:
        pass


class FakeEvent:
    """``query()`` answers "is the copy done": a copy flagged late is still in flight the first
    time it is asked about, and finished from then on."""

    def __init__(self, rec: Recorder, **_kw: Any) -> None:
        self.rec = rec
        self.copy_of: Optional[int] = None
        self.late = False

    def record(self, stream: Optional[FakeStream] = None) -> None:
        pending = getattr(self.rec, "pending_copy", None)
        if pending is not None:
            self.copy_of, self.late = pending
            self.rec.pending_copy = None

    def query(self) -> bool:
        if self.late:
            self.late = False
            return False
        return True

    def synchronize(self) -> None:
        pass


class Counters:
    """Stands in for the harness's metrics object: any counter reads as zero until set."""

    def __getattr__(self, name: str) -> Any:
        if name.startswith("__"):
            raise AttributeError(name)
        return None if name.startswith("_pending") or name.endswith("_stats") else 0


class Weight:
    """Placeholder for a weight tensor; ``to(device)`` of a host weight is a copy."""

    def __init__(self, rec: Recorder, eid: int, part: str, on_device: bool) -> None:
        self.rec, self.eid, self.part, self.on_device = rec, eid, part, on_device

    def to(self, *_a: Any, **_k: Any) -> "Weight":
        if self.part == "gate":
            self.rec.trace.append(("h2d", self.rec.lane, self.eid))
        return Weight(self.rec, self.eid, self.part, True)


def make_torch(rec: Recorder):
    """The real ``torch`` with a ``cuda`` namespace made of the stand-ins above."""
    import torch

    class StreamCtx:
        def __init__(self, stream: FakeStream) -> None:
            self.stream = stream

        def __enter__(self):
            self.prev, rec.lane = rec.lane, self.stream.lane
            return self

        def __exit__(self, *exc):
            rec.lane = self.prev
            return False

    compute = FakeStream(rec, "compute")
    by_lane = {"compute": compute}

    def current_stream(*_a: Any, **_k: Any) -> FakeStream:
        # inside ``with torch.cuda.stream(s)`` the current stream is ``s``
        return by_lane.setdefault(rec.lane, FakeStream(rec, rec.lane))

    cuda = NS(is_available=lambda: True, stream=StreamCtx, current_stream=current_stream,
              Event=lambda **kw: FakeEvent(rec, **kw), OutOfMemoryError=torch.cuda.OutOfMemoryError,
              empty_cache=lambda: None, mem_get_info=lambda *_a: (1 << 40, 1 << 40), synchronize=lambda *_a: None)

    class Proxy:
        def __getattr__(self, name: str) -> Any:
            return cuda if name == "cuda" else getattr(torch, name)

    return Proxy(), compute


def extract(rec: Recorder, env: Dict[str, str], context: NS):
    import torch
    import torch.nn.functional as F
    tree = ast.parse(REF.read_text())
    classes = [n for n in tree.body if isinstance(n, ast.ClassDef) and n.name in CLASSES]
    block = next(n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == "DistributedSparseMoeBlock")
    methods = [n for n in block.body if isinstance(n, ast.FunctionDef) and n.name in METHODS]
    missing = set(METHODS) - {m.name for m in methods}
    if missing:
        sys.exit(f"methods not found in the reference: {sorted(missing)}")
    future = ast.ImportFrom(module="__future__", names=[ast.alias(name="annotations")], level=0)
    module = ast.Module(body=[future, *classes, *methods], type_ignores=[])
    proxy, compute = make_torch(rec)

    def env_flag(name: str, default: str = "0") -> bool:
        return str(env.get(name, default)).strip().lower() not in ("", "0", "false", "no", "off")

    ns: Dict[str, Any] = dict(
        OrderedDict=OrderedDict, dataclass=dataclass, Any=Any, Dict=Dict, List=List, Optional=Optional, Tuple=Tuple,
        Sequence=Sequence, Set=Set, os=NS(environ=env), torch=proxy, F=F, nullcontext=nullcontext,
        SparseContext=context, _env_flag=env_flag,
        _env_int=lambda name, default=0: int(env.get(name, default)),
        _env_float=lambda name, default=0.0: float(env.get(name, default)),
        _hclm_cp_now_ns=lambda: 0, tensor_nbytes=lambda t: 0, _append_prefetch_h2d_event=lambda *a, **k: None,
        Metrics=object, time=__import__("time"), nn=torch.nn)
    exec(compile(ast.fix_missing_locations(module), str(REF), "exec"), ns)
    return ns, compute, torch


# ------------------------------------------------------------------------------------ the stub block
class StubBlock:
    """``self`` for the extracted methods: state and configuration are real attributes,
    extracted methods bind on lookup, accounting calls are swallowed."""

    def __init__(self, ns, torch, rec: Recorder, compute: FakeStream, layer: int, cfg: Dict[str, Any], E: int, K: int,
                 env: Dict[str, str]) -> None:
        d = self.__dict__
        d["_ns"], d["_rec"], d["_env"] = ns, rec, env
        self.layer_idx, self.num_layers = layer, cfg["layers"]
        self.num_experts, self.top_k = E, K
        self.device = NS(type="cuda")
        self.expert_offload, self.experts_kind = "cpu", "modulelist"
        self.planner_mode = cfg["planner_mode"]
        self.placement_mode, self.oracle_mode = "round_robin", "none"
        self.expert_source = self.exec_routing_mode = "router"
        self.comm_rank = self.rank = 0
        self.metrics = Counters()
        self.norm_topk_prob = False
        self.local_expert_ids = list(range(E))
        self._local_eid_set = set(range(E))
        self._rr_local_eid_set = set(range(E))
        self.local_gate_cpu = {e: Weight(rec, e, "gate", False) for e in range(E)}
        self.local_up_cpu = {e: Weight(rec, e, "up", False) for e in range(E)}
        self.local_down_cpu2 = {e: Weight(rec, e, "down", False) for e in range(E)}
        self.prefetch_stream = FakeStream(rec, "prefetch")
        self.epipe_stream = FakeStream(rec, "epipe")
        if cfg["cache_policy"] == "tiered":
            self._cache = ns["TieredExpertWeightCache"](cfg["tiered"][0], hot_capacity=cfg["tiered"][1],
                                                        prefetch_reserved=cfg["tiered"][2])
        else:
            self._cache = ns["ExpertWeightCache"](cfg["capacity"])
        self._base_expert_cache_capacity = cfg["capacity"]
        self.cache_policy = cfg["cache_policy"]
        self._epipe_prefill_extra_cache = ns["EpipePrefillExtraCache"](cfg["epipe_prefill_extra_cache_slots"])
        # request state (constructor defaults of the reference, :4560-4600)
        self._prefetched_ids_this_group, self._prefetch_used_ids_this_group = set(), set()
        self._prefetch_events, self._prefetch_expire_layer = {}, {}
        self._transition_prefetched_ids, self._transition_used_ids = set(), set()
        self._prefetch_current_group_start = self._prefetch_current_group_end = None
        self._prefetch_current_cycle_key = None
        self._expert_access_freq, self._last_used_decode_step = {}, {}
        self._light_policy = None
        self._current_forward_batch_size, self._current_forward_seq_len = 0, 0
        self._epipe_rs_gate_calls = self._epipe_rs_gate_triggers = self._epipe_rs_gate_skip_remaining = 0
        # configuration, under the reference's attribute names (:4939-5027)
        late_only = cfg["epipe_decode_rs_mode"] == "late_only"
        demand_only = cfg["epipe_decode_rs_mode"] == "demand_only"
        for name, value in dict(
            _epipe_enable=cfg["epipe_enable"], _epipe_shadow=cfg["epipe_shadow"], _epipe_mode=cfg["epipe_mode"],
            _epipe_decode_with_rs_mode=cfg["epipe_decode_rs_mode"], _epipe_decode_only=True,
            _epipe_no_evict=cfg["epipe_no_evict"], _epipe_transient_staging=cfg["epipe_transient_staging"],
            _epipe_max_staged_experts=cfg["epipe_max_staged_experts"], _epipe_min_free_mb=0.0,
            _epipe_prefill_min_free_mb=0.0, _epipe_lookahead_experts=cfg["epipe_lookahead_experts"],
            _epipe_lookahead_min_ready_items=cfg["epipe_lookahead_min_ready_items"],
            _epipe_prefill_lookahead_min_ready_items=cfg["epipe_prefill_lookahead_min_ready_items"],
            _epipe_sort_ready_by_work=cfg["epipe_sort_ready_by_work"],
            _epipe_rs_buffer_max_groups=cfg["epipe_rs_buffer_max_groups"],
            _epipe_rs_buffer_max_items=cfg["epipe_rs_buffer_max_items"],
            _epipe_rs_min_buffer_groups=cfg["epipe_rs_min_buffer_groups"],
            _epipe_rs_min_buffer_items=cfg["epipe_rs_min_buffer_items"],
            # the constructor narrows the two handlers by mode (:4975-4984)
            _epipe_rs_handle_late_prefetch=cfg["epipe_rs_handle_late_prefetch"] and not demand_only,
            _epipe_rs_handle_demand_miss=cfg["epipe_rs_handle_demand_miss"] and not late_only,
            _epipe_rs_demand_commit=cfg["epipe_rs_demand_commit"],
            _epipe_rs_force_demand_stage=cfg["epipe_rs_force_demand_stage"],
            _epipe_rs_demand_stage_threshold_ms=cfg["epipe_rs_demand_stage_threshold_ms"],
            _epipe_rs_rolling_gate=cfg["epipe_rs_rolling_gate"],
            _epipe_rs_gate_window=cfg["epipe_rs_gate_window"],
            _epipe_rs_gate_min_triggers=cfg["epipe_rs_gate_min_triggers"],
            _epipe_rs_gate_skip_steps=cfg["epipe_rs_gate_skip_steps"], _epipe_stage_first_missing_only=True,
            _epipe_min_ready_experts=cfg["epipe_min_ready_experts"],
            _epipe_min_missing_experts=cfg["epipe_min_missing_experts"],
            _epipe_min_ready_items=cfg["epipe_min_ready_items"], _epipe_min_missing_h2d_bytes=1,
            _epipe_deferred_lru_commit=cfg["epipe_deferred_lru_commit"],
            _epipe_decode_rs_commit=cfg["epipe_decode_rs_commit"],
            _epipe_decode_no_rs_commit=cfg["epipe_decode_no_rs_commit"],
            _epipe_prefill_enable=cfg["epipe_prefill_enable"], _epipe_prefill_shadow=cfg["epipe_prefill_shadow"],
            _epipe_prefill_multistage_shadow=cfg["epipe_prefill_multistage_shadow"],
            _epipe_prefill_multistage_max_n=cfg["epipe_prefill_multistage_max_n"],
            _epipe_prefill_commit=cfg["epipe_prefill_commit"],
            _epipe_prefill_mark_transient=cfg["epipe_prefill_mark_transient"],
            _epipe_prefill_no_touch_ready=cfg["epipe_prefill_no_touch_ready"],
            _epipe_timing=False, _epipe_debug_counters=False, _epipe_validate_output=False,
            _epipe_prefill_extra_cache_decode_read=cfg["epipe_prefill_extra_cache_decode_read"],
            _epipe_prefill_extra_cache_clear_at_decode=cfg["epipe_prefill_extra_cache_clear_at_decode"],
            _epipe_prefill_extra_cache_persist_requests=cfg["epipe_prefill_extra_cache_persist_requests"],
            _epipe_prefill_extra_cache_max_mb=cfg["epipe_prefill_extra_cache_max_mb"],
            _epipe_prefill_extra_cache_min_free_mb=0.0,
            _prefetch_min_candidate_score=cfg["min_candidate_score"],
            _prefetch_replace_advantage=cfg["replace_advantage"], _prefetch_replace_margin=cfg["replace_margin"],
            _prefetch_allow_active_replace=cfg["allow_active_replace"], _transition_prefetch_enabled=False,
            _global_expert_cache_enabled=False, prefetch_top_m=cfg["prefetch_top_m"],
            _cache_ttl_steps=cfg["cache_ttl_steps"],
        ).items():
            setattr(self, name, value)

    # ---- lookup: extracted methods bind here; accounting is swallowed ----------------------
    def __getattr__(self, name: str) -> Any:
        fn = self._ns.get(name)
        if callable(fn) and name in METHODS:
            return lambda *a, **k: fn(self, *a, **k)
        if "_record_" in name:             # accounting (counters, timing windows): nothing to keep
            return lambda *a, **k: None
        raise AttributeError(name)

    # ---- what the device / harness would provide --------------------------------------------
    def _record_epipe_counter(self, name: str, value: int = 1) -> None:
        counts = self.__dict__.setdefault("_counts", {})
        counts[str(name)] = counts.get(str(name), 0) + int(value)

    def _record_cache_hit(self, is_prefetch_hit: bool = False) -> None:
        self._rec.trace.append(("prefetch_hit" if is_prefetch_hit else "hit",))

    def _record_cache_miss(self) -> None:
        self._rec.trace.append(("miss",))

    def _record_demand_h2d_window_begin(self):
        return None

    def _record_demand_h2d_window_end(self, _start) -> None:
        pass

    def _module_expert_forward(self, cur, gw, uw, dw):
        import torch
        self._rec.trace.append(("compute", gw.eid))
        return torch.zeros_like(cur)

    def _materialize_local_expert_for_prefetch(self, eid: int):
        self._rec.trace.append(("h2d", "prefetch", int(eid)))
        self._rec.pending_copy = (int(eid), copy_is_late(self._rec.seed, self.layer_idx, self._rec.step, int(eid),
                                                         self._rec.late_rate))
        return tuple(Weight(self._rec, int(eid), p, True) for p in ("gate", "up", "down"))

    def _epipe_load_payload_to_device(self, eid: int):
        self._rec.trace.append(("h2d", "epipe", int(eid)))
        self._rec.pending_copy = (int(eid), False)
        return tuple(Weight(self._rec, int(eid), p, True) for p in ("gate", "up", "down")), 100

    def _epipe_estimate_expert_nbytes(self, eid: int) -> int:
        return 100

    _estimate_local_expert_bytes = _epipe_estimate_expert_nbytes

    def _epipe_memory_headroom_ok(self, *_a, **_k) -> bool:
        return True

    def _demand_h2d_make_memory_room(self, *_a, **_k) -> bool:
        return True

    def _global_cache_make_room(self, *_a, **_k) -> bool:
        return True

    def _prefetch_has_memory_headroom(self, *_a, **_k) -> bool:
        return True

    def _global_cache_enforce_after_demand(self) -> None:
        pass

    def _global_cache_enabled(self) -> bool:
        return False

    def _epipe_timing_sampled(self, *_a, **_k) -> bool:
        return False

    def _timing_sampled(self, *_a, **_k) -> bool:
        return False

    def _stage_uses_scp(self, *_a, **_k) -> bool:
        return False

    def _stage_prefetch_eid_set(self):
        return set(range(self.num_experts))

    def resolve_prefetch_target_rank(self, **_kw):
        return NS(target_rank=0)

    def _rs_prefetch_policy(self) -> str:
        return str(self._env.get("SPARSE_RS_PREFETCH_POLICY", "default"))

    def _epipe_record_stage_success_by_stage(self) -> None:
        pass

    def _epipe_record_staged_demand_h2d(self, *_a) -> None:
        pass

    def _epipe_record_prefill_no_commit_payload(self) -> None:
        pass

    def _epipe_record_executor_call_by_stage(self) -> None:
        pass

    def _epipe_record_stage_enabled(self) -> None:
        pass


# ------------------------------------------------------------------------------------ the driver
def execute(blk: StubBlock, torch, cfg: Dict[str, Any], segments: Sequence[Tuple[int, int]]) -> str:
    """Executor choice of ``_execute_local_recv_groups`` (utils/eval_core.py:13264-13357); the
    function itself works on routed tensors, so its dispatch is followed here and every
    branch calls the reference's own executor."""
    if not segments:
        return "empty"
    rows = sum(n for _, n in segments)
    hidden = torch.zeros(rows, 4)
    weights = torch.zeros(rows)
    segs, at = [], 0
    for eid, n in segments:
        segs.append((int(eid), at, at + n, True))
        at += n
    kw = dict(hidden_sorted=hidden, recv_i_sorted=None, w_sorted=weights, segments=segs, allow_nonlocal=False,
              cp_cuda_timing=False, cp_sampled=False, cp_compute_events=[])
    stage = blk._current_stage()
    rs_active = blk.planner_mode == "rs_prefetch"
    rs_mode, mode = blk._epipe_decode_with_rs_mode, blk._epipe_mode
    result, name = None, None
    if blk._epipe_stage_enabled() and mode != "off":
        if stage == "decode" and rs_active and rs_mode == "off":
            pass
        elif stage == "decode" and rs_active and rs_mode == "residual_scan":
            result, name = blk._try_execute_local_recv_groups_epipe_rs_residual_scan(**kw), "epipe_rs_residual_scan"
        elif stage == "decode" and rs_active and rs_mode in ("buffered", "late_only", "demand_only"):
            result, name = blk._try_execute_local_recv_groups_epipe_rs_buffered(**kw), "epipe_rs_buffered"
        elif stage == "decode" and not rs_active and mode != "miss_triggered":
            result, name = blk._try_execute_local_recv_groups_epipe(**kw), "epipe_upfront"
        elif mode == "upfront_scan":
            result, name = blk._try_execute_local_recv_groups_epipe(**kw), "epipe_upfront"
        else:
            result, name = blk._try_execute_local_recv_groups_epipe_miss_triggered(**kw), "epipe_miss_triggered"
    if result is not None:
        return name
    for eid, s, e, local in segs:
        blk._plain_ep_compute_segment(eid=eid, cur=hidden[s:e], cur_w=weights[s:e].unsqueeze(1), eid_is_local=local,
                                      allow_nonlocal=False)
    return "plain"


POLICY_COSTS = dict(h2d_bytes_per_ms=100.0, h2d_latency_ms=0.1, expert_ms=0.3, item_ms=0.05, next_attention_ms=0.4,
                    split_overhead_ms=0.5)


def policy_expert_bytes(eid: int) -> float:
    """Uneven expert sizes so that the policy's choices are not all ties."""
    return 100.0 + 40.0 * (eid % 5)


def config_dict(method: str, kw: Dict[str, Any]) -> Dict[str, Any]:
    from dataclasses import asdict
    from sparse_amd.cache import tiered_capacity_split
    from sparse_amd.methods import residency_config
    cfg = asdict(residency_config(method, kw["capacity"], kw["top_m"], formal_thresholds=kw["formal"],
                                  **kw["overrides"]))
    cfg["layers"] = kw["layers"]
    if cfg["cache_policy"] == "tiered":
        cfg["tiered"] = list(tiered_capacity_split(cfg["capacity"], cfg["planner_mode"] == "rs_prefetch",
                                                   cfg["prefetch_reserved"], cfg["prefetch_extra_capacity"]))
    return cfg


def reference_env(cfg: Dict[str, Any]) -> Dict[str, str]:
    return {
        "SPARSE_RS_PREFETCH_POLICY": cfg["rs_policy"],
        "SPARSE_RS_CACHE_SAFE_MIN_SCORE": str(cfg["cache_safe_min_score"]),
        "SPARSE_RS_CACHE_SAFE_REPLACE_ADVANTAGE": str(cfg["cache_safe_replace_advantage"]),
        "SPARSE_RS_CACHE_SAFE_REPLACE_MARGIN": str(cfg["cache_safe_replace_margin"]),
        "SPARSE_RS_PREFETCH_RECENT_PROTECT_STEPS": str(cfg["recent_protect_steps"]),
        "SPARSE_PREFETCH_PROTECT_MODE": cfg["protect_mode"],
        "SPARSE_PREFETCH_WAIT_BEFORE_EVICT": "1" if cfg["wait_before_evict"] else "0",
        "SPARSE_CACHE_TTL_STEPS": str(cfg["cache_ttl_steps"]),
        "SPARSE_EPIPE_PROMOTE_TRANSIENT_ON_DECODE_HIT": "1" if cfg["epipe_promote_transient_on_decode_hit"] else "0",
    }


def run_case(method: str, kw: Dict[str, Any]) -> Dict[str, Any]:
    from tests.test_residency import RoutingModel
    cfg = config_dict(method, kw)
    env = reference_env(cfg)
    if cfg["pred_topk"] is not None:
        env["SPARSE_RS_PREFETCH_PRED_TOPK"] = str(cfg["pred_topk"])
    context = NS(current_phase="none", runtime_call_id=-1, layer_blocks={}, global_expert_cache_enabled=False,
                 prefill_scp_transient_demoted_for_decode=False, rs_bank=None, rs_bank_layout="next_layer",
                 rs_bank_source_layers=[l - 1 for l in range(kw["layers"])], routing_cache={})
    recs, blocks = [], []
    torch_mod = None
    for layer in range(kw["layers"]):
        rec = Recorder()
        rec.seed, rec.late_rate, rec.pending_copy = kw["seed"], kw["late_rate"], None
        ns, compute, torch_mod = extract(rec, env, context)
        blocks.append(StubBlock(ns, torch_mod, rec, compute, layer, cfg, kw["E"], kw["K"], env))
        if kw.get("observed_exposed_ms"):
            # what the harness's metrics would hold once demand copies of the decode phase were timed
            blocks[-1].metrics.demand_h2d_exposed_decode_ms = float(kw["observed_exposed_ms"])
        recs.append(rec)
    costs = kw.get("policy_costs")
    if costs:
        # the reference's own policy class (a dependency-free module) on every layer
        import importlib.util
        import tempfile
        spec = importlib.util.spec_from_file_location("ref_lightweight_policy", REF.parent / "lightweight_policy.py")
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        with tempfile.TemporaryDirectory() as d:
            path = Path(d) / "costs.json"
            path.write_text(json.dumps(dict(schema_version=1, world_size=1, calibrated=False, rank_defaults=costs)))
            profile = mod.CostProfile(path, 1)
        sizes = {e: policy_expert_bytes(e) for e in range(kw["E"])}
        for l, blk in enumerate(blocks):
            blk._light_policy = mod.LocalPolicy(profile, 0, l, sizes, ())
    dense = bool(kw.get("dense"))
    if dense:
        # the reference's own scheduling function runs, fed by stand-in predictors that return a
        # dense probability matrix rebuilt from the seed by the tests
        current = {}
        context.rs_bank = [None] + [(lambda x, _l=l: current[_l]) for l in range(1, kw["layers"])]
        context.layer_blocks = {l: blk for l, blk in enumerate(blocks)}
        for blk in blocks:
            blk.norm_topk_prob = bool(kw.get("norm_topk_prob", False))
    model = RoutingModel(kw["E"], kw["K"], kw["T"], kw["seed"])
    steps, executors = [], []
    for step in range(kw["steps"]):
        phase = "prefill" if step < kw["prefill_steps"] else "decode"
        if kw["prefill_steps"] and step == kw["prefill_steps"]:
            for blk in blocks:                       # the prefill -> decode boundary hook, per layer
                blk._cache.demote_prefill_scp_transients()
                if blk._epipe_prefill_extra_cache_clear_at_decode:
                    blk._epipe_prefill_extra_cache_clear()
        for at, clear in kw.get("resets", []):
            if at == step:                           # a new request begins (scripts/perf.py:553-588)
                context.prefill_scp_transient_demoted_for_decode = False
                for blk in blocks:
                    blk.reset_runtime_state_for_new_request(clear_expert_cache=bool(clear), clear_cache_metadata=True)
        context.current_phase, context.runtime_call_id = phase, step
        routes = [model.route() for _ in range(kw["layers"])]
        planning = cfg["planner_mode"] == "rs_prefetch" and phase == "decode" and not dense
        pred_k = blocks[0]._rs_prefetch_predict_topk() if planning else kw["K"]
        preds = [model.predict(routes[l + 1], pred_k) if planning and l + 1 < kw["layers"] else None
                 for l in range(kw["layers"])]
        steps.append(dict(phase=phase, routes=[[list(s) for s in r] for r in routes],
                          preds=[None if p is None else [list(p[0]), list(p[1])] for p in preds]))
        for rec in recs:
            rec.step = step
        for l, blk in enumerate(blocks):
            blk._current_forward_batch_size = kw["T"] if phase == "decode" else 1
            blk._current_forward_seq_len = 1 if phase == "decode" else kw["T"]
            if dense:
                if l + 1 < kw["layers"]:
                    current[l + 1] = seeded_prediction(kw["seed"], step, l, kw["T"], kw["E"])
                    tgt = blocks[l + 1]
                    before = set(tgt._prefetched_ids_this_group)
                    x = torch_mod.zeros(kw["T"], 4, dtype=torch_mod.bfloat16)
                    blk._compute_and_schedule_next_layer_rs(x=x, seq_len=1 if phase == "decode" else kw["T"])
                executors.append(execute(blk, torch_mod, cfg, routes[l]))
                continue
            if cfg["planner_mode"] == "rs_prefetch" and l + 1 < kw["layers"] and phase == "decode":
                tgt = blocks[l + 1]
                key = ("next_layer_rs", phase, step, l, l + 1)
                budget = tgt._prefetch_target_budget(l + 1, l + 2, count_metrics=True, cycle_key=key)
                if budget > 0:
                    if costs:
                        # what the source layer's forward sets before planning (:10993-10996)
                        source = tgt._light_policy.profile.cost(0, l)
                        tgt._light_policy.window_ms = (source.compute(kw["K"], kw["T"] * kw["K"])
                                                       + tgt._light_policy.cost.attention)
                    ids, probs = preds[l]
                    topi = torch_mod.tensor(ids, dtype=torch_mod.long).view(kw["T"], pred_k)
                    topv = torch_mod.tensor(probs, dtype=torch_mod.float32).view(kw["T"], pred_k).to(torch_mod.bfloat16)
                    plan = tgt._build_prefetch_plan_from_prob_predictions(
                        topi, topv, protect_ids=tgt._prefetch_protect_ids(), budget=int(budget))
                    if len(plan) > 0:
                        tgt._rec.trace.append(("plan", [[int(e), None if v is None else int(v)] for e, v in plan]))
                        tgt._admit_prefetch_plan(plan, group_end=l + 2)
            executors.append(execute(blk, torch_mod, cfg, routes[l]))
    expect = []
    for blk, rec in zip(blocks, recs):
        t = rec.trace
        expect.append(dict(
            events=[x[0] for x in t if x[0] in ("hit", "prefetch_hit", "miss")],
            h2d=[[x[1], x[2]] for x in t if x[0] == "h2d"],
            compute=[x[1] for x in t if x[0] == "compute"],
            waits=[x[1] for x in t if x[0] == "wait"],
            side_waits=[[x[0], x[1]] for x in t if x[0].startswith("wait_")],
            plans=None if dense else [x[1] for x in t if x[0] == "plan"],
            residents=[int(e) for e in blk._cache.resident_ids()],
            extra=[int(e) for e in blk._epipe_prefill_extra_cache.resident_ids()]))
        if kw.get("counters"):
            counts = blk.__dict__.get("_counts", {})
            expect[-1]["counters"] = {name: int(counts.get(name, 0)) for name in kw["counters"]}
    return dict(method=method, kw=kw, steps=steps, executors=executors, expect=expect)


SHADOW_COUNTERS = [
    "epipe_shadow_count", "epipe_prefill_shadow_opportunity_count", "epipe_ready_expert_count",
    "epipe_missing_expert_count", "epipe_ready_item_count", "epipe_missing_item_count",
    "epipe_missing_h2d_bytes_est", "epipe_cache_free_slot_count", "epipe_cache_full_staged_count",
    "epipe_lookahead_ready_group_count", "epipe_lookahead_ready_item_count",
    "epipe_prefill_multistage_shadow_count", "epipe_prefill_multistage_ready_expert_count",
    "epipe_prefill_multistage_missing_expert_count", "epipe_prefill_multistage_ready_item_count",
    "epipe_prefill_multistage_missing_item_count", "epipe_prefill_multistage_top_missing_item_count_sum",
    "epipe_prefill_multistage_est_expert_h2d_bytes", "epipe_prefill_multistage_est_ready_compute_items",
    "epipe_prefill_multistage_est_hidden_h2d_items_n1", "epipe_prefill_multistage_est_hidden_h2d_items_n2",
    "epipe_prefill_multistage_est_hidden_h2d_items_n4",
]


def cases() -> List[Tuple[str, Dict[str, Any]]]:
    base = dict(steps=24, layers=3, E=16, K=2, T=4, capacity=4, top_m=3, seed=0, late_rate=0.0, prefill_steps=0,
                overrides={}, formal=True, policy_costs=None, resets=[], dense=False,
                norm_topk_prob=False)

    def c(method: str, **kw: Any) -> Tuple[str, Dict[str, Any]]:
        return method, {**base, **kw}

    mt = dict(epipe_mode="miss_triggered", epipe_lookahead_min_ready_items=1)
    return [
        c("rr"), c("rr", capacity=1), c("rr", capacity=0),
        c("rs"), c("rs", formal=False, seed=1), c("rs", capacity=15, E=60, K=4, T=8, top_m=8, seed=2, steps=16),
        c("epipe"), c("epipe", capacity=2, T=8, seed=3),
        c("epipe", overrides=dict(epipe_sort_ready_by_work=True), seed=4),
        c("rs-epipe"), c("rs-epipe", late_rate=0.5, seed=5), c("rs-epipe", formal=False, late_rate=0.3, seed=6),
        c("rs-epipe", capacity=15, E=60, K=4, T=8, top_m=8, late_rate=0.3, seed=7, steps=16),
        c("sparse", late_rate=0.2, seed=8),
        # prefill with EPIPE: commits carry the transient mark; side cache instead of commits
        c("epipe", prefill_steps=5, capacity=8, T=2, overrides=dict(epipe_prefill_enable=True), seed=9),
        c("epipe", prefill_steps=5, capacity=8, T=2,
          overrides=dict(epipe_prefill_enable=True, epipe_prefill_mark_transient=False), seed=9),
        c("epipe", prefill_steps=4, capacity=6, T=8,
          overrides=dict(epipe_prefill_enable=True, epipe_prefill_commit=False, epipe_prefill_extra_cache_slots=2),
          seed=10),
        # bounded ready buffer
        c("rs-epipe", late_rate=0.5, overrides=dict(epipe_decode_rs_mode="late_only"), seed=11),
        c("rs-epipe", late_rate=0.3, formal=False, overrides=dict(epipe_decode_rs_mode="buffered"), seed=12),
        c("rs-epipe", late_rate=0.3, overrides=dict(epipe_decode_rs_mode="demand_only"), seed=13),
        c("rs-epipe", late_rate=0.4, capacity=15, E=60, K=4, T=8, top_m=8,
          overrides=dict(epipe_decode_rs_mode="buffered", epipe_rs_buffer_max_groups=2), seed=14, steps=16),
        c("rs-epipe", late_rate=0.4, overrides=dict(epipe_decode_rs_mode="buffered", epipe_rs_min_buffer_groups=2,
                                                    epipe_rs_min_buffer_items=3), seed=15),
        # miss-triggered look-ahead
        c("epipe", overrides=dict(mt), seed=16),
        c("epipe", capacity=6, T=8, overrides=dict(mt, epipe_lookahead_min_ready_items=4, epipe_lookahead_experts=2),
          seed=17),
        c("rs-epipe", late_rate=0.3, overrides=dict(mt, epipe_decode_rs_mode="stream"), seed=18),
        c("epipe", prefill_steps=4, capacity=6, T=8,
          overrides=dict(mt, epipe_prefill_enable=True, epipe_prefill_lookahead_min_ready_items=1), seed=19),
        c("epipe", prefill_steps=4, capacity=6, T=8,
          overrides=dict(mt, epipe_prefill_enable=True, epipe_prefill_commit=False,
                         epipe_prefill_extra_cache_slots=2, epipe_prefill_lookahead_min_ready_items=1), seed=20),
        # the reference's own next-layer scheduling function on dense predictor outputs
        c("rs", dense=True, seed=31), c("rs", dense=True, formal=False, capacity=6, T=8, top_m=5, seed=32),
        c("rs-epipe", dense=True, late_rate=0.4, seed=33),
        c("rs", dense=True, norm_topk_prob=True, overrides=dict(pred_topk=3), seed=34),
        c("rs-epipe", dense=True, late_rate=0.3, prefill_steps=2, seed=35),
        # less travelled switches of the prefetch planner and the cache guard
        c("rs", overrides=dict(cache_ttl_steps=2), seed=36),
        c("rs-epipe", late_rate=0.3, overrides=dict(cache_ttl_steps=3, recent_protect_steps=3), seed=37),
        c("rs", overrides=dict(protect_mode="minimal"), seed=38),
        c("rs-epipe", late_rate=0.5, overrides=dict(wait_before_evict=False), seed=39),
        c("rs", overrides=dict(allow_active_replace=False), capacity=6, seed=40),
        c("rs", formal=False, overrides=dict(rs_policy="cache_safe"), seed=41),
        c("rs", formal=False, top_m=6, capacity=8, overrides=dict(min_candidate_score=0.0, replace_advantage=0.0,
                                                                  replace_margin=1.0), seed=42),
        c("rr", overrides=dict(cache_ttl_steps=2), seed=43),
        c("epipe", overrides=dict(epipe_min_ready_experts=2, epipe_min_ready_items=3, epipe_min_missing_experts=2),
          T=8, capacity=6, seed=44),
        c("epipe", overrides=dict(epipe_transient_staging=False), seed=45),
        c("rs-epipe", late_rate=0.3, overrides=dict(epipe_rs_rolling_gate=False), seed=46),
        c("rs-epipe", late_rate=0.1, overrides=dict(epipe_rs_gate_window=4, epipe_rs_gate_skip_steps=3,
                                                    epipe_rs_handle_demand_miss=False), seed=47),
        c("rs-epipe", late_rate=0.3, overrides=dict(epipe_rs_demand_commit=False), seed=48),
        # requests following one another: metadata reset, and reset with the cache cleared
        c("rs-epipe", late_rate=0.3, resets=[[8, 0], [16, 1]], seed=27),
        c("rs", resets=[[6, 0], [12, 0], [18, 1]], formal=False, seed=28),
        c("epipe", prefill_steps=3, capacity=6, T=8, resets=[[10, 0]],
          overrides=dict(epipe_prefill_enable=True, epipe_prefill_commit=False, epipe_prefill_extra_cache_slots=2),
          seed=29),
        c("rs", capacity=8, E=24, T=8, top_m=4, resets=[[8, 0], [16, 1]],
          overrides=dict(cache_policy="tiered", prefetch_reserved=1), seed=30),
        # cost-aware local policy installed (rescored plans, cost-based residual choice)
        c("rs-epipe", late_rate=0.4, policy_costs=POLICY_COSTS, seed=24),
        c("sparse", late_rate=0.3, T=8, capacity=6, policy_costs=POLICY_COSTS, seed=25),
        c("rs", policy_costs=POLICY_COSTS, seed=26),
        # counting-only (shadow) variants: classify, count, leave the call to the demand path
        c("epipe", overrides=dict(epipe_enable=False, epipe_shadow=True), seed=50, counters=SHADOW_COUNTERS),
        c("epipe", capacity=2, T=8, overrides=dict(epipe_enable=False, epipe_shadow=True, epipe_transient_staging=False),
          seed=51, counters=SHADOW_COUNTERS),
        c("epipe", prefill_steps=5, capacity=8, T=2, overrides=dict(epipe_prefill_shadow=True), seed=52,
          counters=SHADOW_COUNTERS),
        c("epipe", prefill_steps=6, capacity=6, T=8,
          overrides=dict(epipe_prefill_enable=True, epipe_prefill_multistage_shadow=True,
                         epipe_prefill_multistage_max_n=2), seed=53, counters=SHADOW_COUNTERS),
        c("rr", prefill_steps=6, capacity=6, T=8,
          overrides=dict(epipe_prefill_multistage_shadow=True, epipe_prefill_extra_cache_slots=2), seed=54,
          counters=SHADOW_COUNTERS),
        c("epipe", overrides=dict(mt, epipe_enable=False, epipe_shadow=True), seed=55, counters=SHADOW_COUNTERS),
        c("epipe", prefill_steps=5, capacity=6, T=8,
          overrides=dict(mt, epipe_prefill_shadow=True, epipe_prefill_lookahead_min_ready_items=1), seed=56,
          counters=SHADOW_COUNTERS),
        # prefill reads ready experts without moving them in the LRU
        c("epipe", prefill_steps=6, capacity=6, T=8,
          overrides=dict(epipe_prefill_enable=True, epipe_prefill_no_touch_ready=True), seed=57),
        c("epipe", prefill_steps=6, capacity=6, T=8,
          overrides=dict(epipe_prefill_enable=True, epipe_prefill_no_touch_ready=True, epipe_prefill_commit=False,
                         epipe_prefill_extra_cache_slots=2), seed=58),
        c("epipe", prefill_steps=6, capacity=6, T=8,
          overrides=dict(mt, epipe_prefill_enable=True, epipe_prefill_no_touch_ready=True,
                         epipe_prefill_lookahead_min_ready_items=1, epipe_prefill_commit=False,
                         epipe_prefill_extra_cache_slots=2), seed=59),
        # the demand stage behind the exposed-stall threshold instead of the force flag
        c("rs-epipe", late_rate=0.3, overrides=dict(epipe_rs_force_demand_stage=False,
                                                    epipe_rs_demand_stage_threshold_ms=1.0),
          observed_exposed_ms=5.0, seed=60),
        c("rs-epipe", late_rate=0.3, overrides=dict(epipe_rs_force_demand_stage=False,
                                                    epipe_rs_demand_stage_threshold_ms=1.0),
          observed_exposed_ms=0.5, seed=60),
        c("rs-epipe", late_rate=0.3, overrides=dict(epipe_decode_rs_mode="buffered", epipe_rs_force_demand_stage=False,
                                                    epipe_rs_demand_stage_threshold_ms=2.0),
          observed_exposed_ms=2.5, seed=61),
        # tiered cache under the same state machine
        c("rr", capacity=8, E=24, T=8, overrides=dict(cache_policy="tiered"), seed=21),
        c("rs", capacity=8, E=24, T=8, top_m=4, overrides=dict(cache_policy="tiered", prefetch_reserved=1), seed=22),
        c("rs-epipe", capacity=8, E=24, T=8, top_m=4, formal=False, late_rate=0.2,
          overrides=dict(cache_policy="tiered", prefetch_reserved=1), seed=23),
    ]


def main() -> None:
    if not REF.exists():
        sys.exit("the reference checkout is not mounted; fixtures are only written in the build container")
    out = [run_case(method, kw) for method, kw in cases()]
    (OUT / "layer_traces.json").write_text(json.dumps(out, separators=(",", ":")))
    print("wrote", OUT / "layer_traces.json", "cases:", len(out))


if __name__ == "__main__":
    main()
