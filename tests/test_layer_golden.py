"""Oracle and product against golden traces recorded from the reference's own methods.

``tests/golden/layer_traces.json`` was written by ``tests/golden/make_layer_golden.py``: the
reference's demand path, its four EPIPE executors, its prefetch cycle / budget / plan /
admission methods and its cache classes, taken out of the reference source and run against
recording stand-ins for streams, events and weights.  Each case stores its inputs (routing
per step and layer, predictor top-k lists) and what the reference did with them; here the
oracle (``oracle/ref_layer.py``) and the product (``sparse_amd/residency.py``) replay the
same calls and must produce the same cache events, copies, waits, execution order, prefetch
plans, executor choice and final cache contents."""
import json
from pathlib import Path

import pytest

import torch

from oracle import ref_rs
from oracle.ref_layer import RefLayer
from sparse_amd.rs import topk_for_planning
from sparse_amd.methods import residency_config
from tests.helpers import copy_is_late, seeded_prediction
from tests.test_residency import product_layer, split, to_ref_config

CASES = json.loads((Path(__file__).resolve().parent / "golden" / "layer_traces.json").read_text())


def _label(case):
    kw = case["kw"]
    extra = ",".join(f"{k}={v}" for k, v in sorted(kw["overrides"].items()))
    if kw.get("policy_costs"):
        extra = (extra + "," if extra else "") + "local_policy"
    if kw.get("dense"):
        extra = (extra + "," if extra else "") + "dense_prediction"
    return f"{case['method']}-cap{kw['capacity']}-E{kw['E']}-seed{kw['seed']}" + (f"-{extra}" if extra else "")


def replay(case, which):
    kw = case["kw"]
    cfg = residency_config(case["method"], kw["capacity"], kw["top_m"], formal_thresholds=kw["formal"],
                           **kw["overrides"])
    admitted, fresh = {}, set()
    now = [0]

    def copy_done(layer):
        def fn(eid):
            key = (layer, eid)
            if key in fresh:
                fresh.discard(key)
                return not copy_is_late(kw["seed"], layer, admitted[key], eid, kw["late_rate"])
            return True
        return fn

    lays, backs, mets = [], [], []
    for l in range(kw["layers"]):
        observed = float(kw.get("observed_exposed_ms") or 0.0)   # exposed demand-copy ms the metrics hold
        if which == "oracle":
            lay = RefLayer(l, kw["E"], kw["K"], to_ref_config(cfg), copy_done=copy_done(l))
            lay.expert_bytes = 100
            lay.observed_exposed_ms = observed
        else:
            lay, be, m = product_layer(cfg, E=kw["E"], K=kw["K"], copy_done=copy_done(l), layer=l)
            m.demand_h2d_exposed_decode_ms = observed
            backs.append(be)
            mets.append(m)
        lays.append(lay)
    costs = kw.get("policy_costs")
    if costs:
        import tempfile
        from sparse_amd.local_policy import CostProfile, LocalPolicy
        sizes = {e: 100.0 + 40.0 * (e % 5) for e in range(kw["E"])}
        with tempfile.TemporaryDirectory() as d:
            path = Path(d) / "costs.json"
            path.write_text(json.dumps(dict(schema_version=1, world_size=1, calibrated=False, rank_defaults=costs)))
            profile = CostProfile(path, 1)
        for l, lay in enumerate(lays):
            if which == "oracle":
                lay.policy = dict(costs=dict(costs), expert_bytes=sizes, window_ms=0.0, ready_ms=0.0, feedback=True,
                                  prefetch=True)
            else:
                lay.light_policy = LocalPolicy(profile, 0, l, sizes, ())
    executors, plans = [], [[] for _ in lays]
    for step, rec in enumerate(case["steps"]):
        now[0] = step
        phase = rec["phase"]
        for at, clear in kw.get("resets", []):
            if at == step:
                for lay in lays:
                    lay.reset_for_new_request(clear_expert_cache=bool(clear), clear_cache_metadata=True)
        if kw["prefill_steps"] and step == kw["prefill_steps"]:
            for lay in lays:
                lay.cache.demote_prefill_scp_transients()
        for l, lay in enumerate(lays):
            if cfg.planner_mode == "rs_prefetch" and l + 1 < kw["layers"] and phase == "decode":
                tgt = lays[l + 1]
                tgt.phase, tgt.call_id = phase, step
                budget = tgt.prefetch_budget(("next_layer_rs", phase, step, l, l + 1))
                if budget > 0:
                    if costs:
                        window = costs["expert_ms"] * kw["K"] + costs["item_ms"] * kw["T"] * kw["K"] \
                            + costs["next_attention_ms"]
                        if which == "oracle":
                            tgt.policy["window_ms"] = window
                        else:
                            tgt.light_policy.window_ms = window
                    if kw.get("dense"):
                        # dense predictor output rebuilt from the seed, then what the block does with it
                        pred = seeded_prediction(kw["seed"], step, l, kw["T"], kw["E"])
                        norm = bool(kw.get("norm_topk_prob", False))
                        if which == "oracle":
                            ids, probs = ref_rs.plan_inputs(pred, tgt.predict_topk(), norm, torch.bfloat16)
                        else:
                            topi, topv = topk_for_planning(pred, tgt.predict_topk(), norm, torch.bfloat16)
                            ids, probs = topi.reshape(-1).tolist(), topv.reshape(-1).tolist()
                    else:
                        ids, probs = rec["preds"][l]
                    before = set(tgt.events) if which == "oracle" else set(tgt.prefetch_events)
                    plan = tgt.schedule_prefetch(ids, probs, budget)
                    after = set(tgt.events) if which == "oracle" else set(tgt.prefetch_events)
                    for eid in after - before:
                        admitted[(l + 1, eid)] = step
                        fresh.add((l + 1, eid))
                    if plan:
                        plans[l + 1].append([[int(e), None if v is None else int(v)] for e, v in plan])
            lay.phase, lay.call_id, lay.stage = phase, step, phase
            executors.append(lay.execute([tuple(s) for s in rec["routes"][l]]))
    out = []
    for l, lay in enumerate(lays):
        if which == "oracle":
            trace = lay.trace
            events, h2d, compute, waits = split(trace)
            extra = lay.extra.resident_ids()
        else:
            trace = backs[l].trace
            events = [(k, e) for k, _l, e in mets[l].events]
            _ev, h2d, compute, waits = split(trace)
            extra = lay.extra_cache.resident_ids()
        side = [[t[0], t[1]] for t in trace if isinstance(t[0], str) and t[0].startswith("wait_")]
        out.append(dict(events=[k for k, _e in events], h2d=[[lane, e] for _h, lane, e in h2d], compute=compute,
                        waits=[e for _w, e in waits], side_waits=side, plans=plans[l],
                        residents=lay.cache.resident_ids(), extra=extra))
        if kw.get("counters"):
            counts = lay.counters if which == "oracle" else mets[l].counters
            out[-1]["counters"] = {name: int(counts.get(name, 0)) for name in kw["counters"]}
    return out, executors


@pytest.mark.parametrize("which", ["oracle", "product"])
@pytest.mark.parametrize("case", CASES, ids=[_label(c) for c in CASES])
def test_replay_matches_the_reference(case, which):
    got, executors = replay(case, which)
    assert executors == case["executors"], "executor choice differs from the reference"
    for l, (g, w) in enumerate(zip(got, case["expect"])):
        for key in ("plans", "events", "h2d", "waits", "side_waits", "compute", "residents", "extra"):
            if w[key] is None:
                continue        # the reference's own scheduling function keeps no record of its plans
            assert g[key] == w[key], f"layer {l}: {key} differs from the reference"
        if "counters" in w:
            assert g["counters"] == w["counters"], f"layer {l}: counters differ from the reference"


def test_fixture_covers_every_executor_and_feature():
    names = {n for c in CASES for n in c["executors"]}
    assert {"plain", "epipe_upfront", "epipe_rs_residual_scan", "epipe_rs_buffered", "epipe_miss_triggered"} <= names
    assert any(c["kw"]["late_rate"] > 0 and any(e["waits"] for e in c["expect"]) for c in CASES)
    assert any(any(e["extra"] for e in c["expect"]) for c in CASES)            # side cache in use
    assert any("prefetch_hit" in e["events"] for c in CASES for e in c["expect"])
    assert any(e["plans"] for c in CASES for e in c["expect"])
    assert sum(1 for c in CASES if c["kw"].get("dense")) >= 5
    assert sum(len(e["events"]) for c in CASES for e in c["expect"]) > 10000
    # the counting-only variants did count, the no-touch switch and the stall threshold are in
    shadow = [c for c in CASES if c["kw"].get("counters")]
    assert len(shadow) >= 7
    for name in ("epipe_shadow_count", "epipe_prefill_shadow_opportunity_count", "epipe_lookahead_ready_item_count",
                 "epipe_prefill_multistage_est_hidden_h2d_items_n2", "epipe_cache_full_staged_count"):
        assert any(e["counters"][name] > 0 for c in shadow for e in c["expect"]), name
    assert any(c["kw"]["overrides"].get("epipe_prefill_no_touch_ready") for c in CASES)
    assert sum(1 for c in CASES if c["kw"].get("observed_exposed_ms")) >= 3
