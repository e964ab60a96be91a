#!/usr/bin/env python3
"""Write golden vectors for the cache and the RS prefetch planner.

Runs ONLY in the build container, where the reference checkout is mounted at
/root/reference; the fixtures it writes (``cache_ops.json``, ``rs_plan.json``) are what the
tests read, so nothing at test time touches the reference.  ``tiered_ops.json`` holds the
same kind of traces for ``TieredExpertWeightCache`` (utils/eval_core.py:3953-4338) and the
capacity split of a tiered layer (:4843-4890).

The reference's classes and methods are taken out of ``utils/eval_core.py`` by name with
``ast`` (the technique of the reference's own tests, tests/test_rs_staging.py:18-34) and
executed against a stub ``self``; the reference package is never imported, so neither
transformers nor a GPU is needed.  What is recorded:

  cache_ops.json   random operation sequences on ``ExpertWeightCache`` (get / put with pins,
                   protect sets and transient flags / admit_prefetch / discard / unpin /
                   unpin_all / promote_hot / evictable_prefetch_ids): return value and
                   ``resident_ids()`` after every operation.
  rs_plan.json     random cache states, access frequencies, prefetched sets and predictor
                   top-k lists -> ``_build_target_layer_prob_score_map`` output (as ordered
                   pairs), ``_pick_victims_by_low_value`` and
                   ``_build_prefetch_plan_from_score_map`` output, for the default and the
                   cache_safe policy.
"""
from __future__ import annotations

import ast
import json
import os
import random
import sys
from collections import OrderedDict
from dataclasses import dataclass
from pathlib import Path
from types import SimpleNamespace as NS
from typing import Any, Dict, List, Optional, Sequence, Set, Tuple

REF = Path("/root/reference/utils/eval_core.py")
OUT = Path(__file__).resolve().parent

BLOCK_METHODS = (
    "_resident_keep_bias", "_pick_victims_by_low_value", "_build_prefetch_plan_from_score_map",
    "_build_target_layer_prob_score_map", "_prefetch_evictable_ids", "_prefetch_free_slots",
)


def extract():
    import torch
    tree = ast.parse(REF.read_text())
    classes = [n for n in tree.body if isinstance(n, ast.ClassDef)
               and n.name in ("CacheEntry", "ExpertWeightCache", "TieredExpertWeightCache")]
    block = next(n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == "DistributedSparseMoeBlock")
    methods = [n for n in block.body if isinstance(n, ast.FunctionDef) and n.name in BLOCK_METHODS]
    future = ast.ImportFrom(module="__future__", names=[ast.alias(name="annotations")], level=0)
    module = ast.Module(body=[future, *classes, *methods], type_ignores=[])
    ns: Dict[str, Any] = dict(OrderedDict=OrderedDict, dataclass=dataclass, Any=Any, Dict=Dict, List=List,
                              Optional=Optional, Tuple=Tuple, Sequence=Sequence, Set=Set, os=os, torch=torch,
                              SparseContext=NS(current_phase="decode", runtime_call_id=0))
    exec(compile(ast.fix_missing_locations(module), str(REF), "exec"), ns)
    return ns


def cache_cases(ns, rng: random.Random, n_cases: int = 40, n_ops: int = 120):
    cases = []
    for case in range(n_cases):
        cap = rng.choice([0, 1, 2, 3, 4, 6, 8])
        universe = rng.choice([6, 10, 16])
        cache = ns["ExpertWeightCache"](cap)
        ops, results = [], []
        for _ in range(n_ops):
            op = rng.choices(["get", "put", "admit", "discard", "unpin", "unpin_all", "promote", "evictable", "has",
                              "peek"], weights=[30, 30, 12, 5, 5, 2, 5, 5, 3, 3])[0]
            eid = rng.randrange(universe)
            protect = sorted(rng.sample(range(universe), rng.randrange(0, 4))) if rng.random() < 0.4 else []
            if op == "get":
                r = cache.get(eid)
                rec = ["get", eid]
            elif op == "put":
                pinned, transient = rng.random() < 0.15, rng.random() < 0.15
                r = cache.put(eid, "w%d" % eid, pinned=pinned, protect_ids=set(protect), prefill_scp_transient=transient)
                rec = ["put", eid, pinned, transient, protect]
            elif op == "admit":
                victim = rng.randrange(universe) if rng.random() < 0.6 else None
                r = cache.admit_prefetch(eid, "p%d" % eid, protect_ids=set(protect), preferred_victim=victim)
                rec = ["admit", eid, victim, protect]
            elif op == "discard":
                r = cache.discard(eid)
                rec = ["discard", eid]
            elif op == "unpin":
                r = cache.unpin(eid)
                rec = ["unpin", eid]
            elif op == "unpin_all":
                r = cache.unpin_all()
                rec = ["unpin_all"]
            elif op == "promote":
                r = cache.promote_hot(eid)
                rec = ["promote", eid]
            elif op == "evictable":
                r = cache.evictable_prefetch_ids(set(protect))
                rec = ["evictable", protect]
            elif op == "has":
                r = cache.has(eid)
                rec = ["has", eid]
            else:
                r = cache.peek(eid)
                rec = ["peek", eid]
            ops.append(rec)
            results.append([r, list(cache.resident_ids()), cache.prefetch_free_slots()])
        cases.append(dict(capacity=cap, ops=ops, results=results))
    return cases


def make_block(ns, cache, freq, prefetched, policy, thresholds):
    blk = NS()
    blk._cache = cache
    blk._expert_access_freq = dict(freq)
    blk._prefetched_ids_this_group = set(prefetched)
    blk._prefetch_min_candidate_score, blk._prefetch_replace_advantage, blk._prefetch_replace_margin = thresholds
    blk._prefetch_allow_active_replace = True
    blk.comm_rank, blk.layer_idx, blk.planner_mode = 0, 1, "rs_prefetch"
    blk._rs_prefetch_policy = lambda: policy
    blk._rank_env_float = lambda name, default: float(default)
    blk._rs_env_float = lambda name, default: float(default)
    blk._stage_prefetch_eid_set = lambda: set(range(10 ** 6))
    blk._current_stage = lambda: "decode"
    blk.resolve_prefetch_target_rank = lambda **kw: NS(target_rank=0)
    blk._record_rs_resolver_match = lambda **kw: None
    blk._record_rs_counter = lambda *a, **k: None
    for name in BLOCK_METHODS:
        fn = ns[name]
        setattr(blk, name, (lambda f: (lambda *a, **k: f(blk, *a, **k)))(fn))
    return blk


def plan_cases(ns, rng: random.Random, n_cases: int = 200):
    import torch
    cases = []
    for case in range(n_cases):
        E = rng.choice([16, 60, 64])
        cap = rng.choice([2, 4, 8, 15])
        cache = ns["ExpertWeightCache"](cap)
        n_res = rng.randrange(0, cap + 1)
        residents = rng.sample(range(E), n_res)
        pinned = []
        for e in residents:
            p = rng.random() < 0.2
            cache.put(e, "w", pinned=p)
            if p:
                pinned.append(e)
        freq = {e: rng.randrange(0, 20) for e in rng.sample(range(E), rng.randrange(0, min(E, 12)))}
        prefetched = [e for e in residents if rng.random() < 0.25]
        protect = sorted(set(prefetched) | set(rng.sample(range(E), rng.randrange(0, 3))))
        T, pk = rng.choice([1, 4, 8]), rng.choice([4, 8])
        # predictor output rounded to bf16 then widened, as the reference feeds it
        probs = torch.softmax(torch.randn(T, E, generator=torch.Generator().manual_seed(case)) * 2.0, dim=-1)
        topv, topi = torch.topk(probs, pk, dim=-1)
        topv = topv.to(torch.bfloat16)
        policy = rng.choice(["default", "cache_safe"])
        thresholds = rng.choice([(0.02, 0.02, 1.05), (0.04, 0.08, 1.20)])
        budget = rng.randrange(0, 9)
        blk = make_block(ns, cache, freq, prefetched, policy, thresholds)
        score = blk._build_target_layer_prob_score_map(topi, topv, count_metrics=False)
        victims = blk._pick_victims_by_low_value(score, set(protect))
        plan = blk._build_prefetch_plan_from_score_map(score, protect_ids=set(protect), budget=budget)
        cases.append(dict(
            E=E, capacity=cap, residents=residents, pinned=pinned, freq=sorted(freq.items()), prefetched=prefetched,
            protect=protect, topi=topi.reshape(-1).tolist(), topv=topv.float().reshape(-1).tolist(), policy=policy,
            thresholds=list(thresholds), budget=budget,
            score=[[int(k), float(v)] for k, v in score.items()], victims=[int(v) for v in victims],
            plan=[[int(e), (None if v is None else int(v))] for e, v in plan]))
    return cases


def tiered_cases(ns, rng: random.Random, n_cases: int = 24, n_ops: int = 150):
    """Random operation sequences on the reference's ``TieredExpertWeightCache``."""
    cases = []
    for case in range(n_cases):
        cap = rng.choice([2, 3, 4, 6, 8, 12])
        hot = rng.randrange(0, cap + 1)
        reserved = rng.randrange(0, 3)
        universe = rng.choice([8, 12, 20])
        cache = ns["TieredExpertWeightCache"](cap, hot_capacity=hot, prefetch_reserved=reserved)
        ops, results = [], []
        for _ in range(n_ops):
            op = rng.choices(["get", "put", "admit", "discard", "unpin", "unpin_all", "promote", "evictable", "has",
                              "peek", "reset", "demote_transients", "clear_transient"],
                             weights=[30, 30, 14, 4, 4, 2, 8, 5, 3, 3, 1, 2, 2])[0]
            eid = rng.randrange(universe)
            protect = sorted(rng.sample(range(universe), rng.randrange(0, 4))) if rng.random() < 0.4 else []
            if op == "get":
                r, rec = cache.get(eid), ["get", eid]
            elif op == "put":
                pinned, transient, hotp = rng.random() < 0.2, rng.random() < 0.15, rng.random() < 0.25
                r = cache.put(eid, "w%d" % eid, pinned=pinned, prefer_hot=hotp, protect_ids=set(protect),
                              prefill_scp_transient=transient)
                rec = ["put", eid, pinned, transient, hotp, protect]
            elif op == "admit":
                victim = rng.randrange(universe) if rng.random() < 0.6 else None
                r = cache.admit_prefetch(eid, "p%d" % eid, protect_ids=set(protect), preferred_victim=victim)
                rec = ["admit", eid, victim, protect]
            elif op == "discard":
                r, rec = cache.discard(eid), ["discard", eid]
            elif op == "unpin":
                r, rec = cache.unpin(eid), ["unpin", eid]
            elif op == "unpin_all":
                r, rec = cache.unpin_all(), ["unpin_all"]
            elif op == "promote":
                r, rec = cache.promote_hot(eid), ["promote", eid]
            elif op == "evictable":
                r, rec = cache.evictable_prefetch_ids(set(protect)), ["evictable", protect]
            elif op == "has":
                r, rec = cache.has(eid), ["has", eid]
            elif op == "peek":
                r, rec = cache.peek(eid), ["peek", eid]
            elif op == "reset":
                demote = rng.random() < 0.5
                r, rec = cache.reset_request_metadata(unpin=True, demote_hot=demote), ["reset", demote]
            elif op == "demote_transients":
                r, rec = cache.demote_prefill_scp_transients(), ["demote_transients"]
            else:
                r, rec = cache.clear_prefill_scp_transient(eid), ["clear_transient", eid]
            ops.append(rec)
            occ = cache.occupancy()
            results.append([r, list(cache.resident_ids()), cache.prefetch_free_slots(),
                            [occ["hot"], occ["transient_demand"], occ["transient_prefetch"], occ["prefill_scp_transient"]],
                            bool(cache.last_evicted_was_prefill_scp_transient())])
        cases.append(dict(capacity=cap, hot=hot, reserved=reserved, ops=ops, results=results))
    return cases


def split_cases():
    """The capacity split of a tiered layer is inline code of the block's constructor
    (utils/eval_core.py:4843-4890); those lines are run as they stand against a stub."""
    lines = REF.read_text().splitlines()[4842:4890]
    indent = len(lines[0]) - len(lines[0].lstrip())
    body = "\n".join(line[indent:] if line.strip() else "" for line in lines)
    code = compile(body, str(REF), "exec")
    cases = []
    for cache in range(0, 21):
        for planner in ("none", "rs_prefetch"):
            for reserved in (0, 1, 2, 5):
                for extra in (0, 2):
                    env = {"SPARSE_PREFETCH_RESERVED": str(reserved), "SPARSE_PREFETCH_EXTRA_CAPACITY": str(extra)}
                    ns = dict(self=NS(planner_mode=planner), expert_cache=cache, os=NS(environ=env), int=int, max=max,
                              min=min)
                    exec(code, ns)
                    cases.append([cache, planner == "rs_prefetch", reserved, extra,
                                  [int(ns["total_capacity"]), int(ns["hot_capacity"]), int(ns["prefetch_reserved"])]])
    return cases


def main() -> None:
    if not REF.exists():
        sys.exit("the reference checkout is not mounted; fixtures are only written in the build container")
    ns = extract()
    rng = random.Random(20261125)
    (OUT / "cache_ops.json").write_text(json.dumps(cache_cases(ns, rng)))
    (OUT / "rs_plan.json").write_text(json.dumps(plan_cases(ns, rng)))
    (OUT / "tiered_ops.json").write_text(json.dumps(dict(ops=tiered_cases(ns, rng), split=split_cases())))
    print("wrote", OUT / "cache_ops.json", OUT / "rs_plan.json", OUT / "tiered_ops.json")


if __name__ == "__main__":
    main()
