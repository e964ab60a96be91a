#!/usr/bin/env python3
"""Write golden vectors for the host logic of the bounded RS staging adapter.

Runs ONLY in the build container, where the reference checkout is mounted at
/root/reference; the fixture it writes (``staging_ops.json``) is what the tests read.

``utils/rs_staging.py`` and ``utils/rs_overlap.py`` of the reference import nothing but the
standard library at module level (their docstrings allow a standalone deployment next to
each other), so they are loaded by path and run as they are; the resident cache under the
demand view is the reference's ``ExpertWeightCache``, taken out of ``utils/eval_core.py``
with ``ast`` as in the reference's own tests (tests/test_rs_staging.py:18-34).  Recorded:

  select    random ``select_candidates`` calls: chosen experts and the diagnostics dict.
  sessions  random sequences on one layer: experts are staged into the demand view, looked up
            (get / peek / has), a miss is noted, the empty-forecast cool-down is armed and
            queried, and at "layer exit" every staged expert that was used is admitted by
            ``BoundedRS._retain_used`` -- return values, resident order, first-use order,
            cool-down state and counters after every operation.
"""
from __future__ import annotations

import ast
import json
import random
import sys
from collections import OrderedDict
from dataclasses import dataclass
from pathlib import Path
from types import SimpleNamespace as NS
from typing import Any, Dict, List, Optional, Sequence, Set, Tuple

REF = Path("/root/reference/utils")
OUT = Path(__file__).resolve().parent


def load():
    sys.path.insert(0, str(REF))
    import rs_overlap
    import rs_staging
    tree = ast.parse((REF / "eval_core.py").read_text())
    classes = [n for n in tree.body if isinstance(n, ast.ClassDef) and n.name in ("CacheEntry", "ExpertWeightCache")]
    future = ast.ImportFrom(module="__future__", names=[ast.alias(name="annotations")], level=0)
    ns: Dict[str, Any] = dict(OrderedDict=OrderedDict, dataclass=dataclass, Any=Any, Dict=Dict, List=List,
                              Optional=Optional, Tuple=Tuple, Sequence=Sequence, Set=Set)
    exec(compile(ast.fix_missing_locations(ast.Module(body=[future, *classes], type_ignores=[])),
                 str(REF / "eval_core.py"), "exec"), ns)
    return rs_staging, rs_overlap, ns["ExpertWeightCache"]


STATS = ("observed_decode_misses", "cooldown_miss_invalidations", "cooldown_cache_invalidations", "skipped_cooldown",
         "retained", "recycled_payloads", "allocated_replacements")


def select_cases(staging, rng: random.Random, n: int = 200):
    out = []
    for _ in range(n):
        E = rng.choice([8, 16, 60])
        count = rng.randrange(0, 40)
        ids = [rng.randrange(E + 4) for _ in range(count)]              # some ids belong to nobody
        weights = [round(rng.random() ** 2, 4) for _ in range(count)]
        allowed = sorted(rng.sample(range(E), rng.randrange(1, E + 1)))
        resident = sorted(rng.sample(range(E), rng.randrange(0, min(E, 8))))
        minimum = rng.choice([0.0, 0.02, 0.04, 0.2, 0.5])
        budget = rng.randrange(0, 6)
        diag: Dict[str, int] = {}
        chosen = staging.select_candidates(ids, weights, allowed=set(allowed), resident=set(resident), minimum=minimum,
                                           budget=budget, diagnostics=diag)
        out.append(dict(ids=ids, weights=weights, allowed=allowed, resident=resident, minimum=minimum, budget=budget,
                        chosen=[int(e) for e in chosen], diagnostics=diag))
    return out


def session_cases(staging, overlap, Cache, rng: random.Random, n: int = 24, n_ops: int = 100):
    out = []
    for _ in range(n):
        cap = rng.choice([1, 2, 3, 4, 6])
        E = rng.choice([8, 12, 16])
        empty_steps = rng.choice([0, 4, 16])
        cache = Cache(cap)
        seed_ids = rng.sample(range(E), rng.randrange(0, cap + 1))
        def weights(tag):
            return (NS(shape=(3, 2), dtype="bf16", tag=tag),)

        for e in seed_ids:
            cache.put(e, weights(f"res{e}"))
        view = staging.DemandCacheView(cache)
        owner = overlap.BoundedRS.__new__(overlap.BoundedRS)
        owner.jobs, owner.retired, owner.views = {}, [], {0: view}
        owner.next_probe, owner.cooldown_residents = {}, {}
        owner.empty_steps = empty_steps
        owner.stats = dict(observed_decode_misses=0, cooldown_miss_invalidations=0, cooldown_cache_invalidations=0,
                           skipped_cooldown=0, retained=0, recycled_payloads=0, allocated_replacements=0)
        owner.torch = NS(empty_like=lambda x: NS(shape=x.shape, dtype=x.dtype, tag="fresh"))
        freq: Dict[int, int] = {}

        def access(eid):
            freq[eid] = freq.get(eid, 0) + 1

        block = NS(layer_idx=0, _on_demand_access=access,
                   _cache_put_guarded=lambda eid, value, **kw: cache.put(eid, value),
                   _should_prefer_hot=lambda *a: False)
        step = 0
        ops, results = [], []
        for _ in range(n_ops):
            op = rng.choices(["stage", "get", "peek", "has", "miss", "arm", "skip", "exit", "put"],
                             weights=[18, 30, 8, 8, 5, 6, 12, 8, 5])[0]
            eid = rng.randrange(E)
            if op == "stage":
                if cache.has(eid) or eid in view.staged:
                    continue
                payload = weights(f"staged{eid}")
                view.staged[eid] = staging.Transfer(eid, payload, None, {"payload": payload}, 12)
                r, rec = None, ["stage", eid]
            elif op == "get":
                got = view.get(eid)
                r, rec = (None if got is None else _tag(got)), ["get", eid]
            elif op == "peek":
                got = view.peek(eid)
                r, rec = (None if got is None else _tag(got)), ["peek", eid]
            elif op == "has":
                r, rec = bool(view.has(eid)), ["has", eid]
            elif op == "miss":
                owner.note_demand_miss(block)
                r, rec = None, ["miss"]
            elif op == "arm":
                # what the worker does after an empty forecast (utils/rs_overlap.py:232-237)
                owner.next_probe[0] = step + rng.randrange(1, 20)
                owner.cooldown_residents[0] = frozenset(view.resident_ids())
                r, rec = None, ["arm", owner.next_probe[0]]
            elif op == "skip":
                step += rng.randrange(0, 4)
                r, rec = bool(owner._skip_cooldown(0, step)), ["skip", step]
            elif op == "put":
                # an ordinary demand load by the layer itself
                cache.put(eid, weights(f"res{eid}"))
                r, rec = None, ["put", eid]
            else:
                retained = []
                for transfer in view.used_in_order:
                    owner._retain_used(block, transfer)
                    retained.append([transfer.expert, bool(transfer.retained), _tag(transfer.slot["payload"])])
                view.staged, view.used_in_order = {}, []
                r, rec = retained, ["exit"]
            ops.append(rec)
            results.append([r, [int(e) for e in cache.resident_ids()], [int(t.expert) for t in view.used_in_order],
                            sorted(view.staged), owner.next_probe.get(0), [owner.stats[k] for k in STATS],
                            sorted(freq.items()) if op == "exit" else None])
        out.append(dict(capacity=cap, E=E, empty_steps=empty_steps, seed_ids=seed_ids, ops=ops, results=results))
    return out


def _tag(payload) -> str:
    return str(payload[0].tag)


def main() -> None:
    if not REF.exists():
        sys.exit("the reference checkout is not mounted; fixtures are only written in the build container")
    staging, overlap, Cache = load()
    rng = random.Random(20261126)
    data = dict(stats=list(STATS), select=select_cases(staging, rng),
                sessions=session_cases(staging, overlap, Cache, rng))
    (OUT / "staging_ops.json").write_text(json.dumps(data, separators=(",", ":")))
    print("wrote", OUT / "staging_ops.json")


if __name__ == "__main__":
    main()
