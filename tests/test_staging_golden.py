"""Host logic of forecast staging against vectors recorded from the reference's
own modules (``tests/golden/staging_ops.json``, written by
``tests/golden/make_staging_golden.py`` from utils/rs_staging.py and utils/rs_overlap.py run
as they are): candidate selection, what a demand lookup sees while copies are staged, the
empty-forecast cool-down, and the admission of used experts at layer exit with its exchange
of storage.  The reference's operations are mapped onto this build's slot table: a payload
is a slot index, a staged transfer a ``StagedExpert`` in a lent ring position."""
import json
from pathlib import Path
from types import SimpleNamespace as NS

import pytest

from oracle import ref_rs, ref_staging
from sparse_amd.residency import ResidencyConfig, StagedExpert
from sparse_amd.ring import LENT
from sparse_amd.staging import BoundedRS, select_candidates
from tests.test_residency import FakeEvent, product_layer

DATA = json.loads((Path(__file__).resolve().parent / "golden" / "staging_ops.json").read_text())
STATS = DATA["stats"]


@pytest.mark.parametrize("impl", [select_candidates, ref_rs.select_candidates], ids=["product", "oracle"])
def test_select_candidates_matches_the_reference(impl):
    for c in DATA["select"]:
        diag = {}
        got = impl(c["ids"], c["weights"], allowed=set(c["allowed"]), resident=set(c["resident"]),
                   minimum=c["minimum"], budget=c["budget"], diagnostics=diag)
        assert list(got) == c["chosen"]
        assert diag == c["diagnostics"]


def _product_session(case):
    E = case["E"]
    res, backend, _metrics = product_layer(ResidencyConfig(capacity=case["capacity"], staging_pool_slots=E), E=E)
    res.phase, res.stage, res.call_id = "decode", "decode", 0
    tags = {}

    def load(eid):                      # an ordinary load into the resident cache, no access counted
        slot = res._acquire_slot()
        res._upload(eid, slot, "compute")
        tags[slot] = f"res{eid}"
        res._cache_put(eid, slot)

    for e in case["seed_ids"]:
        load(e)
    ring = res.ring
    engine = BoundedRS(slots=2, empty_steps=case["empty_steps"])
    engine.layers = {0: NS(layer_idx=0, residency=res)}
    engine.begin()
    block = engine.layers[0]
    for (op, *args), want in zip(case["ops"], case["results"]):
        r = None
        if op == "stage":
            pos = ring.state.index("idle")
            slot, ring.state[pos] = ring.slots[pos], LENT
            tags[slot] = f"staged{args[0]}"
            backend.slot_content[slot] = args[0]
            res.staged[args[0]] = StagedExpert(pos, slot, FakeEvent("copy", args[0]))
        elif op in ("get", "peek"):
            got = res.find(args[0], touch=op == "get")
            r = None if got is None else tags[got]
        elif op == "has":
            r = res.holds(args[0])
        elif op == "miss":
            engine.demand_miss(0)
        elif op == "arm":
            engine.pause.until[0] = args[0]
            engine.pause.members[0] = frozenset(res.cache.resident_ids())
        elif op == "skip":
            r = engine._paused(0, args[0])
        elif op == "put":
            if res.cache.has(args[0]):
                # the reference replaces the payload object of a resident entry; here the bytes
                # already sit in the entry's slot, so only the recency moves
                res.cache.get(args[0])
                tags[res.cache.peek(args[0])] = f"res{args[0]}"
            else:
                load(args[0])
                res.flush()
        else:
            free_before = set(res._free_slots)
            r = []
            for eid, rec in engine.settle(block):
                if rec.touched:
                    now = ring.slots[rec.pos]       # what the ring holds in the staged expert's place
                    r.append([eid, rec.kept, "fresh" if (rec.kept and now in free_before) else tags[now]])
            assert ring.all_idle() and not res.staged
        freq = sorted(res.access_freq.items()) if op == "exit" else None
        got = [r, res.cache.resident_ids(), list(res.staged_touched), sorted(res.staged),
               engine.pause.until.get(0), [engine.stats[k] for k in STATS], freq]
        yield op, args, got, want


@pytest.mark.parametrize("index", range(len(DATA["sessions"])))
def test_product_session_matches_the_reference(index):
    for n, (op, args, got, want) in enumerate(_product_session(DATA["sessions"][index])):
        want = list(want)
        if want[6] is not None:
            want[6] = [tuple(x) for x in want[6]]
        assert got == want, f"operation {n}: {op} {args}"


@pytest.mark.parametrize("index", range(len(DATA["sessions"])))
def test_oracle_lookup_matches_the_reference(index):
    """The oracle restates the demand view only (lookups over plain data); resident loads and
    layer exits are applied to its plain lists with textbook LRU so that the lookups keep
    seeing the same state."""
    case = DATA["sessions"][index]
    cap = case["capacity"]
    resident = [(e, f"res{e}") for e in case["seed_ids"]]
    staged, used = {}, []

    def put(eid, payload):
        for i, (e, _p) in enumerate(resident):
            if e == eid:
                resident.pop(i)
                break
        resident.append((eid, payload))
        while len(resident) > cap:
            resident.pop(0)

    for (op, *args), want in zip(case["ops"], case["results"]):
        r = want[0]
        if op == "stage":
            staged[args[0]] = [f"staged{args[0]}", False]
        elif op == "get":
            r = ref_staging.lookup(resident, staged, used, args[0], touch=True)
        elif op == "peek":
            r = ref_staging.lookup(resident, staged, used, args[0], touch=False)
        elif op == "has":
            r = ref_staging.has(resident, staged, args[0])
        elif op == "put":
            put(args[0], f"res{args[0]}")
        elif op == "exit":
            for eid in used:
                put(eid, staged[eid][0])
            staged, used = {}, []
        assert r == want[0], f"{op} {args}"
        assert [e for e, _p in resident] == want[1] and used == want[2] and sorted(staged) == want[3], f"{op} {args}"
