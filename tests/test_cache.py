"""Cache semantics: the oracle restatement and the product cache against the reference's own
known answers, a textbook LRU model, the 4-class victim rule, and golden operation traces
recorded from the reference's class (tests/golden/cache_ops.json)."""
import itertools
import json
import random
from collections import OrderedDict
from pathlib import Path

import pytest

from oracle.ref_cache import RefEpipePrefillExtraCache, RefExpertWeightCache
from sparse_amd.cache import EpipePrefillExtraCache, ExpertWeightCache

GOLDEN = Path(__file__).resolve().parent / "golden"
IMPLS = [RefExpertWeightCache, ExpertWeightCache]
EXTRA_IMPLS = [RefEpipePrefillExtraCache, EpipePrefillExtraCache]


@pytest.mark.parametrize("impl", IMPLS)
def test_reference_known_answers(impl):
    # reference tests/test_rs_staging.py:52-66: access moves to the MRU end
    c = impl(2)
    c.put(0, "w0")
    c.put(4, "w4")
    assert c.resident_ids() == [0, 4]
    assert c.get(0) == "w0"
    assert c.resident_ids() == [4, 0]
    assert c.get(8) is None and c.resident_ids() == [4, 0]
    # reference tests/test_rs_staging.py:152-180: insertion evicts the oldest; order is oldest first
    c = impl(2)
    c.put(0, "old0")
    c.put(4, "old4")
    assert c.put(12, "new12") == 0
    assert c.put(8, "new8") == 4
    assert c.resident_ids() == [12, 8]
    assert c.peek(12) == "new12" and c.resident_ids() == [12, 8]


@pytest.mark.parametrize("impl", IMPLS)
def test_all_access_sequences_over_two_residents(impl):
    # reference tests/test_rs_staging.py:134-145 (64 sequences), against a textbook model
    for seq in itertools.product((0, 4), repeat=6):
        c = impl(2)
        model = OrderedDict()
        for e in (0, 4):
            c.put(e, str(e))
            model[e] = str(e)
        for e in seq:
            assert c.get(e) == model[e]
            model.move_to_end(e)
            assert c.resident_ids() == list(model)


@pytest.mark.parametrize("impl", IMPLS)
def test_replay_counts_of_the_reference_cache_replay_tests(impl):
    """tests/test_scp_cache_replay.py:89-98: experts 0,1,0 with capacity 1 -> 3 loads; capacity 0 -> no hits."""
    def replay(cap, seq):
        c, loads, hits = impl(cap), 0, 0
        for e in seq:
            if c.get(e) is None:
                loads += 1
                c.put(e, e)
            else:
                hits += 1
        return loads, hits
    assert replay(1, [0, 1, 0]) == (3, 0)
    assert replay(0, [0, 1, 0]) == (3, 0)
    assert replay(2, [0, 1, 0]) == (2, 1)
    # tests/test_scp_cache_replay.py:52-61: one expert requested 3 times on one layer, once on another
    assert replay(8, [2, 2, 2]) == (1, 2)


@pytest.mark.parametrize("impl", IMPLS)
def test_textbook_lru_on_random_traces(impl):
    rng = random.Random(1)
    for cap in (1, 2, 3, 5, 8):
        c, model = impl(cap), OrderedDict()
        for _ in range(2000):
            e = rng.randrange(12)
            got = c.get(e)
            if e in model:
                model.move_to_end(e)
                assert got == e
            else:
                assert got is None
                evicted = c.put(e, e)
                model[e] = e
                if len(model) > cap:
                    victim, _ = model.popitem(last=False)
                    assert evicted == victim
                else:
                    assert evicted is None
            assert c.resident_ids() == list(model)


@pytest.mark.parametrize("impl", IMPLS)
def test_victim_classes(impl):
    # oldest unpinned+unprotected transient beats an older plain entry
    c = impl(3)
    c.put(1, "a")
    c.put(2, "b", prefill_scp_transient=True)
    c.put(3, "c")
    assert c.put(4, "d") == 2
    # protected entries are skipped while an unprotected one exists
    c = impl(2)
    c.put(1, "a")
    c.put(2, "b")
    assert c.put(3, "c", protect_ids={1}) == 2
    # pinned entries are skipped; if all others are pinned the new entry itself goes
    c = impl(2)
    c.put(1, "a", pinned=True)
    c.put(2, "b", pinned=True)
    assert c.put(3, "c") == 3
    assert c.resident_ids() == [1, 2]
    # everything pinned, including the newcomer -> the oldest goes
    c = impl(2)
    c.put(1, "a", pinned=True)
    c.put(2, "b", pinned=True)
    assert c.put(3, "c", pinned=True) == 1
    # protected + transient is preferred over protected + plain when nothing is unprotected
    c = impl(2)
    c.put(1, "a")
    c.put(2, "b", prefill_scp_transient=True)
    assert c.put(3, "c", protect_ids={1, 2, 3}) == 2


@pytest.mark.parametrize("impl", IMPLS)
def test_admit_prefetch_rules(impl):
    c = impl(2)
    assert c.admit_prefetch(5, "p5") is True          # free slot, pinned
    c.put(6, "w6")
    assert c.evictable_prefetch_ids() == [6]
    assert c.admit_prefetch(7, "p7", preferred_victim=5) is True   # 5 is pinned -> falls back to 6
    assert c.resident_ids() == [5, 7]
    assert c.admit_prefetch(8, "p8") is False          # both pinned: refused
    c.unpin(5)
    assert c.admit_prefetch(8, "p8", protect_ids={5}) is False
    assert c.admit_prefetch(8, "p8") is True
    assert c.resident_ids() == [7, 8]
    assert impl(0).admit_prefetch(1, "x") is False


@pytest.mark.parametrize("impl", IMPLS)
def test_golden_traces_from_the_reference_class(impl):
    cases = json.loads((GOLDEN / "cache_ops.json").read_text())
    assert len(cases) >= 20
    for case in cases:
        c = impl(case["capacity"])
        for op, (want, resident, free) in zip(case["ops"], case["results"]):
            kind = op[0]
            if kind == "get":
                got = c.get(op[1])
            elif kind == "put":
                got = c.put(op[1], "w%d" % op[1], pinned=op[2], protect_ids=set(op[4]), prefill_scp_transient=op[3])
            elif kind == "admit":
                got = c.admit_prefetch(op[1], "p%d" % op[1], protect_ids=set(op[3]), preferred_victim=op[2])
            elif kind == "discard":
                got = c.discard(op[1])
            elif kind == "unpin":
                got = c.unpin(op[1])
            elif kind == "unpin_all":
                got = c.unpin_all()
            elif kind == "promote":
                got = c.promote_hot(op[1])
            elif kind == "evictable":
                got = c.evictable_prefetch_ids(set(op[1]))
            elif kind == "has":
                got = c.has(op[1])
            else:
                got = c.peek(op[1])
            assert got == want, (kind, op)
            assert c.resident_ids() == resident
            assert c.prefetch_free_slots() == free


@pytest.mark.parametrize("impl", EXTRA_IMPLS)
def test_extra_cache(impl):
    c = impl(2)
    assert c.put(1, "a", nbytes=10) == (True, False, None)
    assert c.put(2, "b", nbytes=20) == (True, False, None)
    assert c.get(1) == "a" and c.resident_ids() == [2, 1]
    assert c.put(3, "c", nbytes=5) == (True, False, 2)
    assert c.put(1, "a2", nbytes=7) == (True, True, None)
    assert c.resident_ids() == [3, 1] and c.resident_nbytes() == 12 and c.resident_count() == 2
    assert c.peek(3) == "c" and c.resident_ids() == [3, 1]
    assert c.clear() == 2 and not c.has(1)
    z = impl(0)
    assert z.put(1, "a") == (False, False, None) and z.get(1) is None


def test_product_and_oracle_agree_on_random_operations():
    rng = random.Random(7)
    for trial in range(30):
        cap = rng.choice([1, 2, 4, 7])
        a, b = RefExpertWeightCache(cap), ExpertWeightCache(cap)
        for _ in range(400):
            e = rng.randrange(14)
            protect = set(rng.sample(range(14), rng.randrange(0, 4)))
            op = rng.randrange(8)
            if op <= 2:
                assert a.get(e) == b.get(e)
            elif op <= 4:
                kw = dict(pinned=rng.random() < 0.2, protect_ids=protect, prefill_scp_transient=rng.random() < 0.2)
                assert a.put(e, e, **kw) == b.put(e, e, **kw)
            elif op == 5:
                v = rng.choice([None, rng.randrange(14)])
                assert a.admit_prefetch(e, e, protect_ids=protect, preferred_victim=v) == \
                    b.admit_prefetch(e, e, protect_ids=protect, preferred_victim=v)
            elif op == 6:
                assert a.discard(e) == b.discard(e)
            else:
                a.unpin(e), b.unpin(e)
                if rng.random() < 0.1:
                    assert a.demote_prefill_scp_transients() == b.demote_prefill_scp_transients()
            assert a.resident_ids() == b.resident_ids()
            assert a.evictable_prefetch_ids(protect) == b.evictable_prefetch_ids(protect)
            assert a.prefill_scp_transient_ids() == b.prefill_scp_transient_ids()


# ---------------------------------------------------------------------------- tiered cache
def _tiered_impls():
    from oracle.ref_cache import RefTieredExpertWeightCache
    from sparse_amd.cache import TieredExpertWeightCache
    return {"product": TieredExpertWeightCache, "oracle": RefTieredExpertWeightCache}


def _tiered_counts(cache):
    if hasattr(cache, "occupancy_counts"):
        return cache.occupancy_counts()
    occ = cache.occupancy()
    return [occ["hot"], occ["transient_demand"], occ["transient_prefetch"], occ["prefill_scp_transient"]]


def _tiered_flag(cache):
    fn = getattr(cache, "last_evicted_was_prefill_scp_transient", None)
    return bool(fn()) if fn is not None else bool(cache.last_evicted_transient)


def _apply_tiered(cache, rec):
    op = rec[0]
    if op == "get":
        return cache.get(rec[1])
    if op == "put":
        return cache.put(rec[1], "w%d" % rec[1], pinned=rec[2], prefer_hot=rec[4], protect_ids=set(rec[5]),
                         prefill_scp_transient=rec[3])
    if op == "admit":
        return cache.admit_prefetch(rec[1], "p%d" % rec[1], protect_ids=set(rec[3]), preferred_victim=rec[2])
    if op == "discard":
        return cache.discard(rec[1])
    if op == "unpin":
        return cache.unpin(rec[1])
    if op == "unpin_all":
        return cache.unpin_all()
    if op == "promote":
        return cache.promote_hot(rec[1])
    if op == "evictable":
        return cache.evictable_prefetch_ids(set(rec[1]))
    if op == "has":
        return cache.has(rec[1])
    if op == "peek":
        return cache.peek(rec[1])
    if op == "reset":
        return cache.reset_request_metadata(unpin=True, demote_hot=rec[1])
    if op == "demote_transients":
        return cache.demote_prefill_scp_transients()
    if op == "clear_transient":
        return cache.clear_prefill_scp_transient(rec[1])
    raise AssertionError(op)


@pytest.mark.parametrize("impl", ["product", "oracle"])
def test_tiered_cache_golden_traces_from_the_reference_class(impl):
    """Every operation of every recorded sequence: return value, resident order (hot, then
    transient demand, then transient prefetch), free speculative slots, tier occupancy and
    the last-evicted flag equal what the reference's own class produced."""
    import json
    from pathlib import Path
    data = json.loads((Path(__file__).parent / "golden" / "tiered_ops.json").read_text())
    cls = _tiered_impls()[impl]
    assert len(data["ops"]) >= 20
    for case in data["ops"]:
        cache = cls(case["capacity"], hot_capacity=case["hot"], prefetch_reserved=case["reserved"])
        for step, (rec, want) in enumerate(zip(case["ops"], case["results"])):
            got = _apply_tiered(cache, rec)
            state = [got, list(cache.resident_ids()), cache.prefetch_free_slots(), _tiered_counts(cache),
                     _tiered_flag(cache)]
            assert state == want, (case["capacity"], case["hot"], case["reserved"], step, rec)


def test_tiered_capacity_split_matches_the_reference_constructor():
    import json
    from pathlib import Path
    from oracle.ref_cache import ref_tiered_capacity_split
    from sparse_amd.cache import tiered_capacity_split
    data = json.loads((Path(__file__).parent / "golden" / "tiered_ops.json").read_text())
    assert len(data["split"]) > 300
    for cache, planner, reserved, extra, want in data["split"]:
        assert list(tiered_capacity_split(cache, planner, reserved, extra)) == want, (cache, planner, reserved, extra)
        assert list(ref_tiered_capacity_split(cache, planner, reserved, extra)) == want


def test_tiered_cache_speculation_never_displaces_hot_residents():
    """Closed-form property of the design (:3954-3962): whatever is admitted by prefetch, an
    expert in the hot tier stays resident and hot."""
    import random
    from sparse_amd.cache import TieredExpertWeightCache
    rng = random.Random(5)
    for _ in range(50):
        cache = TieredExpertWeightCache(8, hot_capacity=4, prefetch_reserved=1)
        hot = rng.sample(range(32), 4)
        for eid in hot:
            cache.put(eid, eid, prefer_hot=True)
        for _ in range(60):
            cache.admit_prefetch(rng.randrange(32, 64), "p", preferred_victim=rng.choice(hot))
            if rng.random() < 0.3:
                cache.unpin_all()
        assert all(cache.has(eid) for eid in hot) and cache.occupancy()["hot"] == 4
        assert len(cache) <= 8
