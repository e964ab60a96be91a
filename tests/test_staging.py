"""CPU tests of the bounded RS staging rules (sparse_amd/staging.py).

The scenarios and expected values are those of the reference's own tests for this
component (tests/test_rs_staging.py, cited per test), run against this build's classes;
random sequences are checked against the oracle in oracle/ref_staging.py and
oracle/ref_rs.py."""
import itertools
import random
import threading
from types import SimpleNamespace as NS

import pytest

from oracle import ref_rs, ref_staging
from sparse_amd.cache import ExpertWeightCache
from sparse_amd.residency import Backend, LayerResidency, ResidencyConfig
from sparse_amd.staging import BoundedRS, DemandCacheView, TargetJob, Transfer, select_candidates


class Event:
    def __init__(self, complete=True):
        self.complete = complete

    def query(self):
        return self.complete

    def synchronize(self):
        raise AssertionError("demand must not CPU-synchronize an expert copy")


def _cache():
    cache = ExpertWeightCache(2)
    cache.put(0, "w0")
    cache.put(4, "w4")
    return cache


def _transfer(eid, complete=True):
    return Transfer(eid, "w%d" % eid, Event(complete), object(), 16)


def test_wrong_prefetch_never_evicts_or_changes_lru():
    """tests/test_rs_staging.py:60-66."""
    cache = _cache()
    view = DemandCacheView(cache)
    view.staged = {8: _transfer(8)}
    assert cache.resident_ids() == [0, 4]
    assert view.get(0) == "w0"
    assert cache.resident_ids() == [4, 0]
    assert not view.staged[8].used
    assert view.capacity == 2 and len(view) == 2


def test_staged_copy_is_visible_without_touching_recency():
    """tests/test_rs_staging.py:68-72: the EPIPE ready classification sees staged payloads."""
    cache = _cache()
    view = DemandCacheView(cache)
    view.staged = {8: _transfer(8)}
    assert view.has(8) and view.peek(8) == "w8" and not view.staged[8].used
    assert cache.resident_ids() == [0, 4]


def test_native_hit_has_precedence_over_staging():
    """tests/test_rs_staging.py:94-99."""
    view = DemandCacheView(_cache())
    shadow = _transfer(0)
    shadow.payload = "wrong-shadow"
    view.staged = {0: shadow}
    assert view.get(0) == "w0" and not shadow.used


def test_future_not_joined_when_target_closes():
    """tests/test_rs_staging.py:101-108."""
    job = TargetJob((1, 1, 2), [])

    class Future:
        def result(self, *args, **kwargs):
            raise AssertionError("no prediction join")
    job.future = Future()
    assert job.close() == {}
    assert not job.publish(8, lambda: pytest.fail("late duplicate H2D"))


def test_close_and_submission_have_single_owner():
    """tests/test_rs_staging.py:110-132: close() waits for a submission in progress and
    declines everything after."""
    entered, go, closed = threading.Event(), threading.Event(), threading.Event()
    job = TargetJob((1, 1, 2), [])

    def submit():
        entered.set()
        assert go.wait(2)
        return _transfer(8, False)
    worker = threading.Thread(target=lambda: job.publish(8, submit))
    worker.start()
    assert entered.wait(2)
    result = []

    def close():
        result.append(job.close())
        closed.set()
    consumer = threading.Thread(target=close)
    consumer.start()
    assert not closed.wait(0.05)
    go.set()
    worker.join(2)
    consumer.join(2)
    assert closed.is_set() and set(result[0]) == {8}
    assert not job.publish(4, lambda: pytest.fail("target already executing"))


def test_no_wrong_forecast_changes_any_resident_access_sequence():
    """tests/test_rs_staging.py:134-145: all 64 sequences over two residents."""
    for sequence in itertools.product((0, 4), repeat=6):
        baseline, candidate = ExpertWeightCache(2), ExpertWeightCache(2)
        for eid in (0, 4):
            baseline.put(eid, str(eid))
            candidate.put(eid, str(eid))
        view = DemandCacheView(candidate)
        for eid in sequence:
            view.staged = {8: _transfer(8)}
            assert view.get(eid) == baseline.get(eid)
            assert view.resident_ids() == baseline.resident_ids()
            assert not view.staged[8].used


def test_selection_known_answers_of_the_reference():
    """tests/test_rs_staging.py:147-150 and :308-312."""
    assert select_candidates([0, 8, 8, 9, 12], [.9, .1, .1, 1., .15], allowed={0, 8, 12}, resident={0},
                             minimum=.2, budget=2) == [8]
    diag = {}
    assert select_candidates([0, 1, 8], [.9, .9, .01], allowed={0, 8}, resident={0}, minimum=.2, budget=2,
                             diagnostics=diag) == []
    assert diag == dict(nonlocal_entries=1, resident_entries=1, scored=1, below_threshold=1)


def test_selection_equals_the_oracle_on_random_inputs():
    rng = random.Random(3)
    for _ in range(300):
        n = rng.randint(0, 40)
        ids = [rng.randrange(16) for _ in range(n)]
        w = [rng.random() * rng.choice((0.05, 0.3, 1.0)) for _ in range(n)]
        allowed = set(rng.sample(range(16), rng.randint(0, 16)))
        resident = set(rng.sample(range(16), rng.randint(0, 6)))
        kw = dict(allowed=allowed, resident=resident, minimum=rng.choice((0.0, 0.04, 0.2)), budget=rng.randint(0, 5))
        assert select_candidates(ids, w, **kw) == ref_rs.select_candidates(ids, w, **kw)


def test_view_equals_the_oracle_on_random_sequences():
    rng = random.Random(11)
    for _ in range(200):
        cache = ExpertWeightCache(3)
        resident = []
        for eid in rng.sample(range(10), 3):
            cache.put(eid, "r%d" % eid)
            resident.append((eid, "r%d" % eid))
        staged_ids = rng.sample(range(10), rng.randint(0, 4))
        view = DemandCacheView(cache)
        view.staged = {e: Transfer(e, "s%d" % e, Event(), object(), 16) for e in staged_ids}
        staged = {e: ["s%d" % e, False] for e in staged_ids}
        used = []
        for _ in range(20):
            eid, touch = rng.randrange(10), rng.random() < 0.7
            got = view.get(eid) if touch else view.peek(eid)
            assert got == ref_staging.lookup(resident, staged, used, eid, touch)
            assert view.has(eid) == ref_staging.has(resident, staged, eid)
            assert view.resident_ids() == [e for e, _ in resident]
        assert [t.expert for t in view.used_in_order] == used


class _NullBackend(Backend):
    def upload(self, eid, slot, lane):
        return Event()

    def event_done(self, event):
        return True

    def wait_event(self, event, lane, ordering=False):
        pass

    def run_segments(self, segments):
        pass

    def fence(self):
        return Event()


def _residency(capacity=2, pool=2):
    cfg = ResidencyConfig(capacity=capacity, staging_slots=2, staging_pool_slots=pool)
    return LayerResidency(0, 16, 4, cfg, _NullBackend(), expert_bytes=12)


def test_actual_use_defers_cache_update_and_recycles_victim_storage():
    """tests/test_rs_staging.py:152-180 on this build's slot model: the staged experts'
    slots become the cache's, the evicted residents' slots become the pool's, in first-use
    order, and nothing moves before the layer's exit."""
    res = _residency()
    res.phase, res.stage, res.call_id = "decode", "decode", 0
    s0, s4 = res._acquire_slot(), res._acquire_slot()
    res._cache_put(0, s0)
    res._cache_put(4, s4)
    p8, p12 = res.claim_staging_pool(2)
    engine = BoundedRS(slots=2)
    engine.stats = dict(retained=0, recycled_payloads=0, allocated_replacements=0)
    view = DemandCacheView(res.cache)
    res.cache = view
    engine.views = {0: view}
    rec8, rec12 = dict(payload=p8, busy=True), dict(payload=p12, busy=True)
    view.staged[8] = Transfer(8, p8, Event(), rec8, 12)
    view.staged[12] = Transfer(12, p12, Event(), rec12, 12)
    block = NS(layer_idx=0, residency=res)
    assert view.get(12) == p12 and view.get(8) == p8 and view.get(12) == p12
    assert view.resident.resident_ids() == [0, 4]
    assert [t.expert for t in view.used_in_order] == [12, 8]
    for transfer in view.used_in_order:
        engine._retain_used(block, transfer)
    assert view.resident.resident_ids() == [12, 8]
    assert rec12["payload"] == s0 and rec8["payload"] == s4      # victims' storage recycled
    assert view.resident.peek(12) == p12 and view.resident.peek(8) == p8
    assert engine.stats == dict(retained=2, recycled_payloads=2, allocated_replacements=0)
    assert sorted(res._pool_slots) == sorted([s0, s4])
    assert res._slot_of == {12: p12, 8: p8}


def test_cold_retention_takes_a_free_slot_as_replacement():
    """tests/test_rs_staging.py:182-197."""
    res = _residency()
    res.phase, res.stage, res.call_id = "decode", "decode", 0
    (p8,) = res.claim_staging_pool(1)
    free_before = list(res._free_slots)
    engine = BoundedRS(slots=2)
    engine.stats = dict(retained=0, recycled_payloads=0, allocated_replacements=0)
    view = DemandCacheView(res.cache)
    res.cache = view
    rec = dict(payload=p8, busy=True)
    transfer = Transfer(8, p8, Event(), rec, 12)
    view.staged[8] = transfer
    view.get(8)
    engine._retain_used(NS(layer_idx=0, residency=res), transfer)
    assert view.resident.peek(8) == p8
    assert rec["payload"] != p8 and rec["payload"] in free_before
    assert engine.stats["allocated_replacements"] == 1 and transfer.retained


def _cooldown_owner(view, empty_steps=16):
    owner = BoundedRS(slots=2, empty_steps=empty_steps)
    owner.views = {1: view}
    owner.next_probe, owner.cooldown_residents = {1: 27}, {1: frozenset({0, 4})}
    owner.stats = dict(observed_decode_misses=0, cooldown_miss_invalidations=0, cooldown_cache_invalidations=0,
                       skipped_cooldown=0)
    return owner


def test_cooldown_rules():
    """tests/test_rs_staging.py:265-306: a new miss or a change of the cache's contents wakes
    the target, a change of recency does not, the deadline does."""
    cache = _cache()
    owner = _cooldown_owner(DemandCacheView(cache))
    assert owner._skip_cooldown(1, 11)
    owner.note_demand_miss(NS(layer_idx=1))
    assert not owner._skip_cooldown(1, 12)
    assert owner.stats["cooldown_miss_invalidations"] == 1

    cache = _cache()
    owner = _cooldown_owner(DemandCacheView(cache))
    cache.put(8, "w8")
    assert not owner._skip_cooldown(1, 11)
    assert owner.stats["cooldown_cache_invalidations"] == 1

    cache = _cache()
    view = DemandCacheView(cache)
    owner = _cooldown_owner(view)
    view.get(0)
    assert owner._skip_cooldown(1, 11)
    assert not owner._skip_cooldown(1, 27)

    owner = _cooldown_owner(DemandCacheView(_cache()))
    owner.views.clear()
    owner.configure(empty_steps=0)
    assert owner.empty_steps == 0 and owner.next_probe == {} and owner.cooldown_residents == {}
    with pytest.raises(ValueError):
        owner.configure(empty_steps=-1)
    with pytest.raises(ValueError):
        owner.configure(empty_steps=True)
    owner.jobs[1] = object()
    with pytest.raises(AssertionError):
        owner.configure(empty_steps=16)


def test_pool_slots_never_enter_the_free_list():
    res = _residency(capacity=2, pool=3)
    pool = res.claim_staging_pool(3)
    assert not set(pool) & set(res._free_slots) and res.num_slots == 2 + 2 + 3
    res.clear()
    assert not set(pool) & set(res._free_slots)
    with pytest.raises(ValueError):
        res.claim_staging_pool(4)
