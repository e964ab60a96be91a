"""CPU tests of the forecast-staging rules (sparse_amd/staging.py, sparse_amd/ring.py and the
staged state of sparse_amd/residency.py).

The scenarios and expected values are those of the reference's own tests for this
component (tests/test_rs_staging.py, cited per test), run against this build's slot table
and ring; random sequences are checked against the oracle in oracle/ref_staging.py and
oracle/ref_rs.py."""
import itertools
import random
import threading
from types import SimpleNamespace as NS

import pytest

from oracle import ref_rs, ref_staging
from sparse_amd.cache import ExpertWeightCache
from sparse_amd.residency import Backend, LayerResidency, ResidencyConfig, StagedExpert
from sparse_amd.ring import LENT, StagingRing
from sparse_amd.staging import BoundedRS, select_candidates


class Event:
    def __init__(self, complete=True):
        self.complete = complete

    def query(self):
        return self.complete

    def synchronize(self):
        raise AssertionError("demand must not CPU-synchronize an expert copy")


class _NullBackend(Backend):
    def upload(self, eid, slot, lane):
        return Event()

    def event_done(self, event):
        return event.query()

    def wait_event(self, event, lane, ordering=False):
        pass

    def run_segments(self, segments):
        pass

    def fence(self):
        return Event()


def _residency(capacity=2, pool=2):
    cfg = ResidencyConfig(capacity=capacity, staging_slots=2, staging_pool_slots=pool)
    res = LayerResidency(0, 16, 4, cfg, _NullBackend(), expert_bytes=12)
    res.phase, res.stage, res.call_id = "decode", "decode", 0
    return res


def _layer(residents=(0, 4), capacity=2, pool=2):
    """A layer whose LRU holds ``residents`` (least recent first); returns it and expert -> slot."""
    res = _residency(capacity, pool)
    where = {}
    for eid in residents:
        where[eid] = res._acquire_slot()
        res._cache_put(eid, where[eid])
    return res, where


def _stage(res, *experts, complete=True):
    """Stage ``experts`` the way a forecast does: window, publication, seal, exposure.
    Returns expert -> ring position."""
    ring = res.ring
    assert ring.open("t", len(experts), lambda ev: ev.query()) == len(experts)
    for eid in experts:
        assert ring.publish("t", eid, lambda slot, pos: Event(complete))
    ticket, filled, chosen = ring.seal()
    assert ticket == "t" and chosen is None
    res.expose_staged(filled)
    return {eid: pos for eid, pos, _ev in filled}


def _engine(res, layer=0, **kw):
    engine = BoundedRS(slots=2, **kw)
    engine.layers = {layer: NS(layer_idx=layer, residency=res)}
    engine.begin()
    return engine


def test_wrong_prefetch_never_evicts_or_changes_lru():
    """tests/test_rs_staging.py:60-66."""
    res, where = _layer()
    _stage(res, 8)
    assert res.cache.resident_ids() == [0, 4]
    assert res.find(0) == where[0]
    assert res.cache.resident_ids() == [4, 0]
    assert not res.staged[8].touched
    assert res.cache.capacity == 2 and len(res.cache) == 2


def test_staged_copy_is_visible_without_touching_recency():
    """tests/test_rs_staging.py:68-72: the EPIPE ready classification sees staged experts."""
    res, _where = _layer()
    pos = _stage(res, 8)
    assert res.holds(8) and res.find(8, touch=False) == res.ring.slots[pos[8]] and not res.staged[8].touched
    assert res._contains_no_touch(8) and not res._contains_no_touch(9)
    assert res.cache.resident_ids() == [0, 4] and res.staged_touched == []


def test_native_hit_has_precedence_over_staging():
    """tests/test_rs_staging.py:94-99."""
    res, where = _layer()
    pos = _stage(res, 0)                # a shadow copy of a resident expert
    assert res.ring.slots[pos[0]] != where[0]
    assert res.find(0) == where[0] and not res.staged[0].touched


def test_forecast_not_joined_when_target_seals():
    """tests/test_rs_staging.py:101-108: the seal never waits for the scoring task, and what
    comes after it is declined."""
    ring = StagingRing([5, 6])
    ticket = (1, 1, 2)
    assert ring.open(ticket, 1, lambda ev: True) == 1

    class Task:
        def result(self, *args, **kwargs):
            raise AssertionError("no prediction join")

        def done(self):
            raise AssertionError("no prediction poll")
    ring.worker = Task()
    assert ring.seal() == (ticket, [], None)
    assert not ring.publish(ticket, 8, lambda slot, pos: pytest.fail("late duplicate H2D"))
    assert ring.all_idle()
    # the engine's hook on top of it: counts the close, waits for nothing
    res, _where = _layer()
    engine = _engine(res, layer=2)
    assert res.ring.open((engine.epoch, 1, 2), 1, lambda ev: True) == 1
    res.ring.worker = Task()
    engine.seal(NS(layer_idx=2, residency=res), 1)
    assert engine.stats["closed_before_publish"] == 1 and engine.stats["unplanned_closes"] == 1
    assert not res.staged


def test_seal_and_publication_have_single_owner():
    """tests/test_rs_staging.py:110-132: the seal waits for a publication in progress and
    everything after it is declined."""
    entered, go, sealed = threading.Event(), threading.Event(), threading.Event()
    ring = StagingRing([5, 6])
    ticket = (1, 1, 2)
    assert ring.open(ticket, 2, lambda ev: True) == 2

    def copy(slot, pos):
        entered.set()
        assert go.wait(2)
        return Event(False)
    worker = threading.Thread(target=lambda: ring.publish(ticket, 8, copy))
    worker.start()
    assert entered.wait(2)
    result = []

    def seal():
        result.append(ring.seal())
        sealed.set()
    consumer = threading.Thread(target=seal)
    consumer.start()
    assert not sealed.wait(0.05)
    go.set()
    worker.join(2)
    consumer.join(2)
    assert sealed.is_set() and [e for e, _p, _ev in result[0][1]] == [8]
    assert not ring.publish(ticket, 4, lambda slot, pos: pytest.fail("target already executing"))


def test_publication_for_another_window_is_declined():
    """A scoring task that wakes up after its window was sealed and the next one opened must
    not write into the new window."""
    ring = StagingRing([5, 6, 7, 8])
    assert ring.open("old", 2, lambda ev: True) == 2
    ring.seal()
    assert ring.open("new", 2, lambda ev: True) == 2
    assert not ring.publish("old", 3, lambda slot, pos: pytest.fail("stale window"))
    assert ring.publish("new", 3, lambda slot, pos: Event())
    assert ring.publish("new", 4, lambda slot, pos: Event())
    assert not ring.publish("new", 5, lambda slot, pos: pytest.fail("window is full"))
    _t, filled, _c = ring.seal()
    # a position is only handed out again when it is back and its fence has passed
    busy = Event(False)
    ring.give_back(filled[0][1], busy)
    assert ring.open("next", 4, lambda ev: ev.query()) == 2     # two never used; one lent, one fenced
    ring.seal()
    busy.complete = True
    assert ring.open("after", 4, lambda ev: ev.query()) == 3


def test_no_wrong_forecast_changes_any_resident_access_sequence():
    """tests/test_rs_staging.py:134-145: all 64 sequences over two residents."""
    for sequence in itertools.product((0, 4), repeat=6):
        baseline = ExpertWeightCache(2)
        res, where = _layer()
        for eid in (0, 4):
            baseline.put(eid, where[eid])
        for eid in sequence:
            _stage(res, 8)
            assert res.find(eid) == baseline.get(eid)
            assert res.cache.resident_ids() == baseline.resident_ids()
            assert not res.staged[8].touched
            assert [e for e, _rec in res.settle_staged()] == [8]
            assert res.cache.resident_ids() == baseline.resident_ids() and res.ring.all_idle()


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


def test_selection_scores_like_the_inline_planner():
    """Candidates are ranked by the planner's own aggregate: for ids that pass the filter the
    order is that of ``LayerResidency.score_map``."""
    ids, w = [3, 5, 3, 7, 5, 3], [.2, .5, .1, .45, .05, .3]
    score = LayerResidency.score_map(ids, w)
    want = sorted(score, key=score.get, reverse=True)
    assert select_candidates(ids, w, allowed=set(range(16)), resident=set(), minimum=0.0, budget=9) == want


def test_lookups_equal_the_oracle_on_random_sequences():
    rng = random.Random(11)
    for _ in range(200):
        ids = rng.sample(range(10), 3)
        res, where = _layer(ids, capacity=3, pool=4)
        tag = {slot: "r%d" % eid for eid, slot in where.items()}
        resident = [(eid, "r%d" % eid) for eid in ids]
        staged_ids = rng.sample(range(10), rng.randint(0, 4))
        if staged_ids:
            for eid, pos in _stage(res, *staged_ids).items():
                tag[res.ring.slots[pos]] = "s%d" % eid
        staged = {e: ["s%d" % e, False] for e in staged_ids}
        used = []
        for _ in range(20):
            eid, touch = rng.randrange(10), rng.random() < 0.7
            got = res.find(eid, touch)
            assert (None if got is None else tag[got]) == ref_staging.lookup(resident, staged, used, eid, touch)
            assert res.holds(eid) == ref_staging.has(resident, staged, eid)
            assert res.cache.resident_ids() == [e for e, _ in resident]
        assert res.staged_touched == used


def test_actual_use_defers_cache_update_and_recycles_victim_storage():
    """tests/test_rs_staging.py:152-180 on this build's slot model: the staged experts'
    slots become the cache's, the evicted residents' slots become the ring's, in first-use
    order, and nothing moves before the layer's exit."""
    res, where = _layer()
    s0, s4 = where[0], where[4]
    engine = _engine(res)
    pos = _stage(res, 8, 12)
    p8, p12 = res.ring.slots[pos[8]], res.ring.slots[pos[12]]
    assert res.find(12) == p12 and res.find(8) == p8 and res.find(12) == p12
    assert res.cache.resident_ids() == [0, 4]
    assert res.staged_touched == [12, 8]
    settled = engine.settle(NS(layer_idx=0, residency=res))
    assert [e for e, _rec in settled] == [12, 8] and all(rec.kept and rec.recycled for _e, rec in settled)
    assert res.cache.resident_ids() == [12, 8]
    assert res.ring.slots[pos[12]] == s0 and res.ring.slots[pos[8]] == s4      # victims' storage recycled
    assert res.cache.peek(12) == p12 and res.cache.peek(8) == p8
    got = {k: engine.stats[k] for k in ("retained", "recycled_payloads", "allocated_replacements", "used", "wasted")}
    assert got == dict(retained=2, recycled_payloads=2, allocated_replacements=0, used=2, wasted=0)
    assert sorted(res._pool_slots) == sorted([s0, s4])
    assert res._slot_of == {12: p12, 8: p8}
    assert not res.staged and not res.staged_touched and res.ring.all_idle()


def test_cold_retention_takes_a_free_slot_as_replacement():
    """tests/test_rs_staging.py:182-197."""
    res, _where = _layer(residents=())
    engine = _engine(res)
    pos = _stage(res, 8)
    p8 = res.ring.slots[pos[8]]
    free_before = list(res._free_slots)
    assert res.find(8) == p8
    ((eid, rec),) = engine.settle(NS(layer_idx=0, residency=res))
    assert eid == 8 and rec.kept and not rec.recycled
    assert res.cache.peek(8) == p8
    assert res.ring.slots[pos[8]] != p8 and res.ring.slots[pos[8]] in free_before
    assert engine.stats["allocated_replacements"] == 1 and engine.stats["retained"] == 1


def test_unused_copy_is_wasted_and_its_slot_waits_for_the_copy():
    """A staged expert nobody asked for leaves no trace in the LRU; its ring position comes
    back behind its own copy event (the copy may still be in flight)."""
    res, _where = _layer()
    engine = _engine(res)
    pos = _stage(res, 8, complete=False)
    before = res.metrics.prefetch_wasted_count
    ((eid, rec),) = engine.settle(NS(layer_idx=0, residency=res))
    assert eid == 8 and not rec.touched and not rec.kept
    assert res.cache.resident_ids() == [0, 4] and engine.stats["wasted"] == 1
    assert res.metrics.prefetch_wasted_count == before + 1 and res.staged_unconfirmed == 1
    assert res.ring.fence[pos[8]] is rec.event
    assert res.ring.open("t2", 2, lambda ev: ev.query()) == 1      # the other position only
    res.ring.seal()
    res.confirm_staged_copies()
    assert res.staged_unconfirmed == 0


def _paused(res, empty_steps=16):
    engine = _engine(res, layer=1, empty_steps=empty_steps)
    engine.pause.until[1], engine.pause.members[1] = 27, frozenset({0, 4})
    return engine


def test_cooldown_rules():
    """tests/test_rs_staging.py:265-306: a new miss or a change of the cache's contents wakes
    the target, a change of recency does not, the deadline does."""
    res, _where = _layer()
    engine = _paused(res)
    assert engine._paused(1, 11) and engine.stats["skipped_cooldown"] == 1
    engine.demand_miss(1)
    assert not engine._paused(1, 12)
    assert engine.stats["cooldown_miss_invalidations"] == 1 and engine.stats["observed_decode_misses"] == 1

    res, _where = _layer()
    engine = _paused(res)
    res._cache_put(8, res._acquire_slot())
    assert not engine._paused(1, 11)
    assert engine.stats["cooldown_cache_invalidations"] == 1

    res, _where = _layer()
    engine = _paused(res)
    res.find(0)
    assert engine._paused(1, 11)
    assert not engine._paused(1, 27)
    assert engine.pause.until == {} and engine.pause.members == {}

    engine = _paused(res)
    engine.configure(empty_steps=0)
    assert engine.empty_steps == 0 and engine.pause.until == {} and engine.pause.members == {}
    with pytest.raises(ValueError):
        engine.configure(empty_steps=-1)
    with pytest.raises(ValueError):
        engine.configure(empty_steps=True)
    res.ring.open("t", 1, lambda ev: True)      # a window is open: the request is not drained
    with pytest.raises(AssertionError):
        engine.configure(empty_steps=16)


def test_an_empty_forecast_arms_the_cooldown_at_the_seal():
    """utils/rs_overlap.py:321-323: only a window whose scoring ran and chose nothing starts
    the pause, for ``empty_steps`` steps after this one."""
    res, _where = _layer()
    engine = _engine(res, layer=1, empty_steps=4)
    block = NS(layer_idx=1, residency=res)
    res.ring.open((engine.epoch, 7, 1), 1, lambda ev: True)
    engine.seal(block, 7)                                   # not scored yet: no pause
    assert engine.pause.until == {} and engine.stats["unplanned_closes"] == 1
    res.ring.open((engine.epoch, 8, 1), 1, lambda ev: True)
    res.ring.note_chosen((engine.epoch, 8, 1), 0)
    engine.seal(block, 8)
    assert engine.pause.until == {1: 13} and engine.pause.members == {1: frozenset({0, 4})}
    assert engine.stats["empty_plan_closes"] == 1 and engine.stats["closed_before_publish"] == 2
    assert engine._paused(1, 12) and not engine._paused(1, 13)


def test_ring_slots_never_enter_the_free_list():
    res = _residency(capacity=2, pool=3)
    ring = res.staging_ring(3)
    assert not set(ring.slots) & set(res._free_slots) and res.num_slots == 2 + 2 + 3
    res.clear()
    assert not set(ring.slots) & set(res._free_slots)
    with pytest.raises(ValueError):
        res.staging_ring(4)
