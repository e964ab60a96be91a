"""Prefill -> decode boundary hooks of the block and the prefill side cache, on the CPU.

The first three tests restate the reference's own tests of the hooks
(tests/test_prefill_cache_boundary.py:52-78) with the same stub caches and numbers; the
rest pin the side cache's rules (utils/eval_core.py:5637-5720, :6146-6147, :16591-16627):
a payload found there is an ordinary hit, it is filled during prefill only, decode keeps
reading it unless told otherwise, and a new request drops it."""
from types import SimpleNamespace

import pytest

from oracle.ref_layer import RefConfig, RefLayer
from sparse_amd.block import DistributedSparseMoeBlock as Block
from sparse_amd.context import Metrics, SparseContext
from sparse_amd.residency import ResidencyConfig
from tests.test_residency import product_layer


class StubCache:
    def __init__(self, ids):
        self.ids, self.calls = list(ids), 0

    def prefill_scp_transient_ids(self):
        return list(self.ids)

    def demote_prefill_scp_transients(self):
        self.calls += 1
        return len(self.ids)


def _plain_metrics():
    return SimpleNamespace(prefill_scp_transient_resident_at_decode_start=0, prefill_scp_transient_demote_count=0,
                           epipe_prefill_transient_demote_count=0, prefill_scp_transient_resident_at_decode_end=0)


@pytest.fixture
def caches():
    SparseContext.reset()
    caches = [StubCache([3, 7]), StubCache([11])]
    SparseContext.layer_blocks = {i: SimpleNamespace(_cache=c) for i, c in enumerate(caches)}
    yield caches
    SparseContext.reset()


def test_demotes_registered_layers_once_per_request(caches):
    first = _plain_metrics()
    Block.demote_prefill_scp_transients_for_decode(first)
    Block.demote_prefill_scp_transients_for_decode(first)
    assert [c.calls for c in caches] == [1, 1]
    assert first.prefill_scp_transient_resident_at_decode_start == 3
    assert first.prefill_scp_transient_demote_count == 3
    assert first.epipe_prefill_transient_demote_count == 3
    SparseContext.prefill_scp_transient_demoted_for_decode = False
    second = _plain_metrics()
    Block.demote_prefill_scp_transients_for_decode(second)
    assert [c.calls for c in caches] == [2, 2]
    assert second.prefill_scp_transient_demote_count == 3


def test_request_context_decides_not_class_state(caches):
    Block.prefill_scp_transient_demoted_for_decode = True     # stale class attributes must not matter
    Block.layer_blocks = {}
    try:
        Block.demote_prefill_scp_transients_for_decode()
        assert [c.calls for c in caches] == [1, 1]
        assert SparseContext.prefill_scp_transient_demoted_for_decode
    finally:
        del Block.prefill_scp_transient_demoted_for_decode, Block.layer_blocks


def test_end_accounting_reads_current_registered_caches(caches):
    result = _plain_metrics()
    caches[0].ids.clear()
    Block.record_prefill_scp_transient_decode_end(result)
    assert result.prefill_scp_transient_resident_at_decode_end == 1
    Block.record_prefill_scp_transient_decode_end(None)
    own = Metrics()                                            # this package's counters work too
    Block.record_prefill_scp_transient_decode_end(own)
    assert own.counters["prefill_scp_transient_resident_at_decode_end"] == 1


# ---- the prefill side cache -------------------------------------------------------------
EXTRA = dict(capacity=2, epipe_enable=True, epipe_prefill_enable=True, epipe_prefill_commit=False,
             epipe_prefill_extra_cache_slots=2)


def _both(**cfg):
    ref = RefLayer(0, 16, 2, RefConfig(**cfg))
    prod, backend, metrics = product_layer(ResidencyConfig(**cfg))
    ref.expert_bytes = 100
    return ref, prod, backend, metrics


def _step(ref, prod, metrics, stage, call, segments):
    for lay in (ref, prod):
        lay.phase, lay.call_id, lay.stage = stage, call, stage
    before_r, before_p = len(ref.trace), len(metrics.events)
    names = (ref.execute(segments), prod.execute(segments))
    assert names[0] == names[1]
    ev_r = [t for t in ref.trace[before_r:] if t[0] in ("hit", "prefetch_hit", "miss")]
    ev_p = [(k, e) for k, _l, e in metrics.events[before_p:]]
    assert ev_r == ev_p
    return names[0], ev_r


def test_side_cache_is_filled_in_prefill_and_read_as_hits_in_decode():
    ref, prod, _be, metrics = _both(**EXTRA)
    _step(ref, prod, metrics, "prefill", 0, [(1, 4)])                       # expert 1 resident
    name, ev = _step(ref, prod, metrics, "prefill", 1, [(1, 4), (5, 4)])
    assert name == "epipe_upfront" and ev == [("hit", 1), ("miss", 5)]
    assert ref.extra.resident_ids() == [5] == prod.extra_cache.resident_ids()      # not committed: kept aside
    assert ref.cache.resident_ids() == [1] == prod.cache.resident_ids()
    # decode finds expert 5 in the side cache: a hit, no copy
    copies = len([t for t in ref.trace if t[0] == "h2d"])
    _name, ev = _step(ref, prod, metrics, "decode", 2, [(5, 1)])
    assert ev == [("hit", 5)] and len([t for t in ref.trace if t[0] == "h2d"]) == copies
    assert ref.counters["epipe_prefill_extra_cache_hit_count"] == 1
    assert metrics.counters["epipe_prefill_extra_cache_hit_count"] == 1
    # decode never stores there
    _step(ref, prod, metrics, "decode", 3, [(5, 1), (9, 1)])
    assert ref.extra.resident_ids() == [5] == prod.extra_cache.resident_ids()
    # a new request drops it (and the product's slot goes back to the pool)
    free_before = len(prod._free_slots)
    ref.reset_for_new_request()
    prod.reset_for_new_request()
    assert ref.extra.resident_ids() == [] == prod.extra_cache.resident_ids()
    assert len(prod._free_slots) == free_before + 1


def test_side_cache_switches():
    # decode reads switched off: the staged expert is a miss again in decode
    ref, prod, _be, metrics = _both(**dict(EXTRA, epipe_prefill_extra_cache_decode_read=False))
    _step(ref, prod, metrics, "prefill", 0, [(1, 4)])
    _step(ref, prod, metrics, "prefill", 1, [(1, 4), (5, 4)])
    _name, ev = _step(ref, prod, metrics, "decode", 2, [(5, 1)])
    assert ev == [("miss", 5)]
    # kept across requests when asked to
    ref, prod, _be, metrics = _both(**dict(EXTRA, epipe_prefill_extra_cache_persist_requests=True))
    _step(ref, prod, metrics, "prefill", 0, [(1, 4)])
    _step(ref, prod, metrics, "prefill", 1, [(1, 4), (5, 4)])
    ref.reset_for_new_request()
    prod.reset_for_new_request()
    assert ref.extra.resident_ids() == [5] == prod.extra_cache.resident_ids()
    # the byte bound: one expert of 100 bytes does not fit under a bound of 64 bytes
    small = 64.0 / (1024.0 * 1024.0)
    ref, prod, _be, metrics = _both(**dict(EXTRA, epipe_prefill_extra_cache_max_mb=small))
    _step(ref, prod, metrics, "prefill", 0, [(1, 4)])
    _step(ref, prod, metrics, "prefill", 1, [(1, 4), (5, 4)])
    assert ref.extra.resident_ids() == [] == prod.extra_cache.resident_ids()
    assert ref.counters["epipe_prefill_extra_cache_no_room_count"] == 1
    assert metrics.counters["epipe_prefill_extra_cache_no_room_count"] == 1


def test_boundary_hook_counts_and_clears_the_side_cache_only_on_request():
    SparseContext.reset()
    try:
        lays = []
        for clear in (False, True):
            prod, _be, metrics = product_layer(ResidencyConfig(**dict(
                EXTRA, epipe_prefill_extra_cache_clear_at_decode=clear)))
            for call, segs in enumerate([[(1, 4)], [(1, 4), (5, 4)]]):
                prod.phase, prod.call_id, prod.stage = "prefill", call, "prefill"
                prod.execute(segs)
            lays.append(prod)
        SparseContext.layer_blocks = {i: SimpleNamespace(residency=l, _cache=l.cache) for i, l in enumerate(lays)}
        m = Metrics()
        Block.handle_epipe_prefill_extra_cache_decode_boundary(m)
        assert m.counters["epipe_prefill_extra_cache_resident_at_decode_start"] == 2
        assert m.counters["epipe_prefill_extra_cache_evict_count"] == 1
        assert lays[0].extra_cache.resident_ids() == [5] and lays[1].extra_cache.resident_ids() == []
        Block.record_epipe_prefill_extra_cache_decode_end(m)
        assert m.counters["epipe_prefill_extra_cache_resident_at_decode_end"] == 1
    finally:
        SparseContext.reset()


def test_workspace_tables_are_bounded():
    """Per-shape workspaces are kept for the most recently used shapes only."""
    from sparse_amd._lru import LruTable
    made = []
    table = LruTable(3)
    for key in (1, 2, 3, 1, 4):          # 1 is refreshed before 4 arrives, so 2 is the one dropped
        table.get_or_make(key, lambda key=key: made.append(key) or object())
    assert table.keys() == [3, 1, 4] and made == [1, 2, 3, 4] and 2 not in table
    assert table.get_or_make(1, lambda: pytest.fail("still held")) is not None
    with pytest.raises(ValueError):
        LruTable(0)
    from sparse_amd import ops
    from sparse_amd.block import _Workspace
    assert isinstance(_Workspace._cache, LruTable) and isinstance(ops._TILE_WS, LruTable)


def test_workspace_used_under_graph_capture_is_never_dropped():
    """A captured graph holds raw pointers into a workspace and no reference: an entry that was
    looked up while the stream was capturing stays, whatever else is used afterwards."""
    from sparse_amd._lru import LruTable
    capturing = [False]
    table = LruTable(2, capturing=lambda: capturing[0])
    table.get_or_make("a", object)
    capturing[0] = True
    held = table.get_or_make("graph", object)          # looked up during capture: pinned
    assert table.get_or_make("a", lambda: pytest.fail("held")) is not None and table.pinned() == {"graph", "a"}
    capturing[0] = False
    for key in range(10):                                # eager shapes come and go
        table.get_or_make(key, object)
    assert "graph" in table and "a" in table
    assert table.get_or_make("graph", lambda: pytest.fail("a pinned entry was dropped")) is held
    # pinned entries do not count against the limit: the two most recent eager shapes are still there
    assert [k for k in table.keys() if k not in ("graph", "a")] == [8, 9]
    table.pin(9)
    table.get_or_make(10, object)
    table.get_or_make(11, object)
    assert 9 in table and 8 not in table
    table.clear()
    assert len(table) == 0 and table.pinned() == set()


def test_prefill_expert_math_is_validated_like_the_reference(monkeypatch):
    """``SPARSE_PREFILL_EXPERT_MATH`` must be ``native`` or ``fixed64`` (utils/eval_core.py:4795-4798): anything
    else is a ``ValueError`` of the constructor, before a weight is touched; both accepted values (and
    ``SPARSE_EP_NATIVE_DECODE_GRANULARITY``) are read and recorded."""
    import torch
    from sparse_amd.context import DistEnv
    from sparse_amd.synthetic import make_mlp_block
    shape = dict(family="qwen_shared", hidden=64, num_experts=4, inter=64, top_k=2, shared_inter=64)
    mlp = make_mlp_block(shape, dtype=torch.float32, seed=0)
    env = DistEnv(0, 1, 0, torch.device("cpu"))
    monkeypatch.setenv("SPARSE_PREFILL_EXPERT_MATH", "fixed32")
    SparseContext.reset()
    try:
        with pytest.raises(ValueError, match="SPARSE_PREFILL_EXPERT_MATH must be native or fixed64"):
            Block(0, mlp, None, env, num_layers=1, num_experts=4, top_k=2, dtype=torch.float32)
        assert 0 not in SparseContext.layer_blocks
    finally:
        SparseContext.reset()
