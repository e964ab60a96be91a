"""Cost-aware local readiness policy: the product's classes (``sparse_amd/local_policy.py``)
and the oracle's plain functions (``oracle/ref_policy.py``) against the reference's own
known-answer tests (tests/test_lightweight_policy.py:31-54, restated here with the same
numbers), closed forms, and each other on random inputs."""
import ast
import json
import random
from pathlib import Path

import pytest

from oracle import ref_policy
from sparse_amd.local_policy import COST_FIELDS, CostProfile, Costs, LocalPolicy, write_profile

ROOT = Path(__file__).resolve().parents[1]
# cost table of the reference's tests (tests/test_lightweight_policy.py:22-27)
REF_COSTS = dict(h2d_bytes_per_ms=10, h2d_latency_ms=0, expert_ms=.2, item_ms=.1, next_attention_ms=1,
                 split_overhead_ms=.01)


def _profile(tmp_path, world=2, **extra):
    path = tmp_path / "costs.json"
    path.write_text(json.dumps(dict(schema_version=1, world_size=world, calibrated=False, rank_defaults=REF_COSTS,
                                    **extra)))
    return CostProfile(path, world)


def test_prefetch_scores_known_answers_of_the_reference(tmp_path):
    # tests/test_lightweight_policy.py:31-44
    policy = LocalPolicy(_profile(tmp_path), 0, 1, {0: 10, 1: 100, 2: 10}, ())
    policy.window_ms = 2
    policy.observe_ready(2, 8)              # 1.2 ms already available for overlap
    assert policy.ready_ms == pytest.approx(1.2)
    values = policy.scores({0: .5, 1: .5, 2: .9}, {2})
    assert values[0] == 0 and values[1] == .5 and values[2] == .9
    assert policy.stats["candidate_scores"] == 3
    policy.reset()
    assert policy.ready_ms == 0 and policy.stats["candidate_scores"] == 0
    # the oracle's formulation on the same numbers
    sizes = {0: 10, 1: 100, 2: 10}
    got = ref_policy.adjusted_scores(REF_COSTS, sizes, {0: .5, 1: .5, 2: .9}, {2}, 2, 1.2)
    assert got == {0: 0, 1: .5, 2: .9}


def test_residual_known_answers_of_the_reference(tmp_path):
    # tests/test_lightweight_policy.py:46-54
    sizes = {0: 1, 1: 100, 2: 100}
    policy = LocalPolicy(_profile(tmp_path), 0, 1, sizes, ())
    choices = [(0, 0, "late"), (1, 1, "late"), (2, 2, "demand")]
    assert policy.residual(1, 1, choices) == (1, "late")          # equal overlap: the first one stays
    assert policy.residual(0, 0, choices) is None
    policy.window_ms = 0
    assert policy.scores({1: .7}, set()) == {1: .7}
    assert ref_policy.choose_residual(REF_COSTS, sizes, 1, 1, choices) == (1, "late")
    assert ref_policy.choose_residual(REF_COSTS, sizes, 0, 0, choices) is None
    assert ref_policy.adjusted_scores(REF_COSTS, sizes, {1: .7}, set(), 0, 0) == {1: .7}


def test_closed_forms(tmp_path):
    policy = LocalPolicy(_profile(tmp_path), 0, 0, {0: 50, 1: 5}, ())
    assert policy.transfer == {0: 5.0, 1: 0.5}
    assert policy.cost.compute(3, 10) == pytest.approx(.2 * 3 + .1 * 10)
    # window shorter than the copy, nothing covered: the whole window is gain -> score unchanged
    policy.window_ms = 2
    assert policy.scores({0: .8}, set())[0] == pytest.approx(.8)
    # 4 of the copy's 5 ms are covered: 1 ms of a 2 ms window can still be gained
    policy.observe_ready(20, 0)
    assert policy.scores({0: .8}, set())[0] == pytest.approx(.4)
    # without feedback the covered time is ignored
    blind = LocalPolicy(_profile(tmp_path), 0, 0, {0: 50}, (), feedback=False)
    blind.window_ms = 2
    blind.observe_ready(20, 0)
    assert blind.ready_ms == 0 and blind.scores({0: .8}, set())[0] == pytest.approx(.8)
    # prefetch part switched off: the very same mapping comes back
    off = LocalPolicy(_profile(tmp_path), 0, 0, {0: 50}, (), prefetch=False)
    values = {0: .8}
    assert off.scores(values, set()) is values
    # the split overhead is a strict threshold
    assert policy.residual(0, 0, [(0, 0, "late")]) is None
    summary = policy.summary()
    assert summary["metadata_collectives"] == 0 and summary["device_to_host_copies"] == 0
    assert summary["calibrated"] is False and len(summary["profile_sha256"]) == 64


def test_product_and_oracle_agree_on_random_inputs(tmp_path):
    rng = random.Random(5)
    for _ in range(200):
        costs = dict(h2d_bytes_per_ms=rng.uniform(1, 100), h2d_latency_ms=rng.uniform(0, 1),
                     expert_ms=rng.uniform(0, 1), item_ms=rng.uniform(0, .2), next_attention_ms=rng.uniform(0, 2),
                     split_overhead_ms=rng.uniform(0, 1))
        path = tmp_path / "c.json"
        path.write_text(json.dumps(dict(schema_version=1, world_size=1, calibrated=True, rank_defaults=costs)))
        sizes = {e: rng.uniform(1, 300) for e in range(12)}
        policy = LocalPolicy(CostProfile(path, 1), 0, 0, sizes, ())
        policy.window_ms = rng.choice([0.0, rng.uniform(0, 5)])
        groups, items = rng.randrange(0, 6), rng.randrange(0, 30)
        policy.observe_ready(groups, items)
        values = {e: rng.random() for e in rng.sample(range(12), 6)}
        residents = set(rng.sample(range(12), 3))
        want = ref_policy.adjusted_scores(costs, sizes, values, residents, policy.window_ms,
                                          ref_policy.compute_ms(costs, groups, items))
        got = policy.scores(values, residents)
        assert list(got) == list(want)
        for e in want:
            assert got[e] == pytest.approx(want[e], rel=1e-12, abs=1e-15)
        cands = [(i, e, rng.choice(["late", "demand"])) for i, e in enumerate(rng.sample(range(12), 4))]
        assert policy.residual(groups, items, cands) == ref_policy.choose_residual(costs, sizes, groups, items, cands)


def test_profile_override_order_and_validation(tmp_path):
    prof = _profile(tmp_path, rank_overrides={"1": {"expert_ms": .5}},
                    layers={"3": {"defaults": {"item_ms": .7}, "rank_overrides": {"1": {"item_ms": .9}}}})
    assert prof.cost(0, 0).expert == .2 and prof.cost(1, 0).expert == .5
    assert prof.cost(0, 3).item == .7 and prof.cost(1, 3).item == .9 and prof.cost(1, 3).expert == .5
    assert prof.cost(1, 3) is prof.cost(1, 3)
    want = ref_policy.resolve_costs(prof.data, 1, 3)
    got = prof.cost(1, 3)
    assert [want[k] for k in COST_FIELDS] == [got.bandwidth, got.latency, got.expert, got.item, got.attention,
                                              got.split]
    with pytest.raises(ValueError):
        _profile(tmp_path, world=2) and CostProfile(tmp_path / "costs.json", 4)      # world mismatch
    bad = tmp_path / "bad.json"
    bad.write_text(json.dumps(dict(schema_version=2, world_size=1, calibrated=False, rank_defaults=REF_COSTS)))
    with pytest.raises(ValueError):
        CostProfile(bad, 1)
    bad.write_text(json.dumps(dict(schema_version=1, world_size=1, calibrated="no", rank_defaults=REF_COSTS)))
    with pytest.raises(ValueError):
        CostProfile(bad, 1)
    for field, value in (("h2d_bytes_per_ms", 0), ("item_ms", -1), ("expert_ms", float("nan"))):
        with pytest.raises(ValueError):
            Costs.from_dict(dict(REF_COSTS, **{field: value}))
    write_profile(tmp_path / "w.json", dict(REF_COSTS), calibrated=True, provenance="test")
    assert CostProfile(tmp_path / "w.json", 1).cost(0, 0) == Costs.from_dict(REF_COSTS)


def test_policy_module_has_no_device_or_distributed_imports_at_module_level():
    # the reference holds its module to the same rule (tests/test_lightweight_policy.py:56-60)
    tree = ast.parse((ROOT / "sparse_amd" / "local_policy.py").read_text())
    names = [n.module for n in tree.body if isinstance(n, ast.ImportFrom)]
    names += [a.name for n in tree.body if isinstance(n, ast.Import) for a in n.names]
    assert not any(name and ("torch" in name or "distributed" in name) for name in names)
