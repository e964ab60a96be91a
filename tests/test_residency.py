"""Residency state machine: oracle (``oracle/ref_layer.py``) against the reference's known
answers and golden planner vectors, and the product (``sparse_amd/residency.py``) against
the oracle on long random traces for every method switch.  Runs on the CPU: the product's
device services are replaced by a recording backend that also checks slot safety."""
import json
import random
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import ref_rs
from oracle.ref_layer import RefConfig, RefLayer
from sparse_amd.context import Metrics
from sparse_amd.methods import METHODS, method_settings, residency_config
from sparse_amd.residency import Backend, LayerResidency, ResidencyConfig

GOLDEN = Path(__file__).resolve().parent / "golden"


# ----------------------------------------------------------------------------- fake device
class FakeEvent:
    def __init__(self, kind, eid=None):
        self.kind, self.eid = kind, eid


class RecordingBackend(Backend):
    """Records device effects and asserts the physical invariants of the slot pool."""

    def __init__(self, copy_done=None):
        self.trace = []
        self.slot_content = {}
        self.copy_done = copy_done or (lambda eid: True)

    def upload(self, eid, slot, lane):
        self.trace.append(("h2d", lane, eid))
        self.slot_content[slot] = eid
        return FakeEvent("copy", eid)

    def event_done(self, event):
        return True if event.kind == "fence" else bool(self.copy_done(event.eid))

    def wait_event(self, event, lane, ordering=False):
        if ordering:
            self.trace.append(("order_wait", lane, event.eid))
        elif event.kind == "copy":
            self.trace.append(("wait" if lane == "compute" else "wait_%s_lane" % lane, event.eid))

    def run_segments(self, segments):
        seen = set()
        for eid, slot in segments:
            assert self.slot_content.get(slot) == eid, f"slot {slot} holds {self.slot_content.get(slot)}, not {eid}"
            assert slot not in seen, "two segments of one batch share a slot"
            seen.add(slot)
            self.trace.append(("compute", eid))

    def fence(self):
        return FakeEvent("fence")


def product_layer(cfg: ResidencyConfig, E=16, K=2, copy_done=None, layer=0):
    m = Metrics()
    m.events = []
    be = RecordingBackend(copy_done)
    return LayerResidency(layer, E, K, cfg, be, m, expert_bytes=100), be, m


def to_ref_config(cfg: ResidencyConfig) -> RefConfig:
    names = [n for n in vars(RefConfig()) if hasattr(cfg, n)]
    return RefConfig(**{n: getattr(cfg, n) for n in names})


def split(trace):
    events = [t for t in trace if t[0] in ("hit", "prefetch_hit", "miss")]
    h2d = [t for t in trace if t[0] == "h2d"]
    compute = [t[1] for t in trace if t[0] == "compute"]
    waits = [t for t in trace if t[0] == "wait"]
    return events, h2d, compute, waits


# ----------------------------------------------------------------------------- scoring known answers
def test_select_candidates_known_answers_of_the_reference():
    # reference tests/test_rs_staging.py:147-150
    assert ref_rs.select_candidates([0, 8, 8, 9, 12], [.9, .1, .1, 1., .15], allowed={0, 8, 12}, resident={0},
                                    minimum=.2, budget=2) == [8]
    # reference tests/test_rs_staging.py:308-312
    diag = {}
    assert ref_rs.select_candidates([0, 1, 8], [.9, .9, .01], allowed={0, 8}, resident={0}, minimum=.2, budget=2,
                                    diagnostics=diag) == []
    assert diag == dict(nonlocal_entries=1, resident_entries=1, scored=1, below_threshold=1)


@pytest.mark.parametrize("impl", [RefLayer.score_map, LayerResidency.score_map])
def test_score_map_formula(impl):
    ids, w = [0, 8, 8, 9, 12], [.9, .1, .1, 1., .15]
    s = impl(ids, w)
    assert list(s) == [0, 8, 9, 12]                      # first-seen order
    assert s[8] == pytest.approx((.1 + .1) * 1.15 + .05 * .1)
    assert s[12] == pytest.approx(.15 + .05 * .15)
    assert s[9] == pytest.approx(1.05)
    # agrees with the staging adapter's selection on the same data
    chosen = [e for e in sorted(s, key=s.get, reverse=True) if e in {8, 12} and s[e] >= .2][:2]
    assert chosen == ref_rs.select_candidates(ids, w, allowed={0, 8, 12}, resident={0}, minimum=.2, budget=2)
    # brute force on random data
    rng = random.Random(3)
    for _ in range(50):
        n = rng.randrange(1, 40)
        ids = [rng.randrange(10) for _ in range(n)]
        w = [rng.random() for _ in range(n)]
        s = impl(ids, w)
        for e in set(ids):
            ws = [x for i, x in zip(ids, w) if i == e]
            assert s[e] == pytest.approx(sum(ws) * (1 + .15 * (len(ws) - 1)) + .05 * max(ws), rel=1e-12)


# ----------------------------------------------------------------------------- golden planner vectors
def _load_plan_cases():
    return json.loads((GOLDEN / "rs_plan.json").read_text())


def _setup_case(case, which):
    kw = dict(capacity=case["capacity"], planner_mode="rs_prefetch", prefetch_top_m=8, rs_policy=case["policy"],
              min_candidate_score=case["thresholds"][0], replace_advantage=case["thresholds"][1],
              replace_margin=case["thresholds"][2])
    if which == "oracle":
        lay = RefLayer(1, case["E"], 4, RefConfig(**kw))
        cache, freq, pre = lay.cache, lay.freq, lay.prefetched
    else:
        lay, _be, _m = product_layer(ResidencyConfig(**kw), E=case["E"], K=4, layer=1)
        cache, freq, pre = lay.cache, lay.access_freq, lay.prefetched_ids
    for e in case["residents"]:
        cache.put(e, ("w", e) if which == "oracle" else 0, pinned=e in case["pinned"])
    freq.update({int(k): int(v) for k, v in case["freq"]})
    pre.update(case["prefetched"])
    return lay


@pytest.mark.parametrize("which", ["oracle", "product"])
def test_planner_matches_golden_vectors_of_the_reference(which):
    cases = _load_plan_cases()
    assert len(cases) >= 100
    nontrivial = 0
    for case in cases:
        lay = _setup_case(case, which)
        score = lay.score_map(case["topi"], case["topv"])
        assert [[k, v] for k, v in score.items()] == case["score"]       # same floats, same order
        protect = set(case["protect"])
        if which == "oracle":
            assert lay.pick_victims_by_low_value(score, protect) == case["victims"]
        plan = lay.build_plan(score, protect, case["budget"])
        assert [[e, v] for e, v in plan] == case["plan"]
        nontrivial += any(v is not None for _e, v in plan)
        # invariants
        assert len(plan) <= case["budget"]
        assert all(not lay.cache.has(e) for e, _ in plan)
        assert all(v is None or (v not in protect and v in case["residents"] and v not in case["pinned"])
                   for _, v in plan)
    assert nontrivial > 20


# ----------------------------------------------------------------------------- predictor
def test_routing_scout_forward_closed_form():
    from sparse_amd.rs import RoutingScoutMLP
    torch.manual_seed(0)
    m = RoutingScoutMLP(32, 10, hidden_dim=16).eval()
    bn = m.mlp[1]
    bn.running_mean.uniform_(-1, 1)
    bn.running_var.uniform_(0.5, 2.0)
    x = torch.randn(5, 32)
    with torch.no_grad():
        want = m(x).numpy()
    got = ref_rs.routing_scout_forward(
        x.numpy(), m.mlp[0].weight.detach().numpy(), m.mlp[0].bias.detach().numpy(), bn.weight.detach().numpy(),
        bn.bias.detach().numpy(), bn.running_mean.numpy(), bn.running_var.numpy(), m.mlp[4].weight.detach().numpy(),
        m.mlp[4].bias.detach().numpy())
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got.sum(-1), 1.0, rtol=1e-5)
    assert sorted(m.state_dict()) == sorted(
        ["mlp.0.weight", "mlp.0.bias", "mlp.1.weight", "mlp.1.bias", "mlp.1.running_mean", "mlp.1.running_var",
         "mlp.1.num_batches_tracked", "mlp.4.weight", "mlp.4.bias"])


# ----------------------------------------------------------------------------- demand path
def test_inflight_prefetch_hit_waits_once_and_does_not_reload():
    """Restates reference tests/test_rs_staging.py:74-92 for both implementations."""
    for which in ("oracle", "product"):
        cfg = dict(capacity=4, planner_mode="rs_prefetch", prefetch_top_m=2)
        if which == "oracle":
            lay = RefLayer(0, 16, 2, RefConfig(**cfg), copy_done=lambda e: False)
            trace = lay.trace
        else:
            lay, be, m = product_layer(ResidencyConfig(**cfg), copy_done=lambda e: False)
        lay.phase, lay.call_id, lay.stage = "decode", 0, "decode"
        assert lay.prefetch_budget(("k", 0)) == 2
        lay.schedule_prefetch([8], [0.9], 2)
        lay.execute([(8, 1)])
        if which == "product":
            trace = [(k, e) for k, _l, e in m.events] + be.trace
        events, h2d, compute, waits = split(trace)
        assert events == [("prefetch_hit", 8)]
        assert h2d == [("h2d", "prefetch", 8)]        # no second load
        assert waits == [("wait", 8)]                 # exactly one stream wait, never a host sync
        assert compute == [8]
        assert lay.cache.resident_ids() == [8]


# ----------------------------------------------------------------------------- random traces, all methods
class RoutingModel:
    """Seeded routing with skewed popularity and an optional noisy predictor."""

    def __init__(self, E, K, T, seed):
        self.E, self.K, self.T = E, K, T
        self.rng = random.Random(seed)
        self.weights = [1.0 / (r + 1) ** 1.1 for r in range(E)]
        self.rng.shuffle(self.weights)

    def route(self):
        counts = {}
        for _ in range(self.T):
            picked = set()
            while len(picked) < self.K:
                picked.add(self.rng.choices(range(self.E), self.weights)[0])
            for e in picked:
                counts[e] = counts.get(e, 0) + 1
        return sorted(counts.items())

    def predict(self, next_segments, pred_k):
        ids, probs = [], []
        truth = [e for e, _ in next_segments]
        for _ in range(self.T):
            row = set()
            while len(row) < pred_k:
                if truth and self.rng.random() < 0.6:
                    row.add(self.rng.choice(truth))
                else:
                    row.add(self.rng.randrange(self.E))
            p = sorted((self.rng.random() for _ in row), reverse=True)
            s = sum(p)
            for e, v in zip(row, p):
                ids.append(e)
                probs.append(float(torch.tensor(v / s).to(torch.bfloat16)))
        return ids, probs


def run_trace(method, which, *, steps=60, layers=3, E=16, K=2, T=4, capacity=4, top_m=3, seed=0, late_rate=0.0,
              prefill_first=False, prefill_steps=0, overrides=None, formal=True, policy_costs=None, model=None):
    cfg = residency_config(method, capacity, top_m, formal_thresholds=formal, **(overrides or {}))
    late_rng = random.Random(seed + 99)
    late = {}

    def copy_done(layer):
        def fn(eid):
            key = (layer, eid)
            if key not in late:
                late[key] = late_rng.random() >= late_rate
            done = late[key]
            late[key] = True          # a second query finds the copy finished
            return done
        return fn

    lays, backs, mets = [], [], []
    for l in range(layers):
        if which == "oracle":
            lays.append(RefLayer(l, E, K, to_ref_config(cfg), copy_done=copy_done(l)))
        else:
            lay, be, m = product_layer(cfg, E=E, K=K, copy_done=copy_done(l), layer=l)
            lays.append(lay)
            backs.append(be)
            mets.append(m)
    if policy_costs is not None:
        # the cost-aware local policy on every layer: the product's class, the oracle's plain state
        import json
        import tempfile
        from sparse_amd.local_policy import CostProfile, LocalPolicy
        sizes = {e: 100.0 + 40.0 * (e % 5) for e in range(E)}
        with tempfile.TemporaryDirectory() as d:
            path = Path(d) / "costs.json"
            path.write_text(json.dumps(dict(schema_version=1, world_size=1, calibrated=False,
                                            rank_defaults=policy_costs)))
            profile = CostProfile(path, 1)
        for l, lay in enumerate(lays):
            if which == "oracle":
                lay.policy = dict(costs=dict(policy_costs), expert_bytes=sizes, window_ms=0.0, ready_ms=0.0,
                                  feedback=True, prefetch=True)
            else:
                lay.light_policy = LocalPolicy(profile, 0, l, sizes, ())
    model = RoutingModel(E, K, T, seed) if model is None else model
    executors = []
    prefill_steps = max(int(prefill_steps), 1 if prefill_first else 0)
    for step in range(steps):
        phase = "prefill" if step < prefill_steps else "decode"
        if prefill_steps and step == prefill_steps:
            # the prefill -> decode boundary hook: entries staged during prefill go to the LRU end
            for lay in lays:
                lay.cache.demote_prefill_scp_transients()
        routes = [model.route() for _ in range(layers)]
        preds = [model.predict(routes[l + 1], lays[l + 1].predict_topk()) if l + 1 < layers else None
                 for l in range(layers)]
        for l in range(layers):
            if cfg.planner_mode == "rs_prefetch" and l + 1 < layers and phase == "decode":
                tgt = lays[l + 1]
                tgt.phase, tgt.call_id = phase, step
                budget = tgt.prefetch_budget(("next_layer_rs", phase, step, l, l + 1))
                if budget > 0:
                    if policy_costs is not None:
                        # what the source layer's forward sets before planning (reference :10993-10996)
                        window = (policy_costs["expert_ms"] * K + policy_costs["item_ms"] * T * K
                                  + policy_costs["next_attention_ms"])
                        if which == "oracle":
                            tgt.policy["window_ms"] = window
                        else:
                            tgt.light_policy.window_ms = window
                    tgt.schedule_prefetch(preds[l][0], preds[l][1], budget)
            lay = lays[l]
            lay.phase, lay.call_id, lay.stage = phase, step, phase
            executors.append(lay.execute(routes[l]))
    out = []
    for l in range(layers):
        if which == "oracle":
            trace = lays[l].trace
            events, h2d, compute, waits = split(trace)
            plans = [list(t[1]) for t in trace if t[0] == "plan"]
        else:
            events = [(k, e) for k, _l, e in mets[l].events]
            _ev, h2d, compute, waits = split(backs[l].trace)
            plans = None
        out.append(dict(events=events, h2d=h2d, compute=compute, waits=waits, residents=lays[l].cache.resident_ids(),
                        plans=plans))
    return out, executors


METHOD_CASES = [
    ("rr", {}), ("rs", {}), ("epipe", {}), ("rs-epipe", {}), ("sparse", {}),
    ("rs-epipe", dict(late_rate=0.5)), ("rs", dict(formal=False)), ("rs-epipe", dict(formal=False, late_rate=0.3)),
    ("epipe", dict(prefill_first=True, overrides=dict(epipe_prefill_enable=True))),
    ("rr", dict(capacity=1)), ("rr", dict(capacity=0)), ("epipe", dict(capacity=2, T=8)),
    ("rs", dict(capacity=15, E=60, K=4, T=8, top_m=8)), ("rs-epipe", dict(capacity=15, E=60, K=4, T=8, top_m=8)),
    ("epipe", dict(overrides=dict(epipe_sort_ready_by_work=True))),
    ("epipe", dict(prefill_first=True, overrides=dict(epipe_prefill_enable=True, epipe_prefill_extra_cache_slots=2,
                                                      epipe_prefill_commit=False))),
    # --cache-policy tiered: hot / transient tiers, prefetch into its reserved area first
    ("rr", dict(capacity=8, E=24, T=8, overrides=dict(cache_policy="tiered"))),
    ("rs", dict(capacity=8, E=24, T=8, top_m=4, overrides=dict(cache_policy="tiered", prefetch_reserved=1))),
    ("rs", dict(capacity=12, E=60, K=4, T=8, top_m=8, formal=False,
                overrides=dict(cache_policy="tiered", prefetch_reserved=2))),
    ("epipe", dict(capacity=6, E=24, T=8, overrides=dict(cache_policy="tiered"))),
    ("rs-epipe", dict(capacity=8, E=24, T=8, top_m=4, formal=False,
                      overrides=dict(cache_policy="tiered", prefetch_reserved=1))),
    # several prefill calls: staged commits carry the transient mark and are evicted first
    ("epipe", dict(prefill_steps=5, capacity=8, T=2, overrides=dict(epipe_prefill_enable=True))),
    ("epipe", dict(prefill_steps=5, capacity=8, T=2,
                   overrides=dict(epipe_prefill_enable=True, epipe_prefill_mark_transient=False))),
    # bounded ready buffer: the code default (late_only), with demand staging, demand only
    ("rs-epipe", dict(late_rate=0.5, overrides=dict(epipe_decode_rs_mode="late_only"))),
    ("rs-epipe", dict(late_rate=0.3, formal=False, overrides=dict(epipe_decode_rs_mode="buffered"))),
    ("rs-epipe", dict(late_rate=0.3, overrides=dict(epipe_decode_rs_mode="demand_only"))),
    ("rs-epipe", dict(late_rate=0.4, capacity=15, E=60, K=4, T=8, top_m=8,
                      overrides=dict(epipe_decode_rs_mode="buffered", epipe_rs_buffer_max_groups=2))),
    ("rs-epipe", dict(late_rate=0.4, overrides=dict(epipe_decode_rs_mode="buffered", epipe_rs_min_buffer_groups=2,
                                                    epipe_rs_min_buffer_items=3))),
    # miss-triggered look-ahead: decode, decode with RS active, prefill with and without commit
    ("epipe", dict(overrides=dict(epipe_mode="miss_triggered", epipe_lookahead_min_ready_items=1))),
    ("epipe", dict(capacity=6, T=8, overrides=dict(epipe_mode="miss_triggered", epipe_lookahead_min_ready_items=4,
                                                   epipe_lookahead_experts=2))),
    ("rs-epipe", dict(late_rate=0.3, overrides=dict(epipe_mode="miss_triggered", epipe_decode_rs_mode="stream",
                                                    epipe_lookahead_min_ready_items=1))),
    ("epipe", dict(prefill_steps=4, capacity=6, T=8,
                   overrides=dict(epipe_mode="miss_triggered", epipe_prefill_enable=True,
                                  epipe_prefill_lookahead_min_ready_items=1, epipe_lookahead_min_ready_items=1))),
    ("epipe", dict(prefill_steps=4, capacity=6, T=8,
                   overrides=dict(epipe_mode="miss_triggered", epipe_prefill_enable=True, epipe_prefill_commit=False,
                                  epipe_prefill_extra_cache_slots=2, epipe_prefill_lookahead_min_ready_items=1,
                                  epipe_lookahead_min_ready_items=1))),
    # stream-all EPIPE (this build's addition): every miss of an EPIPE call on the EPIPE lane
    ("epipe", dict(overrides=dict(epipe_stream_all=True))),
    ("rs-epipe", dict(late_rate=0.3, overrides=dict(epipe_stream_all=True))),
    ("sparse", dict(capacity=15, E=60, K=4, T=8, top_m=8, overrides=dict(epipe_stream_all=True))),
    ("epipe", dict(prefill_steps=4, capacity=6, T=8, overrides=dict(epipe_stream_all=True, epipe_prefill_enable=True))),
    ("epipe", dict(capacity=6, T=8, overrides=dict(epipe_stream_all=True, epipe_mode="miss_triggered",
                                                   epipe_lookahead_min_ready_items=1))),
]


@pytest.mark.parametrize("method,kw", METHOD_CASES)
def test_product_reproduces_the_oracle_event_for_event(method, kw):
    for seed in range(3):
        want, ex_o = run_trace(method, "oracle", seed=seed, **kw)
        got, ex_p = run_trace(method, "product", seed=seed, **kw)
        assert ex_o == ex_p
        for l, (w, g) in enumerate(zip(want, got)):
            assert g["events"] == w["events"], f"layer {l}: cache events differ"
            assert g["h2d"] == w["h2d"], f"layer {l}: H2D sequence differs"
            assert g["compute"] == w["compute"], f"layer {l}: execution order differs"
            assert g["waits"] == w["waits"], f"layer {l}: stream waits differ"
            assert g["residents"] == w["residents"], f"layer {l}: final LRU order differs"
    if method in ("epipe", "rs-epipe", "sparse"):
        assert any(e.startswith("epipe") for e in ex_o), "EPIPE never triggered in this trace"


class SyntheticStackRouting:
    """The routing the cached-decode benchmark produces, computed on the host: per layer a bias-free gate
    carrying Zipf(1.1) popularity and clusters of four co-selected experts (``sparse_amd.synthetic``), the
    hidden states of ``make_structured_hidden`` (every layer reads the same rows), the router of the CPU
    oracle, and next-layer predictions from a bank of routing-scout MLPs (random-init, as the
    cached-decode configuration says, or built to reproduce the next router), reduced to the planner's inputs by the
    oracle's ``plan_inputs``.  Everything is computed once for all steps; ``route`` / ``predict`` then
    hand it out in the order ``run_trace`` asks."""

    def __init__(self, steps, layers, E, K, T, hidden, bank_kind, pred_k, dtype=torch.bfloat16):
        from types import SimpleNamespace as NS
        from oracle import ref_moe
        from sparse_amd.rs import informed_bank, random_init_bank
        from sparse_amd.synthetic import add_routing_structure, make_structured_hidden
        gates, structure = [], None
        for layer in range(layers):
            g = torch.Generator().manual_seed(layer)
            blk = NS(gate=NS(weight=(torch.randn(E, hidden, generator=g) * 0.02).to(dtype)))
            structure = add_routing_structure(blk, E, seed=layer)
            gates.append(blk.gate.weight)
        rows = torch.cat([make_structured_hidden(T, hidden, E // 4, structure["cluster_prob"], dtype, seed=5000 + i)
                          for i in range(steps)])
        self.routes, self.plans = [], []
        bank = (informed_bank([None] + gates[1:], hidden_dim=512) if bank_kind == "informed"
                else random_init_bank(layers, hidden, E, hidden_dim=512, seed=0))
        for layer in range(layers):
            _v, topi, _ = ref_moe.routing_router(rows, gates[layer], K, False)
            per_step = []
            for ids in topi.view(steps, T * K).tolist():
                counts = {}
                for e in ids:
                    counts[e] = counts.get(e, 0) + 1
                per_step.append(sorted(counts.items()))
            self.routes.append(per_step)
            if layer >= 1:
                with torch.no_grad():
                    pred = bank[layer](rows.float())
                ids, probs = ref_rs.plan_inputs(pred, pred_k, False, dtype)
                n = T * min(pred_k, E)
                self.plans.append([(ids[i * n:(i + 1) * n], probs[i * n:(i + 1) * n]) for i in range(steps)])
        self.layers, self._route_calls, self._predict_calls = layers, 0, 0

    def route(self):
        step, layer = divmod(self._route_calls, self.layers)
        self._route_calls += 1
        return self.routes[layer][step]

    def predict(self, next_segments, pred_k):
        step, src = divmod(self._predict_calls, self.layers - 1)
        self._predict_calls += 1
        return self.plans[src][step]


@pytest.mark.parametrize("method,bank", [("rr", "random"), ("rs", "random"), ("rs", "informed"),
                                         ("rs-epipe", "informed")])
def test_full_length_cached_decode_event_parity(method, bank):
    """The benchmark's cached-decode configuration at its full length on the host: 512 decode steps over 24
    layers, 60 experts, top-4, batch 8, a cache of 15, prefetch top-8, with its skewed co-activating routing.
    The product's policy against the oracle (utils/eval_core.py:11388-11435, :10916-11010, :12169-12512):
    every cache event, copy, execution order and wait of every layer equal, the final LRU order equal."""
    steps, layers, E, K, T = 512, 24, 60, 4, 8
    kw = dict(steps=steps, layers=layers, E=E, K=K, T=T, capacity=15, top_m=8)
    pred_k = product_layer(residency_config(method, 15, 8), E=E, K=K)[0].predict_topk()
    make = lambda: SyntheticStackRouting(steps, layers, E, K, T, 2048, bank, pred_k)
    first = make()
    import copy
    want, ex_o = run_trace(method, "oracle", model=copy.copy(first), **kw)
    got, ex_p = run_trace(method, "product", model=copy.copy(first), **kw)
    assert ex_o == ex_p
    misses = 0
    for l, (w, g) in enumerate(zip(want, got)):
        assert len(w["events"]) >= steps                        # every layer ran every step
        assert g["events"] == w["events"], f"layer {l}: cache events differ"
        assert g["h2d"] == w["h2d"], f"layer {l}: H2D sequence differs"
        assert g["compute"] == w["compute"], f"layer {l}: execution order differs"
        assert g["waits"] == w["waits"], f"layer {l}: stream waits differ"
        assert g["residents"] == w["residents"] and len(g["residents"]) == 15, f"layer {l}: final LRU order differs"
        misses += sum(1 for e in w["events"] if e[0] == "miss")
    accesses = sum(len(w["events"]) for w in want)
    # the routing is the skewed one: ~14 distinct experts per layer-step, far from uniform 60
    assert 10 * steps * layers < accesses < 20 * steps * layers
    assert 0.2 < 1 - misses / accesses < 0.95
    if method == "rs-epipe":
        assert any(e.startswith("epipe") for e in ex_o)


@pytest.mark.parametrize("method,kw", [
    ("epipe", {}), ("rs-epipe", dict(late_rate=0.3)), ("sparse", dict(capacity=15, E=60, K=4, T=8, top_m=8)),
    ("epipe", dict(prefill_steps=4, capacity=6, T=8, overrides=dict(epipe_prefill_enable=True))),
])
def test_stream_all_changes_lanes_and_waits_only(method, kw):
    """Stream-all EPIPE against the reference's one-staged-expert executors on the same trace:
    the same cache events in the same order, the same execution order, the same final LRU
    order and executor per call; every copy that was a demand copy on the compute lane inside
    an EPIPE call now travels on the EPIPE lane and is awaited exactly once; nothing else moves."""
    kw = dict(kw)
    over = dict(kw.pop("overrides", {}))
    for which in ("oracle", "product"):
        base, ex_b = run_trace(method, which, seed=5, overrides=over, **kw)
        strm, ex_s = run_trace(method, which, seed=5, overrides=dict(over, epipe_stream_all=True), **kw)
        assert ex_b == ex_s
        moved = 0
        for b, s_ in zip(base, strm):
            assert s_["events"] == b["events"] and s_["compute"] == b["compute"] and s_["residents"] == b["residents"]
            assert [(e) for _h, _lane, e in s_["h2d"]] == [(e) for _h, _lane, e in b["h2d"]]     # same copies, same order
            for (_h, lane_b, e), (_h2, lane_s, _e) in zip(b["h2d"], s_["h2d"]):
                assert lane_s == lane_b or (lane_b == "compute" and lane_s == "epipe")
                moved += lane_s != lane_b
            assert len(s_["waits"]) == len(b["waits"]) + sum(
                1 for (_h, lb, _e), (_h2, ls, _e2) in zip(b["h2d"], s_["h2d"]) if lb != ls)
        assert moved > 0, "no copy ever moved to the EPIPE lane"


def test_stream_all_runs_resident_segments_before_it_waits(which="product"):
    """In the product's device trace of a stream-all call the resident segments are launched
    before the compute lane waits for the first streamed copy, and every streamed segment is
    launched after its own wait."""
    cfg = residency_config("epipe", 4, 2, epipe_stream_all=True)
    lay, be, m = product_layer(cfg)
    lay.phase, lay.call_id, lay.stage = "decode", 0, "decode"
    lay.execute([(1, 2), (3, 1)])                        # cold: plain path, still streamed? (no EPIPE trigger)
    be.trace.clear()
    lay.call_id = 1
    name = lay.execute([(1, 1), (2, 2), (3, 1), (5, 1), (7, 3)])
    assert name == "epipe_upfront"
    t = be.trace
    first_wait = min(i for i, x in enumerate(t) if x[0] == "wait")
    for eid in (1, 3):
        assert t.index(("compute", eid)) < first_wait
    for eid in (2, 5, 7):
        assert ("h2d", "epipe", eid) in t
        assert t.index(("h2d", "epipe", eid)) < t.index(("wait", eid)) < t.index(("compute", eid))
    # all three copies are enqueued before the second streamed segment runs (they are back to back on their lane)
    assert t.index(("h2d", "epipe", 5)) < t.index(("compute", 5))


def test_transient_mark_of_prefill_commits_changes_later_evictions():
    """An expert staged during prefill and committed to a free slot is the preferred victim
    (reference :12083-12089 with :3770-3796) until a decode hit clears the mark: with the
    mark switched off the same trace evicts differently."""
    kw = dict(seed=0, prefill_steps=5, capacity=8, T=2)
    marked, _ = run_trace("epipe", "oracle", overrides=dict(epipe_prefill_enable=True), **kw)
    plain, _ = run_trace("epipe", "oracle",
                         overrides=dict(epipe_prefill_enable=True, epipe_prefill_mark_transient=False), **kw)
    assert any(a["events"] != b["events"] for a, b in zip(marked, plain))
    # the mark is set on commits in prefill only, and a decode hit clears it
    lay = RefLayer(0, 16, 2, RefConfig(capacity=4, epipe_enable=True, epipe_prefill_enable=True))
    lay.phase, lay.call_id, lay.stage = "prefill", 0, "prefill"
    lay.execute([(1, 3)])
    assert lay.execute([(1, 2), (2, 2)]) == "epipe_upfront"
    assert lay.cache.prefill_scp_transient_ids() == [2]
    lay.phase, lay.call_id, lay.stage = "decode", 1, "decode"
    lay.execute([(2, 1)])
    assert lay.cache.prefill_scp_transient_ids() == [] and lay.counters["prefill_scp_transient_promote_count"] == 1


POLICY_COSTS = dict(h2d_bytes_per_ms=100.0, h2d_latency_ms=0.1, expert_ms=0.3, item_ms=0.05, next_attention_ms=0.4,
                    split_overhead_ms=0.5)


@pytest.mark.parametrize("method,kw", [
    ("rs", {}), ("rs-epipe", dict(late_rate=0.4)), ("sparse", dict(late_rate=0.3, T=8, capacity=6)),
    ("rs-epipe", dict(late_rate=0.5, capacity=15, E=60, K=4, T=8, top_m=8)),
])
def test_local_policy_through_the_layer_state_machine(method, kw):
    """With the cost-aware policy installed the product still follows the oracle event for
    event, and where the residual scan runs the policy does change decisions (plans or
    residual choices) on these traces."""
    changed = False
    for seed in range(3):
        want, ex_o = run_trace(method, "oracle", seed=seed, policy_costs=POLICY_COSTS, **kw)
        got, ex_p = run_trace(method, "product", seed=seed, policy_costs=POLICY_COSTS, **kw)
        base, ex_b = run_trace(method, "oracle", seed=seed, **kw)
        assert ex_o == ex_p
        for w, g in zip(want, got):
            for key in ("events", "h2d", "compute", "waits", "residents"):
                assert g[key] == w[key], key
        changed = changed or ex_b != ex_o or any(b["h2d"] != w["h2d"] for b, w in zip(base, want))
    # without the residual scan nothing ever reports covered time, and the discount is then 1
    assert changed == (method != "rs"), "the policy changed decisions" if method == "rs" else "never changed one"


def _walk(lay, stage, call, segments):
    lay.phase, lay.call_id, lay.stage = stage, call, stage
    before = len(lay.trace)
    name = lay.execute(segments)
    return name, lay.trace[before:]


def test_buffered_executor_walkthrough():
    """The bounded-buffer pass of the reference (:12514-12843) on a hand-made call: a resident
    expert is counted at once and buffered; the expert whose prefetch is still in flight
    triggers, the buffer runs first, only then the copy is waited for; the miss that follows
    takes the demand path (``late_only`` never stages)."""
    late = {4}
    lay = RefLayer(1, 16, 2, RefConfig(capacity=4, planner_mode="rs_prefetch", epipe_enable=True,
                                       epipe_decode_rs_mode="late_only"),
                   copy_done=lambda eid: eid not in late)
    lay.cache.put(2, ("w", 2))
    lay.cache.admit_prefetch(4, ("w", 4))
    lay.prefetched.add(4)
    lay.events[4] = 1
    name, trace = _walk(lay, "decode", 0, [(2, 3), (4, 1), (9, 2)])
    assert name == "epipe_rs_buffered"
    assert trace == [("hit", 2), ("compute", 2), ("wait", 4), ("prefetch_hit", 4), ("compute", 4),
                     ("miss", 9), ("h2d", "compute", 9), ("compute", 9)]
    # with demand staging the miss is copied on the side lane while the buffer runs
    lay = RefLayer(1, 16, 2, RefConfig(capacity=4, planner_mode="rs_prefetch", epipe_enable=True,
                                       epipe_decode_rs_mode="buffered", epipe_rs_handle_demand_miss=True,
                                       epipe_rs_force_demand_stage=True))
    lay.cache.put(2, ("w", 2))
    lay.cache.put(3, ("w", 3))
    name, trace = _walk(lay, "decode", 0, [(2, 1), (3, 1), (9, 2), (11, 1)])
    assert trace == [("hit", 2), ("hit", 3), ("h2d", "epipe", 9), ("compute", 2), ("compute", 3), ("wait", 9),
                     ("miss", 9), ("compute", 9),
                     # nothing is buffered any more, so the second miss is not staged
                     ("miss", 11), ("h2d", "compute", 11), ("compute", 11)]
    assert lay.cache.resident_ids() == [2, 3, 9, 11]
    # a full buffer runs at once: with max_groups=1 nothing is left to cover a late copy
    lay = RefLayer(1, 16, 2, RefConfig(capacity=4, planner_mode="rs_prefetch", epipe_enable=True,
                                       epipe_decode_rs_mode="late_only", epipe_rs_buffer_max_groups=1),
                   copy_done=lambda eid: eid != 4)
    lay.cache.put(2, ("w", 2))
    lay.cache.admit_prefetch(4, ("w", 4))
    lay.prefetched.add(4)
    lay.events[4] = 1
    _name, trace = _walk(lay, "decode", 0, [(2, 3), (4, 1)])
    assert trace == [("hit", 2), ("compute", 2), ("prefetch_hit", 4), ("wait", 4), ("compute", 4)]


def test_miss_triggered_executor_walkthrough():
    """The look-ahead executor of the reference (:12845-13154): the first miss is staged on
    the side lane while up to ``lookahead`` later resident experts run; a later miss of the
    same call is an ordinary demand miss; with a full cache the staged expert is not kept."""
    cfg = dict(capacity=2, epipe_enable=True, epipe_mode="miss_triggered", epipe_lookahead_min_ready_items=1)
    lay = RefLayer(0, 16, 2, RefConfig(**cfg))
    lay.cache.put(3, ("w", 3))
    lay.cache.put(5, ("w", 5))
    name, trace = _walk(lay, "decode", 0, [(1, 1), (3, 2), (5, 1), (7, 1)])
    assert name == "epipe_miss_triggered"
    assert trace == [("h2d", "epipe", 1), ("hit", 3), ("compute", 3), ("hit", 5), ("compute", 5), ("wait", 1),
                     ("miss", 1), ("compute", 1), ("miss", 7), ("h2d", "compute", 7), ("compute", 7)]
    assert lay.cache.resident_ids() == [5, 7]              # expert 1 was transient, 7 evicted 3
    # look-ahead window of one segment: expert 5 is out of reach, too little work -> demand path
    lay = RefLayer(0, 16, 2, RefConfig(**dict(cfg, epipe_lookahead_experts=1, epipe_lookahead_min_ready_items=3)))
    lay.cache.put(3, ("w", 3))
    lay.cache.put(5, ("w", 5))
    _name, trace = _walk(lay, "decode", 0, [(1, 1), (3, 2), (5, 1)])
    assert trace[:3] == [("miss", 1), ("h2d", "compute", 1), ("compute", 1)]
    # loading expert 1 evicted expert 3 (capacity 2), whose own look-ahead is again too small
    assert trace[3:6] == [("miss", 3), ("h2d", "compute", 3), ("compute", 3)]
    assert lay.counters["epipe_fallback_low_ready_items"] == 2
    # prefill: a free slot commits the staged expert with the transient mark
    lay = RefLayer(0, 16, 2, RefConfig(**dict(cfg, capacity=3, epipe_prefill_enable=True,
                                              epipe_prefill_lookahead_min_ready_items=1)))
    lay.cache.put(3, ("w", 3))
    _name, trace = _walk(lay, "prefill", 0, [(1, 4), (3, 4)])
    assert trace == [("h2d", "epipe", 1), ("hit", 3), ("compute", 3), ("wait", 1), ("miss", 1), ("compute", 1)]
    assert lay.cache.prefill_scp_transient_ids() == [1] and lay.freq[1] == 1


def test_world1_exact_runs_the_plain_loop_whatever_the_epipe_switches_say():
    """The reference's single-process forward never reaches the EPIPE executors
    (utils/eval_core.py:16520-16526); with ``world1_exact`` the product does the same, and its
    events are those of the same method without EPIPE."""
    got, ex = run_trace("rs-epipe", "product", seed=3, late_rate=0.4, overrides=dict(world1_exact=True))
    want, ex_rs = run_trace("rs", "product", seed=3, late_rate=0.4)
    assert set(ex) == {"plain"} == set(ex_rs)
    for g, w in zip(got, want):
        assert g["events"] == w["events"] and g["compute"] == w["compute"] and g["h2d"] == w["h2d"]


def test_decode_rs_mode_spellings():
    from sparse_amd.residency import normalize_decode_rs_mode
    assert [normalize_decode_rs_mode(m) for m in
            (None, "", "Disabled", "late", "demand", "scan", "residual-scan", "buffered_scan", "buffered", "off")] == \
        ["late_only", "late_only", "off", "late_only", "demand_only", "residual_scan", "residual_scan",
         "residual_scan", "buffered", "off"]


def test_invariants_of_every_method():
    for method in METHODS:
        if method.startswith("executor") or method.startswith("scp"):
            continue
        res, _ex = run_trace(method, "oracle", seed=11, steps=40)
        rr, _ = run_trace("rr", "oracle", seed=11, steps=40)
        for l, r in enumerate(res):
            # every routed segment is computed exactly once, whatever the order
            assert sorted(r["compute"]) == sorted(rr[l]["compute"])
            n_miss = sum(1 for k, _ in r["events"] if k == "miss")
            n_demand_h2d = sum(1 for _, lane, _e in r["h2d"] if lane in ("compute", "epipe"))
            assert n_miss == n_demand_h2d                    # one copy per miss, staged experts included
            assert len(r["events"]) == len(r["compute"])     # one cache event per executed segment
    # rr is textbook LRU
    from collections import OrderedDict
    model = OrderedDict()
    lay = RefLayer(0, 16, 2, RefConfig(capacity=4))
    m = RoutingModel(16, 2, 4, 5)
    for step in range(50):
        segs = m.route()
        lay.phase, lay.call_id, lay.stage = "decode", step, "decode"
        before = len(lay.trace)
        lay.execute(segs)
        ev = [t for t in lay.trace[before:] if t[0] in ("hit", "miss")]
        for (kind, eid), (e, _n) in zip(ev, segs):
            assert eid == e and kind == ("hit" if e in model else "miss")
            if e in model:
                model.move_to_end(e)
            else:
                model[e] = 1
                if len(model) > 4:
                    model.popitem(last=False)
        assert lay.cache.resident_ids() == list(model)


def test_method_table_matches_the_reference_launcher():
    # scripts/run/run_case.sh:85-138
    assert METHODS["rr"] == ("none", False, "off", "unique_mask", "round_robin")
    assert METHODS["rs"] == ("rs_prefetch", False, "off", "unique_mask", "round_robin")
    assert METHODS["epipe"] == ("none", True, "off", "sorted_segment", "round_robin")
    assert METHODS["rs-epipe"] == ("rs_prefetch", True, "residual_scan", "sorted_segment", "round_robin")
    assert METHODS["sparse"] == ("rs_prefetch", True, "residual_scan", "sorted_segment", "scp_ep")
    s = method_settings("sparse")
    assert s["kwargs"]["planner_mode"] == "rs_prefetch" and s["kwargs"]["expert_offload"] == "cpu"
    assert s["env"]["SPARSE_EPIPE_RS_FORCE_DEMAND_STAGE"] == "1" and s["env"]["SPARSE_EPIPE_PREFILL_ENABLE"] == "0"
    assert method_settings("rr")["env"]["SPARSE_PREFETCH_ALLOW_ACTIVE_REPLACE"] == "0"
    with pytest.raises(ValueError):
        method_settings("nope")
    cfg = residency_config("rs-epipe", 8, 2)
    assert (cfg.min_candidate_score, cfg.replace_advantage, cfg.replace_margin) == (0.04, 0.08, 1.20)
    assert cfg.recent_protect_steps == 1 and cfg.epipe_decode_rs_mode == "residual_scan"


def test_rolling_gate_skips_after_a_quiet_window():
    for which in ("oracle", "product"):
        cfg = residency_config("rs-epipe", 4, 2)
        if which == "oracle":
            lay = RefLayer(0, 16, 2, to_ref_config(cfg))
        else:
            lay, _be, _m = product_layer(cfg)
        for e in (1, 2, 3):
            lay.cache.put(e, ("w", e) if which == "oracle" else e)
            if which == "product":
                lay._slot_of[e] = e
                lay.backend.slot_content[e] = e
                lay._free_slots.remove(e)
        names = []
        for step in range(30):
            lay.phase, lay.call_id, lay.stage = "decode", step, "decode"
            names.append(lay.execute([(1, 1), (2, 1)]))     # everything resident: never a residual
        assert set(names) == {"plain"}
        skip = lay.gate_skip if which == "oracle" else lay._gate_skip_remaining
        calls = lay.gate_calls if which == "oracle" else lay._gate_calls
        # the 16th call fills the window and is the first of 8 skipped calls (steps 15..22);
        # the remaining 7 calls (steps 23..29) are counted again
        assert (skip, calls) == (0, 7)
