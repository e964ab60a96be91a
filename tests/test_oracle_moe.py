"""Pins the arithmetic oracle (``oracle/ref_moe.py``, ``oracle/ref_permute.py``) with
closed forms, brute force, invariants and special cases, so that a dropped term, a wrong
sign or index or a transposed operand fails here rather than hiding in a GPU comparison."""
import itertools

import numpy as np
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import ref_moe, ref_permute
from tests.helpers import make_hidden, make_layer


def test_router_closed_form_and_invariants():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(40, 32, generator=g)
    w = torch.randn(12, 32, generator=g) * 0.3
    topv, topi, logits = ref_moe.routing_router(x, w, 4)
    # fp64 restatement of softmax(x W^T) and a brute-force top-k
    l64 = x.double() @ w.double().T
    p64 = torch.exp(l64 - l64.max(1, keepdim=True).values)
    p64 = p64 / p64.sum(1, keepdim=True)
    for t in range(40):
        best = sorted(range(12), key=lambda e: (-p64[t, e].item(), e))[:4]
        assert topi[t].tolist() == best
        assert torch.allclose(topv[t].double(), p64[t, best], rtol=1e-5)
    torch.testing.assert_close(logits.double(), l64, rtol=1e-5, atol=1e-6)
    assert (topv[:, :-1] >= topv[:, 1:]).all() and (topv.sum(1) <= 1 + 1e-6).all()
    assert all(len(set(r.tolist())) == 4 for r in topi)
    assert topi.dtype == torch.int64
    # renormalisation
    tv2, ti2, _ = ref_moe.routing_router(x, w, 4, norm_topk_prob=True)
    assert torch.equal(ti2, topi)
    torch.testing.assert_close(tv2.sum(1), torch.ones(40))
    torch.testing.assert_close(tv2, topv / topv.sum(1, keepdim=True))
    # weights are cast to the activation dtype, logits stay in it
    xb, wb = x.to(torch.bfloat16), w.to(torch.bfloat16)
    tvb, _tib, lb = ref_moe.routing_router(xb, wb, 4)
    assert tvb.dtype == torch.bfloat16 and lb.dtype == torch.bfloat16


def test_router_tie_rule():
    logits = torch.zeros(3, 8)
    logits[1, [6, 2]] = 1.0
    logits[2, 7] = 3.0
    _v, topi, _ = ref_moe.routing_router(torch.zeros(3, 4), torch.zeros(8, 4), 3, router_logits=logits)
    assert topi.tolist() == [[0, 1, 2], [2, 6, 0], [7, 0, 1]]


def test_ranking_on_logits_is_the_probability_ranking_wherever_probabilities_differ():
    """``topk_by_logit`` against the plain top-k of the probabilities (what the reference
    computes): identical indices and values on every row whose k+1 largest probabilities are
    distinct or come from equal logits -- softmax is monotone."""
    g = torch.Generator().manual_seed(3)
    for dtype in (torch.float32, torch.bfloat16):
        logits = (torch.randn(2000, 60, generator=g) * 2.0).to(dtype)
        probs = torch.softmax(logits, dim=-1, dtype=torch.float32)
        v1, i1 = ref_moe.topk_by_logit(logits, probs, 4)
        v2, i2 = ref_moe.topk_lower_id_first(probs, 4)
        top5 = torch.sort(probs, dim=-1, descending=True).values[:, :5]
        lt5 = torch.sort(logits.float(), dim=-1, descending=True).values[:, :5]
        clear = ((top5[:, :-1] != top5[:, 1:]) | (lt5[:, :-1] == lt5[:, 1:])).all(dim=1)
        assert clear.float().mean() > 0.99
        assert torch.equal(i1[clear], i2[clear]) and torch.equal(v1[clear], v2[clear])
        tv, ti = torch.topk(probs, 4, dim=-1)                 # the reference's call
        assert torch.equal(v1, tv)                            # values never depend on the tie order
        distinct = (top5[:, :-1] != top5[:, 1:]).all(dim=1)   # torch.topk leaves equal values in any order
        assert torch.equal(i1[distinct], ti[distinct])


def test_ranking_on_logits_when_two_logits_collapse_to_one_probability():
    """Two logits one ulp apart close to the maximum round to the same probability; the rule
    still prefers the larger logit, whichever id it has, and the selected set is a valid top-k
    of the probabilities either way."""
    lo = torch.tensor(-0.1)
    logits = torch.stack([torch.tensor(0.0), torch.nextafter(lo, torch.tensor(-100.0)), lo]).view(1, 3)
    probs = torch.softmax(logits, dim=-1)
    assert probs[0, 1] == probs[0, 2]                         # collapsed
    v, i = ref_moe.topk_by_logit(logits, probs, 2)
    assert i.tolist() == [[0, 2]]
    assert ref_moe.topk_lower_id_first(probs, 2)[1].tolist() == [[0, 1]]
    assert torch.equal(v, torch.topk(probs, 2).values)


def test_deepseek_router_is_fp32_and_builds_pseudo_logits():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(10, 16, generator=g)).to(torch.bfloat16)
    w = (torch.randn(8, 16, generator=g) * 0.5).to(torch.bfloat16)
    topv, topi, pseudo = ref_moe.deepseek_router(x, w, 3)
    l32 = x.float() @ w.float().T
    p = torch.softmax(l32, -1)
    want_v, want_i = ref_moe.topk_lower_id_first(p, 3)
    assert torch.equal(topi, want_i) and topv.dtype == torch.bfloat16
    assert torch.equal(topv, want_v.to(torch.bfloat16))
    assert pseudo.dtype == torch.float32 and torch.isinf(pseudo).sum() == 10 * 5
    torch.testing.assert_close(torch.gather(pseudo, 1, topi), topv.float().log())


def _closed_form(x, topi, topv, experts, shared=None, sgw=None):
    """fp64 per-token restatement: sum_k w_k down(silu(gate x) * up x) (+ shared expert)."""
    out = torch.zeros(x.shape, dtype=torch.float64)
    for t in range(x.shape[0]):
        xt = x[t].double()
        for k in range(topi.shape[1]):
            gw, uw, dw = (m.double() for m in experts[int(topi[t, k])])
            h = F.silu(gw @ xt) * (uw @ xt)
            out[t] += (dw @ h) * topv[t, k].double()
        if shared is not None:
            gw, uw, dw = (m.double() for m in shared)
            s = dw @ (F.silu(gw @ xt) * (uw @ xt))
            if sgw is not None:
                s = torch.sigmoid(sgw.double() @ xt) * s
            out[t] += s
    return out


def test_expert_loop_closed_form_fp32():
    layer = make_layer(64, 6, 32, 2, Is=48, shared_gate=True, seed=2, std=0.2)
    x = make_hidden(9, 64, seed=3)
    out, topv, topi, _ = ref_moe.moe_forward(x, layer["gate_w"], layer["experts"], 2, layer["shared"],
                                             layer["shared_gate_w"])
    want = _closed_form(x, topi, topv, layer["experts"], layer["shared"], layer["shared_gate_w"])
    torch.testing.assert_close(out.double(), want, rtol=1e-4, atol=1e-5)
    # without the shared gate / without a shared expert
    out2, tv2, ti2, _ = ref_moe.moe_forward(x, layer["gate_w"], layer["experts"], 2, layer["shared"], None,
                                            family="deepseek_shared")
    torch.testing.assert_close(out2.double(), _closed_form(x, ti2, tv2, layer["experts"], layer["shared"]),
                               rtol=1e-4, atol=1e-5)
    out3, tv3, ti3, _ = ref_moe.moe_forward(x, layer["gate_w"], layer["experts"], 2)
    torch.testing.assert_close(out3.double(), _closed_form(x, ti3, tv3, layer["experts"]), rtol=1e-4, atol=1e-5)
    # a transposed operand or a swapped gate/up would not survive: silu is not symmetric
    swapped = [(u, g, d) for g, u, d in layer["experts"]]
    bad = ref_moe.experts_world1_exact(x, ti3, tv3, swapped)
    assert not torch.allclose(bad, out3, rtol=1e-2, atol=1e-3)


def test_expert_loop_invariances():
    layer = make_layer(64, 8, 32, 3, seed=4, std=0.2)
    x = make_hidden(17, 64, seed=5)
    topv, topi, _ = ref_moe.routing_router(x, layer["gate_w"], 3)
    base = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    # token permutation commutes
    p = torch.randperm(17, generator=torch.Generator().manual_seed(6))
    torch.testing.assert_close(ref_moe.experts_world1_exact(x[p], topi[p], topv[p], layer["experts"]), base[p],
                               rtol=1e-6, atol=1e-7)
    # linear in the route weights
    torch.testing.assert_close(ref_moe.experts_world1_exact(x, topi, 2 * topv, layer["experts"]), 2 * base,
                               rtol=1e-6, atol=1e-7)
    # the sorted-segment executor + combine is the same function, in any execution order
    seg = ref_moe.execute_sorted_segments(x, topi, topv, layer["experts"])
    torch.testing.assert_close(seg, base, rtol=1e-6, atol=1e-7)
    active = sorted(set(topi.reshape(-1).tolist()))
    rev = ref_moe.execute_sorted_segments(x, topi, topv, layer["experts"], order=list(reversed(active)))
    assert torch.equal(rev, seg)


def test_bf16_rounding_points_of_the_expert_loop():
    """In bf16 every Linear output, the activation, the product and the weighted result are
    rounded; the exact-loop and the segment executor then agree bit for bit, because both
    add the same bf16 terms in ascending expert id."""
    layer = make_layer(64, 8, 32, 3, dtype=torch.bfloat16, seed=7, std=0.2)
    x = make_hidden(11, 64, torch.bfloat16, seed=8)
    topv, topi, _ = ref_moe.routing_router(x, layer["gate_w"], 3)
    a = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    b = ref_moe.execute_sorted_segments(x, topi, topv, layer["experts"])
    assert a.dtype == torch.bfloat16 and torch.equal(a, b)
    # one token, by hand
    t = 0
    acc = torch.zeros(64, dtype=torch.bfloat16)
    for e in sorted(topi[t].tolist()):
        k = topi[t].tolist().index(e)
        gw, uw, dw = layer["experts"][e]
        xt = x[t:t + 1]
        g = F.linear(xt, gw)
        u = F.linear(xt, uw)
        h = F.silu(g) * u
        y = F.linear(h, dw) * topv[t, k]
        acc = acc + y[0]
    assert torch.equal(acc, a[t])


def test_combine_is_an_ordered_sum_in_the_activation_dtype():
    parts = torch.tensor([[[1.0], [256.0], [-256.0]]], dtype=torch.bfloat16)   # 1 token, 3 slots
    for ids, want in (([[0, 1, 2]], 0.0), ([[1, 2, 0]], 1.0), ([[2, 0, 1]], 1.0)):
        # ascending expert id decides the order: (1+256)-256 = 0 in bf16 but (256-256)+1 = 1
        got = ref_moe.combine_expert_outputs(parts, torch.tensor(ids))
        assert got.item() == want
    # brute force
    g = torch.Generator().manual_seed(9)
    parts = torch.randn(5, 4, 3, generator=g)
    ids = torch.stack([torch.randperm(10, generator=g)[:4] for _ in range(5)])
    got = ref_moe.combine_expert_outputs(parts, ids)
    for t in range(5):
        acc = torch.zeros(3)
        for k in sorted(range(4), key=lambda k: ids[t, k].item()):
            acc = acc + parts[t, k]
        assert torch.equal(acc, got[t])
    with pytest.raises(ValueError):
        ref_moe.combine_expert_outputs(parts, ids[:, :3])


def test_shared_expert_special_cases():
    layer = make_layer(32, 2, 16, 1, Is=24, shared_gate=True, seed=10, std=0.3)
    x = make_hidden(4, 32, seed=11)
    assert torch.equal(ref_moe.shared_expert_forward(x, None, None), torch.zeros_like(x))
    plain = ref_moe.shared_expert_forward(x, layer["shared"], None)
    torch.testing.assert_close(plain, ref_moe.expert_forward(x, layer["shared"]))
    # a zero gate vector gives sigmoid(0) = 1/2
    half = ref_moe.shared_expert_forward(x, layer["shared"], torch.zeros(32))
    torch.testing.assert_close(half, 0.5 * plain)


# ----------------------------------------------------------------------------- permutation
def _brute_perm(flat, E):
    n = len(flat)
    pos = [sum(1 for g in range(n) if (flat[g], g) < (flat[f], f)) for f in range(n)]
    perm = [0] * n
    for f, p in enumerate(pos):
        perm[p] = f
    return perm, pos


def test_permute_brute_force_and_invariants():
    rng = np.random.default_rng(0)
    for T, K, E in [(1, 4, 60), (8, 4, 60), (7, 3, 5), (40, 6, 64)]:
        topi = np.stack([rng.permutation(E)[:K] for _ in range(T)])
        perm, inv, off, active = ref_permute.permute_build(topi, E)
        bp, binv = _brute_perm(topi.reshape(-1).tolist(), E)
        assert perm.tolist() == bp and inv.tolist() == binv
        assert sorted(perm.tolist()) == list(range(T * K))
        assert (inv[perm] == np.arange(T * K)).all()
        s = topi.reshape(-1)[perm]
        assert (np.diff(s) >= 0).all()
        counts = np.bincount(topi.reshape(-1), minlength=E)
        assert off.tolist() == [0] + np.cumsum(counts).tolist()
        assert active.tolist() == [e for e in range(E) if counts[e]]
        # inside a segment the items are in ascending flat index (token-major)
        for e, a, b in ref_permute.segments(topi, E):
            assert (np.diff(perm[a:b]) > 0).all() and (s[a:b] == e).all()
    # the permutation is what the segment executor of the arithmetic oracle uses
    topi = torch.tensor([[3, 1], [1, 0], [3, 2]])
    perm, _, _, _ = ref_permute.permute_build(topi.numpy(), 4)
    assert perm.tolist() == torch.argsort(topi.reshape(-1), stable=True).tolist()


def test_rs_routing_closed_form():
    """Routing replayed from predictor probabilities: a hand-made row and brute force."""
    pred = torch.tensor([[.05, .4, .1, .3, .15], [.2, .2, .5, .05, .05]])
    w, idx, logits = ref_moe.rs_routing(pred, 2, torch.float32)
    assert idx.tolist() == [[1, 3], [2, 0]]                       # tie between experts 0 and 1: lower id
    torch.testing.assert_close(w, torch.tensor([[.4, .3], [.5, .2]]))
    assert logits[0, 1].item() == pytest.approx(math.log(.4), rel=1e-6)
    assert logits[0, 0].item() == -1e9 and logits.dtype == torch.float32
    w, _, _ = ref_moe.rs_routing(pred, 2, torch.float32, norm_topk_prob=True)
    torch.testing.assert_close(w, torch.tensor([[.4 / .7, .3 / .7], [.5 / .7, .2 / .7]]))
    wb, _, lb = ref_moe.rs_routing(pred, 2, torch.bfloat16)
    assert wb.dtype == torch.bfloat16
    assert lb[0, 3].item() == pytest.approx(math.log(float(torch.tensor(.3).bfloat16())), rel=1e-6)
    # a zero probability is clamped before the log
    _, _, lz = ref_moe.rs_routing(torch.tensor([[1., 0., 0.]]), 2, torch.float32, eps=1e-12)
    assert lz[0, 1].item() == pytest.approx(math.log(1e-12), rel=1e-6)
    g = torch.Generator().manual_seed(3)
    pred = torch.softmax(torch.randn(20, 9, generator=g), -1)
    w, idx, _ = ref_moe.rs_routing(pred, 3, torch.float32)
    for t in range(20):
        want = sorted(range(9), key=lambda e: (-pred[t, e].item(), e))[:3]
        assert idx[t].tolist() == want
    # given routing: same as routing by a gate that produces those logits
    H, E, I = 16, 6, 8
    x = torch.randn(5, H, generator=g)
    experts = [(torch.randn(I, H, generator=g) * .1, torch.randn(I, H, generator=g) * .1,
                torch.randn(H, I, generator=g) * .1) for _ in range(E)]
    gate_w = torch.randn(E, H, generator=g)
    out, topv, topi, _ = ref_moe.moe_forward(x, gate_w, experts, 2)
    torch.testing.assert_close(ref_moe.moe_forward_routed(x, topv, topi, experts), out)


def test_deepseek_router_against_the_transformers_port_of_the_gate():
    """The reference delegates DeepSeek routing to the checkpoint's own gate, which is not in
    its tree.  The installed ``transformers`` carries a port of that gate
    (``DeepseekV2TopkRouter``); with the ``greedy`` method DeepSeek-V2-Lite uses, the oracle
    must choose the same experts with the same weights."""
    transformers = pytest.importorskip("transformers")
    try:
        from transformers import DeepseekV2Config
        from transformers.models.deepseek_v2.modeling_deepseek_v2 import DeepseekV2TopkRouter
    except ImportError:
        pytest.skip("this transformers has no DeepSeek-V2")
    g = torch.Generator().manual_seed(11)
    for dtype, scale in ((torch.float32, 1.0), (torch.bfloat16, 1.0), (torch.float32, 2.5)):
        cfg = DeepseekV2Config(hidden_size=64, n_routed_experts=16, num_experts_per_tok=6, topk_method="greedy",
                               routed_scaling_factor=scale, num_hidden_layers=1, vocab_size=32)
        gate = DeepseekV2TopkRouter(cfg)
        gate.weight.data = (torch.randn(16, 64, generator=g) * 0.3)
        x = torch.randn(40, 64, generator=g).to(dtype)
        gate = gate.to(dtype)
        with torch.no_grad():
            logits, weights, idx = gate(x)
        topv, topi, pseudo = ref_moe.deepseek_router(x, gate.weight.data, 6, routed_scaling_factor=scale)
        # the third output is the reference's pseudo logits: log(weight) at the chosen experts
        assert torch.isinf(pseudo).sum() == 40 * (16 - 6)
        order_ref, order_hf = torch.sort(topi, 1), torch.sort(idx, 1)
        assert torch.equal(order_ref.values, order_hf.values)
        # the reference casts the gate's weights to the activation dtype at its call site (:9514)
        torch.testing.assert_close(torch.gather(topv.float(), 1, order_ref.indices),
                                   torch.gather(weights.to(dtype).float(), 1, order_hf.indices), rtol=1e-6, atol=1e-7)


def test_deepseek_group_limited_router_against_the_transformers_port():
    """The ``group_limited_greedy`` method of the full-size DeepSeek-V2 gate (experts in equal
    groups, only the best groups compete): same experts and weights as the transformers port,
    a hand-made case where the limit changes the answer, and the degenerate settings that
    must reduce to plain top-k."""
    pytest.importorskip("transformers")
    try:
        from transformers import DeepseekV2Config
        from transformers.models.deepseek_v2.modeling_deepseek_v2 import DeepseekV2TopkRouter
    except ImportError:
        pytest.skip("this transformers has no DeepSeek-V2")
    g = torch.Generator().manual_seed(12)
    for dtype, scale, E, ng, kg, K in ((torch.float32, 1.0, 16, 4, 2, 6), (torch.bfloat16, 16.0, 32, 8, 3, 6),
                                       (torch.float32, 1.0, 160, 8, 3, 6)):
        cfg = DeepseekV2Config(hidden_size=64, n_routed_experts=E, num_experts_per_tok=K,
                               topk_method="group_limited_greedy", n_group=ng, topk_group=kg,
                               routed_scaling_factor=scale, num_hidden_layers=1, vocab_size=32)
        gate = DeepseekV2TopkRouter(cfg)
        gate.weight.data = (torch.randn(E, 64, generator=g) * 0.3)
        x = torch.randn(50, 64, generator=g).to(dtype)
        gate = gate.to(dtype)
        with torch.no_grad():
            _, weights, idx = gate(x)
        topv, topi, _ = ref_moe.deepseek_router(x, gate.weight.data, K, routed_scaling_factor=scale,
                                                n_group=ng, topk_group=kg)
        order_ref, order_hf = torch.sort(topi, 1), torch.sort(idx, 1)
        assert torch.equal(order_ref.values, order_hf.values)
        torch.testing.assert_close(torch.gather(topv.float(), 1, order_ref.indices),
                                   torch.gather(weights.to(dtype).float(), 1, order_hf.indices), rtol=1e-6, atol=1e-7)
        # every chosen expert sits in one of kg groups
        assert (torch.div(topi, E // ng, rounding_mode="floor").sort(1).values.diff(dim=1) != 0).sum(1).max() < kg
        plain = ref_moe.deepseek_router(x, gate.weight.data, K, routed_scaling_factor=scale)
        assert not torch.equal(torch.sort(plain[1], 1).values, order_ref.values)      # the limit matters here
        for ng2, kg2 in ((1, 1), (ng, ng)):
            same = ref_moe.deepseek_router(x, gate.weight.data, K, routed_scaling_factor=scale, n_group=ng2,
                                           topk_group=kg2)
            assert torch.equal(same[1], plain[1]) and torch.equal(same[0], plain[0])
    # by hand: 2 groups of 3, one group allowed, K=2: the runner-up overall (id 3) is outside the best group
    probs = torch.tensor([[0.30, 0.05, 0.10, 0.28, 0.02, 0.25]])
    masked = ref_moe.group_limited_scores(probs, 2, 1)
    assert torch.equal(masked, torch.tensor([[0.30, 0.05, 0.10, 0.0, 0.0, 0.0]]))
    assert ref_moe.topk_lower_id_first(masked, 2)[1].tolist() == [[0, 2]]
    # equal group scores: the lower group wins
    tie = torch.tensor([[0.25, 0.0, 0.25, 0.0]])
    assert ref_moe.group_limited_scores(tie, 2, 1).tolist() == [[0.25, 0.0, 0.0, 0.0]]
