"""CPU tests of the synthetic workloads the benchmarks use: skewed co-activating routing
and the predictor bank that reproduces a router."""
import torch

from sparse_amd.rs import informed_bank
from sparse_amd.synthetic import (QWEN, add_routing_structure, make_mlp_block, make_structured_hidden,
                                  routing_structure)


def _routed(shape, seed, tokens):
    mlp = make_mlp_block(shape, dtype=torch.float32, seed=seed)
    st = add_routing_structure(mlp, shape["num_experts"], seed=seed)
    x = make_structured_hidden(tokens, shape["hidden"], shape["num_experts"] // 4, st["cluster_prob"],
                               torch.float32, seed=5)
    logits = x @ mlp.gate.weight.T
    top = torch.topk(torch.softmax(logits, -1), shape["top_k"]).indices
    return mlp, st, x, top


def test_popularity_is_skewed_and_clusters_are_co_selected():
    shape = dict(QWEN, hidden=256, inter=64, shared_inter=64)
    _mlp, st, _x, top = _routed(shape, 3, 4096)
    counts = torch.bincount(top.reshape(-1), minlength=shape["num_experts"]).float()
    by_rank = counts[torch.argsort(st["bias"], descending=True)]
    # Zipf: the most popular quarter of the experts takes most of the traffic
    assert by_rank[:15].sum() / counts.sum() > 0.6
    assert by_rank[:15].mean() > 4 * by_rank[-15:].mean()
    clusters = [set(c.tolist()) for c in st["clusters"]]
    whole = sum(1 for row in top.tolist() if set(row) in clusters) / top.shape[0]
    assert whole > 0.4   # 60 % of the tokens activate one cluster (more coincide by popularity alone)


def test_structure_is_seeded_and_cluster_probabilities_depend_on_rank_only():
    a = routing_structure(60, seed=1)
    b = routing_structure(60, seed=1)
    c = routing_structure(60, seed=2)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert not torch.equal(a[1], c[1])
    torch.testing.assert_close(a[2], c[2])
    assert abs(float(a[2].sum()) - 1.0) < 1e-6


def test_informed_bank_reproduces_the_router():
    shape = dict(QWEN, hidden=256, inter=64, shared_inter=64)
    mlp, _st, x, top = _routed(shape, 4, 256)
    bank = informed_bank([None, mlp.gate.weight], hidden_dim=512)
    assert bank[0] is None
    probs = bank[1](x)
    want = torch.softmax(x @ mlp.gate.weight.T, -1)
    torch.testing.assert_close(probs, want, rtol=1e-3, atol=1e-6)
    pred = torch.topk(probs, shape["top_k"]).indices
    assert torch.equal(pred.sort(-1).values, top.sort(-1).values)
