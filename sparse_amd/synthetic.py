"""Seeded synthetic MoE layers in the shapes the benchmarks name.

There are no checkpoints to load, so layers are random-init: weights ~N(0, 0.02) from a
per-layer seed, hidden states ~N(0, 1).  ``make_mlp_block`` returns the duck-typed
``mlp_block`` the block constructor takes (``.gate``, ``.experts``, and
``.shared_expert`` + ``.shared_expert_gate`` or ``.shared_experts``), the same surface the
reference reads from a Hugging Face MoE module (utils/eval_core.py:4342-4362).
"""
from __future__ import annotations

from types import SimpleNamespace as NS
from typing import Optional

import torch
import torch.nn.functional as F

# Qwen1.5-MoE-A2.7B-shaped and DeepSeek-V2-Lite-shaped MoE layers
QWEN = dict(family="qwen_shared", hidden=2048, num_experts=60, inter=1408, top_k=4, shared_inter=5632,
            num_layers=24)
DEEPSEEK = dict(family="deepseek_shared", hidden=2048, num_experts=64, inter=1408, top_k=6, shared_inter=2816,
                num_layers=26)


def _mlp(gate_w, up_w, down_w):
    return NS(gate_proj=NS(weight=gate_w), up_proj=NS(weight=up_w), down_proj=NS(weight=down_w), act_fn=F.silu)


def make_mlp_block(shape: dict, dtype: torch.dtype = torch.bfloat16, seed: int = 0, device="cpu",
                   std: float = 0.02, fused: bool = False):
    """One seeded layer.  Drawn in fp32 from a generator on ``device`` and cast to
    ``dtype``; the same (seed, device type) always gives the same layer."""
    H, E, I, Is = shape["hidden"], shape["num_experts"], shape["inter"], shape.get("shared_inter", 0)
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(int(seed))

    def w(*dims):
        return (torch.randn(*dims, generator=g, device=dev, dtype=torch.float32) * std).to(dtype)

    block = NS(norm_topk_prob=False)
    block.gate = NS(weight=w(E, H))
    if fused:
        block.experts = NS(gate_up_proj=w(E, 2 * I, H), down_proj=w(E, H, I), act_fn=F.silu)
    else:
        block.experts = [_mlp(w(I, H), w(I, H), w(H, I)) for _ in range(E)]
    if Is:
        shared = _mlp(w(Is, H), w(Is, H), w(H, Is))
        if shape.get("family", "qwen_shared") == "qwen_shared":
            block.shared_expert = shared
            block.shared_expert_gate = NS(weight=w(1, H))
        else:
            block.shared_experts = shared
    return block


def make_hidden(tokens: int, hidden: int, dtype: torch.dtype = torch.bfloat16, seed: int = 1000, device="cpu"):
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(int(seed))
    return torch.randn(tokens, hidden, generator=g, device=dev, dtype=torch.float32).to(dtype)


# ---- skewed, co-activating routing -------------------------------------------------
# The router is a bias-free Linear, so structure is put into the data: a few reserved
# hidden dimensions carry control values and the matching gate columns turn them into logit
# offsets.  Dimension 0 holds a constant and gate column 0 the per-expert popularity bias;
# dimension 1+c is raised for tokens that activate cluster c and gate column 1+c lifts the
# experts of that cluster together.
ROUTING_CONST = 4.0


def routing_structure(num_experts: int, seed: int = 0, s: float = 1.1, cluster: int = 4):
    """(bias[E], clusters[C][cluster], cluster_prob[C]) for one layer: popularity Zipf(s)
    over a seeded permutation; consecutive popularity ranks form a cluster."""
    g = torch.Generator().manual_seed(int(seed))
    order = torch.randperm(num_experts, generator=g)          # order[r] = expert of rank r+1
    rank = torch.empty(num_experts, dtype=torch.float32)
    rank[order] = torch.arange(1, num_experts + 1, dtype=torch.float32)
    bias = (-s) * torch.log(rank)
    n_clusters = num_experts // cluster
    clusters = order[: n_clusters * cluster].reshape(n_clusters, cluster)
    weight = torch.exp(bias)[clusters].sum(dim=1)
    return bias, clusters, weight / weight.sum()


def add_routing_structure(mlp_block, num_experts: int, seed: int = 0, s: float = 1.1, cluster: int = 4,
                          boost: float = 5.0):
    """Write the popularity bias and the cluster columns into ``mlp_block.gate.weight`` (in
    place) and return the structure for ``make_structured_hidden``."""
    bias, clusters, prob = routing_structure(num_experts, seed, s, cluster)
    w = mlp_block.gate.weight
    n_clusters = clusters.shape[0]
    if w.shape[1] < 1 + n_clusters:
        raise ValueError("hidden size too small for the reserved routing dimensions")
    w[:, : 1 + n_clusters] = 0
    w[:, 0] = (bias / ROUTING_CONST).to(w.dtype).to(w.device)
    for c in range(n_clusters):
        w[clusters[c].to(w.device), 1 + c] = boost / ROUTING_CONST
    return dict(bias=bias, clusters=clusters, cluster_prob=prob)


def make_structured_hidden(tokens: int, hidden: int, n_clusters: int, cluster_prob: torch.Tensor,
                           dtype: torch.dtype = torch.bfloat16, seed: int = 1000, device="cpu", p: float = 0.6):
    """Hidden states ~N(0,1) whose reserved dimensions say which cluster (if any, with
    probability ``p``) each token activates.  All layers of a synthetic stack read the same
    hidden state, so one cluster draw per token serves every layer's own cluster table."""
    x = make_hidden(tokens, hidden, torch.float32, seed, device)
    g = torch.Generator().manual_seed(int(seed) + 77)
    active = torch.rand(tokens, generator=g) < p
    which = torch.multinomial(cluster_prob, tokens, replacement=True, generator=g)
    ctrl = torch.zeros(tokens, 1 + n_clusters)
    ctrl[:, 0] = ROUTING_CONST
    ctrl[torch.arange(tokens)[active], 1 + which[active]] = ROUTING_CONST
    x[:, : 1 + n_clusters] = ctrl.to(x.device)
    return x.to(dtype)
