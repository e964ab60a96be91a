"""CPU oracle for the arithmetic of the MoE layer path.  TEST INFRASTRUCTURE ONLY.

This file restates, with PyTorch CPU ops, what louislichen/SPARSE's
``DistributedSparseMoeBlock`` computes on the all-resident path.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import it,
and only as the checker or the timed CPU baseline -- never the product path.

Every function cites the reference lines it follows (paths relative to the reference
checkout, ``utils/eval_core.py`` unless stated).

How each function is pinned (see tests/test_oracle_moe.py):
  routing_router            closed form (fp64 softmax + brute-force top-k on small E),
                            invariants (distinct ids, descending, sum <= 1), the chosen
                            tie rule on hand-made ties.  torch.topk leaves tie order
                            unspecified; the rule here is "higher LOGIT first, then lower
                            expert id" (``topk_by_logit``).  Softmax is monotone, so this is
                            the probability order wherever two probabilities differ; where
                            two distinct logits round to one probability the reference's
                            own order is whatever torch.topk happens to do, and the rule
                            here picks the mathematically larger one.
  deepseek_router           the reference delegates to the model's own ``MoEGate`` (third-party,
                            loaded with trust_remote_code, no version pin, source not in the
                            reference tree), so no reference code exists to run.  Restated
                            from the published DeepSeek-V2 gate (fp32 logits, fp32 softmax,
                            top-k, times routed_scaling_factor) and pinned against the port
                            of that gate in the installed ``transformers``
                            (``DeepseekV2TopkRouter``, ``greedy`` and
                            ``group_limited_greedy`` methods): same experts and weights in
                            fp32 and bf16.
  experts_world1_exact      fp64 per-token closed form sum_k w_k*down(silu(gate x)*up x)
                            (the expected value of the reference's own
                            tests/test_lightweight_policy.py:122-127), permutation
                            invariance, equality with execute_sorted_segments+combine.
  combine_expert_outputs    brute force on tiny inputs, order sensitivity in bf16.
  shared_expert_forward     closed form.
  every function above      bit-for-bit equality on the CPU with vectors recorded from the
                            reference's own functions, taken out of its source and run on
                            small fp32 and bf16 inputs (tests/golden/make_moe_golden.py,
                            tests/test_moe_golden.py).
  rs_routing                closed form on hand-made probabilities (top-k of a known row,
                            renormalised sum, log / -1e9 pseudo logits), brute-force top-k.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

ExpertWeights = Tuple[torch.Tensor, torch.Tensor, torch.Tensor]  # gate [I,H], up [I,H], down [H,I]


def topk_lower_id_first(probs: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k along the last dim, descending, ties resolved to the lower index."""
    order = torch.sort(probs, dim=-1, descending=True, stable=True)
    return order.values[..., :k].contiguous(), order.indices[..., :k].contiguous()


def topk_by_logit(logits: torch.Tensor, probs: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k of ``probs = softmax(logits)`` ranked on the logits: logit descending, ties to the
    lower index; the values are the probabilities of the winners.  ``logits`` may carry -inf
    for entries whose probability was forced to 0."""
    order = torch.sort(logits.to(torch.float32), dim=-1, descending=True, stable=True).indices[..., :k].contiguous()
    return torch.gather(probs, -1, order), order


def routing_router(x: torch.Tensor, gate_w: torch.Tensor, top_k: int, norm_topk_prob: bool = False,
                   router_logits: Optional[torch.Tensor] = None):
    """Qwen-family router, :9519-9520 and :9590-9595.

    ``router_logits = gate(x)`` in x.dtype, fp32 softmax, top-k, optional renorm, cast.
    ``router_logits`` may be supplied to route on given logits (the parity contract is
    "bit-exact indices given identical router logits").
    Returns (topv [T,K] x.dtype, topi [T,K] int64, router_logits [T,E]).
    """
    if router_logits is None:
        router_logits = F.linear(x, gate_w)
    probs = torch.softmax(router_logits, dim=-1, dtype=torch.float32)
    topv, topi = topk_by_logit(router_logits, probs, top_k)
    if norm_topk_prob:
        topv = topv / topv.sum(dim=-1, keepdim=True).clamp_min(1e-12)
    return topv.to(dtype=x.dtype), topi.to(torch.long), router_logits


def group_limited_scores(probs: torch.Tensor, n_group: int, topk_group: int, logits: Optional[torch.Tensor] = None):
    """DeepSeek-V2's ``group_limited_greedy`` mask: experts form ``n_group`` equal runs of ids, a
    group scores its largest probability, the ``topk_group`` best groups (ties to the lower
    group id) keep their probabilities, every other entry becomes 0.  With ``logits`` the
    groups are ranked on their largest logit (the same order, see ``topk_by_logit``) and the
    masked logits (-inf where the probability became 0) are returned as well."""
    T, E = probs.shape
    ranked = probs if logits is None else logits.to(torch.float32)
    group_scores = ranked.view(T, n_group, E // n_group).max(dim=-1).values
    _, keep = topk_lower_id_first(group_scores, topk_group)
    mask = torch.zeros_like(group_scores, dtype=torch.bool)
    mask.scatter_(1, keep, True)
    full = mask.repeat_interleave(E // n_group, dim=1)
    masked = torch.where(full, probs, torch.zeros_like(probs))
    if logits is None:
        return masked
    return masked, torch.where(full, ranked, torch.full_like(ranked, float("-inf")))


def deepseek_router(x: torch.Tensor, gate_w: torch.Tensor, top_k: int, routed_scaling_factor: float = 1.0,
                    router_logits: Optional[torch.Tensor] = None, n_group: int = 1, topk_group: int = 1):
    """DeepSeek-family router as seen at the reference's call site :9503-9517.

    The gate itself is third-party (see the module docstring for what pins this restatement): fp32
    logits from fp32-cast x and W, fp32 softmax, greedy top-k (optionally limited to the best
    groups, the method of the full-size DeepSeek-V2), weights scaled and cast to x.dtype.
    Returns (topv, topi, pseudo_logits) with pseudo_logits built as :9490-9499.
    """
    if router_logits is None:
        router_logits = F.linear(x.to(torch.float32), gate_w.to(torch.float32))
    probs = torch.softmax(router_logits, dim=-1, dtype=torch.float32)
    keys = router_logits.to(torch.float32)
    if n_group > 1 and topk_group < n_group:
        probs, keys = group_limited_scores(probs, n_group, topk_group, logits=keys)
    topv, topi = topk_by_logit(keys, probs, top_k)
    topv = (topv * routed_scaling_factor).to(dtype=x.dtype)
    pseudo = torch.full((x.shape[0], gate_w.shape[0]), float("-inf"), dtype=torch.float32)
    pseudo.scatter_(1, topi, topv.to(torch.float32).clamp_min(1e-12).log())
    return topv, topi.to(torch.long), pseudo


def expert_forward(cur: torch.Tensor, weights: ExpertWeights) -> torch.Tensor:
    """``down(act(gate(cur)) * up(cur))`` with SiLU, :11793-11796 (module layout)."""
    gw, uw, dw = weights
    return F.linear(F.silu(F.linear(cur, gw)) * F.linear(cur, uw), dw)


def experts_world1_exact(x: torch.Tensor, idx: torch.Tensor, w: torch.Tensor,
                         experts: Sequence[ExpertWeights]) -> torch.Tensor:
    """All-resident expert loop, :14690-14721: ascending expert id, rows of an expert in
    (slot, token) order, ``index_add_`` in x.dtype."""
    T, H = x.shape
    E = len(experts)
    final = torch.zeros((T, H), dtype=x.dtype)
    mask = F.one_hot(idx.to(torch.long), num_classes=E).permute(2, 1, 0)
    for e in range(E):
        slot, tok = torch.where(mask[e])
        if tok.numel() == 0:
            continue
        cur = x[None, tok].reshape(-1, H)
        y = expert_forward(cur, experts[e])
        y = y * w[tok, slot, None]
        final.index_add_(0, tok, y.to(x.dtype))
    return final


def combine_expert_outputs(parts: torch.Tensor, expert_ids: torch.Tensor) -> torch.Tensor:
    """Per-token sum of the K slot outputs in ascending expert id, accumulated in the
    activation dtype, :523-538."""
    T, K, H = parts.shape
    if tuple(expert_ids.shape) != (T, K):
        raise ValueError("expert output/ID shape mismatch")
    by_id = torch.argsort(expert_ids, dim=1, stable=True)
    total = parts.new_zeros((T, H))
    tok = torch.arange(T)
    for j in range(K):
        total.add_(parts[tok, by_id[:, j]])
    return total


def execute_sorted_segments(x: torch.Tensor, idx: torch.Tensor, w: torch.Tensor,
                            experts: Sequence[ExpertWeights],
                            order: Optional[Sequence[int]] = None, stable: bool = True) -> torch.Tensor:
    """World-size-1 form of the EP executor: token x K expansion (:14728-14730), sort by
    expert id and contiguous segments (:13240-13262), per-segment SwiGLU times route
    weight (:13340-13357, :11700-11765), un-permute (:13359-13360), then
    ``combine_expert_outputs`` (:14861-14863).  ``order`` optionally gives the expert
    execution order (EPIPE changes the order, never the values).  The sort is the stable
    one by default; the reference's plain ``argsort`` leaves the order of equal ids
    unspecified, and only row order inside a segment depends on it.  ``stable=False`` makes
    the very call the reference makes: on the CPU a row's fp32 result can depend on its
    position inside the segment's matrix product in the last bit, so bit-for-bit comparison
    with vectors recorded from the reference needs the same row order."""
    T, H = x.shape
    K = idx.shape[1]
    expanded = x.unsqueeze(1).expand(-1, K, -1).reshape(-1, H)
    flat_i = idx.reshape(-1).to(torch.long)
    flat_w = w.reshape(-1).to(expanded.dtype)
    perm = torch.argsort(flat_i, stable=True) if stable else torch.argsort(flat_i)
    sorted_i = flat_i[perm]
    hidden_sorted = expanded[perm]
    w_sorted = flat_w[perm]
    out_sorted = torch.zeros_like(hidden_sorted)
    bounds = {}
    n = int(sorted_i.numel())
    start = 0
    while start < n:
        e = int(sorted_i[start])
        end = start
        while end < n and int(sorted_i[end]) == e:
            end += 1
        bounds[e] = (start, end)
        start = end
    for e in (sorted(bounds) if order is None else order):
        s, t = bounds[e]
        y = expert_forward(hidden_sorted[s:t], experts[e])
        out_sorted[s:t] = y * w_sorted[s:t].unsqueeze(1)
    out = torch.zeros_like(expanded)
    out[perm] = out_sorted
    return combine_expert_outputs(out.view(T, K, H), idx)


def shared_expert_forward(x: torch.Tensor, shared: Optional[ExpertWeights],
                          shared_gate_w: Optional[torch.Tensor]) -> torch.Tensor:
    """:9455-9463.  Qwen: ``sigmoid(shared_expert_gate(x)) * shared_expert(x)``; DeepSeek:
    ``shared_experts(x)`` (pass ``shared_gate_w=None``); no shared expert: zeros."""
    if shared is None:
        return torch.zeros_like(x)
    out = expert_forward(x, shared)
    if shared_gate_w is not None:
        out = torch.sigmoid(F.linear(x, shared_gate_w.reshape(1, -1))) * out
    return out


def rs_routing(pred: torch.Tensor, top_k: int, dtype: torch.dtype, norm_topk_prob: bool = False,
               eps: float = 1e-12):
    """Routing replayed from a predictor's probabilities ``pred [T,E]`` instead of the router
    (``expert_source="rs"``): top-k of the prediction (:10971-10983), optional renormalisation,
    weights in the activation dtype, and pseudo logits that hold ``log(clamp(w, eps))`` at the
    chosen experts and -1e9 elsewhere (:11137-11155)."""
    topv, topi = topk_lower_id_first(pred.float(), top_k)
    if norm_topk_prob:
        topv = topv / topv.sum(dim=-1, keepdim=True).clamp_min(1e-12)
    w = topv.to(dtype)
    logits = torch.full((pred.shape[0], pred.shape[1]), -1e9, dtype=torch.float32)
    logits.scatter_(1, topi, torch.log(w.float().clamp_min(eps)))
    return w, topi, logits


def moe_forward_routed(x: torch.Tensor, topv: torch.Tensor, topi: torch.Tensor, experts: Sequence[ExpertWeights],
                       shared: Optional[ExpertWeights] = None,
                       shared_gate_w: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``forward`` with the routing given (:16488, :16520-16526)."""
    return experts_world1_exact(x, topi, topv, experts) + shared_expert_forward(x, shared, shared_gate_w)


def moe_forward(x: torch.Tensor, gate_w: torch.Tensor, experts: Sequence[ExpertWeights], top_k: int,
                shared: Optional[ExpertWeights] = None, shared_gate_w: Optional[torch.Tensor] = None,
                norm_topk_prob: bool = False, family: str = "qwen_shared",
                router_logits: Optional[torch.Tensor] = None):
    """``forward`` at world size 1, :16488 and :16520-16526: route, expert loop, shared
    expert, sum.  Returns (out [T,H], topv, topi, router_logits)."""
    if family == "deepseek_shared":
        topv, topi, logits = deepseek_router(x, gate_w, top_k, router_logits=router_logits)
    else:
        topv, topi, logits = routing_router(x, gate_w, top_k, norm_topk_prob, router_logits=router_logits)
    expert_out = experts_world1_exact(x, topi, topv, experts)
    shared_out = shared_expert_forward(x, shared, shared_gate_w)
    return expert_out + shared_out, topv, topi, logits
