"""CPU oracle of the RS predictor and of candidate selection.  TEST INFRASTRUCTURE ONLY:
only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may
import this.

``routing_scout_forward`` restates ``RoutingScoutMLP.forward`` in eval mode
(utils/eval_core.py:3402-3417: Linear, BatchNorm1d with running statistics, ReLU, Dropout
as identity, Linear, Softmax) in numpy float32.  Pinned by closed form against
``torch.nn`` layers with the same parameters (tests/test_residency.py).

``routing_scout_residual_forward`` restates ``RoutingScoutResidualMLP.forward`` in eval mode
(utils/eval_core.py:3419-3461: LayerNorm, Linear, GELU; units ``x + Linear(GELU(Linear(LayerNorm(x))))``;
LayerNorm, Linear, softmax) in numpy float32.  Pinned against ``torch.nn.LayerNorm`` / ``nn.GELU`` /
``nn.Linear`` stacks holding the same parameters, and by hand-made cases (a unit whose second Linear is
zero is the identity; constant rows normalise to the LayerNorm's bias) in tests/test_rs_fused.py.

``select_candidates`` restates utils/rs_staging.py:97-118, the staging adapter's scoring
(the same formula as utils/eval_core.py:10104-10106).  Pinned by the reference's own
known-answer tests, tests/test_rs_staging.py:147-150 and :308-312.

``router_topk_feature`` restates utils/eval_core.py:10903-10908, the extra predictor input of
``feature_mode="hidden_router_topk"``.  Pinned by vectors recorded from the reference's own
method (tests/golden/make_rs_golden.py, tests/test_rs_golden.py) and by hand-made rows.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Sequence, Set

import numpy as np


def routing_scout_forward(x: np.ndarray, w1, b1, bn_weight, bn_bias, bn_mean, bn_var, w2, b2,
                          eps: float = 1e-5) -> np.ndarray:
    h = x.astype(np.float32) @ np.asarray(w1, np.float32).T + np.asarray(b1, np.float32)
    h = (h - bn_mean) / np.sqrt(np.asarray(bn_var, np.float32) + eps) * bn_weight + bn_bias
    h = np.maximum(h, 0.0)
    z = h @ np.asarray(w2, np.float32).T + np.asarray(b2, np.float32)
    z = z - z.max(axis=-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)


def _layer_norm(x: np.ndarray, weight, bias, eps: float) -> np.ndarray:
    mean = x.mean(axis=-1, keepdims=True, dtype=np.float32)
    var = np.square(x - mean).mean(axis=-1, keepdims=True, dtype=np.float32)      # biased, as nn.LayerNorm
    return ((x - mean) / np.sqrt(var + np.float32(eps)) * np.asarray(weight, np.float32)
            + np.asarray(bias, np.float32)).astype(np.float32)


def _gelu(x: np.ndarray) -> np.ndarray:
    from scipy.special import erf
    return (0.5 * x * (1.0 + erf(x.astype(np.float64) / np.sqrt(2.0)))).astype(np.float32)    # nn.GELU's default


def _linear(x: np.ndarray, weight, bias) -> np.ndarray:
    return (x @ np.asarray(weight, np.float32).T + np.asarray(bias, np.float32)).astype(np.float32)


def routing_scout_residual_forward(x: np.ndarray, stem, units, out_norm, head, eps: float = 1e-5) -> np.ndarray:
    """``stem = (ln_weight, ln_bias, w, b)``; ``units`` = list of ``(ln_weight, ln_bias, w_up, b_up, w_down,
    b_down)``; ``out_norm = (ln_weight, ln_bias)``; ``head = (w, b)``.  Returns ``[T, E]`` probabilities."""
    h = np.asarray(x, np.float32)
    h = _gelu(_linear(_layer_norm(h, stem[0], stem[1], eps), stem[2], stem[3]))
    for ln_w, ln_b, w_up, b_up, w_down, b_down in units:
        h = (h + _linear(_gelu(_linear(_layer_norm(h, ln_w, ln_b, eps), w_up, b_up)), w_down, b_down)).astype(np.float32)
    z = _linear(_layer_norm(h, out_norm[0], out_norm[1], eps), head[0], head[1])
    z = z - z.max(axis=-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)


def select_candidates(ids: Sequence[int], weights: Sequence[float], *, allowed: Set[int], resident: Set[int],
                      minimum: float, budget: int, diagnostics: Optional[Dict[str, int]] = None) -> List[int]:
    total: Dict[int, float] = {}
    seen: Dict[int, int] = {}
    best: Dict[int, float] = {}
    skipped_nonlocal = skipped_resident = 0
    for eid, w in zip(ids, weights):
        eid, w = int(eid), float(w)
        if eid not in allowed:
            skipped_nonlocal += 1
        elif eid in resident:
            skipped_resident += 1
        else:
            total[eid] = total.get(eid, 0.0) + w
            seen[eid] = seen.get(eid, 0) + 1
            best[eid] = max(best.get(eid, 0.0), w)
    score = {e: s * (1 + 0.15 * (seen[e] - 1)) + 0.05 * best[e] for e, s in total.items()}
    if diagnostics is not None:
        diagnostics.update(nonlocal_entries=skipped_nonlocal, resident_entries=skipped_resident, scored=len(score),
                           below_threshold=sum(1 for v in score.values() if v < minimum))
    ranked = sorted(score, key=score.get, reverse=True)
    return [e for e in ranked if score[e] >= minimum][:budget]


def plan_inputs(pred, pred_k: int, norm_topk_prob: bool, dtype):
    """Flattened ``[T * pred_k]`` expert ids and probabilities the planner scans, from a dense
    predictor output (utils/eval_core.py:10985-10996): per token the ``pred_k`` largest
    probabilities in descending order (lower id first among equals), optionally renormalised,
    rounded to the activation dtype.  Plain Python lists of ints and floats."""
    import torch
    pred = torch.as_tensor(pred, dtype=torch.float32)
    k = min(int(pred.shape[-1]), int(pred_k))
    order = torch.sort(pred, dim=-1, descending=True, stable=True)
    vals, ids = order.values[:, :k], order.indices[:, :k]
    if norm_topk_prob:
        vals = vals / vals.sum(dim=-1, keepdim=True).clamp_min(1e-12)
    return ids.reshape(-1).tolist(), vals.to(dtype).to(torch.float32).reshape(-1).tolist()


def router_topk_feature(idx, w, num_experts: int) -> np.ndarray:
    """``[T, E]`` float32: token t's routing weights, divided by their sum (at least 1e-12),
    added at its chosen experts; zero elsewhere (utils/eval_core.py:10903-10908).  The sum
    and the division run in float32 as in the reference."""
    idx = np.asarray(idx, dtype=np.int64)
    ww = np.asarray(w, dtype=np.float32)
    total = np.zeros(ww.shape[0], dtype=np.float32)
    for k in range(ww.shape[1]):                     # left to right, as a float32 row sum
        total = (total + ww[:, k]).astype(np.float32)
    ww = (ww / np.maximum(total, np.float32(1e-12))[:, None]).astype(np.float32)
    feat = np.zeros((idx.shape[0], int(num_experts)), dtype=np.float32)
    for t in range(idx.shape[0]):
        for k in range(idx.shape[1]):
            feat[t, idx[t, k]] = np.float32(feat[t, idx[t, k]] + ww[t, k])
    return feat
