"""CPU oracle for the token x K expansion and permutation.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may
import this.  Restates utils/eval_core.py:14728-14730 (flat index f = t*K + k),
:13240-13262 (``argsort`` by expert id, contiguous segments) and :13359-13360
(``out[order] = out_sorted``).  The reference's ``argsort`` is not ``stable=True``; the
permutation is therefore defined here by the stable rule, order (expert id, f).

Pinned by (tests/test_oracle_moe.py): a brute-force O(n^2) rank computation on small
inputs, ``perm`` being a permutation, ``inv_perm[perm[p]] == p``, segment offsets equal to
the exclusive prefix sum of ``bincount``, sortedness of ``topi.flat[perm]``.
"""
from __future__ import annotations

import numpy as np


def permute_build(topi: np.ndarray, num_experts: int):
    """topi [T,K] integer -> (perm [T*K] int32, inv_perm [T*K] int32,
    seg_offsets [E+1] int32, active_eids int32 ascending)."""
    flat = np.asarray(topi).reshape(-1).astype(np.int64)
    perm = np.argsort(flat, kind="stable").astype(np.int32)
    inv_perm = np.empty_like(perm)
    inv_perm[perm] = np.arange(perm.size, dtype=np.int32)
    counts = np.bincount(flat, minlength=num_experts)[:num_experts]
    seg_offsets = np.zeros(num_experts + 1, dtype=np.int32)
    seg_offsets[1:] = np.cumsum(counts)
    active = np.nonzero(counts)[0].astype(np.int32)
    return perm, inv_perm, seg_offsets, active


def segments(topi: np.ndarray, num_experts: int):
    """The reference's segment tuples ``(eid, start, end)`` in ascending expert id."""
    _, _, off, active = permute_build(topi, num_experts)
    return [(int(e), int(off[e]), int(off[e + 1])) for e in active]
