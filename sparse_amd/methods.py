"""The reference launcher's method switches (scripts/run/run_case.sh:75-138, :220-264).

``method_settings(name)`` gives the constructor keywords and the ``SPARSE_*`` environment a
formal run of that method uses; ``residency_config(name, ...)`` turns them into a
``ResidencyConfig`` without touching ``os.environ``.  On one GPU every expert resolves to
rank 0, so ``sparse`` (SCP placement + RS + EPIPE) executes exactly like ``rs-epipe``.
"""
from __future__ import annotations

from typing import Dict, Tuple

from .residency import ResidencyConfig

# method -> (planner_mode, epipe_enable, epipe_decode_rs_mode, plain_ep_exec_mode, placement_mode)
METHODS: Dict[str, Tuple[str, bool, str, str, str]] = {
    "rr": ("none", False, "off", "unique_mask", "round_robin"),
    "scp": ("none", False, "off", "unique_mask", "scp_ep"),
    "rs": ("rs_prefetch", False, "off", "unique_mask", "round_robin"),
    "epipe": ("none", True, "off", "sorted_segment", "round_robin"),
    "scp-rs": ("rs_prefetch", False, "off", "unique_mask", "scp_ep"),
    "rs-epipe": ("rs_prefetch", True, "residual_scan", "sorted_segment", "round_robin"),
    "sparse": ("rs_prefetch", True, "residual_scan", "sorted_segment", "scp_ep"),
    "executor-no-epipe": ("rs_prefetch", False, "off", "sorted_segment", "scp_ep"),
    "executor-with-epipe": ("rs_prefetch", True, "residual_scan", "sorted_segment", "scp_ep"),
}


def method_settings(method: str) -> Dict[str, object]:
    """Constructor keywords and environment of a formal run of ``method``."""
    if method not in METHODS:
        raise ValueError(f"unknown method: {method} (expected one of {', '.join(METHODS)})")
    planner, epipe, rs_mode, plain_exec, placement = METHODS[method]
    run_rs = planner == "rs_prefetch"
    env = {
        "SPARSE_RS_PREFETCH_POLICY": "cache_safe",
        "SPARSE_RS_CACHE_SAFE_MIN_SCORE": "0.04",
        "SPARSE_RS_CACHE_SAFE_REPLACE_ADVANTAGE": "0.08",
        "SPARSE_RS_CACHE_SAFE_REPLACE_MARGIN": "1.20",
        "SPARSE_RS_PREFETCH_RECENT_PROTECT_STEPS": "1",
        "SPARSE_PREFETCH_MIN_CAND_SCORE": "0.04",
        "SPARSE_PREFETCH_REPLACE_ADVANTAGE": "0.08",
        "SPARSE_PREFETCH_REPLACE_MARGIN": "1.20",
        "SPARSE_PREFETCH_ALLOW_ACTIVE_REPLACE": "1" if run_rs else "0",
        "SPARSE_EPIPE_ENABLE": "1" if epipe else "0",
        "SPARSE_EPIPE_PREFILL_ENABLE": "0",
        "SPARSE_EPIPE_MODE": "upfront_scan",
        "SPARSE_EPIPE_DECODE_RS_MODE": rs_mode,
        "SPARSE_EPIPE_RS_HANDLE_LATE_PREFETCH": "1" if epipe else "0",
        "SPARSE_EPIPE_RS_HANDLE_DEMAND_MISS": "1" if epipe else "0",
        "SPARSE_EPIPE_RS_FORCE_DEMAND_STAGE": "1" if epipe else "0",
        "SPARSE_EPIPE_NO_EVICT": "1",
        "SPARSE_EPIPE_TRANSIENT_STAGING": "1",
        "SPARSE_EPIPE_MAX_STAGED_EXPERTS": "1",
        "SPARSE_PLAIN_EP_EXEC_MODE": plain_exec,
    }
    kwargs = {
        "planner_mode": planner,
        "placement_mode": placement,
        "expert_offload": "cpu",
        "cache_policy": "lru",
        "routing_mode": "router",
        "expert_source": "router",
    }
    return {"kwargs": kwargs, "env": env}


def residency_config(method: str, expert_cache: int, prefetch_top_m: int = 2, *, formal_thresholds: bool = True,
                     **overrides) -> ResidencyConfig:
    """``ResidencyConfig`` of ``method`` with the launcher's values (or the code defaults
    when ``formal_thresholds`` is false)."""
    planner, epipe, rs_mode, plain_exec, _placement = METHODS[method] if method in METHODS else (None,) * 5
    if planner is None:
        raise ValueError(f"unknown method: {method}")
    run_rs = planner == "rs_prefetch"
    cfg = ResidencyConfig(capacity=int(expert_cache), planner_mode=planner, prefetch_top_m=int(prefetch_top_m))
    cfg.allow_active_replace = run_rs
    cfg.epipe_enable = epipe
    cfg.epipe_decode_rs_mode = rs_mode
    cfg.epipe_rs_handle_late_prefetch = epipe
    cfg.epipe_rs_handle_demand_miss = epipe
    cfg.epipe_rs_force_demand_stage = epipe
    cfg.plain_ep_exec_mode = plain_exec
    if formal_thresholds:
        cfg.rs_policy = "cache_safe"
        cfg.min_candidate_score = 0.04
        cfg.replace_advantage = 0.08
        cfg.replace_margin = 1.20
        cfg.cache_safe_min_score = 0.04
        cfg.cache_safe_replace_advantage = 0.08
        cfg.cache_safe_replace_margin = 1.20
        cfg.recent_protect_steps = 1
    for k, v in overrides.items():
        if not hasattr(cfg, k):
            raise ValueError(f"unknown residency option {k}")
        setattr(cfg, k, v)
    return cfg
