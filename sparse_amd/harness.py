"""Decoder-stack harness around the MoE block: module swap and the phase protocol.

The block depends on three things its caller does (utils/eval_core.py:17940-17991,
:18463-18607): every sparse MLP of a decoder stack is replaced by a
``DistributedSparseMoeBlock`` built from it; ``SparseContext.current_phase`` and
``begin_runtime_call(call_id)`` are set before each pass over the stack (call 0 is the
prefill, call n the n-th decode step); and the prefill -> decode boundary hooks run once
between them.  ``install_sparse_blocks`` does the first for any model whose decoder layers
hold an ``.mlp`` with ``.gate`` and ``.experts``; ``greedy_decode`` does the other two for
any causal LM with the Hugging Face call convention (``input_ids``, ``attention_mask``,
``use_cache``, ``past_key_values``, ``return_dict`` -> ``.logits``, ``.past_key_values``).
"""
from __future__ import annotations

import os
import time
from typing import Any, Iterable, List, Optional

import torch

from .block import DistributedSparseMoeBlock
from .context import DistEnv, Metrics, SparseContext
from .rs import load_rs_bank


def looks_like_sparse_moe_block(mlp: Any) -> bool:
    """Same duck test as the reference (:4342-4347): a router gate and an expert container."""
    return hasattr(mlp, "gate") and hasattr(mlp, "experts")


def decoder_layers(model: Any) -> List[Any]:
    """The decoder layers of a causal LM (``model.model.layers``), of a bare decoder
    (``model.layers``) or of a plain sequence of layers."""
    inner = getattr(model, "module", model)
    for owner in (getattr(inner, "model", None), inner):
        layers = getattr(owner, "layers", None)
        if layers is not None:
            return list(layers)
    if isinstance(model, Iterable):
        return list(model)
    raise RuntimeError("cannot find decoder layers (expected .model.layers or .layers)")


def _expert_count(mlp: Any, default: int = 0) -> int:
    for owner in (mlp, getattr(mlp, "gate", None)):
        for name in ("num_experts", "n_routed_experts"):
            if int(getattr(owner, name, 0) or 0) > 0:
                return int(getattr(owner, name))
    experts = mlp.experts
    if hasattr(experts, "gate_up_proj"):
        return int(experts.gate_up_proj.shape[0])
    try:
        return len(list(experts))
    except TypeError:
        if default > 0:
            return default
        raise RuntimeError("Cannot infer num_experts") from None


def install_sparse_blocks(model: Any, *, env: Optional[DistEnv] = None, dtype: torch.dtype = torch.bfloat16,
                          top_k: Optional[int] = None, metrics: Optional[Metrics] = None,
                          rs_dir: Optional[str] = None, rs_require_complete: bool = True,
                          **block_kwargs: Any) -> List[DistributedSparseMoeBlock]:
    """Replace every sparse MLP of ``model``'s decoder layers by a block built from it.

    Expert count and top-k are read from the module (``num_experts`` / ``n_routed_experts``,
    ``top_k`` / ``num_experts_per_tok``) as the reference does (:17943-17955), or from its router
    module where newer Hugging Face layouts keep them; ``top_k`` overrides.  Remaining keywords (``expert_offload``, ``expert_cache``, ``planner_mode``,
    ``prefetch_top_m``, ``cache_policy`` ...) go to every block unchanged.  With ``rs_dir``
    the next-layer predictor bank is loaded and registered.  Returns the blocks in layer order.
    """
    env = env if env is not None else DistEnv()
    metrics = metrics if metrics is not None else Metrics()
    layers = decoder_layers(model)
    blocks: List[DistributedSparseMoeBlock] = []
    for idx, layer in enumerate(layers):
        mlp = getattr(layer, "mlp", None)
        if mlp is None or isinstance(mlp, DistributedSparseMoeBlock) or not looks_like_sparse_moe_block(mlp):
            continue
        router = getattr(mlp, "gate", None)
        k = top_k if top_k is not None else int(
            getattr(mlp, "top_k", 0) or getattr(mlp, "num_experts_per_tok", 0) or getattr(router, "top_k", 0) or 0)
        if k <= 0:
            raise RuntimeError(f"Cannot infer top_k at layer {idx}")
        block = DistributedSparseMoeBlock(
            layer_idx=idx, mlp_block=mlp, env=env, num_layers=len(layers), num_experts=_expert_count(mlp),
            top_k=k, dtype=dtype, metrics=metrics, rs_dir=rs_dir, rs_require_complete=rs_require_complete,
            **block_kwargs)
        if hasattr(router, "top_k") and hasattr(mlp, "shared_expert"):
            # Hugging Face layouts whose router module does the top-k: their decoder layer
            # consumes a tensor, not (tensor, router_logits)
            block.return_router_logits = False
        layer.mlp = block
        blocks.append(block)
    if rs_dir and blocks:
        first = blocks[0]
        modules, sources, _ = load_rs_bank(rs_dir, len(layers), first.hidden_size, first.num_experts,
                                           device=first.device, require_complete=rs_require_complete)
        SparseContext.set_rs_bank(modules, sources)
    return blocks


def begin_request(*, clear_expert_cache: bool = True, clear_cache_metadata: bool = True) -> None:
    """What the formal runs do before each repeat (scripts/perf.py:553-588): every block
    forgets the previous request."""
    SparseContext.prefill_scp_transient_demoted_for_decode = False
    for blk in SparseContext.layer_blocks.values():
        blk.reset_runtime_state_for_new_request(clear_expert_cache=clear_expert_cache,
                                                clear_cache_metadata=clear_cache_metadata)


def _env_flag(name: str, default: str) -> bool:
    return str(os.environ.get(name, default)).strip().lower() not in ("", "0", "false", "no", "off")


def _demote_at_boundary() -> bool:
    """The reference's switch for the transient demotion and its end-of-decode count
    (:18530-18531, :18588-18589); on unless both variables say otherwise."""
    return (_env_flag("SPARSE_SCP_TRANSIENT_PREFILL_CACHE", "0")
            or _env_flag("SPARSE_EPIPE_DECODE_DEMOTE_PREFILL_TRANSIENT", "1"))


def prefill_decode_boundary(metrics: Optional[Metrics] = None) -> None:
    """Hooks between the prefill pass and the first decode step (:18530-18537)."""
    if _demote_at_boundary():
        DistributedSparseMoeBlock.demote_prefill_scp_transients_for_decode(metrics)
    DistributedSparseMoeBlock.handle_epipe_prefill_extra_cache_decode_boundary(metrics)
    if _env_flag("SPARSE_SCP_CLEAR_CACHE_BEFORE_DECODE", "0"):
        DistributedSparseMoeBlock.clear_all_expert_caches()


@torch.no_grad()
def greedy_decode(model: Any, input_ids: torch.Tensor, attention_mask: Optional[torch.Tensor],
                  max_new_tokens: int, metrics: Optional[Metrics] = None) -> torch.Tensor:
    """Greedy generation with the phase protocol of ``greedy_decode_profiled``
    (:18463-18600): prefill as call 0 in phase ``prefill``, the boundary hooks, then one
    ``decode`` call per further token with call id = tokens generated so far.  Wall times go
    to ``metrics.timings_ms['wall_prefill']`` / ``['wall_decode']``.  Returns prompt +
    generated ids."""
    if hasattr(model, "eval"):
        model.eval()
    device = input_ids.device

    def sync() -> None:
        if device.type == "cuda":
            torch.cuda.synchronize(device)

    SparseContext.current_phase = "prefill"
    SparseContext.begin_runtime_call(0)
    t0 = time.perf_counter()
    out = model(input_ids=input_ids, attention_mask=attention_mask, use_cache=True, return_dict=True)
    sync()
    prefill_ms = (time.perf_counter() - t0) * 1e3
    prefill_decode_boundary(metrics)

    past = out.past_key_values
    cur = torch.argmax(out.logits[:, -1, :], dim=-1, keepdim=True)
    generated = [cur]
    mask = attention_mask
    decode_ms = 0.0
    for _ in range(int(max_new_tokens) - 1):
        if mask is not None:
            mask = torch.cat([mask, torch.ones((mask.shape[0], 1), device=mask.device, dtype=mask.dtype)], dim=1)
        SparseContext.current_phase = "decode"
        SparseContext.begin_runtime_call(len(generated))
        t0 = time.perf_counter()
        out = model(input_ids=cur, attention_mask=mask, use_cache=True, past_key_values=past, return_dict=True)
        sync()
        decode_ms += (time.perf_counter() - t0) * 1e3
        past = out.past_key_values
        cur = torch.argmax(out.logits[:, -1, :], dim=-1, keepdim=True)
        generated.append(cur)
    if _demote_at_boundary():
        DistributedSparseMoeBlock.record_prefill_scp_transient_decode_end(metrics)
    DistributedSparseMoeBlock.record_epipe_prefill_extra_cache_decode_end(metrics)
    SparseContext.current_phase = "none"
    if metrics is not None:
        metrics.timings_ms["wall_prefill"] = metrics.timings_ms.get("wall_prefill", 0.0) + prefill_ms
        metrics.timings_ms["wall_decode"] = metrics.timings_ms.get("wall_decode", 0.0) + decode_ms
        if device.type == "cuda":
            metrics.harvest_timings()
    return torch.cat([input_ids, torch.cat(generated, dim=1)], dim=1)
