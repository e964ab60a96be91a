#!/usr/bin/env python3
"""Write the golden call sequence of the reference's generation loop.

Runs ONLY in the build container, where the reference checkout is mounted at
/root/reference; the fixture it writes (``decode_protocol.json``) is what the tests read.

``greedy_decode_profiled`` (utils/eval_core.py:18463-18600) is taken out of the reference
source with ``ast`` and run on the CPU against recording stand-ins: a toy causal LM with the
Hugging Face call convention, a ``SparseContext`` that logs phase changes and call ids, and a
block class whose boundary hooks log their names.  Recorded: the order of phase changes,
``begin_runtime_call`` ids, model calls (input shape, mask length, whether a cache was passed)
and hook calls, plus the generated ids.
"""
from __future__ import annotations

import ast
import json
import sys
from pathlib import Path
from types import SimpleNamespace as NS
from typing import Any, Dict

import torch
import torch.nn.functional as F

REF = Path("/root/reference/utils/eval_core.py")
OUT = Path(__file__).resolve().parent
ROOT = OUT.parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


class LoggingContext:
    """Stands in for the reference's ``SparseContext`` class object."""

    def __init__(self, log):
        object.__setattr__(self, "log", log)
        object.__setattr__(self, "oracle_mode", "none")
        object.__setattr__(self, "_phase", "none")

    def __setattr__(self, name, value):
        if name == "current_phase":
            self.log.append(["phase", value])
            object.__setattr__(self, "_phase", value)
        else:
            object.__setattr__(self, name, value)

    @property
    def current_phase(self):
        return self._phase

    def begin_runtime_call(self, call_id):
        self.log.append(["begin_runtime_call", int(call_id)])

    def __getattr__(self, name):                  # clear_group_plan, end_oracle_call, ...
        return lambda *a, **k: None


def main() -> None:
    if not REF.exists():
        sys.exit("the reference checkout is not mounted; fixtures are only written in the build container")
    from tests.toy_lm import ToyCausalLM
    tree = ast.parse(REF.read_text())
    fn = next(n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == "greedy_decode_profiled")
    future = ast.ImportFrom(module="__future__", names=[ast.alias(name="annotations")], level=0)
    out = []
    for env, tokens, batch, prompt in (({}, 5, 2, 3), ({}, 1, 1, 4), ({"SPARSE_EPIPE_DECODE_DEMOTE_PREFILL_TRANSIENT": "0"}, 3, 1, 2)):
        log = []
        context = LoggingContext(log)

        class Hooks:
            def __getattr__(self, name):
                return lambda *a, **k: log.append(["hook", name])

        class Timer:
            def __enter__(self):
                return lambda: 0.001

            def __exit__(self, *exc):
                return False

        proxy_cuda = NS(reset_peak_memory_stats=lambda *_a: None, synchronize=lambda *_a: None,
                        is_available=lambda: False, max_memory_allocated=lambda *_a: 0, max_memory_reserved=lambda *_a: 0)

        class TorchProxy:
            def __getattr__(self, name):
                return proxy_cuda if name == "cuda" else getattr(torch, name)

        ns: Dict[str, Any] = dict(
            torch=TorchProxy(), F=F, SparseContext=context, DistributedSparseMoeBlock=Hooks(),
            _hclm_cp_create_from_env=lambda *_a: NS(start_step=lambda *a, **k: None, end_step=lambda *a: None,
                                                     close=lambda: None),
            _hclm_cp_set_global=lambda *_a: None, _HCLMCPNoOp=lambda: None, _phase_trace=lambda *_a: None,
            wall_timer_s=Timer, time=__import__("time"),
            _env_flag=lambda name, default="0": str(env.get(name, default)).strip().lower() not in ("", "0", "false", "no", "off"),
            _unwrap_causal_lm_for_logits=lambda model: (None, None),
            _finalize_pending_demand_h2d_events=lambda *_a: None, _finalize_pending_prefetch_events=lambda *_a: None,
            _finalize_pending_epipe_timing_events=lambda *_a: None, _consume_skvs_accounting=lambda *_a: None,
            _normalize_past_key_values_for_runtime=lambda past: past)
        exec(compile(ast.fix_missing_locations(ast.Module(body=[future, fn], type_ignores=[])), str(REF), "exec"), ns)

        class Plain(torch.nn.Module):
            def forward(self, x):
                return torch.tanh(x)

        model = ToyCausalLM(50, 16, [Plain(), Plain()])
        real_forward = model.forward

        def logged(input_ids, attention_mask=None, use_cache=True, past_key_values=None, return_dict=True):
            log.append(["model", list(input_ids.shape), None if attention_mask is None else int(attention_mask.shape[1]),
                        past_key_values is not None])
            return real_forward(input_ids, attention_mask=attention_mask, use_cache=use_cache,
                                past_key_values=past_key_values, return_dict=return_dict)

        model.forward = logged
        ids = torch.arange(1, 1 + batch * prompt).view(batch, prompt)
        metrics = NS(wall_prefill_ms=0.0, wall_decode_ms=0.0, wall_ttft_ms=0.0, decode_step_stats=None,
                     warmup_time_ms=0.0, peak_allocated_mb=0.0, peak_reserved_mb=0.0)
        result = ns["greedy_decode_profiled"](model, ids, torch.ones_like(ids), tokens, NS(rank=0, world=1, device="cpu"),
                                              metrics, True)
        out.append(dict(env=env, max_new_tokens=tokens, input_ids=ids.tolist(), log=log, output_ids=result.tolist()))
    (OUT / "decode_protocol.json").write_text(json.dumps(out))
    print("wrote", OUT / "decode_protocol.json")


if __name__ == "__main__":
    main()
