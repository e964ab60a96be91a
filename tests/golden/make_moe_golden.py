#!/usr/bin/env python3
"""Write golden vectors for the arithmetic of the MoE layer from the reference's own code.

Runs ONLY in the build container, where the reference checkout is mounted at
/root/reference; the fixture it writes (``moe_math.json``) is what the tests read.

The reference package cannot be imported here (it needs transformers and a GPU at import
time), so -- as in the reference's own tests (tests/test_lightweight_policy.py:63-71) -- the
functions are taken out of ``utils/eval_core.py`` by name with ``ast`` and run on the CPU
against a stub block that holds small ``torch.nn`` modules:

  _routing_router            Qwen branch: gate Linear, fp32 softmax, top-k, optional renorm
  _experts_world1_exact      all-resident expert loop with ``index_add_`` in the activation dtype
  _execute_local_recv_groups sorted-segment executor over the token x K expansion
                             (both ``unique_mask`` and ``sorted_segment`` modes)
  combine_expert_outputs     K ordered adds in the activation dtype
  _shared_expert_forward     shared MLP, with and without the sigmoid gate
  _module_expert_forward / _plain_ep_compute_segment   one expert's SwiGLU times route weight

Inputs are small seeded tensors (fp32 and bf16); inputs and outputs are stored as raw
little-endian bytes in base64, so the comparison in the tests is bit for bit.
"""
from __future__ import annotations

import ast
import base64
import json
import os
import sys
import time
from pathlib import Path
from types import SimpleNamespace as NS
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F
from torch import nn

REF = Path("/root/reference/utils/eval_core.py")
OUT = Path(__file__).resolve().parent
ROOT = OUT.parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

from tests.helpers import seeded_moe_layer  # noqa: E402

METHODS = ("_routing_router", "_experts_world1_exact", "_execute_local_recv_groups", "_shared_expert_forward",
           "_module_expert_forward", "_plain_ep_compute_segment", "_current_stage", "_epipe_stage_enabled")
FUNCTIONS = ("combine_expert_outputs", "_plain_ep_exec_mode")


def pack(t: torch.Tensor) -> Dict[str, Any]:
    t = t.detach().contiguous()
    if t.dtype == torch.bfloat16:
        raw, kind = t.view(torch.int16).numpy().tobytes(), "bf16"
    elif t.dtype == torch.float32:
        raw, kind = t.numpy().tobytes(), "f32"
    else:
        raw, kind = t.to(torch.int64).numpy().tobytes(), "i64"
    return dict(dtype=kind, shape=list(t.shape), data=base64.b64encode(raw).decode())


def extract(env: Dict[str, str]):
    tree = ast.parse(REF.read_text())
    block = next(n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == "DistributedSparseMoeBlock")
    methods = [n for n in block.body if isinstance(n, ast.FunctionDef) and n.name in METHODS]
    functions = [n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name in FUNCTIONS]
    assert {m.name for m in methods} == set(METHODS) and {f.name for f in functions} == set(FUNCTIONS)
    future = ast.ImportFrom(module="__future__", names=[ast.alias(name="annotations")], level=0)
    ns: Dict[str, Any] = dict(
        torch=torch, F=F, os=NS(environ=env), time=time, Any=Any, Dict=Dict, List=List, Optional=Optional, Tuple=Tuple,
        Sequence=Sequence, SparseContext=NS(current_phase="decode", runtime_call_id=0),
        _hclm_cp_profiler=lambda: NS(should_sample=lambda _step: False), _hclm_cp_now_ns=lambda: 0,
        _env_flag=lambda name, default="0": str(env.get(name, default)).strip().lower() not in ("", "0", "false", "no", "off"))
    exec(compile(ast.fix_missing_locations(ast.Module(body=[future, *functions, *methods], type_ignores=[])),
                 str(REF), "exec"), ns)
    return ns


class Mlp(nn.Module):
    def __init__(self, hidden: int, inter: int) -> None:
        super().__init__()
        self.gate_proj = nn.Linear(hidden, inter, bias=False)
        self.up_proj = nn.Linear(hidden, inter, bias=False)
        self.down_proj = nn.Linear(inter, hidden, bias=False)
        self.act_fn = nn.SiLU()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


class StubBlock:
    def __init__(self, ns, shape, dtype, seed, renorm, shared_gate, given=None):
        self.__dict__["_ns"] = ns
        torch.manual_seed(seed)
        H, E, I, K, Is = shape
        self.num_experts, self.top_k, self.norm_topk_prob = E, K, renorm
        self.hidden_size = H
        self.moe_family = "qwen_shared"
        self.gate = nn.Linear(H, E, bias=False).to(dtype)
        self.experts = [Mlp(H, I).to(dtype) for _ in range(E)]
        self.shared_experts = None
        self.shared_expert = Mlp(H, Is).to(dtype) if Is else None
        self.shared_expert_gate = nn.Linear(H, 1, bias=False).to(dtype) if (Is and shared_gate) else None
        for m in [self.gate, *self.experts, self.shared_expert, self.shared_expert_gate]:
            if m is not None:
                for p in m.parameters():
                    p.data.mul_(2.0)          # a little more spread than the default init
        if given is not None:                  # weights from the seeded helper instead of the default init
            def fill(mlp, triple):
                mlp.gate_proj.weight.data, mlp.up_proj.weight.data, mlp.down_proj.weight.data = triple

            self.gate.weight.data = given["gate_w"]
            for m, triple in zip(self.experts, given["experts"]):
                fill(m, triple)
            if self.shared_expert is not None:
                fill(self.shared_expert, given["shared"])
            if self.shared_expert_gate is not None:
                self.shared_expert_gate.weight.data = given["shared_gate_w"].view(1, -1)
        self.act_fn = nn.SiLU()
        self.experts_kind, self.expert_offload = "modulelist", "cpu"
        self.local_expert_ids = list(range(E))
        self._local_eid_set = set(range(E))
        self.device = torch.device("cpu")
        self.layer_idx = 0
        self.planner_mode = "none"
        self._epipe_enable = self._epipe_shadow = self._epipe_prefill_enable = False
        self._epipe_prefill_shadow = self._epipe_prefill_multistage_shadow = False
        self._epipe_mode, self._epipe_decode_with_rs_mode = "upfront_scan", "off"
        self._current_forward_batch_size, self._current_forward_seq_len = 1, 1

    def __getattr__(self, name):
        fn = self._ns.get(name)
        if callable(fn) and name in METHODS:
            return lambda *a, **k: fn(self, *a, **k)
        if "_record_" in name:
            return lambda *a, **k: None
        raise AttributeError(name)

    def _nodepatch_phase_enabled(self) -> bool:
        return False

    def _get_local_module_weights(self, eid: int):
        m = self.experts[int(eid)]
        return m.gate_proj.weight, m.up_proj.weight, m.down_proj.weight


def run_case(shape, dtype, T, seed, renorm, shared_gate, seeded=False):
    H, E, I, K, Is = shape
    out: Dict[str, Any] = dict(shape=list(shape), T=T, seed=seed, renorm=renorm, shared_gate=shared_gate,
                               dtype="bf16" if dtype == torch.bfloat16 else "f32", seeded=seeded)
    with torch.no_grad():
        env = {"SPARSE_PLAIN_EP_EXEC_MODE": "sorted_segment"}
        ns = extract(env)
        if seeded:
            # device-sized layer: the inputs are rebuilt from the seed by the test, only their
            # checksum is stored
            given = seeded_moe_layer(shape, T, dtype, seed, shared_gate)
            blk = StubBlock(ns, shape, dtype, seed, renorm, shared_gate, given)
            x = given["x"]
            out["checksum"] = given["checksum"]
        else:
            blk = StubBlock(ns, shape, dtype, seed, renorm, shared_gate)
            x = torch.randn(T, H, generator=torch.Generator().manual_seed(seed + 1)).to(dtype)
            out["x"] = pack(x)
            out["gate_w"] = pack(blk.gate.weight)
            out["experts"] = [[pack(m.gate_proj.weight), pack(m.up_proj.weight), pack(m.down_proj.weight)]
                              for m in blk.experts]
            sh = blk.shared_expert
            out["shared"] = ([pack(sh.gate_proj.weight), pack(sh.up_proj.weight), pack(sh.down_proj.weight)]
                             if sh else None)
            out["shared_gate_w"] = (pack(blk.shared_expert_gate.weight.reshape(-1))
                                    if blk.shared_expert_gate else None)

        topv, topi, logits = blk._routing_router(x)
        out["topv"], out["topi"], out["logits"] = pack(topv), pack(topi), pack(logits)
        exact = blk._experts_world1_exact(x, topi, topv)
        out["experts_world1_exact"] = pack(exact)
        # the EP form at world size 1: expansion (:14728-14733), executor, combine (:14861-14863)
        expanded = x.unsqueeze(1).expand(-1, K, -1).reshape(-1, H)
        flat_i = topi.reshape(-1).to(torch.long)
        flat_w = topv.reshape(-1).to(expanded.dtype)
        parts = blk._execute_local_recv_groups(expanded, flat_i, flat_w)
        if not seeded:
            out["parts_sorted_segment"] = pack(parts)
        env["SPARSE_PLAIN_EP_EXEC_MODE"] = "unique_mask"
        parts_mask = blk._execute_local_recv_groups(expanded, flat_i, flat_w)
        # rows of a segment come in another order in this mode, which a CPU matrix product can
        # show in the last fp32 bit: keep the size of the difference, not the tensor
        out["parts_unique_mask_maxdiff"] = float((parts.float() - parts_mask.float()).abs().max())
        combined = ns["combine_expert_outputs"](parts.view(T, K, H), topi)
        shared = blk._shared_expert_forward(x)
        out["layer_out"] = pack(exact + shared)
        if seeded:
            # bulky outputs of the device-sized cases are kept as what they must add up to
            out["combined_equals_exact"] = bool(torch.equal(combined, exact))
            out["combined_maxdiff"] = float((combined.float() - exact.float()).abs().max())
        else:
            out["combined"] = pack(combined)
            out["shared_out"] = pack(shared)
            y, _ms = blk._plain_ep_compute_segment(eid=1, cur=x[:3], cur_w=topv[:3, :1].to(x.dtype),
                                                   eid_is_local=True, allow_nonlocal=False)
            out["segment_expert1"] = pack(y)
    return out


def main() -> None:
    if not REF.exists():
        sys.exit("the reference checkout is not mounted; fixtures are only written in the build container")
    cases = []
    seed = 100
    for dtype in (torch.float32, torch.bfloat16):
        for shape, T, renorm, gate in (((16, 5, 8, 2, 12), 7, False, True), ((32, 12, 16, 4, 24), 9, False, True),
                                       ((16, 8, 8, 6, 16), 5, False, False), ((32, 6, 16, 2, 0), 4, True, False),
                                       ((16, 4, 8, 1, 8), 1, False, True)):
            seed += 1
            cases.append(run_case(shape, dtype, T, seed, renorm, gate))
        # layers of the granularity the HIP kernels accept (H, I, Is multiples of 64)
        for shape, T, renorm, gate in (((128, 12, 64, 4, 128), 8, False, True), ((64, 16, 128, 6, 64), 40, False, False),
                                       ((128, 8, 64, 2, 64), 70, True, True)):
            seed += 1
            cases.append(run_case(shape, dtype, T, seed, renorm, gate, seeded=True))
    (OUT / "moe_math.json").write_text(json.dumps(cases, separators=(",", ":")))
    print("wrote", OUT / "moe_math.json", "cases:", len(cases))


if __name__ == "__main__":
    main()
