#!/usr/bin/env python3
"""Write golden vectors for the RS predictors and their checkpoint directories.

Runs ONLY in the build container, where the reference checkout is mounted at
/root/reference; the fixture it writes (``rs_bank.json``) is what the tests read.

The predictor classes (``RoutingScoutMLP``, ``RoutingScoutResidualMLP``) and the loader
functions (``_build_rs_module_from_payload``, ``_load_runtime_rs_bank`` and their helpers) are
top-level definitions of ``utils/eval_core.py``; they are taken out of the source with ``ast``
and run on the CPU.  Recorded: state dicts of small predictors, their eval-mode outputs on a
fixed input, and what the loader returns for directories with complete, incomplete and
differently named checkpoint sets (layout, source layers, missing list, module classes,
outputs of the loaded bank), the block method that builds the ``hidden_router_topk`` input
feature, and a checkpoint that asks for it.
"""
from __future__ import annotations

import ast
import json
import re
import sys
import tempfile
from pathlib import Path
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F
from torch import nn

REF = Path("/root/reference/utils/eval_core.py")
OUT = Path(__file__).resolve().parent
NAMES = ("RoutingScoutMLP", "_RSResidualBlock", "RoutingScoutResidualMLP", "CacheValueScoutMLP", "_extract_state_dict",
         "_build_rs_module_from_payload", "_is_next_layer_rs_layout", "_next_layer_rs_target_layers",
         "_is_optional_next_layer_rs_miss", "_load_runtime_rs_bank")


def extract():
    tree = ast.parse(REF.read_text())
    nodes = [n for n in tree.body if isinstance(n, (ast.ClassDef, ast.FunctionDef)) and n.name in NAMES]
    assert {n.name for n in nodes} == set(NAMES)
    future = ast.ImportFrom(module="__future__", names=[ast.alias(name="annotations")], level=0)
    ns: Dict[str, Any] = dict(torch=torch, nn=nn, F=F, re=re, Path=Path, Any=Any, Dict=Dict, List=List,
                              Optional=Optional, Tuple=Tuple, Sequence=Sequence)
    exec(compile(ast.fix_missing_locations(ast.Module(body=[future, *nodes], type_ignores=[])), str(REF), "exec"), ns)
    return ns


def block_method(name: str):
    """A method of the reference's ``DistributedSparseMoeBlock`` as a plain function."""
    tree = ast.parse(REF.read_text())
    cls = next(n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == "DistributedSparseMoeBlock")
    fn = next(n for n in cls.body if isinstance(n, ast.FunctionDef) and n.name == name)
    future = ast.ImportFrom(module="__future__", names=[ast.alias(name="annotations")], level=0)
    ns: Dict[str, Any] = dict(torch=torch)
    exec(compile(ast.fix_missing_locations(ast.Module(body=[future, fn], type_ignores=[])), str(REF), "exec"), ns)
    return ns[name]


def lists(state: Dict[str, torch.Tensor]) -> Dict[str, Any]:
    return {k: dict(shape=list(v.shape), dtype=str(v.dtype).replace("torch.", ""), data=v.reshape(-1).tolist())
            for k, v in state.items()}


def randomize(module: nn.Module, seed: int) -> None:
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, t in module.state_dict().items():
            if t.dtype.is_floating_point:
                t.copy_(torch.randn(t.shape, generator=g) * 0.5 + (1.0 if name.endswith("running_var") else 0.0))
            if name.endswith("running_var"):
                t.abs_().add_(0.1)


def main() -> None:
    if not REF.exists():
        sys.exit("the reference checkout is not mounted; fixtures are only written in the build container")
    ns = extract()
    D, E, W = 8, 5, 16
    x = torch.randn(6, D, generator=torch.Generator().manual_seed(7))
    out: Dict[str, Any] = dict(input_dim=D, num_experts=E, hidden_dim=W, x=x.tolist(), modules=[], directories=[])
    payloads = {}
    for kind, cls, extra in (("independent_light_logits_rs", "RoutingScoutMLP", {}),
                             ("next_layer_residual_logits_rs", "RoutingScoutResidualMLP", dict(num_hidden_layers=2))):
        kw = dict(extra)
        mod = ns[cls](D, E, hidden_dim=W, **kw).eval()
        randomize(mod, 11 + len(payloads))
        with torch.no_grad():
            y = mod(x)
            y3 = mod(x.view(2, 3, D))                       # [B,S,H] inputs are flattened
        assert torch.equal(y, y3)
        meta = dict(model_type=kind, input_dim=D, num_experts=E, hidden_dim=W, **kw)
        payloads[kind] = (meta, mod.state_dict())
        out["modules"].append(dict(meta=meta, state=lists(mod.state_dict()), output=y.tolist()))

    def write_dir(d: Path, files: Dict[str, Tuple[Dict[str, Any], Dict[str, torch.Tensor], Dict[str, Any]]]):
        for name, (meta, state, more) in files.items():
            torch.save({**meta, **more, "state_dict": state}, d / name)

    light, deep = payloads["independent_light_logits_rs"], payloads["next_layer_residual_logits_rs"]
    scenarios = [
        ("complete", 3, {"rs_l1_inL0.pth": (*light, {}), "rs_l2_inL1.pth": (*deep, dict(source_layer=1))}, True),
        ("gap", 4, {"rs_l1_inL0.pth": (*light, {}), "rs_l3_inL2.pth": (*deep, {})}, False),
        ("gap_required", 4, {"rs_l1_inL0.pth": (*light, {}), "rs_l3_inL2.pth": (*deep, {})}, True),
        ("late_start", 4, {"rs_l2_inL1.pth": (*light, {}), "rs_l3_inL2.pth": (*light, {})}, True),
        ("model_state_dict_key", 2, {"rs_l1_inL0.pth": (light[0], light[1], dict(_rename=True))}, True),
    ]
    for name, layers, files, require in scenarios:
        with tempfile.TemporaryDirectory() as tmp:
            d = Path(tmp)
            listing = []
            for fname, (meta, state, more) in files.items():
                more = dict(more)
                key = "model_state_dict" if more.pop("_rename", False) else "state_dict"
                torch.save({**meta, **more, key: state}, d / fname)
                listing.append(dict(file=fname, model_type=meta["model_type"], extra=more, state_key=key))
            rec: Dict[str, Any] = dict(name=name, num_layers=layers, files=listing, require_complete=require)
            try:
                bank, task, layout, sources, missing = ns["_load_runtime_rs_bank"](
                    rs_path=d, num_layers=layers, hidden_dim=D, num_experts=E, device=torch.device("cpu"),
                    require_complete=require)
                with torch.no_grad():
                    rec.update(task=task, layout=layout, sources=[int(s) for s in sources], missing=list(missing),
                               classes=[type(m).__name__ for m in bank],
                               trained=[f"rs_l{l}_inL{l - 1}.pth" in files for l in range(layers)],
                               outputs=[bank[l](x).tolist() if f"rs_l{l}_inL{l - 1}.pth" in files else None
                                        for l in range(layers)])
            except RuntimeError as err:
                rec.update(error=str(err).splitlines()[0])
            out["directories"].append(rec)
    # the extra predictor input of ``feature_mode="hidden_router_topk"``: the source layer's own
    # routing as a dense [T, E] row of renormalised weights
    from types import SimpleNamespace
    build = block_method("_build_router_topk_feature")
    g = torch.Generator().manual_seed(21)
    out["router_topk_feature"] = []
    for dtype, T, E2, K in ((torch.float32, 4, 5, 2), (torch.bfloat16, 3, 7, 3), (torch.float32, 2, 4, 4)):
        w = torch.rand(T, K, generator=g).to(dtype)
        idx = torch.stack([torch.randperm(E2, generator=g)[:K] for _ in range(T)])
        feat = build(SimpleNamespace(num_experts=E2), idx, w)
        out["router_topk_feature"].append(dict(dtype=str(dtype).replace("torch.", ""), num_experts=E2,
                                               idx=idx.tolist(), w=w.float().tolist(), feat=feat.tolist()))
    # a checkpoint that asks for that input: what the loader leaves on the module
    mod = ns["RoutingScoutMLP"](D + E, E, hidden_dim=W).eval()
    randomize(mod, 31)
    meta = dict(model_type="independent_light_logits_rs", input_dim=D + E, num_experts=E, hidden_dim=W,
                feature_mode="hidden_router_topk")
    with tempfile.TemporaryDirectory() as tmp:
        d = Path(tmp)
        torch.save({**meta, "state_dict": mod.state_dict()}, d / "rs_l1_inL0.pth")
        bank, task, layout, sources, missing = ns["_load_runtime_rs_bank"](
            rs_path=d, num_layers=2, hidden_dim=D, num_experts=E, device=torch.device("cpu"), require_complete=True)
        w = torch.rand(6, 2, generator=g)
        idx = torch.stack([torch.randperm(E, generator=g)[:2] for _ in range(6)])
        full = torch.cat([x, build(SimpleNamespace(num_experts=E), idx, w)], dim=-1)
        with torch.no_grad():
            out["feature_checkpoint"] = dict(
                meta=meta, state=lists(mod.state_dict()), layout=layout, task=task,
                feature_modes=[str(getattr(m, "rs_feature_mode", "hidden")) for m in bank],
                idx=idx.tolist(), w=w.tolist(), output=bank[1](full).tolist())
    (OUT / "rs_bank.json").write_text(json.dumps(out, separators=(",", ":")))
    print("wrote", OUT / "rs_bank.json")


if __name__ == "__main__":
    main()
