"""RS predictors and checkpoint directories against vectors recorded from the reference's own
classes and loader (``tests/golden/rs_bank.json``, written by ``tests/golden/make_rs_golden.py``
from ``RoutingScoutMLP``, ``RoutingScoutResidualMLP``, ``_build_rs_module_from_payload`` and
``_load_runtime_rs_bank`` of utils/eval_core.py, run on the CPU)."""
import json
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import ref_rs
from sparse_amd.rs import RoutingScoutMLP, RoutingScoutResidualMLP, load_rs_bank, module_from_payload

DATA = json.loads((Path(__file__).resolve().parent / "golden" / "rs_bank.json").read_text())
X = torch.tensor(DATA["x"], dtype=torch.float32)
D, E = DATA["input_dim"], DATA["num_experts"]


def state_dict(rec):
    return {k: torch.tensor(v["data"], dtype=getattr(torch, v["dtype"])).reshape(v["shape"]) for k, v in rec.items()}


@pytest.mark.parametrize("rec", DATA["modules"], ids=[m["meta"]["model_type"] for m in DATA["modules"]])
def test_predictor_output_matches_the_reference(rec):
    module = module_from_payload({**rec["meta"], "state_dict": state_dict(rec["state"])}, D, E).eval()
    want = torch.tensor(rec["output"], dtype=torch.float32)
    with torch.no_grad():
        torch.testing.assert_close(module(X), want, rtol=1e-6, atol=1e-7)
        torch.testing.assert_close(module(X.view(2, 3, D)), want, rtol=1e-6, atol=1e-7)   # [B,S,H] is flattened
    assert set(module.state_dict()) == set(rec["state"])
    if rec["meta"]["model_type"] == "independent_light_logits_rs":
        sd = {k: np.asarray(v["data"], np.float32).reshape(v["shape"]) for k, v in rec["state"].items()}
        got = ref_rs.routing_scout_forward(X.numpy(), sd["mlp.0.weight"], sd["mlp.0.bias"], sd["mlp.1.weight"],
                                           sd["mlp.1.bias"], sd["mlp.1.running_mean"], sd["mlp.1.running_var"],
                                           sd["mlp.4.weight"], sd["mlp.4.bias"])
        np.testing.assert_allclose(got, want.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("rec", DATA["directories"], ids=[d["name"] for d in DATA["directories"]])
def test_directory_loading_matches_the_reference(rec, tmp_path):
    by_type = {m["meta"]["model_type"]: m for m in DATA["modules"]}
    for f in rec["files"]:
        src = by_type[f["model_type"]]
        torch.save({**src["meta"], **f["extra"], f["state_key"]: state_dict(src["state"])}, tmp_path / f["file"])
    if "error" in rec:
        with pytest.raises(RuntimeError, match=rec["error"].rstrip(":")):
            load_rs_bank(str(tmp_path), rec["num_layers"], D, E, require_complete=rec["require_complete"])
        return
    bank, sources, missing = load_rs_bank(str(tmp_path), rec["num_layers"], D, E,
                                          require_complete=rec["require_complete"])
    assert sources == rec["sources"] and missing == rec["missing"]
    assert [type(m).__name__ for m in bank] == rec["classes"]
    assert all(isinstance(m, (RoutingScoutMLP, RoutingScoutResidualMLP)) and not m.training for m in bank)
    for module, want in zip(bank, rec["outputs"]):
        if want is not None:
            with torch.no_grad():
                torch.testing.assert_close(module(X), torch.tensor(want), rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("rec", DATA["router_topk_feature"], ids=lambda r: f"{r['dtype']}-E{r['num_experts']}")
def test_router_topk_feature_matches_the_reference(rec):
    """The extra predictor input of ``feature_mode="hidden_router_topk"`` against the rows the
    reference's own method returned: bit for bit from the host code (same PyTorch ops on the
    same CPU), to float32 rounding from the numpy oracle."""
    from sparse_amd.rs import router_topk_feature
    idx = torch.tensor(rec["idx"])
    w = torch.tensor(rec["w"], dtype=torch.float32).to(getattr(torch, rec["dtype"]))
    want = torch.tensor(rec["feat"], dtype=torch.float32)
    got = router_topk_feature(idx, w, rec["num_experts"])
    assert got.dtype == torch.float32 and torch.equal(got, want)
    np.testing.assert_allclose(ref_rs.router_topk_feature(rec["idx"], w.float().numpy(), rec["num_experts"]),
                               want.numpy(), rtol=2e-7, atol=0)
    assert torch.allclose(got.sum(1), torch.ones(len(idx)))


def test_router_topk_feature_by_hand():
    feat = ref_rs.router_topk_feature([[2, 0], [1, 3]], [[1.0, 3.0], [0.0, 0.0]], 4)
    assert feat.tolist() == [[0.75, 0.0, 0.25, 0.0], [0.0, 0.0, 0.0, 0.0]]      # an all-zero row stays zero


def test_checkpoint_asking_for_the_router_topk_feature(tmp_path):
    """What the loader leaves on the modules, and the prediction from hidden state + feature."""
    from sparse_amd.rs import router_topk_feature
    rec = DATA["feature_checkpoint"]
    torch.save({**rec["meta"], "state_dict": state_dict(rec["state"])}, tmp_path / "rs_l1_inL0.pth")
    bank, sources, missing = load_rs_bank(str(tmp_path), 2, D, E, require_complete=True)
    assert [str(getattr(m, "rs_feature_mode", "hidden")) for m in bank] == rec["feature_modes"]
    feat = router_topk_feature(torch.tensor(rec["idx"]), torch.tensor(rec["w"]), E)
    with torch.no_grad():
        got = bank[1](torch.cat([X, feat], dim=-1))
    torch.testing.assert_close(got, torch.tensor(rec["output"]), rtol=1e-6, atol=1e-7)
