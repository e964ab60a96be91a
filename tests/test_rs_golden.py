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
