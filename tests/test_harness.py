"""Host logic of the decoder-stack harness: the phase / call-id protocol and the loader of
next-layer predictor directories.  The protocol is the one the reference's generation loop
follows (utils/eval_core.py:18463-18600) and its boundary test pins
(tests/test_prefill_cache_boundary.py:52-78); the directory rules are those of
utils/eval_core.py:3553-3658."""
import os

import pytest
import torch

from sparse_amd import harness
from sparse_amd.context import Metrics, SparseContext
from sparse_amd.rs import (RoutingScoutMLP, RoutingScoutResidualMLP, load_rs_bank, module_from_payload)
from tests.toy_lm import ToyCausalLM


class _Plain(torch.nn.Module):
    def forward(self, x):
        return torch.tanh(x)


def test_greedy_decode_sets_phase_and_call_ids():
    SparseContext.reset()
    model = ToyCausalLM(50, 16, [_Plain(), _Plain()])
    ids = torch.tensor([[1, 2, 3], [4, 5, 6]])
    mask = torch.ones_like(ids)
    m = Metrics()
    out = harness.greedy_decode(model, ids, mask, max_new_tokens=4, metrics=m)
    assert out.shape == (2, 7) and torch.equal(out[:, :3], ids)
    assert [c[:2] for c in model.calls] == [("prefill", 0), ("decode", 1), ("decode", 2), ("decode", 3)]
    assert [c[2] for c in model.calls] == [(2, 3), (2, 1), (2, 1), (2, 1)]
    assert [c[3] for c in model.calls] == [3, 4, 5, 6]            # the mask grows by one column per step
    assert [c[4] for c in model.calls] == [False, True, True, True]
    assert SparseContext.current_phase == "none"
    assert SparseContext.prefill_scp_transient_demoted_for_decode     # boundary hook ran once
    assert m.timings_ms["wall_prefill"] > 0 and m.timings_ms["wall_decode"] > 0
    # greedy: each new token is the argmax of the previous call's last logits
    model2 = ToyCausalLM(50, 16, [_Plain(), _Plain()])
    first = model2(ids).logits[:, -1].argmax(-1)
    assert torch.equal(out[:, 3], first)


def test_begin_request_clears_the_boundary_flag():
    SparseContext.reset()
    SparseContext.prefill_scp_transient_demoted_for_decode = True
    harness.begin_request()
    assert not SparseContext.prefill_scp_transient_demoted_for_decode


def test_decoder_layers_lookup():
    model = ToyCausalLM(10, 8, [_Plain()])
    assert harness.decoder_layers(model) == list(model.model.layers)
    assert harness.decoder_layers(model.model) == list(model.model.layers)
    assert not harness.looks_like_sparse_moe_block(_Plain())


# ---- predictor checkpoints ---------------------------------------------------------------
# Parameter names a checkpoint of the deeper predictor carries (module tree of
# utils/eval_core.py:3419-3464 with two residual units).
RESIDUAL_KEYS = {
    "input.0.weight", "input.0.bias", "input.1.weight", "input.1.bias",
    "blocks.0.net.0.weight", "blocks.0.net.0.bias", "blocks.0.net.1.weight", "blocks.0.net.1.bias",
    "blocks.0.net.4.weight", "blocks.0.net.4.bias",
    "blocks.1.net.0.weight", "blocks.1.net.0.bias", "blocks.1.net.1.weight", "blocks.1.net.1.bias",
    "blocks.1.net.4.weight", "blocks.1.net.4.bias",
    "out_norm.weight", "out_norm.bias", "head.weight", "head.bias",
}
LIGHT_KEYS = {"mlp.0.weight", "mlp.0.bias", "mlp.1.weight", "mlp.1.bias", "mlp.1.running_mean",
              "mlp.1.running_var", "mlp.1.num_batches_tracked", "mlp.4.weight", "mlp.4.bias"}


def test_predictor_state_dict_keys():
    assert set(RoutingScoutResidualMLP(8, 5, hidden_dim=16, num_hidden_layers=2).state_dict()) == RESIDUAL_KEYS
    assert set(RoutingScoutMLP(8, 5, hidden_dim=16).state_dict()) == LIGHT_KEYS


def test_residual_predictor_is_a_distribution_and_matches_its_formula():
    torch.manual_seed(0)
    mod = RoutingScoutResidualMLP(8, 5, hidden_dim=16, num_hidden_layers=1).eval()
    x = torch.randn(3, 1, 8)
    p = mod(x)
    assert p.shape == (3, 5)
    torch.testing.assert_close(p.sum(-1), torch.ones(3))
    sd = mod.state_dict()
    ln = torch.nn.functional.layer_norm
    h = torch.nn.functional.gelu(ln(x.view(3, 8), (8,), sd["input.0.weight"], sd["input.0.bias"]) @ sd["input.1.weight"].T
                                 + sd["input.1.bias"])
    r = ln(h, (16,), sd["blocks.0.net.0.weight"], sd["blocks.0.net.0.bias"])
    r = torch.nn.functional.gelu(r @ sd["blocks.0.net.1.weight"].T + sd["blocks.0.net.1.bias"])
    h = h + r @ sd["blocks.0.net.4.weight"].T + sd["blocks.0.net.4.bias"]
    want = torch.softmax(ln(h, (16,), sd["out_norm.weight"], sd["out_norm.bias"]) @ sd["head.weight"].T
                         + sd["head.bias"], -1)
    torch.testing.assert_close(p, want)


def _save(dirname, layer, module, **meta):
    payload = dict(meta)
    payload["state_dict"] = module.state_dict()
    torch.save(payload, os.path.join(dirname, f"rs_l{layer}_inL{layer - 1}.pth"))


def test_load_rs_bank_next_layer_directory(tmp_path):
    d = str(tmp_path)
    torch.manual_seed(1)
    light = RoutingScoutMLP(8, 5, hidden_dim=16)
    deep = RoutingScoutResidualMLP(8, 5, hidden_dim=16, num_hidden_layers=2)
    _save(d, 1, light, model_type="independent_light_logits_rs", input_dim=8, num_experts=5, hidden_dim=16)
    _save(d, 2, deep, model_type="next_layer_residual_logits_rs", input_dim=8, num_experts=5, hidden_dim=16,
          num_hidden_layers=2, source_layer=1)
    bank, sources, missing = load_rs_bank(d, 3, 8, 5)
    assert len(bank) == 3 and sources == [-1, 0, 1] and missing == []   # layer 0 is never a target
    assert isinstance(bank[1], RoutingScoutMLP) and isinstance(bank[2], RoutingScoutResidualMLP)
    assert not bank[2].training
    x = torch.randn(4, 8)
    torch.testing.assert_close(bank[2](x), deep.eval()(x))
    torch.testing.assert_close(bank[1](x), light.eval()(x))


def test_load_rs_bank_missing_layers(tmp_path):
    d = str(tmp_path)
    _save(d, 1, RoutingScoutMLP(8, 5, hidden_dim=16), model_type="independent_light_logits_rs", input_dim=8,
          num_experts=5, hidden_dim=16)
    with pytest.raises(RuntimeError, match="incomplete"):
        load_rs_bank(d, 3, 8, 5, require_complete=True)
    bank, _, missing = load_rs_bank(d, 3, 8, 5, require_complete=False)
    assert len(bank) == 3 and len(missing) == 1 and "rs_l2_inL1.pth" in missing[0]
    with pytest.raises(NotImplementedError):
        load_rs_bank(str(tmp_path / "nothing_here_yet") if os.makedirs(tmp_path / "nothing_here_yet") is None else d,
                     3, 8, 5)


def test_payload_variants():
    plain = RoutingScoutMLP(8, 5, hidden_dim=1024)
    assert isinstance(module_from_payload(plain.state_dict(), 8, 5), RoutingScoutMLP)       # bare state dict
    assert isinstance(module_from_payload({"model_state_dict": plain.state_dict()}, 8, 5), RoutingScoutMLP)
    with pytest.raises(NotImplementedError):
        module_from_payload({"task": "cache_value_rs", "state_dict": {}}, 8, 5)
    wide = RoutingScoutMLP(8 + 5, 5, hidden_dim=1024)
    mod = module_from_payload({"model_type": "independent_light_logits_rs", "feature_mode": "hidden_router_topk",
                               "input_dim": 13, "state_dict": wide.state_dict()}, 8, 5)
    assert mod.rs_feature_mode == "hidden_router_topk"
    with pytest.raises(RuntimeError):
        module_from_payload([1, 2, 3], 8, 5)


# ---- the reference's generation loop, recorded ------------------------------------------
PROTOCOL = __import__("json").loads((__import__("pathlib").Path(__file__).resolve().parent / "golden" /
                                     "decode_protocol.json").read_text())


@pytest.mark.parametrize("rec", PROTOCOL, ids=[f"tokens{r['max_new_tokens']}-{len(r['env'])}env" for r in PROTOCOL])
def test_greedy_decode_follows_the_recorded_sequence_of_the_reference(rec, monkeypatch):
    """``tests/golden/decode_protocol.json`` holds what the reference's own
    ``greedy_decode_profiled`` did with a toy LM (written by
    ``tests/golden/make_protocol_golden.py``): phases, call ids, model calls and boundary hooks
    in order, and the generated ids."""
    from sparse_amd.block import DistributedSparseMoeBlock
    for name in ("SPARSE_SCP_TRANSIENT_PREFILL_CACHE", "SPARSE_EPIPE_DECODE_DEMOTE_PREFILL_TRANSIENT",
                 "SPARSE_SCP_CLEAR_CACHE_BEFORE_DECODE"):
        monkeypatch.delenv(name, raising=False)
    for name, value in rec["env"].items():
        monkeypatch.setenv(name, value)
    SparseContext.reset()
    log = []
    for hook in ("demote_prefill_scp_transients_for_decode", "handle_epipe_prefill_extra_cache_decode_boundary",
                 "record_prefill_scp_transient_decode_end", "record_epipe_prefill_extra_cache_decode_end",
                 "clear_all_expert_caches"):
        monkeypatch.setattr(DistributedSparseMoeBlock, hook,
                            classmethod(lambda cls, *a, _n=hook, **k: log.append(["hook", _n])))
    begin = SparseContext.begin_runtime_call.__func__
    monkeypatch.setattr(SparseContext, "begin_runtime_call",
                        classmethod(lambda cls, call_id: (log.append(["begin_runtime_call", int(call_id)]),
                                                          begin(cls, call_id))[1]))
    model = ToyCausalLM(50, 16, [_Plain(), _Plain()])
    forward = model.forward

    def logged(input_ids, attention_mask=None, use_cache=True, past_key_values=None, return_dict=True):
        log.append(["phase", SparseContext.current_phase])
        log.append(["model", list(input_ids.shape), None if attention_mask is None else int(attention_mask.shape[1]),
                    past_key_values is not None])
        return forward(input_ids, attention_mask=attention_mask, use_cache=use_cache,
                       past_key_values=past_key_values, return_dict=return_dict)

    model.forward = logged
    ids = torch.tensor(rec["input_ids"])
    out = harness.greedy_decode(model, ids, torch.ones_like(ids), rec["max_new_tokens"])
    assert out.tolist() == rec["output_ids"]

    def normal(entries):
        """One entry per model call, carrying the phase and call id in force, and the hooks."""
        seq, phase, call = [], None, None
        for e in entries:
            if e[0] == "phase":
                phase = e[1]
            elif e[0] == "begin_runtime_call":
                call = e[1]
            elif e[0] == "model":
                seq.append(["model", phase, call, *e[1:]])
            else:
                seq.append(e)
        return seq, phase

    want, want_phase = normal(rec["log"])
    got, _ = normal(log)
    assert got == want
    assert SparseContext.current_phase == want_phase == "none"
