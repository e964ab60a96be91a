"""The decoder-stack harness on the GPU: sparse MLPs of a toy causal LM are swapped for the
HIP block and greedy generation must follow the same tokens as the CPU oracle evaluating the
same weights, with all experts resident and with experts offloaded behind a small cache and
a predictor bank loaded from a checkpoint directory."""
import copy
import os

import pytest
import torch

from tests.toy_lm import OracleMoe, ToyCausalLM

pytestmark = pytest.mark.gpu

SHAPE = dict(family="qwen_shared", hidden=512, num_experts=12, inter=256, top_k=4, shared_inter=384)
LAYERS, VOCAB = 3, 97


def _mlps(dtype):
    from sparse_amd.synthetic import make_mlp_block
    return [make_mlp_block(SHAPE, dtype=dtype, seed=10 + l) for l in range(LAYERS)]


def _reference_tokens(ids, mask, new_tokens):
    from sparse_amd import harness
    from sparse_amd.context import SparseContext
    SparseContext.reset()
    model = ToyCausalLM(VOCAB, SHAPE["hidden"], [OracleMoe(m, SHAPE["top_k"]) for m in _mlps(torch.float32)])
    out = harness.greedy_decode(model, ids, mask, new_tokens)
    first_logits = ToyCausalLM.forward(model, ids).logits
    return out, first_logits


@pytest.mark.parametrize("family", ["qwen_shared", "deepseek_shared"])
def test_swap_and_generate_resident(device, family):
    from sparse_amd import harness
    from sparse_amd.block import DistributedSparseMoeBlock
    from sparse_amd.context import DistEnv, Metrics, SparseContext
    from sparse_amd.synthetic import make_mlp_block
    shape = dict(SHAPE, family=family)
    ids = torch.tensor([[3, 14, 15, 92, 65], [35, 89, 79, 32, 38]])
    mask = torch.ones_like(ids)

    def mlps():
        return [make_mlp_block(shape, dtype=torch.float32, seed=10 + l) for l in range(LAYERS)]

    SparseContext.reset()
    ref = ToyCausalLM(VOCAB, shape["hidden"], [OracleMoe(m, shape["top_k"]) for m in mlps()])
    want = harness.greedy_decode(ref, ids, mask, 6)
    want_logits = ref(ids).logits

    SparseContext.reset()
    model = ToyCausalLM(VOCAB, shape["hidden"], mlps())
    for m in model.model.layers:
        m.mlp.top_k = shape["top_k"]        # where Hugging Face modules keep it
    metrics = Metrics()
    blocks = harness.install_sparse_blocks(model, env=DistEnv(0, 1, 0, device), dtype=torch.float32,
                                           metrics=metrics, expert_offload="gpu")
    assert len(blocks) == LAYERS and all(isinstance(l.mlp, DistributedSparseMoeBlock) for l in model.model.layers)
    assert [b.layer_idx for b in blocks] == [0, 1, 2] and SparseContext.layer_blocks[2] is blocks[2]
    model = model.to(device)
    got_logits = model(ids.to(device)).logits.cpu()
    torch.testing.assert_close(got_logits, want_logits, rtol=1e-4, atol=1e-4)
    got = harness.greedy_decode(model, ids.to(device), mask.to(device), 6, metrics)
    assert torch.equal(got.cpu(), want)
    assert harness.install_sparse_blocks(model, env=DistEnv(0, 1, 0, device), dtype=torch.float32) == []


def test_offloaded_generation_with_predictor_directory(device, tmp_path):
    from sparse_amd import harness
    from sparse_amd.context import DistEnv, Metrics, SparseContext
    from sparse_amd.rs import informed_bank
    ids = torch.tensor([[3, 14, 15, 92, 65, 35], [89, 79, 32, 38, 46, 26]])
    mask = torch.ones_like(ids)
    want, _ = _reference_tokens(ids, mask, 8)

    # a directory of predictors, one per target layer, in the reference's naming
    mlps = _mlps(torch.float32)
    bank = informed_bank([None] + [m.gate.weight.detach() for m in mlps[1:]], hidden_dim=32)
    for layer in range(1, LAYERS):
        torch.save(dict(model_type="independent_light_logits_rs", input_dim=SHAPE["hidden"],
                        num_experts=SHAPE["num_experts"], hidden_dim=32, state_dict=bank[layer].state_dict()),
                   os.path.join(tmp_path, f"rs_l{layer}_inL{layer - 1}.pth"))

    SparseContext.reset()
    model = ToyCausalLM(VOCAB, SHAPE["hidden"], mlps)
    metrics = Metrics()
    blocks = harness.install_sparse_blocks(
        model, env=DistEnv(0, 1, 0, device), dtype=torch.float32, top_k=SHAPE["top_k"], metrics=metrics,
        rs_dir=str(tmp_path), expert_offload="cpu", expert_cache=5, planner_mode="rs_prefetch", prefetch_top_m=4)
    assert len(SparseContext.rs_bank) == LAYERS and SparseContext.rs_bank_source_layers == [-1, 0, 1]
    model = model.to(device)
    harness.begin_request()
    got = harness.greedy_decode(model, ids.to(device), mask.to(device), 8, metrics)
    assert torch.equal(got.cpu(), want)
    assert metrics.cache_miss_count > 0
    assert metrics.rs_next_layer_pred_calls > 0
    # a second request after a reset reproduces the first
    first = (metrics.cache_hit_count, metrics.prefetch_hit_count, metrics.cache_miss_count)
    harness.begin_request()
    again = harness.greedy_decode(model, ids.to(device), mask.to(device), 8, metrics)
    assert torch.equal(again.cpu(), want)
    second = (metrics.cache_hit_count - first[0], metrics.prefetch_hit_count - first[1],
              metrics.cache_miss_count - first[2])
    assert second == first
