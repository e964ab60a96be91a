"""Arithmetic of the MoE layer against vectors recorded from the reference's own functions.

``tests/golden/moe_math.json`` was written by ``tests/golden/make_moe_golden.py``: the
reference's router, all-resident expert loop, sorted-segment executor, combine, shared
expert and single-segment FFN, taken out of the reference source and run on the CPU on
small seeded inputs in fp32 and bf16.  The oracle (``oracle/ref_moe.py``), computing on the
same CPU with the same PyTorch ops, must reproduce every output bit for bit; the HIP path is
then held to the tolerances of the other GPU tests and to exact expert indices."""
import base64
import json
from pathlib import Path
from types import SimpleNamespace as NS

import numpy as np
import pytest
import torch

from oracle import ref_moe
from tests.helpers import seeded_moe_layer

CASES = json.loads((Path(__file__).resolve().parent / "golden" / "moe_math.json").read_text())


def unpack(rec):
    raw = base64.b64decode(rec["data"])
    if rec["dtype"] == "bf16":
        t = torch.from_numpy(np.frombuffer(raw, dtype=np.int16).copy()).view(torch.bfloat16)
    elif rec["dtype"] == "f32":
        t = torch.from_numpy(np.frombuffer(raw, dtype=np.float32).copy())
    else:
        t = torch.from_numpy(np.frombuffer(raw, dtype=np.int64).copy())
    return t.reshape(rec["shape"])


def load(case):
    c = NS(**{k: v for k, v in case.items() if not isinstance(v, (dict, list)) or k == "shape"})
    if case["seeded"]:
        dtype = torch.bfloat16 if case["dtype"] == "bf16" else torch.float32
        given = seeded_moe_layer(tuple(case["shape"]), case["T"], dtype, case["seed"], case["shared_gate"])
        assert given["checksum"] == case["checksum"], "the seeded inputs are not the ones the fixture was recorded on"
        c.x, c.gate_w, c.experts = given["x"], given["gate_w"], given["experts"]
        c.shared, c.shared_gate_w = given["shared"], given["shared_gate_w"]
    else:
        c.x, c.gate_w = unpack(case["x"]), unpack(case["gate_w"])
        c.experts = [tuple(unpack(w) for w in triple) for triple in case["experts"]]
        c.shared = tuple(unpack(w) for w in case["shared"]) if case["shared"] else None
        c.shared_gate_w = unpack(case["shared_gate_w"]) if case["shared_gate_w"] else None
    c.want = {k: unpack(case[k]) for k in ("topv", "topi", "logits", "experts_world1_exact", "parts_sorted_segment",
                                           "combined", "shared_out", "layer_out", "segment_expert1") if k in case}
    return c


def _id(case):
    return f"{case['dtype']}-H{case['shape'][0]}-E{case['shape'][1]}-K{case['shape'][3]}-T{case['T']}"


@pytest.mark.parametrize("case", CASES, ids=[_id(c) for c in CASES])
def test_oracle_reproduces_the_reference_bit_for_bit(case):
    c = load(case)
    K = c.shape[3]
    topv, topi, logits = ref_moe.routing_router(c.x, c.gate_w, K, c.renorm)
    assert torch.equal(logits, c.want["logits"]) and logits.dtype == c.x.dtype
    assert torch.equal(topv, c.want["topv"]) and topv.dtype == c.x.dtype and topi.dtype == torch.int64
    # equal probabilities (they happen in bf16) come out of torch.topk in no particular order:
    # the oracle's rule is "lower id first", so compare the order only where nothing ties
    probs = torch.softmax(logits, dim=-1, dtype=torch.float32)
    chosen = torch.gather(probs, 1, c.want["topi"])
    kth = chosen[:, -1:]
    tied = ((chosen[:, 1:] == chosen[:, :-1]).any(1) if K > 1 else torch.zeros(len(probs), dtype=torch.bool)) \
        | ((probs == kth).sum(1) > (chosen == kth).sum(1))
    assert torch.equal(topi[~tied], c.want["topi"][~tied])
    assert torch.equal(torch.gather(probs, 1, topi), chosen)           # same probabilities chosen everywhere
    inside = ~((probs == kth).sum(1) > (chosen == kth).sum(1))         # tie inside the chosen set only
    assert torch.equal(torch.sort(topi[inside], 1).values, torch.sort(c.want["topi"][inside], 1).values)
    topi = c.want["topi"]                                              # continue on the reference's choice
    exact = ref_moe.experts_world1_exact(c.x, topi, topv, c.experts)
    assert torch.equal(exact, c.want["experts_world1_exact"])
    # the EP form: same parts per (token, slot), same combined sum
    T, H = c.x.shape
    combined = ref_moe.execute_sorted_segments(c.x, topi, topv, c.experts, stable=False)   # the reference's argsort
    shared = ref_moe.shared_expert_forward(c.x, c.shared, c.shared_gate_w)
    assert torch.equal(exact + shared, c.want["layer_out"])
    if not bool(tied.any()):
        out, _, _, _ = ref_moe.moe_forward(c.x, c.gate_w, c.experts, K, c.shared, c.shared_gate_w, c.renorm)
        assert torch.equal(out, c.want["layer_out"])
    if case["seeded"]:
        assert torch.equal(combined, exact) == case["combined_equals_exact"]
        assert float((combined.float() - exact.float()).abs().max()) == case["combined_maxdiff"]
        return
    assert torch.equal(combined, c.want["combined"])
    torch.testing.assert_close(ref_moe.execute_sorted_segments(c.x, topi, topv, c.experts).float(),
                               c.want["combined"].float(), rtol=1e-6, atol=1e-7)             # rows in stable order
    assert torch.equal(ref_moe.combine_expert_outputs(c.want["parts_sorted_segment"].view(T, K, H), topi),
                       c.want["combined"])
    assert case["parts_unique_mask_maxdiff"] <= 1e-6          # the reference's two executor modes agree
    assert torch.equal(shared, c.want["shared_out"])
    seg = ref_moe.expert_forward(c.x[:3], c.experts[1]) * topv[:3, :1].to(c.x.dtype)
    assert torch.equal(seg, c.want["segment_expert1"])


def test_fixture_shape():
    assert {c["dtype"] for c in CASES} == {"f32", "bf16"}
    assert any(c["renorm"] for c in CASES) and any(c["shape"][4] == 0 for c in CASES)
    assert any(c["shape"][4] and not c["shared_gate"] for c in CASES)
    assert sum(1 for c in CASES if c["seeded"]) >= 6


DEVICE_CASES = [c for c in CASES if c["seeded"]]       # layers of the kernels' granularity (multiples of 64)


@pytest.mark.gpu
@pytest.mark.parametrize("case", DEVICE_CASES, ids=[_id(c) for c in DEVICE_CASES])
def test_hip_block_against_the_reference_vectors(device, case):
    """The whole block on the GPU from the fixture's weights: expert indices exact (the
    fixture's logits are well separated at these sizes), weights, logits and the layer
    output within the bf16 / fp32 tolerances used throughout."""
    from sparse_amd.block import DistributedSparseMoeBlock
    from sparse_amd.context import DistEnv, SparseContext
    c = load(case)
    H, E, I, K, Is = c.shape
    dtype = c.x.dtype

    def lin(w):
        return NS(weight=w)

    def mlp(triple):
        return NS(gate_proj=lin(triple[0]), up_proj=lin(triple[1]), down_proj=lin(triple[2]), act_fn=torch.nn.SiLU())

    block = NS(gate=lin(c.gate_w), experts=[mlp(t) for t in c.experts], norm_topk_prob=c.renorm)
    if c.shared is not None:
        block.shared_expert = mlp(c.shared)
        block.shared_expert_gate = lin(c.shared_gate_w.view(1, -1)) if c.shared_gate_w is not None else None
    SparseContext.reset()
    blk = DistributedSparseMoeBlock(0, block, None, DistEnv(0, 1, 0, device), num_layers=1, num_experts=E, top_k=K,
                                    dtype=dtype, expert_offload="gpu")
    T = c.x.shape[0]
    ret = blk(c.x.view(1, T, H).to(device))
    out, logits = ret if isinstance(ret, tuple) else (ret, None)
    torch.cuda.synchronize()
    ws = blk._workspace(T)
    tol = dict(rtol=2e-2, atol=1e-2) if dtype == torch.bfloat16 else dict(rtol=1e-5, atol=1e-5)
    if logits is not None:
        torch.testing.assert_close(logits.cpu().float(), c.want["logits"].float(),
                                   **(dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else tol))
    # indices: exact, on every row, given the logits the device itself wrote
    if logits is not None:
        _, own_i, _ = ref_moe.routing_router(c.x, c.gate_w, K, c.renorm, router_logits=logits.cpu())
        assert torch.equal(ws.topi.cpu(), own_i)
    # against the reference's recorded run: its logits differ from the device's in the order of
    # the sum, so a token whose K-th and (K+1)-th logits nearly tie may route elsewhere; rows
    # that chose the reference's experts (nearly all) are held to the recorded layer output
    got = out.view(T, H).cpu().float()
    got_i = torch.sort(ws.topi.cpu(), 1).values
    same = (got_i == torch.sort(c.want["topi"], 1).values).all(dim=1)
    assert float(same.float().mean()) >= 0.9, "too few rows route like the reference for the comparison to mean much"
    torch.testing.assert_close(got[same], c.want["layer_out"].float()[same], **tol)
    # the other rows: the oracle on the device's own routing
    if not bool(same.all()):
        want = ref_moe.moe_forward_routed(c.x, ws.topv.cpu(), ws.topi.cpu(), c.experts, c.shared, c.shared_gate_w)
        torch.testing.assert_close(got[~same], want.float()[~same], **tol)
    # the output scale is that of the full-size layers, so atol 1e-2 bites
    assert 0.05 < float(c.want["layer_out"].float().abs().mean()) < 2.0
