"""GPU parity of the fp16 path (the reference's formal dtype, scripts/run/run_case.sh:199) against the CPU
oracle run in fp16: the same kernels as bf16 with IEEE-half conversions and the fp16 MFMA.

Indices and permutations bit for bit; values within rtol 5e-3 / atol 2e-3 (fp16 keeps 11 significant
bits where bf16 keeps 8, so the bound is tighter than the bf16 one the north star states; what remains
is the order of the fp32 sums before each rounding)."""
import pytest
import torch

from oracle import ref_moe
from tests.helpers import make_hidden, make_layer
from tests.test_gpu_kernels import _ops, _routing, _run_routed

pytestmark = pytest.mark.gpu

F16 = torch.float16
FP16_TOL = dict(rtol=5e-3, atol=2e-3)


def _rel(a, b):
    return float((a.float() - b.float()).abs().max() / b.float().abs().max())


@pytest.mark.parametrize("T", [1, 8, 33, 128])
def test_router_logits_fp16(device, T):
    """T >= 64 takes the MFMA kernel, smaller calls the FMA one; logits in fp16 or fp32."""
    ops = _ops()
    layer = make_layer(2048, 60, 64, 4, Is=64, shared_gate=True, dtype=F16, seed=3)
    x = make_hidden(T, 2048, F16, seed=4)
    ref = torch.nn.functional.linear(x.float(), layer["gate_w"].float())
    ref_sg = torch.nn.functional.linear(x.float(), layer["shared_gate_w"].float().reshape(1, -1)).reshape(-1)
    logits, sg = ops.router_logits(x.to(device), layer["gate_w"].to(device), layer["shared_gate_w"].to(device))
    assert logits.dtype == F16 and sg.dtype == F16
    torch.testing.assert_close(logits.float().cpu(), ref, rtol=2e-3, atol=2e-3)
    torch.testing.assert_close(sg.float().cpu(), ref_sg, rtol=2e-3, atol=2e-3)
    l32, _ = ops.router_logits(x.to(device), layer["gate_w"].to(device), logits_dtype=torch.float32)
    assert l32.dtype == torch.float32
    torch.testing.assert_close(l32.cpu(), ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("E,K", [(60, 4), (64, 6), (200, 8)])
def test_gate_topk_fp16_logits_and_weights(device, E, K):
    """Indices are a function of the logits alone (descending, then lower id), also where fp16 logits
    tie around the K-th place; weights are the softmax probabilities rounded to fp16."""
    ops = _ops()
    g = torch.Generator().manual_seed(E * 100 + K)
    logits = (torch.randn(257, E, generator=g) * 2.0).to(F16)
    srt = torch.sort(logits.float(), dim=-1, descending=True)
    for t in range(0, 257, 3):
        a, b = int(srt.indices[t, K - 1]), int(srt.indices[t, K])
        logits[t, b] = logits[t, a]
    probs = torch.softmax(logits, dim=-1, dtype=torch.float32)
    ref_v, ref_i = ref_moe.topk_by_logit(logits, probs, K)
    topv, topi = ops.gate_topk(logits.to(device), K, out_dtype=F16)
    assert topv.dtype == F16
    assert torch.equal(topi.cpu(), ref_i)
    torch.testing.assert_close(topv.cpu().float(), ref_v.to(F16).float(), rtol=2e-3, atol=1e-6)
    topv32, topi32 = ops.gate_topk(logits.to(device), K, out_dtype=torch.float32)
    assert torch.equal(topi32.cpu(), ref_i)
    torch.testing.assert_close(topv32.cpu(), ref_v.float(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("T", [1, 8, 32])
def test_route_decode_fp16_equals_the_three_separate_calls(device, T):
    ops = _ops()
    E, K, H = 60, 4, 2048
    layer = make_layer(H, E, 64, K, Is=64, shared_gate=True, dtype=F16, seed=7)
    wg, wsg = layer["gate_w"].to(device), layer["shared_gate_w"].to(device)
    counter = torch.zeros(1, dtype=torch.int32, device=device)
    for rep in range(2):
        x = make_hidden(T, H, F16, seed=100 + rep).to(device)
        logits_a, sg_a = ops.router_logits(x, wg, wsg)
        logits_b, sg_b = torch.empty_like(logits_a), torch.empty_like(sg_a)
        topv_b = torch.empty(T, K, dtype=F16, device=device)
        topi_b = torch.empty(T, K, dtype=torch.int64, device=device)
        perm_b = ops.Permutation(T, K, E, device)
        ops.route_decode(x, wg, wsg, K, False, logits_b, sg_b, topv_b, topi_b, perm_b, counter)
        torch.cuda.synchronize()
        assert int(counter.item()) == 0
        torch.testing.assert_close(logits_b.float(), logits_a.float(), rtol=1e-3, atol=1e-6)   # one fp16 ulp
        torch.testing.assert_close(sg_b.float(), sg_a.float(), rtol=1e-3, atol=1e-6)
        topv_a, topi_a = ops.gate_topk(logits_b, K, out_dtype=F16)
        perm_a = ops.permute_build(topi_a, E)
        torch.cuda.synchronize()
        assert torch.equal(topv_a, topv_b) and torch.equal(topi_a, topi_b)
        for name in ("perm", "inv_perm", "seg_offsets"):
            assert torch.equal(getattr(perm_a, name), getattr(perm_b, name)), name


@pytest.mark.parametrize("ldt", [F16, torch.float32])
@pytest.mark.parametrize("T,H,E,K,Is", [(1, 2048, 60, 4, 5632), (8, 2048, 60, 4, 5632), (16, 2048, 63, 6, 2816),
                                        (5, 192, 15, 3, 96)])
def test_route_decode_packed_fp16(device, T, H, E, K, Is, ldt):
    """The one-workgroup router on the packed gate matrix in fp16, alone and with the shared expert's gate and up
    projections beside it: logits against fp32 linear algebra, top-k and permutation bit for bit what gate_topk
    and permute_build return on the logits it wrote, SiLU(gate x) * (up x) within the fp16 bound of fp32 linear
    algebra rounded the way the expert kernels round, and the same bits from the stand-alone launch."""
    from sparse_amd.weights import tile_weight
    ops = _ops()
    layer = make_layer(H, E, 64, K, Is=Is, shared_gate=True, dtype=F16, seed=23 + T, std=0.05)
    packed = ops.pack_router_gate(layer["gate_w"].to(device), layer["shared_gate_w"].to(device))
    assert packed is not None and packed.dtype == F16 and packed.numel() == 64 * H
    gw, uw = (tile_weight(w.to(device)).reshape(w.shape).contiguous() for w in layer["shared"][:2])
    x = make_hidden(T, H, F16, seed=400 + T)
    xd = x.to(device)

    def route(shared_up):
        logits = torch.empty(T, E, dtype=ldt, device=device)
        sg = torch.empty(T, dtype=F16, device=device)
        topv = torch.empty(T, K, dtype=F16, device=device)
        topi = torch.empty(T, K, dtype=torch.int64, device=device)
        perm = ops.Permutation(T, K, E, device)
        ops.route_decode_packed(xd, packed, E, True, K, False, logits, sg, topv, topi, perm, shared_up=shared_up)
        torch.cuda.synchronize()
        return logits, sg, topv, topi, perm

    inter = torch.full((T, Is), float("nan"), dtype=F16, device=device)
    a, b = route(None), route((gw, uw, inter))
    for u, v in zip(a[:4], b[:4]):
        assert torch.equal(u, v)
    for name in ("perm", "inv_perm", "seg_offsets", "n_active"):
        assert torch.equal(getattr(a[4], name), getattr(b[4], name)), name
    logits, sg, topv, topi, perm = a
    ref = torch.nn.functional.linear(x.float(), layer["gate_w"].float())
    tol = dict(rtol=2e-3, atol=2e-3) if ldt == F16 else dict(rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(logits.float().cpu(), ref, **tol)
    ref_sg = torch.nn.functional.linear(x.float(), layer["shared_gate_w"].float().reshape(1, -1)).reshape(-1)
    torch.testing.assert_close(sg.float().cpu(), ref_sg, rtol=2e-3, atol=2e-3)
    topv_a, topi_a = ops.gate_topk(logits, K, out_dtype=F16)
    perm_a = ops.permute_build(topi_a, E)
    torch.cuda.synchronize()
    assert torch.equal(topv_a, topv) and torch.equal(topi_a, topi)
    n = int(perm_a.n_active.item())
    assert n == int(perm.n_active.item())
    for name in ("perm", "inv_perm", "seg_offsets"):
        assert torch.equal(getattr(perm_a, name), getattr(perm, name)), name
    g = torch.nn.functional.linear(x.float(), layer["shared"][0].float()).to(F16).float()
    u = torch.nn.functional.linear(x.float(), layer["shared"][1].float()).to(F16).float()
    want = (torch.nn.functional.silu(g).to(F16).float() * u).to(F16)
    got = inter.cpu()
    assert not torch.isnan(got.float()).any()
    torch.testing.assert_close(got.float(), want.float(), **FP16_TOL)
    alone = torch.empty_like(inter)
    ops.shared_gate_up(xd, gw, uw, alone)
    torch.cuda.synchronize()
    assert torch.equal(alone, inter)


@pytest.mark.parametrize("T", [1, 8, 16])
@pytest.mark.parametrize("gated", [True, False])
def test_fused_decode_fp16_with_the_shared_reduction_split(device, T, gated):
    """The fp16 decode launch pair with the shared expert's down projection left as fp32 partial sums: finished
    by combine_split, and by the down launch itself (moe_ffn_decode_combine) with the same bits; routed parts
    those of the one-workgroup form, the output within tolerance of the oracle."""
    from sparse_amd.weights import ExpertSlab, tile_weight
    ops = _ops()
    H, E, I, K, Is = 512, 8, 128, 2, 1024
    layer = make_layer(H, E, I, K, Is=Is, shared_gate=gated, dtype=F16, seed=81, std=0.05)
    xc = make_hidden(T, H, F16, seed=82)
    x = xc.to(device)
    slab = ExpertSlab.resident(layer["experts"], H, I, F16, device)
    experts = ops.make_experts(slab.data, slab.expert_slot, E, H, I)
    logits, sg = ops.router_logits(x, layer["gate_w"].to(device), layer["shared_gate_w"].to(device) if gated else None)
    topv, topi = ops.gate_topk(logits, K, out_dtype=F16)
    perm = ops.permute_build(topi, E)
    segs = ops.seglist_device(perm, min(E, T * K))
    sw = tuple(tile_weight(t).reshape(t.shape).contiguous().to(device) for t in layer["shared"])
    nparts = ops.decode_split_parts(Is)
    ws = ops.decode_split_workspace(T, H, device)

    def run(mode):
        inter = torch.empty((T * K, I), device=device, dtype=F16)
        parts = torch.empty((T * K, H), device=device, dtype=F16)
        sh_inter = torch.empty((T, Is), device=device, dtype=F16)
        sh_out = torch.empty((T, H), device=device, dtype=F16)
        out = torch.full((T, H), float("nan"), device=device, dtype=F16)
        if mode == "plain":
            ops.moe_ffn_decode(experts, x, topv, perm, segs, inter, parts, sw, sg if gated else None, sh_inter, sh_out, None)
            ops.combine(parts, perm, sh_out, T, K, out)
        elif mode == "split":
            ops.moe_ffn_decode(experts, x, topv, perm, segs, inter, parts, sw, sg if gated else None, sh_inter, sh_out, ws)
            ops.combine_split(parts, perm, ws, nparts, sg if gated else None, T, K, out)
        else:
            ops.moe_ffn_decode_combine(experts, x, topv, perm, segs, inter, parts, sw, sg if gated else None, sh_inter,
                                       ws, out)
        torch.cuda.synchronize()
        return parts, out

    parts0, out0 = run("plain")
    ref, _, _, _ = ref_moe.moe_forward(xc, layer["gate_w"], layer["experts"], K, layer["shared"], layer["shared_gate_w"],
                                       router_logits=logits.cpu())
    parts1, out1 = run("split")
    parts2, out2 = run("fold")
    assert torch.equal(parts1, parts0) and torch.equal(parts2, parts0)
    assert not torch.isnan(out1.float()).any() and torch.equal(out1, out2)
    torch.testing.assert_close(out1.float(), out0.float(), rtol=2e-3, atol=1e-6)   # two fp16 roundings apart at most
    torch.testing.assert_close(out1.cpu().float(), ref.float(), **FP16_TOL)
    _, again = run("fold")
    assert torch.equal(again, out2)


@pytest.mark.parametrize("T", [1, 8, 17, 32])
def test_decode_ffn_fp16_matches_oracle(device, T):
    ops = _ops()
    layer = make_layer(512, 12, 256, 4, dtype=F16, seed=11, std=0.05)
    x = make_hidden(T, 512, F16, seed=12)
    topv, topi = _routing(layer, x)
    out, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=True)
    ref = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    torch.testing.assert_close(out.float(), ref.float(), **FP16_TOL)
    assert _rel(out, ref) < 5e-3   # a bf16 instruction on fp16 bits, or a wrong mapping, gives O(1)


@pytest.mark.parametrize("T", [40, 300])
def test_prefill_ffn_fp16_matches_oracle(device, T):
    ops = _ops()
    layer = make_layer(512, 12, 256, 4, dtype=F16, seed=21, std=0.05)
    x = make_hidden(T, 512, F16, seed=22)
    topv, topi = _routing(layer, x)
    out, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=False)
    ref = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    torch.testing.assert_close(out.float(), ref.float(), **FP16_TOL)
    assert _rel(out, ref) < 5e-3


def test_ffn_fp16_at_the_qwen_shape(device):
    ops = _ops()
    layer = make_layer(2048, 60, 1408, 4, dtype=F16, seed=0)
    x = make_hidden(8, 2048, F16, seed=1000)
    topv, topi = _routing(layer, x)
    ref = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    for decode in (True, False):
        out, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=decode)
        torch.testing.assert_close(out.float(), ref.float(), **FP16_TOL)
        assert _rel(out, ref) < 5e-3


@pytest.mark.parametrize("T", [8, 32, 200])
@pytest.mark.parametrize("gated", [True, False])
def test_shared_expert_fp16(device, T, gated):
    ops = _ops()
    layer = make_layer(512, 4, 64, 2, Is=384, shared_gate=gated, dtype=F16, seed=61, std=0.05)
    x = make_hidden(T, 512, F16, seed=62)
    ref = ref_moe.shared_expert_forward(x, layer["shared"], layer["shared_gate_w"])
    xd = x.to(device)
    sg = None
    if gated:
        _, sg = ops.router_logits(xd, layer["gate_w"].to(device), layer["shared_gate_w"].to(device))
    from sparse_amd.weights import tile_weight
    gw, uw, dw = (tile_weight(t).reshape(t.shape).contiguous().to(device) for t in layer["shared"])
    inter = torch.empty((T, 384), device=device, dtype=F16)
    out = torch.empty((T, 512), device=device, dtype=F16)
    ops.shared_expert(xd, gw, uw, dw, sg, inter, out)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **FP16_TOL)


def test_combine_fp16_is_the_ordered_sum(device):
    ops = _ops()
    T, K, H, E = 37, 4, 256, 20
    g = torch.Generator().manual_seed(71)
    topi = torch.topk(torch.rand(T, E, generator=g), K, dim=1).indices.to(torch.int64)
    parts_tkh = (torch.randn(T, K, H, generator=g) * 3).to(F16)
    shared = torch.randn(T, H, generator=g).to(F16)
    ref = ref_moe.combine_expert_outputs(parts_tkh, topi) + shared
    p = ops.permute_build(topi.to(device), E)
    parts_sorted = parts_tkh.reshape(T * K, H)[p.perm.cpu().long()].contiguous().to(device)
    out = torch.empty((T, H), device=device, dtype=F16)
    ops.combine(parts_sorted, p, shared.to(device), T, K, out)
    assert torch.equal(out.cpu(), ref)   # same adds in the same order: bit for bit


SMALL_Q = dict(family="qwen_shared", hidden=512, num_experts=12, inter=256, top_k=4, shared_inter=384)
SMALL_D = dict(family="deepseek_shared", hidden=512, num_experts=16, inter=256, top_k=6, shared_inter=512)


def _check_block(shape, T, device, fused=False, seed=0):
    from sparse_amd.synthetic import make_hidden as mk
    from tests.helpers import oracle_layer
    from tests.test_gpu_block import _build
    mlp, blk = _build(shape, F16, device, seed=seed, fused=fused)
    H = shape["hidden"]
    x = mk(T, H, F16, seed=1000 + seed)
    ret = blk(x.view(1, T, H).to(device))
    torch.cuda.synchronize()
    lay = oracle_layer(mlp)
    ws = blk._workspace(T)
    if lay["family"] == "qwen_shared":
        out, logits = ret
        logits = logits.cpu()
        assert logits.dtype == F16
    else:
        out = ret
        from sparse_amd import ops
        logits, _ = ops.router_logits(x.to(device), blk.gate_weight, None, torch.float32)
        logits = logits.cpu()
    ref_out, ref_topv, ref_topi, _ = ref_moe.moe_forward(
        x, lay["gate_w"], lay["experts"], shape["top_k"], lay["shared"], lay["shared_gate_w"],
        family=lay["family"], router_logits=logits)
    topi_dev = ws.topi.cpu()
    if lay["family"] == "qwen_shared":
        assert torch.equal(topi_dev, ref_topi), "expert indices differ on identical logits"
    else:
        assert torch.equal(torch.sort(topi_dev, 1).values, torch.sort(ref_topi, 1).values)
    out = out.cpu().view(T, H)
    assert out.dtype == F16
    torch.testing.assert_close(out.float(), ref_out.float(), **FP16_TOL)
    assert _rel(out, ref_out) < 5e-3


@pytest.mark.parametrize("T", [1, 8, 32, 33, 130])
def test_small_qwen_block_fp16(device, T):
    _check_block(SMALL_Q, T, device)


@pytest.mark.parametrize("T", [4, 200])
def test_small_deepseek_block_fp16(device, T):
    _check_block(SMALL_D, T, device, fused=True)


def test_qwen_shape_fp16_decode_and_prefill(device):
    from sparse_amd.synthetic import QWEN
    for T in (8, 160):
        _check_block(QWEN, T, device, seed=1)


@pytest.mark.parametrize("method", ["rr", "rs-epipe"])
def test_offloaded_fp16_stack_gives_the_resident_bits(device, method):
    """Residency decides where the weights come from and in which order experts run, never the values:
    an fp16 stack with 4 of 12 experts cached gives, bit for bit, what the all-resident fp16 stack gives,
    over a prefill call and decode steps, with misses, prefetches and staged copies on the way."""
    from tests.test_gpu_offload import _run, _stack
    blocks, metrics = _stack(device, method, 4, 3, "cpu", dtype=F16)
    got = _run(blocks, device, 7, 4, prefill_first=True, dtype=F16)
    assert metrics.cache_miss_count > 0 and got[0].dtype == F16
    resident, _ = _stack(device, method, 4, 3, "gpu", dtype=F16)
    want = _run(resident, device, 7, 4, prefill_first=True, dtype=F16)
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert torch.equal(a, b), f"call {i}: offloaded and resident outputs differ"
