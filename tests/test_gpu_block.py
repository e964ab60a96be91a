"""GPU parity of the whole MoE block (all experts resident) against the CPU oracle.

Routing is compared on identical router logits: the oracle is fed the logits the device
produced, so expert indices must match bit for bit; the logits themselves and the layer
output are compared within the stated tolerances (bf16: rtol 2e-2 / atol 1e-2, fp32: 1e-5).
"""
import pytest
import torch

from oracle import ref_moe
from tests.helpers import oracle_layer

pytestmark = pytest.mark.gpu

BF16_TOL = dict(rtol=2e-2, atol=1e-2)
F32_TOL = dict(rtol=1e-5, atol=1e-5)


def _build(shape, dtype, device, seed=0, fused=False, **kw):
    from sparse_amd.block import DistributedSparseMoeBlock
    from sparse_amd.context import DistEnv, SparseContext
    from sparse_amd.synthetic import make_mlp_block
    SparseContext.reset()
    mlp = make_mlp_block(shape, dtype=dtype, seed=seed, fused=fused)
    blk = DistributedSparseMoeBlock(0, mlp, None, DistEnv(0, 1, 0, device), num_layers=1,
                                    num_experts=shape["num_experts"], top_k=shape["top_k"], dtype=dtype,
                                    expert_offload="gpu", **kw)
    return mlp, blk


def _check(shape, dtype, T, device, B=None, fused=False, seed=0):
    from sparse_amd.synthetic import make_hidden
    mlp, blk = _build(shape, dtype, device, seed=seed, fused=fused)
    H = shape["hidden"]
    x = make_hidden(T, H, dtype, seed=1000 + seed)
    B = B or 1
    hid = x.view(B, T // B, H).to(device)
    ret = blk(hid)
    torch.cuda.synchronize()
    lay = oracle_layer(mlp)
    if lay["family"] == "qwen_shared":
        out, logits = ret
        logits = logits.cpu()
        assert logits.dtype == dtype and tuple(logits.shape) == (T, shape["num_experts"])
        ref_logits = torch.nn.functional.linear(x, lay["gate_w"])
        torch.testing.assert_close(logits.float(), ref_logits.float(),
                                   **(dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else F32_TOL))
    else:
        out = ret
        ws = blk._workspace(T)
        logits = None
    ws = blk._workspace(T)
    topi_dev, topv_dev = ws.topi.cpu(), ws.topv.cpu()
    if logits is None:
        # DeepSeek family: fp32 logits are internal; recompute them on the device
        from sparse_amd import ops
        logits, _ = ops.router_logits(hid.view(T, H), blk.gate_weight, None, torch.float32)
        logits = logits.cpu()
    ref_out, ref_topv, ref_topi, _ = ref_moe.moe_forward(
        x, lay["gate_w"], lay["experts"], shape["top_k"], lay["shared"], lay["shared_gate_w"],
        family=lay["family"], router_logits=logits)
    if lay["family"] == "qwen_shared":
        assert torch.equal(topi_dev, ref_topi), "expert indices differ on identical logits"
    else:
        assert torch.equal(torch.sort(topi_dev, 1).values, torch.sort(ref_topi, 1).values)
    torch.testing.assert_close(topv_dev.float(), ref_topv.float(), rtol=1e-2, atol=1e-5)
    out = out.cpu().view(T, H)
    torch.testing.assert_close(out.float(), ref_out.float(), **(BF16_TOL if dtype == torch.bfloat16 else F32_TOL))
    rel = (out.float() - ref_out.float()).abs().max() / ref_out.float().abs().max()
    assert rel < (3e-2 if dtype == torch.bfloat16 else 1e-4), f"max relative error {rel}"
    return blk


SMALL_Q = dict(family="qwen_shared", hidden=512, num_experts=12, inter=256, top_k=4, shared_inter=384)
SMALL_D = dict(family="deepseek_shared", hidden=512, num_experts=16, inter=256, top_k=6, shared_inter=512)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 8, 32, 33, 130])
def test_small_qwen_block(device, dtype, T):
    _check(SMALL_Q, dtype, T, device)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [4, 200])
def test_small_deepseek_block(device, dtype, T):
    _check(SMALL_D, dtype, T, device, fused=True)


def test_config1_qwen_fp32_128_tokens(device):
    """BASELINE config 1: Q shape, fp32, one layer, 128 tokens, seed 0."""
    from sparse_amd.synthetic import QWEN
    _check(QWEN, torch.float32, 128, device, seed=0)


def test_qwen_bf16_decode_batches(device):
    from sparse_amd.synthetic import QWEN
    for T in (1, 8, 32):
        _check(QWEN, torch.bfloat16, T, device, B=T, seed=1)


def test_deepseek_bf16_prefill_512(device):
    from sparse_amd.synthetic import DEEPSEEK
    _check(DEEPSEEK, torch.bfloat16, 512, device, seed=2)


@pytest.mark.parametrize("shape", [SMALL_Q, SMALL_D], ids=["qwen", "deepseek"])
def test_shared_expert_on_its_own_stream_changes_nothing(device, shape):
    """Prefill-size batches run the shared expert on a second stream beside the routing; the
    kernels and their inputs are the same, so the layer output is bit for bit the one-stream
    result, call after call, also when calls alternate between the two forms."""
    from sparse_amd.synthetic import make_hidden
    _, blk = _build(shape, torch.bfloat16, device, seed=3)
    assert blk.overlap_shared
    H = shape["hidden"]
    outs = {}
    for rep in range(3):
        x = make_hidden(256, H, torch.bfloat16, seed=50 + rep).view(1, 256, H).to(device)
        for overlap in (True, False, True):
            blk.overlap_shared = overlap
            ret = blk(x)
            out = (ret[0] if isinstance(ret, tuple) else ret).clone()
            torch.cuda.synchronize()
            outs.setdefault(rep, out)
            assert torch.equal(out, outs[rep]), (rep, overlap)


def test_constructor_rejects_bad_enums(device):
    from sparse_amd.block import DistributedSparseMoeBlock
    from sparse_amd.context import DistEnv
    from sparse_amd.synthetic import make_mlp_block
    mlp = make_mlp_block(SMALL_Q, dtype=torch.bfloat16)
    env = DistEnv(0, 1, 0, device)
    for kw in (dict(routing_mode="x"), dict(placement_mode="x"), dict(planner_mode="x"), dict(expert_source="x"),
               dict(expert_offload="disk"), dict(cache_policy="x"), dict(runtime_mode="x"),
               dict(expert_source="rs")):
        with pytest.raises(ValueError):
            DistributedSparseMoeBlock(0, mlp, None, env, num_layers=1, num_experts=12, top_k=4, **kw)
    # settings the reference accepts and this build does not
    for kw in (dict(oracle_mode="replay"), dict(oracle_mode="record")):
        with pytest.raises(NotImplementedError):
            DistributedSparseMoeBlock(0, mlp, None, env, num_layers=1, num_experts=12, top_k=4, **kw)


def test_deepseek_full_size_4096_tokens_properties(device):
    """BASELINE config 3 at full size (one layer).  Size-independent properties of the path:
    every output row depends on its own token only, through a k loop whose order does not
    depend on where the row sits in a tile, so (a) permuting the tokens permutes the output
    rows bit for bit and (b) two 2048-token calls give the same rows as one 4096-token call;
    (c) a sample of rows matches the CPU oracle within the bf16 tolerance."""
    from sparse_amd.synthetic import DEEPSEEK, make_hidden
    mlp, blk = _build(DEEPSEEK, torch.bfloat16, device, seed=3, fused=True)
    T, H = 4096, DEEPSEEK["hidden"]
    x = make_hidden(T, H, torch.bfloat16, seed=77)
    xd = x.to(device)
    out = blk(xd.view(1, T, H)).view(T, H).clone()
    g = torch.Generator().manual_seed(5)
    order = torch.randperm(T, generator=g)
    out_perm = blk(xd[order.to(device)].view(1, T, H)).view(T, H).clone()
    assert torch.equal(out_perm, out[order.to(device)]), "token permutation changed some output row"
    halves = torch.cat([blk(xd[:2048].view(1, 2048, H)).view(2048, H).clone(),
                        blk(xd[2048:].view(1, 2048, H)).view(2048, H).clone()])
    assert torch.equal(halves, out), "chunked calls differ from the single call"
    # decode-sized call through the other kernels: same numbers up to bf16 rounding of a few sums
    few = blk(xd[:8].view(8, 1, H)).view(8, H)
    torch.testing.assert_close(few.float(), out[:8].float(), **BF16_TOL)
    torch.cuda.synchronize()
    lay = oracle_layer(mlp)
    rows = torch.arange(0, T, 61)[:64]
    from sparse_amd import ops
    logits, _ = ops.router_logits(xd[rows.to(device)].contiguous(), blk.gate_weight, None, torch.float32)
    ref_out, _v, _i, _ = ref_moe.moe_forward(x[rows], lay["gate_w"], lay["experts"], DEEPSEEK["top_k"],
                                             lay["shared"], lay["shared_gate_w"], family=lay["family"],
                                             router_logits=logits.cpu())
    torch.testing.assert_close(out[rows.to(device)].cpu().float(), ref_out.float(), **BF16_TOL)


def test_prefill_with_empty_and_tiny_segments(device):
    """Routing that leaves most experts without tokens and gives some a single row: tokens are
    copies of a few prototypes, so only a handful of experts are hit, with segment lengths
    from 1 row to several tiles."""
    from sparse_amd.synthetic import make_hidden
    shape = dict(SMALL_D, num_experts=32)
    mlp, blk = _build(shape, torch.bfloat16, device, seed=9, fused=True)
    H = shape["hidden"]
    protos = make_hidden(3, H, torch.bfloat16, seed=4)
    idx = torch.cat([torch.zeros(300, dtype=torch.long), torch.ones(1, dtype=torch.long),
                     torch.full((129,), 2, dtype=torch.long)])
    x = protos[idx]
    T = x.shape[0]
    out = blk(x.to(device).view(1, T, H)).view(T, H).cpu()
    ws = blk._workspace(T)
    counts = torch.bincount(ws.topi.cpu().reshape(-1), minlength=shape["num_experts"])
    assert int((counts == 0).sum()) >= shape["num_experts"] - 18 and int((counts > 0).sum()) >= 6
    lay = oracle_layer(mlp)
    from sparse_amd import ops
    logits, _ = ops.router_logits(x.to(device), blk.gate_weight, None, torch.float32)
    ref_out, _v, _i, _ = ref_moe.moe_forward(x, lay["gate_w"], lay["experts"], shape["top_k"], lay["shared"],
                                             lay["shared_gate_w"], family=lay["family"], router_logits=logits.cpu())
    torch.testing.assert_close(out.float(), ref_out.float(), **BF16_TOL)
    # identical tokens give identical rows
    assert torch.equal(out[0], out[299]) and torch.equal(out[301], out[429])


@pytest.mark.parametrize("dtype,offload", [(torch.float32, "gpu"), (torch.bfloat16, "gpu"), (torch.bfloat16, "cpu")])
def test_expert_source_rs_executes_the_predicted_routing(device, dtype, offload):
    """``expert_source="rs"``: layer l's predictor leaves (weights, ids) for layer l+1, which
    then executes them instead of its own router; layer 0 and prefill calls use the router
    (reference :11118-11155, :10971-10983).  Checked against the oracle fed with the
    device's own prediction."""
    from sparse_amd.block import DistributedSparseMoeBlock
    from sparse_amd.context import DistEnv, SparseContext
    from sparse_amd.rs import random_init_bank
    from sparse_amd.synthetic import make_hidden, make_mlp_block
    shape, T, L = SMALL_Q, 6, 3
    SparseContext.reset()
    mlps = [make_mlp_block(shape, dtype=dtype, seed=20 + l) for l in range(L)]
    kw = dict(expert_offload=offload, expert_cache=4, planner_mode="rs_prefetch", prefetch_top_m=3) \
        if offload == "cpu" else dict(expert_offload="gpu", routing_mode="rs")
    blocks = [DistributedSparseMoeBlock(l, mlps[l], None, DistEnv(0, 1, 0, device), num_layers=L,
                                        num_experts=shape["num_experts"], top_k=shape["top_k"], dtype=dtype,
                                        expert_source="rs", **kw) for l in range(L)]
    SparseContext.set_rs_bank(random_init_bank(L, shape["hidden"], shape["num_experts"], hidden_dim=32, seed=1,
                                               device=device))
    tol = BF16_TOL if dtype == torch.bfloat16 else F32_TOL
    for call, phase in enumerate(["prefill", "decode", "decode"]):
        SparseContext.current_phase = phase
        SparseContext.begin_runtime_call(call)
        x = make_hidden(T, shape["hidden"], dtype, seed=300 + call)
        hid = (x.view(1, T, -1) if phase == "prefill" else x.view(T, 1, -1)).to(device)
        for l, blk in enumerate(blocks):
            replay = phase == "decode" and l > 0
            assert (l in SparseContext.routing_cache) == replay
            if replay:
                w_dev, i_dev = (t.cpu() for t in SparseContext.routing_cache[l])
            out, logits = blk(hid)
            torch.cuda.synchronize()
            lay = oracle_layer(mlps[l])
            xin = hid.view(T, -1).cpu()
            ws = blk._workspace(T)
            if replay:
                assert torch.equal(ws.topi.cpu(), i_dev) and torch.equal(ws.topv.cpu(), w_dev)
                # the prediction itself: the oracle's top-k of the device's probabilities
                pred = SparseContext.rs_bank[l](prev_in.to(device).float()).cpu()
                w_ref, i_ref, logits_ref = ref_moe.rs_routing(pred, shape["top_k"], dtype)
                assert torch.equal(i_ref, i_dev)
                torch.testing.assert_close(w_ref.float(), w_dev.float(), rtol=1e-2, atol=1e-6)
                assert logits.dtype == torch.float32
                torch.testing.assert_close(logits.cpu(), ref_moe.rs_routing(pred, shape["top_k"], dtype)[2],
                                           rtol=1e-2, atol=1e-2)
                want = ref_moe.moe_forward_routed(xin, w_dev, i_dev, lay["experts"], lay["shared"],
                                                  lay["shared_gate_w"])
            else:
                want, _, ref_topi, _ = ref_moe.moe_forward(
                    xin, lay["gate_w"], lay["experts"], shape["top_k"], lay["shared"], lay["shared_gate_w"],
                    router_logits=logits.cpu())
                assert torch.equal(ws.topi.cpu(), ref_topi)
            torch.testing.assert_close(out.view(T, -1).cpu().float(), want.float(), **tol)
            prev_in = xin
            hid = out


@pytest.mark.parametrize("exec_topk", [2, 7])
@pytest.mark.parametrize("offload", ["gpu", "cpu"])
def test_rs_routing_with_its_own_number_of_experts_per_token(device, monkeypatch, exec_topk, offload):
    """``SPARSE_RS_EXEC_TOPK`` (reference :10979-10987): the replayed routing holds that many
    experts per token, fewer or more than the layer's own top-k, and the layer executes
    exactly them; router-routed calls keep the layer's top-k."""
    from sparse_amd.block import DistributedSparseMoeBlock
    from sparse_amd.context import DistEnv, SparseContext
    from sparse_amd.rs import random_init_bank
    from sparse_amd.synthetic import make_hidden, make_mlp_block
    monkeypatch.setenv("SPARSE_RS_EXEC_TOPK", str(exec_topk))
    shape, T, L, dtype = SMALL_Q, 5, 3, torch.bfloat16
    SparseContext.reset()
    mlps = [make_mlp_block(shape, dtype=dtype, seed=40 + l) for l in range(L)]
    kw = dict(expert_offload="cpu", expert_cache=5, planner_mode="rs_prefetch", prefetch_top_m=3) \
        if offload == "cpu" else dict(expert_offload="gpu", routing_mode="rs")
    blocks = [DistributedSparseMoeBlock(l, mlps[l], None, DistEnv(0, 1, 0, device), num_layers=L,
                                        num_experts=shape["num_experts"], top_k=shape["top_k"], dtype=dtype,
                                        expert_source="rs", **kw) for l in range(L)]
    SparseContext.set_rs_bank(random_init_bank(L, shape["hidden"], shape["num_experts"], hidden_dim=32, seed=2,
                                               device=device))
    for call, phase in enumerate(["prefill", "decode", "decode"]):
        SparseContext.current_phase = phase
        SparseContext.begin_runtime_call(call)
        x = make_hidden(T, shape["hidden"], dtype, seed=500 + call)
        hid = (x.view(1, T, -1) if phase == "prefill" else x.view(T, 1, -1)).to(device)
        for l, blk in enumerate(blocks):
            replay = phase == "decode" and l > 0
            if replay:
                w_dev, i_dev = (t.cpu() for t in SparseContext.routing_cache[l])
                assert tuple(i_dev.shape) == (T, exec_topk)
            out, logits = blk(hid)
            torch.cuda.synchronize()
            lay = oracle_layer(mlps[l])
            xin = hid.view(T, -1).cpu()
            if replay:
                ws = blk._workspace(T, exec_topk)
                assert torch.equal(ws.topi.cpu(), i_dev) and torch.equal(ws.topv.cpu(), w_dev)
                assert int((logits.cpu() > -1e8).sum()) == T * exec_topk
                want = ref_moe.moe_forward_routed(xin, w_dev, i_dev, lay["experts"], lay["shared"],
                                                  lay["shared_gate_w"])
            else:
                want, _, ref_topi, _ = ref_moe.moe_forward(
                    xin, lay["gate_w"], lay["experts"], shape["top_k"], lay["shared"], lay["shared_gate_w"],
                    router_logits=logits.cpu())
                # compare the choice where it does not hang on the last bit of exp(): the two
                # probabilities around the top-k boundary are equal or clearly apart
                srt = logits.cpu().float().sort(dim=-1, descending=True, stable=True)
                p = torch.softmax(logits.cpu().float(), -1).gather(1, srt.indices)
                k = shape["top_k"]
                clear = (srt.values[:, k - 1] == srt.values[:, k]) | ((p[:, k - 1] - p[:, k]) / p[:, k - 1] > 1e-4)
                got_topi = blk._workspace(T).topi.cpu()
                assert torch.equal(got_topi[clear], ref_topi[clear])
                want = ref_moe.moe_forward_routed(xin, blk._workspace(T).topv.cpu(), got_topi, lay["experts"],
                                                  lay["shared"], lay["shared_gate_w"])
            torch.testing.assert_close(out.view(T, -1).cpu().float(), want.float(), **BF16_TOL)
            hid = out


@pytest.mark.parametrize("shape_name,T", [("qwen", 1), ("qwen", 8), ("qwen", 16), ("small", 3), ("small", 16)])
def test_combine_folded_into_the_down_projection_gives_the_same_bits(device, shape_name, T):
    """Small all-resident decode calls combine inside the down projection's launch (the
    workgroup that finishes a 32-column tile last sums it): bit for bit the output of the
    separate combine launch, call after call on new inputs (the arrival counters go back to
    zero), and every routed row is still written."""
    from sparse_amd.synthetic import QWEN, make_hidden
    shape = QWEN if shape_name == "qwen" else dict(family="qwen_shared", hidden=512, num_experts=12, inter=256,
                                                     top_k=4, shared_inter=1024)
    _mlp, blk = _build(shape, torch.bfloat16, device, seed=3)
    H = shape["hidden"]
    assert blk._workspace(T).split_ws is not None
    for i in range(6):
        x = make_hidden(T, H, torch.bfloat16, seed=4000 + i).view(T, 1, H).to(device)
        blk.fold_combine = True
        got, _ = blk(x)
        parts_a = blk._workspace(T).parts.clone()
        blk.fold_combine = False
        want, _ = blk(x)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"call {i}"
        assert torch.equal(parts_a, blk._workspace(T).parts)
    # the counters are back at zero
    from sparse_amd import _lib
    ws = blk._workspace(T)
    off = int(_lib.load().sparse_hip_decode_split_counter_offset(T, H)) // 4
    assert int(ws.split_ws[off:].view(torch.int32).abs().sum().item()) == 0


def test_folded_combine_soak_at_the_decode_shape(device):
    """The hand-off inside the down projection's launch (write-through stores, a full wait, a counter) is
    ordered by the hardware's behaviour rather than by fences, so it gets a longer run than the other
    bit-equality tests: 500 calls at the Qwen shape over batch 1, 8 and 16, each on new inputs with routing
    of its own, the folded launch against the separate combine, stopping at the first difference."""
    from sparse_amd.synthetic import QWEN, make_hidden
    _mlp, blk = _build(QWEN, torch.bfloat16, device, seed=9)
    H = QWEN["hidden"]
    calls = 0
    for T, n in ((1, 170), (8, 170), (16, 160)):
        rows = make_hidden(T * n, H, torch.bfloat16, seed=7000 + T).to(device).view(n, T, 1, H)
        for i in range(n):
            blk.fold_combine = True
            got, _ = blk(rows[i])
            got = got.clone()
            blk.fold_combine = False
            want, _ = blk(rows[i])
            # one comparison per call, on the device: the host only learns whether to stop
            assert torch.equal(got, want), f"batch {T}, call {i}: folded combine differs from the separate launch"
            calls += 1
    assert calls == 500


@pytest.mark.parametrize("T", [8, 300])
def test_segment_timing_counters(device, monkeypatch, T):
    """``SPARSE_EXPERT_TIMING=1`` (utils/eval_core.py:14655-14676): router, routed experts and
    shared expert are timed one after the other into ``moe_{router,expert,shared}_ms``; the
    output keeps its bits; without the switch nothing is counted."""
    from sparse_amd.context import Metrics
    from sparse_amd.synthetic import QWEN, make_hidden
    metrics = Metrics()
    _mlp, blk = _build(QWEN, torch.bfloat16, device, seed=5, metrics=metrics)
    H = QWEN["hidden"]
    x = make_hidden(T, H, torch.bfloat16, seed=77).view(T, 1, H).to(device)
    want, want_logits = blk(x)
    torch.cuda.synchronize()
    assert metrics.moe_timing_calls == 0 and metrics.moe_expert_ms == 0.0
    monkeypatch.setenv("SPARSE_EXPERT_TIMING", "1")
    for _ in range(2):
        got, got_logits = blk(x)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(got_logits, want_logits)
    assert metrics.moe_timing_calls == 6
    assert metrics.moe_router_ms > 0 and metrics.moe_expert_ms > 0 and metrics.moe_shared_ms > 0
    assert metrics.moe_router_ms + metrics.moe_expert_ms + metrics.moe_shared_ms < 1000
    monkeypatch.delenv("SPARSE_EXPERT_TIMING")
    again, _ = blk(x)
    torch.cuda.synchronize()
    assert torch.equal(again, want) and metrics.moe_timing_calls == 6


@pytest.mark.parametrize("T", [1, 8, 32, 96])
def test_decode_stack_in_a_hip_graph_replays_like_eager(device, T):
    """The decode path of a small stack captured into a HIP graph (one-launch router, fused FFN
    launch pair, combine; at 96 tokens the prefill-size kernels with the shared expert forked
    onto its second stream inside the capture): every replay, on new inputs and with eager calls and
    synchronisations of the same blocks in between, gives bit for bit what the eager call
    gives on those inputs.  None of the kernels' self-resetting counters or workspaces may
    depend on having been run eagerly last."""
    from sparse_amd.block import DistributedSparseMoeBlock
    from sparse_amd.context import DistEnv, SparseContext
    from sparse_amd.synthetic import make_hidden, make_mlp_block
    shape = dict(family="qwen_shared", hidden=512, num_experts=12, inter=256, top_k=4, shared_inter=1024)
    dtype = torch.bfloat16
    SparseContext.reset()
    SparseContext.current_phase = "decode"
    blocks = [DistributedSparseMoeBlock(l, make_mlp_block(shape, dtype=dtype, seed=60 + l), None, DistEnv(0, 1, 0, device),
                                        num_layers=2, num_experts=12, top_k=4, dtype=dtype, expert_offload="gpu")
              for l in range(2)]

    def step(h):
        outs = []
        for blk in blocks:
            h, logits = blk(h)
            outs += [h, logits]
        return outs

    inputs = [make_hidden(T, 512, dtype, seed=700 + i).view(T, 1, -1).to(device) for i in range(5)]
    static_in = inputs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(static_in)                                   # workspaces exist before capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(static_in)
    for i in (1, 2, 3, 4, 1):
        want = [t.clone() for t in step(inputs[i])]       # eager, between the replays
        torch.cuda.synchronize()
        static_in.copy_(inputs[i])
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(captured, want):
            assert torch.equal(got, ref), (T, i)


def test_folded_combine_does_not_depend_on_what_the_workspace_held(device):
    """The arrival counters of the folded combine sit behind the partial sums, at an offset that depends
    on the token count.  A workspace sized and used for 16 tokens, then reused for 3, puts the counters
    of the second call on top of stale partial sums -- and a workspace may hold anything at all before its
    first call.  Every call clears its own counters first, so both give the bits of the separate combine."""
    from sparse_amd import ops
    from sparse_amd.synthetic import make_hidden
    shape = dict(family="qwen_shared", hidden=512, num_experts=12, inter=256, top_k=4, shared_inter=1024)
    _mlp, blk = _build(shape, torch.bfloat16, device, seed=3)
    H, K = shape["hidden"], shape["top_k"]
    big = ops.decode_split_workspace(16, H, device)
    big.view(torch.int32).fill_(0x7F7F7F7F)          # garbage, also where any counter could be
    for i, T in enumerate((16, 3, 16, 1)):
        x = make_hidden(T, H, torch.bfloat16, seed=4100 + i).view(T, 1, H).to(device)
        blk.fold_combine = False
        want, _ = blk(x)                                # routes, and leaves topv / perm of this call in ws
        ws = blk._workspace(T)
        got = torch.empty_like(want).view(T, H)
        ops.moe_ffn_decode_combine(blk._experts_desc, x.view(T, H), ws.topv, ws.perm, ws.segs_dev, ws.inter,
                                   ws.parts, blk.shared_weights, ws.shared_gate, ws.shared_inter, big, got,
                                   shared_inter_ready=True)   # the routing launch of blk(x) left it there
        torch.cuda.synchronize()
        assert torch.equal(got.view_as(want), want), f"T={T}"


@pytest.mark.parametrize("T", [17, 24, 32])
def test_folded_combine_above_sixteen_tokens_through_the_c_entry(device, T):
    """The block folds the combine only for calls of up to 16 tokens; the entry point takes up to 32.
    Against the split down projection followed by the separate combine launch: the same bits."""
    from sparse_amd import ops
    from sparse_amd.synthetic import make_hidden
    shape = dict(family="qwen_shared", hidden=512, num_experts=12, inter=256, top_k=4, shared_inter=1024)
    _mlp, blk = _build(shape, torch.bfloat16, device, seed=7)
    H, K = shape["hidden"], shape["top_k"]
    split_ws = ops.decode_split_workspace(T, H, device)
    nparts = ops.decode_split_parts(shape["shared_inter"])
    assert nparts > 1
    for i in range(3):
        x = make_hidden(T, H, torch.bfloat16, seed=4200 + i).view(T, 1, H).to(device)
        blk(x)                                          # routing of this call stays in the workspace
        ws = blk._workspace(T)
        x2 = x.view(T, H)
        # (both calls compute the shared expert's gate and up projections themselves, the same way)
        ops.moe_ffn_decode(blk._experts_desc, x2, ws.topv, ws.perm, ws.segs_dev, ws.inter, ws.parts,
                           blk.shared_weights, ws.shared_gate, ws.shared_inter, ws.shared_out, split_ws)
        want = torch.empty((T, H), device=device, dtype=torch.bfloat16)
        ops.combine_split(ws.parts, ws.perm, split_ws, nparts, ws.shared_gate, T, K, want)
        parts_a = ws.parts.clone()
        got = torch.empty_like(want)
        ops.moe_ffn_decode_combine(blk._experts_desc, x2, ws.topv, ws.perm, ws.segs_dev, ws.inter, ws.parts,
                                   blk.shared_weights, ws.shared_gate, ws.shared_inter, split_ws, got)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"call {i}"
        assert torch.equal(parts_a, ws.parts)
