"""GPU parity tests of the individual C-ABI operators against the CPU oracle.

Bit-exact for indices and permutations; bf16 outputs within rtol 2e-2 / atol 1e-2 and fp32
outputs within rtol/atol 1e-5 of the oracle (the tolerances the north star states).
"""
import numpy as np
import pytest
import torch

from oracle import ref_moe, ref_permute
from tests.helpers import make_hidden, make_layer

pytestmark = pytest.mark.gpu

BF16_TOL = dict(rtol=2e-2, atol=1e-2)
F32_TOL = dict(rtol=1e-5, atol=1e-5)


def tol(dtype):
    return BF16_TOL if dtype == torch.bfloat16 else F32_TOL


def _ops():
    from sparse_amd import ops
    return ops


# ------------------------------------------------------------------ gate_topk
@pytest.mark.parametrize("E,K", [(60, 4), (64, 6), (16, 2), (200, 8)])
@pytest.mark.parametrize("ldt", [torch.float32, torch.bfloat16])
def test_gate_topk_matches_oracle(device, E, K, ldt):
    ops = _ops()
    g = torch.Generator().manual_seed(E * 100 + K)
    logits = (torch.randn(257, E, generator=g) * 2.0).to(ldt)
    # a third of the rows get logits one ulp apart around the K-th place: the indices are a
    # function of the logits alone, so they must agree there too
    srt = torch.sort(logits.float(), dim=-1, descending=True)
    for t in range(0, 257, 3):
        a, b = int(srt.indices[t, K - 1]), int(srt.indices[t, K])
        logits[t, b] = torch.nextafter(logits[t, a].float(), torch.tensor(-1e30)).to(ldt) if ldt == torch.float32 \
            else logits[t, a]
    probs = torch.softmax(logits, dim=-1, dtype=torch.float32)
    ref_v, ref_i = ref_moe.topk_by_logit(logits, probs, K)
    topv, topi = ops.gate_topk(logits.to(device), K, out_dtype=ldt)
    topv, topi = topv.cpu(), topi.cpu()
    assert torch.equal(topi, ref_i)
    torch.testing.assert_close(topv.float(), ref_v.to(ldt).float(), rtol=1e-2 if ldt == torch.bfloat16 else 1e-5,
                               atol=1e-6)


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("scale", [1.0, 2.5, 16.0])
def test_gate_topk_scaling_factor_and_pseudo_logits(device, dt, scale):
    """The DeepSeek branch after the gate (utils/eval_core.py:9503-9517, :9490-9499) inside the top-k
    launch: weights times the routed scaling factor, multiplied in fp32 and rounded once (the oracle's
    ``(topv * factor).to(dtype)``), and the pseudo logits: -inf but log(weight) at the chosen experts."""
    ops = _ops()
    E, K, T = 64, 6, 193
    x = make_hidden(T, 128, dt, seed=5)
    gate_w = (torch.randn(E, 128, generator=torch.Generator().manual_seed(6)) * 0.3).to(dt)
    want_v, want_i, want_p = ref_moe.deepseek_router(x, gate_w, K, routed_scaling_factor=scale)
    logits = torch.nn.functional.linear(x.float(), gate_w.float())
    pseudo = torch.empty((T, E), device=device, dtype=torch.float32)
    topv, topi = ops.gate_topk(logits.to(device), K, out_dtype=dt, scale=scale, pseudo_logits=pseudo)
    assert torch.equal(topi.cpu(), want_i)
    got_v = topv.cpu()
    # one rounding of an fp32 product: at most the last bit of the output type apart from the oracle's
    # (exp and the sum of the softmax differ in their last few fp32 bits between host and device, which is
    # all an fp32 output shows: the unscaled test's 1e-5 bounds it there)
    ulp = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 1e-5}[dt]
    assert float(((got_v.float() - want_v.float()).abs() / want_v.float().abs()).max()) <= ulp
    assert (got_v == want_v).float().mean() > (0.9 if dt != torch.float32 else 0.0)
    got_p = pseudo.cpu()
    chosen = torch.zeros((T, E), dtype=torch.bool).scatter_(1, want_i, True)
    assert torch.isneginf(got_p[~chosen]).all() and torch.isfinite(got_p[chosen]).all()
    torch.testing.assert_close(got_p.gather(1, want_i), got_v.float().clamp_min(1e-12).log(), rtol=1e-5, atol=1e-6)
    # the stand-alone kernel on the same weights, with the replay convention (-1e9, a larger eps)
    again = ops.pseudo_logits(topv, topi, E, eps=1e-12, fill=float("-inf")).cpu()
    assert torch.equal(again, got_p)
    replay = ops.pseudo_logits(topv, topi, E, eps=0.05, fill=-1e9).cpu()
    assert (replay[~chosen] == -1e9).all()
    torch.testing.assert_close(replay.gather(1, want_i), got_v.float().clamp_min(0.05).log(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("E,n_group,topk_group,K", [(16, 4, 2, 6), (160, 8, 3, 6), (256, 64, 5, 16), (64, 2, 1, 8),
                                                      (60, 6, 6, 4), (12, 4, 1, 5)])
@pytest.mark.parametrize("ldt", [torch.float32, torch.bfloat16])
def test_gate_topk_group_limited(device, E, n_group, topk_group, K, ldt):
    """Group-limited selection against the oracle, indices exact on every row; K larger than
    the experts left picks zero-probability experts in id order, as the oracle's rule says."""
    ops = _ops()
    g = torch.Generator().manual_seed(E + n_group)
    logits = (torch.randn(300, E, generator=g) * 2.0).to(ldt)
    topv, topi = ops.gate_topk(logits.to(device), K, out_dtype=torch.float32, n_group=n_group, topk_group=topk_group)
    probs = torch.softmax(logits, dim=-1, dtype=torch.float32)
    masked, keys = probs, logits.float()
    if topk_group < n_group:
        masked, keys = ref_moe.group_limited_scores(probs, n_group, topk_group, logits=logits)
    ref_v, ref_i = ref_moe.topk_by_logit(keys, masked, K)
    assert torch.equal(topi.cpu(), ref_i)
    torch.testing.assert_close(topv.cpu(), ref_v, rtol=1e-5, atol=1e-7)
    if topk_group < n_group:
        grp = torch.div(topi.cpu(), E // n_group, rounding_mode="floor")
        live = (masked > 0).sum(1) >= K                     # enough experts left in the kept groups
        assert max((len(set(r.tolist())) for r in grp[live]), default=0) <= topk_group


def test_gate_topk_ties_go_to_lower_id(device):
    ops = _ops()
    logits = torch.zeros(5, 60)
    logits[1, [7, 3, 50]] = 2.0          # three-way tie at the top, K=4 takes all + id 0
    logits[2, [59, 58, 57, 56, 55]] = 1.0  # five-way tie, K=4 takes the four lowest ids
    logits[3, 10] = 5.0
    logits[4] = torch.arange(60, dtype=torch.float32).flip(0) * 0.0  # all equal
    for ldt in (torch.float32, torch.bfloat16):
        probs = torch.softmax(logits.to(ldt), dim=-1, dtype=torch.float32)
        ref_v, ref_i = ref_moe.topk_by_logit(logits.to(ldt), probs, 4)
        topv, topi = ops.gate_topk(logits.to(ldt).to(device), 4)
        assert torch.equal(topi.cpu(), ref_i)
        assert topi.cpu()[0].tolist() == [0, 1, 2, 3]
        assert topi.cpu()[1].tolist() == [3, 7, 50, 0]
        assert topi.cpu()[2].tolist() == [55, 56, 57, 58]
        assert topi.cpu()[3].tolist() == [10, 0, 1, 2]


def test_gate_topk_renorm(device):
    ops = _ops()
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(33, 60, generator=g)
    topv, topi = ops.gate_topk(logits.to(device), 4, renorm=True)
    torch.testing.assert_close(topv.cpu().sum(dim=1), torch.ones(33), rtol=1e-5, atol=1e-5)
    x = torch.zeros(33, 8)
    ref_v, ref_i, _ = ref_moe.routing_router(x, torch.zeros(60, 8), 4, True, router_logits=logits)
    assert torch.equal(topi.cpu(), ref_i)
    torch.testing.assert_close(topv.cpu(), ref_v, rtol=1e-5, atol=1e-6)


def test_gate_topk_rejects_bad_arguments(device):
    ops = _ops()
    logits = torch.zeros(4, 300, device=device)
    with pytest.raises(ValueError):
        ops.gate_topk(logits, 4)
    with pytest.raises(ValueError):
        ops.gate_topk(torch.zeros(4, 8, device=device), 9)


def test_topk_of_given_probabilities(device):
    """``sparse_hip_topk``: rows ranked as they are (no softmax), equal values in id order."""
    ops = _ops()
    g = torch.Generator().manual_seed(9)
    pred = torch.softmax(torch.randn(50, 60, generator=g) * 3.0, dim=-1)
    pred[3, [40, 5, 17]] = pred[3].max() + 0.1          # three-way tie at the top
    pred[4] = 1.0 / 60                                   # all equal
    for K in (1, 8, 16):
        order = torch.sort(pred, dim=-1, descending=True, stable=True)
        topv, topi = ops.topk_values(pred.to(device), K)
        assert torch.equal(topi.cpu(), order.indices[:, :K])
        assert torch.equal(topv.cpu(), order.values[:, :K])
    topv, _ = ops.topk_values(pred.to(device), 8, out_dtype=torch.bfloat16)
    assert torch.equal(topv.cpu(), torch.sort(pred, dim=-1, descending=True).values[:, :8].to(torch.bfloat16))
    with pytest.raises(ValueError):
        ops.topk_values(pred.to(device), 17)


# ------------------------------------------------------------------ router logits
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 8, 33, 128])
def test_router_logits(device, dtype, T):
    ops = _ops()
    layer = make_layer(2048, 60, 64, 4, Is=64, shared_gate=True, dtype=dtype, seed=3)
    x = make_hidden(T, 2048, dtype, seed=4)
    ref = torch.nn.functional.linear(x.float(), layer["gate_w"].float())
    ref_sg = torch.nn.functional.linear(x.float(), layer["shared_gate_w"].float().reshape(1, -1)).reshape(-1)
    logits, sg = ops.router_logits(x.to(device), layer["gate_w"].to(device), layer["shared_gate_w"].to(device))
    assert logits.dtype == dtype and sg.dtype == dtype
    t = dict(rtol=1e-2, atol=1e-2) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(logits.float().cpu(), ref, **t)
    torch.testing.assert_close(sg.float().cpu(), ref_sg, **t)
    if dtype == torch.bfloat16:
        l32, _ = ops.router_logits(x.to(device), layer["gate_w"].to(device), logits_dtype=torch.float32)
        assert l32.dtype == torch.float32
        torch.testing.assert_close(l32.cpu(), ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype,ldt", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                       (torch.float32, torch.float32)])
@pytest.mark.parametrize("T", [1, 8, 32])
def test_route_decode_equals_the_three_separate_calls(device, dtype, ldt, T):
    """The single-launch decode router: its logits agree with router_logits up to the
    summation order, and its top-k and permutation are bit for bit what gate_topk and
    permute_build return for the logits it wrote, call after call (its counter goes back
    to zero)."""
    ops = _ops()
    E, K, H = 60, 4, 2048
    layer = make_layer(H, E, 64, K, Is=64, shared_gate=True, dtype=dtype, seed=7)
    wg, wsg = layer["gate_w"].to(device), layer["shared_gate_w"].to(device)
    counter = torch.zeros(1, dtype=torch.int32, device=device)
    for rep in range(3):
        x = make_hidden(T, H, dtype, seed=100 + rep).to(device)
        logits_a, sg_a = ops.router_logits(x, wg, wsg, logits_dtype=ldt)
        logits_b = torch.empty_like(logits_a)
        sg_b = torch.empty_like(sg_a)
        topv_b = torch.empty(T, K, dtype=dtype, device=device)
        topi_b = torch.empty(T, K, dtype=torch.int64, device=device)
        perm_b = ops.Permutation(T, K, E, device)
        ops.route_decode(x, wg, wsg, K, False, logits_b, sg_b, topv_b, topi_b, perm_b, counter)
        torch.cuda.synchronize()
        assert int(counter.item()) == 0
        # one bf16 ulp where the rounding boundary falls between two summation orders
        tol = dict(rtol=8e-3, atol=1e-6) if ldt == torch.bfloat16 else dict(rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(logits_b.float(), logits_a.float(), **tol)
        tol = dict(rtol=8e-3, atol=1e-6) if dtype == torch.bfloat16 else dict(rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(sg_b.float(), sg_a.float(), **tol)
        topv_a, topi_a = ops.gate_topk(logits_b, K, out_dtype=dtype)
        perm_a = ops.permute_build(topi_a, E)
        torch.cuda.synchronize()
        assert torch.equal(topv_a, topv_b) and torch.equal(topi_a, topi_b)
        n = int(perm_a.n_active.item())
        assert n == int(perm_b.n_active.item())
        for name in ("perm", "inv_perm", "seg_offsets"):
            assert torch.equal(getattr(perm_a, name), getattr(perm_b, name)), name
        assert torch.equal(perm_a.active_eids[:n], perm_b.active_eids[:n])


@pytest.mark.parametrize("T,E,K", [(1, 4, 4), (32, 256, 16), (7, 64, 6), (32, 60, 1)])
def test_route_decode_shapes_against_oracle(device, T, E, K):
    """Corner shapes of the decode router (K == E, the largest E and K, K == 1) against the
    CPU oracle: logits within fp32 summation error, indices exact given the logits the kernel wrote."""
    ops = _ops()
    H = 512
    dtype = torch.float32
    layer = make_layer(H, E, 64, K, Is=64, shared_gate=False, dtype=dtype, seed=11)
    wg = layer["gate_w"].to(device)
    x = make_hidden(T, H, dtype, seed=5).to(device)
    logits = torch.empty(T, E, dtype=dtype, device=device)
    topv = torch.empty(T, K, dtype=dtype, device=device)
    topi = torch.empty(T, K, dtype=torch.int64, device=device)
    perm = ops.Permutation(T, K, E, device)
    counter = torch.zeros(1, dtype=torch.int32, device=device)
    ops.route_decode(x, wg, None, K, False, logits, None, topv, topi, perm, counter)
    torch.cuda.synchronize()
    _, _, ref_logits = ref_moe.routing_router(x.cpu(), layer["gate_w"], K, False)
    torch.testing.assert_close(logits.cpu(), ref_logits, rtol=1e-5, atol=1e-5)
    ref_v, ref_i, _ = ref_moe.routing_router(x.cpu(), layer["gate_w"], K, False, router_logits=logits.cpu())
    assert torch.equal(topi.cpu(), ref_i)
    torch.testing.assert_close(topv.cpu(), ref_v, rtol=1e-5, atol=1e-6)
    p_perm, p_inv, p_off, p_active = ref_permute.permute_build(topi.cpu().numpy(), E)
    assert np.array_equal(perm.perm.cpu().numpy(), p_perm)
    assert np.array_equal(perm.inv_perm.cpu().numpy(), p_inv)
    assert np.array_equal(perm.seg_offsets.cpu().numpy(), p_off)
    n = int(perm.n_active.item())
    assert n == p_active.size and np.array_equal(perm.active_eids.cpu().numpy()[:n], p_active)


@pytest.mark.parametrize("ldt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,H,E,K,shared_gate,renorm", [
    (1, 2048, 60, 4, True, False), (8, 2048, 60, 4, True, False), (3, 2048, 64, 6, False, True),
    (16, 2048, 63, 8, True, False), (8, 64, 60, 4, True, False), (5, 2560, 8, 8, True, True),
    (16, 4096, 64, 1, False, False), (7, 192, 15, 3, True, False), (2, 1088, 33, 16, False, False)])
def test_route_decode_packed_shapes(device, T, H, E, K, shared_gate, renorm, ldt):
    """One-workgroup decode router on the packed gate matrix (one to sixty-four rows, H from
    one 64-wide block to several per wavefront, an odd number of blocks): logits and shared
    gate against fp32 linear algebra, top-k and permutation bit for bit what gate_topk and
    permute_build return on the logits it wrote, indices equal to the oracle's on those logits,
    and the same answer call after call."""
    ops = _ops()
    dtype = torch.bfloat16
    layer = make_layer(H, E, 64, K, Is=64, shared_gate=shared_gate, dtype=dtype, seed=23 + T)
    wsg = layer["shared_gate_w"].to(device) if shared_gate else None
    packed = ops.pack_router_gate(layer["gate_w"].to(device), wsg)
    assert packed is not None and packed.numel() == 64 * H
    for rep in range(2):
        x = make_hidden(T, H, dtype, seed=400 + rep)
        logits = torch.empty(T, E, dtype=ldt, device=device)
        sg = torch.empty(T, dtype=dtype, device=device) if shared_gate else None
        topv = torch.empty(T, K, dtype=dtype, device=device)
        topi = torch.empty(T, K, dtype=torch.int64, device=device)
        perm = ops.Permutation(T, K, E, device)
        ops.route_decode_packed(x.to(device), packed, E, shared_gate, K, renorm, logits, sg, topv, topi, perm)
        torch.cuda.synchronize()
        ref = torch.nn.functional.linear(x.float(), layer["gate_w"].float())
        tol = dict(rtol=1e-2, atol=1e-2) if ldt == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(logits.float().cpu(), ref, **tol)
        if shared_gate:
            ref_sg = torch.nn.functional.linear(x.float(), layer["shared_gate_w"].float().reshape(1, -1)).reshape(-1)
            torch.testing.assert_close(sg.float().cpu(), ref_sg, rtol=1e-2, atol=1e-2)
        topv_a, topi_a = ops.gate_topk(logits, K, renorm=renorm, out_dtype=dtype)
        perm_a = ops.permute_build(topi_a, E)
        torch.cuda.synchronize()
        assert torch.equal(topv_a, topv) and torch.equal(topi_a, topi)
        n = int(perm_a.n_active.item())
        assert n == int(perm.n_active.item())
        for name in ("perm", "inv_perm", "seg_offsets"):
            assert torch.equal(getattr(perm_a, name), getattr(perm, name)), name
        assert torch.equal(perm_a.active_eids[:n], perm.active_eids[:n])
        probs = torch.softmax(logits.cpu(), dim=-1, dtype=torch.float32)
        _, ref_i = ref_moe.topk_by_logit(logits.cpu(), probs, K)
        assert torch.equal(topi.cpu(), ref_i)


@pytest.mark.parametrize("T,H,E,K,Is", [(1, 2048, 60, 4, 5632), (8, 2048, 60, 4, 5632), (16, 2048, 63, 6, 2816),
                                        (5, 192, 15, 3, 96), (13, 4096, 62, 2, 64), (7, 4160, 33, 4, 32)])
def test_route_decode_packed_with_the_shared_gate_up_beside_it(device, T, H, E, K, Is):
    """The routing launch that also computes the shared expert's SiLU(gate x) * (up x): routing
    results bit for bit those of the routing-only launch; the activation equal to fp32 linear
    algebra rounded the way the expert kernels round (gate and up to bf16, SiLU to bf16, the
    product to bf16) within two bf16 steps (a sum that lands on the other side of a rounding
    boundary moves gate or up by one step each), and to what the decode expert kernel writes for
    the same weights within the same bound (their fp32 sums are grouped differently); H from three
    64-wide blocks to more than two per wavefront, T up to the launch's 16 tokens."""
    from sparse_amd.weights import tile_weight
    ops = _ops()
    dtype = torch.bfloat16
    layer = make_layer(H, E, 64, K, Is=Is, shared_gate=True, dtype=dtype, seed=71 + T, std=0.05)
    packed = ops.pack_router_gate(layer["gate_w"].to(device), layer["shared_gate_w"].to(device))
    gw, uw = (tile_weight(w.to(device)).reshape(w.shape).contiguous() for w in layer["shared"][:2])
    x = make_hidden(T, H, dtype, seed=500 + T)
    xd = x.to(device)

    def route(shared_up):
        logits = torch.empty(T, E, dtype=dtype, device=device)
        sg = torch.empty(T, dtype=dtype, device=device)
        topv = torch.empty(T, K, dtype=dtype, device=device)
        topi = torch.empty(T, K, dtype=torch.int64, device=device)
        perm = ops.Permutation(T, K, E, device)
        ops.route_decode_packed(xd, packed, E, True, K, False, logits, sg, topv, topi, perm, shared_up=shared_up)
        torch.cuda.synchronize()
        return logits, sg, topv, topi, perm

    inter = torch.full((T, Is), float("nan"), dtype=dtype, device=device)
    a, b = route(None), route((gw, uw, inter))
    for u, v in zip(a[:4], b[:4]):
        assert torch.equal(u, v)
    for name in ("perm", "inv_perm", "seg_offsets", "n_active"):
        assert torch.equal(getattr(a[4], name), getattr(b[4], name)), name
    g = torch.nn.functional.linear(x.float(), layer["shared"][0].float()).to(dtype).float()
    u = torch.nn.functional.linear(x.float(), layer["shared"][1].float()).to(dtype).float()
    want = (torch.nn.functional.silu(g).to(dtype).float() * u).to(dtype)
    got = inter.cpu()
    assert not torch.isnan(got.float()).any()
    torch.testing.assert_close(got.float(), want.float(), rtol=2 ** -6, atol=1e-3)
    assert float(((got.float() - want.float()).abs() <= want.float().abs() * 2 ** -7 + 1e-3).float().mean()) > 0.995
    alone = torch.empty_like(inter)
    ops.shared_gate_up(xd, gw, uw, alone)       # the same kernel code without the routing
    torch.cuda.synchronize()
    assert torch.equal(alone, inter)
    if Is % 64:
        return      # the expert kernels' down projection needs Is in 64-wide blocks
    # the decode expert kernel on the same weights
    dw = tile_weight(layer["shared"][2].to(device)).reshape(H, Is).contiguous()
    old_inter = torch.empty((T, Is), dtype=dtype, device=device)
    old_out = torch.empty((T, H), dtype=dtype, device=device)
    ops.shared_expert(xd, gw, uw, dw, a[1], old_inter, old_out)
    torch.cuda.synchronize()
    torch.testing.assert_close(got.float(), old_inter.cpu().float(), rtol=2 ** -6, atol=1e-3)
    assert float((got == old_inter.cpu()).float().mean()) > 0.97


def test_pack_router_gate_declines_what_does_not_fit():
    from sparse_amd import ops
    wg = torch.zeros(64, 128, dtype=torch.bfloat16)
    assert ops.pack_router_gate(wg, None) is not None
    assert ops.pack_router_gate(wg, torch.zeros(128, dtype=torch.bfloat16)) is None      # 65 rows
    assert ops.pack_router_gate(wg[:, :96].contiguous(), None) is None                    # H % 64
    assert ops.pack_router_gate(wg.float(), None) is None


# ------------------------------------------------------------------ permute
@pytest.mark.parametrize("T,E,K", [(1, 60, 4), (8, 60, 4), (32, 60, 4), (255, 64, 6), (256, 64, 6),
                                    (257, 64, 6), (2048, 64, 6), (4096, 64, 6), (1000, 256, 16), (3, 4, 4),
                                    (10923, 64, 6), (16384, 60, 4), (20000, 64, 6)])
def test_permute_build_bit_exact(device, T, E, K):
    ops = _ops()
    g = torch.Generator().manual_seed(T * 7 + E)
    scores = torch.rand(T, E, generator=g)
    if T >= 255:
        scores[:, : E // 4] += 0.5  # skewed popularity, some experts possibly empty
        scores[:, E - 1] = -1.0     # one expert never chosen
    topi = torch.topk(scores, K, dim=1).indices.to(torch.int64)
    p = ops.permute_build(topi.to(device), E)
    perm, inv, off, active = ref_permute.permute_build(topi.numpy(), E)
    torch.cuda.synchronize()
    assert np.array_equal(p.perm.cpu().numpy(), perm)
    assert np.array_equal(p.inv_perm.cpu().numpy(), inv)
    assert np.array_equal(p.seg_offsets.cpu().numpy(), off)
    n = int(p.n_active.cpu().item())
    assert n == active.size
    assert np.array_equal(p.active_eids.cpu().numpy()[:n], active)


# ------------------------------------------------------------------ FFN helpers
def _run_routed(ops, layer, x, topv, topi, device, decode, order=None):
    from sparse_amd.weights import ExpertSlab
    H, E, I, K = layer["H"], layer["E"], layer["I"], layer["K"]
    dtype = layer["dtype"]
    T = x.shape[0]
    slab = ExpertSlab.resident(layer["experts"], H, I, dtype, device)
    ex = ops.make_experts(slab.data, slab.expert_slot, E, H, I)
    xd, tvd, tid = x.to(device), topv.to(device), topi.to(device)
    p = ops.permute_build(tid, E)
    inter = torch.zeros((T * K, I), device=device, dtype=dtype)
    parts = torch.zeros((T * K, H), device=device, dtype=dtype)
    if order is None:
        segs = ops.seglist_device(p, min(E, T * K))
    else:
        segs = ops.seglist_host(order)
    ops.grouped_swiglu(ex, xd, tvd, p, segs, inter, parts, decode=decode)
    out = torch.empty((T, H), device=device, dtype=dtype)
    ops.combine(parts, p, None, T, K, out)
    torch.cuda.synchronize()
    return out.cpu(), parts.cpu(), p


def _routing(layer, x):
    topv, topi, _ = ref_moe.routing_router(x, layer["gate_w"], layer["K"])
    return topv, topi


@pytest.mark.parametrize("T", [1, 2, 8, 16, 17, 32])
def test_decode_ffn_bf16_matches_oracle(device, T):
    ops = _ops()
    layer = make_layer(512, 12, 256, 4, dtype=torch.bfloat16, seed=11, std=0.05)
    x = make_hidden(T, 512, torch.bfloat16, seed=12)
    topv, topi = _routing(layer, x)
    out, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=True)
    ref = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    torch.testing.assert_close(out.float(), ref.float(), **BF16_TOL)
    # a wrong row/column mapping would give O(1) relative error; check it is tight
    err = (out.float() - ref.float()).abs().max() / ref.float().abs().max()
    assert err < 2e-2


def test_decode_ffn_bf16_qwen_shape(device):
    ops = _ops()
    layer = make_layer(2048, 60, 1408, 4, dtype=torch.bfloat16, seed=0)
    x = make_hidden(8, 2048, torch.bfloat16, seed=1000)
    topv, topi = _routing(layer, x)
    out, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=True)
    ref = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    torch.testing.assert_close(out.float(), ref.float(), **BF16_TOL)
    assert (out.float() - ref.float()).abs().max() / ref.float().abs().max() < 2e-2


@pytest.mark.parametrize("T", [40, 128, 300])
def test_prefill_ffn_bf16_matches_oracle(device, T):
    ops = _ops()
    layer = make_layer(512, 12, 256, 4, dtype=torch.bfloat16, seed=21, std=0.05)
    x = make_hidden(T, 512, torch.bfloat16, seed=22)
    topv, topi = _routing(layer, x)
    out, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=False)
    ref = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    torch.testing.assert_close(out.float(), ref.float(), **BF16_TOL)
    assert (out.float() - ref.float()).abs().max() / ref.float().abs().max() < 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("H,E,I,K,T", [(320, 6, 192, 2, 200), (576, 5, 448, 3, 333), (192, 4, 64, 2, 150),
                                       (64, 3, 64, 1, 129)])
def test_prefill_ffn_odd_shapes_match_oracle(device, dtype, H, E, I, K, T):
    """Reduction lengths that are an odd number of 64-wide slabs (the k loop runs its slabs in pairs plus a
    tail), output widths that end inside a workgroup's column tile or inside a wavefront's 16-row group
    range, and segments that end inside a 32-row sub-tile."""
    ops = _ops()
    layer = make_layer(H, E, I, K, dtype=dtype, seed=41 + H, std=0.05)
    x = make_hidden(T, H, dtype, seed=42 + T)
    topv, topi = _routing(layer, x)
    out, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=False)
    ref = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    tol = BF16_TOL if dtype == torch.bfloat16 else dict(rtol=5e-3, atol=2e-3)
    torch.testing.assert_close(out.float(), ref.float(), **tol)
    assert not torch.isnan(out.float()).any()


def test_prefill_and_decode_kernels_agree(device):
    ops = _ops()
    layer = make_layer(512, 12, 256, 4, dtype=torch.bfloat16, seed=31, std=0.05)
    x = make_hidden(24, 512, torch.bfloat16, seed=32)
    topv, topi = _routing(layer, x)
    a, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=True)
    b, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=False)
    torch.testing.assert_close(a.float(), b.float(), **BF16_TOL)


@pytest.mark.parametrize("H,E,I,K,T", [(512, 12, 256, 4, 300), (2048, 60, 1408, 4, 1531), (7168, 8, 2048, 2, 777)])
def test_prefill_counted_waits_equal_full_drains(device, H, E, I, K, T):
    """The prefill kernel's k loop waits for a counted number of vector-memory operations.
    The same kernel built with full drains in their place must give the same bits, over
    ragged segments (routing of random rows: segment sizes from empty to several row tiles,
    odd and even numbers of k slabs across the three shapes), for the routed rows, the
    combined output and the shared expert."""
    from sparse_amd import _lib
    ops = _ops()
    lib = _lib.load()
    layer = make_layer(H, E, I, K, Is=I, shared_gate=True, dtype=torch.bfloat16, seed=61)
    x = make_hidden(T, H, torch.bfloat16, seed=62)
    g = torch.Generator().manual_seed(63)
    popularity = 1.0 / torch.arange(1, E + 1, dtype=torch.float32) ** 1.2    # a few busy experts, a long tail
    popularity[E - 1] = 0.0                                                   # and one nobody routes to
    topi = torch.multinomial(popularity.expand(T, E), K, replacement=False, generator=g)
    topv = torch.rand(T, K, generator=g).to(torch.bfloat16)
    counts = torch.bincount(topi.reshape(-1), minlength=E)
    assert int(counts.max()) > 256 and int(counts[counts > 0].min()) < 128 and int(counts.min()) == 0
    sh = [w.to(device) for w in layer["shared"]]
    xd = x.to(device)
    sg = torch.nn.functional.linear(x.float(), layer["shared_gate_w"].float().reshape(1, -1)).reshape(-1)
    sg = sg.to(torch.bfloat16).to(device)

    def run():
        out, parts, _ = _run_routed(ops, layer, x, topv, topi, device, decode=False)
        inter = torch.zeros((T, I), device=device, dtype=torch.bfloat16)
        shared = torch.zeros((T, H), device=device, dtype=torch.bfloat16)
        ops.shared_expert(xd, sh[0], sh[1], sh[2], sg, inter, shared)
        torch.cuda.synchronize()
        return out, parts, shared.cpu()

    assert lib.sparse_hip_prefill_drain_waits(0) == 0
    fast = run()
    assert lib.sparse_hip_prefill_drain_waits(1) == 0
    try:
        safe = run()
    finally:
        assert lib.sparse_hip_prefill_drain_waits(0) == 1
    for a, b, what in zip(fast, safe, ("combined output", "routed rows", "shared expert")):
        assert torch.equal(a, b), f"{what}: counted waits and full drains differ"
    assert float(fast[0].float().abs().max()) > 0


def test_prefill_clock_probe_reads_a_plausible_clock_and_changes_nothing(device):
    """The probe adds up, per workgroup of the prefill FFN kernel, shader-clock cycles and ticks of the
    constant 100 MHz clock: their ratio is a clock between the part's idle and peak clocks, both
    counters grow with every launch, and the kernel's output is the same with and without it."""
    ops = _ops()
    H, E, I, K, T = 512, 12, 256, 4, 600
    layer = make_layer(H, E, I, K, dtype=torch.bfloat16, seed=71)
    x = make_hidden(T, H, torch.bfloat16, seed=72)
    topv, topi = _routing(layer, x)
    plain, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=False)
    clk = torch.zeros(2, dtype=torch.int64, device=device)
    ops.prefill_clock_probe(clk)
    try:
        probed, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=False)
        first = clk.tolist()
        _run_routed(ops, layer, x, topv, topi, device, decode=False)
        second = clk.tolist()
    finally:
        ops.prefill_clock_probe(None)
    assert torch.equal(plain, probed)
    assert first[0] > 0 and first[1] > 0 and second[0] > first[0] and second[1] > first[1]
    assert 100.0 < ops.prefill_shader_clock_mhz(clk) < 3000.0
    _run_routed(ops, layer, x, topv, topi, device, decode=False)
    torch.cuda.synchronize()
    assert clk.tolist() == second   # switched off: nothing is added any more


def test_mfma_probe_reports_a_rate_below_peak_and_a_plausible_clock(device):
    """The probe's loop is nothing but MFMAs (and, in its second form, LDS fragment reads): its rate can
    not exceed what 256 compute units deliver at the clock it measured (4096 flop per clock per unit), it
    is a sizeable fraction of it, and bad arguments are rejected."""
    ops = _ops()
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    for from_lds in (False, True):
        tflops, mhz = ops.mfma_probe(from_lds, iters=4000, device=device)
        assert 100.0 < mhz < 3000.0
        at_clock = cus * 4096 * mhz * 1e6 / 1e12
        assert 0.5 * at_clock < tflops <= 1.02 * at_clock, (from_lds, tflops, mhz)
    with pytest.raises(Exception):
        ops.mfma_probe(False, iters=3, device=device)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T", [1, 8, 32])
def test_rs_predictor_kernel_matches_the_module(device, dtype, T):
    """The two-launch HIP forward pass of the routing-scout MLP (BatchNorm folded into the first Linear)
    against the PyTorch module in eval mode on ``x.float()``, with running statistics and affine
    parameters that are not the identity; probabilities within fp32 summation-order noise, and the
    planner's top-8 equal wherever the ninth probability is not within that noise of the eighth."""
    from sparse_amd.rs import RoutingScoutMLP, fused_scout, stable_topk
    ops = _ops()
    H, E, D = 2048, 60, 512
    torch.manual_seed(5)
    mod = RoutingScoutMLP(H, E, hidden_dim=D)
    bn = mod.mlp[1]
    with torch.no_grad():
        bn.running_mean.copy_(torch.randn(D) * 0.3)
        bn.running_var.copy_(torch.rand(D) * 2 + 0.25)
        bn.weight.copy_(torch.rand(D) + 0.5)
        bn.bias.copy_(torch.randn(D) * 0.2)
        mod.mlp[4].weight.mul_(4.0)          # spread the output distribution
    mod = mod.eval().to(device)
    x = make_hidden(T, H, dtype, seed=81).to(device)
    with torch.no_grad():
        ref = mod(x.float())
    fused = fused_scout(mod, x)
    assert fused is not None and fused_scout(mod, x) is fused          # built once, cached on the module
    pred = fused(x)
    assert pred.dtype == torch.float32 and tuple(pred.shape) == (T, E)
    torch.testing.assert_close(pred, ref, rtol=2e-4, atol=1e-7)
    torch.testing.assert_close(pred.sum(-1), torch.ones(T, device=device), rtol=1e-5, atol=1e-5)
    v_ref, i_ref = stable_topk(ref, 9)
    _, i_dev = stable_topk(pred, 8)
    clear = (v_ref[:, 7] - v_ref[:, 8]) > 1e-4 * v_ref[:, 7]
    assert bool(clear.any())
    assert torch.equal(torch.sort(i_dev[clear], 1).values, torch.sort(i_ref[clear, :8], 1).values)
    # what the kernel does not take falls back to the module: training mode, widths off the 8-grid
    assert fused_scout(mod.train(), x) is None
    assert fused_scout(mod.eval(), x[:, :H - 4].contiguous()) is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T", [33, 100, 4096])
def test_rs_predictor_kernel_at_prefill_sizes(device, dtype, T):
    """The same two launches over blocks of 32 token rows: a prefill-size call against the numpy oracle of
    the predictor (and through it the module), including a last block that is not full."""
    from oracle import ref_rs
    from sparse_amd.rs import RoutingScoutMLP, fused_scout
    H, E, D = 512, 60, 256
    torch.manual_seed(6)
    mod = RoutingScoutMLP(H, E, hidden_dim=D)
    bn = mod.mlp[1]
    with torch.no_grad():
        bn.running_mean.copy_(torch.randn(D) * 0.3)
        bn.running_var.copy_(torch.rand(D) * 2 + 0.25)
        bn.weight.copy_(torch.rand(D) + 0.5)
        bn.bias.copy_(torch.randn(D) * 0.2)
        mod.mlp[4].weight.mul_(4.0)
    mod = mod.eval()
    x = make_hidden(T, H, dtype, seed=83)
    n = lambda t: t.detach().numpy()
    want = ref_rs.routing_scout_forward(x.float().numpy(), n(mod.mlp[0].weight), n(mod.mlp[0].bias), n(bn.weight),
                                        n(bn.bias), n(bn.running_mean), n(bn.running_var), n(mod.mlp[4].weight),
                                        n(mod.mlp[4].bias), eps=bn.eps)
    mod = mod.to(device)
    fused = fused_scout(mod, x.to(device))
    assert fused is not None
    pred = fused(x.to(device))
    assert tuple(pred.shape) == (T, E)
    torch.testing.assert_close(pred.cpu(), torch.from_numpy(want), rtol=2e-4, atol=1e-7)


def _residual_scout(H, E, D, layers, seed):
    from sparse_amd.rs import RoutingScoutResidualMLP
    torch.manual_seed(seed)
    mod = RoutingScoutResidualMLP(H, E, hidden_dim=D, num_hidden_layers=layers)
    with torch.no_grad():
        for m in mod.modules():
            if isinstance(m, torch.nn.LayerNorm):
                m.weight.copy_(torch.rand_like(m.weight) + 0.5)
                m.bias.copy_(torch.randn_like(m.bias) * 0.3)
        mod.head.weight.mul_(4.0)
    return mod.eval()


def _residual_oracle(mod, rows):
    from oracle import ref_rs
    n = lambda t: t.detach().cpu().numpy()
    stem = (n(mod.input[0].weight), n(mod.input[0].bias), n(mod.input[1].weight), n(mod.input[1].bias))
    units = [(n(u.net[0].weight), n(u.net[0].bias), n(u.net[1].weight), n(u.net[1].bias), n(u.net[4].weight),
              n(u.net[4].bias)) for u in mod.blocks]
    return ref_rs.routing_scout_residual_forward(rows, stem, units, (n(mod.out_norm.weight), n(mod.out_norm.bias)),
                                                 (n(mod.head.weight), n(mod.head.bias)), eps=mod.out_norm.eps)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,layers", [(1, 3), (8, 3), (32, 1), (40, 0), (300, 2)])
def test_residual_rs_predictor_chain_matches_oracle(device, dtype, T, layers):
    """The deeper predictor as a chain of LayerNorm, dense (+GELU, +residual) and softmax launches against
    its numpy oracle on the widened token rows; fp32 arithmetic both sides, tolerance for summation order
    (1e-3 relative on probabilities that pass through up to eight matrix products)."""
    from sparse_amd.rs import FusedResidualScout, fused_scout
    H, E, D = 512, 60, 128
    mod = _residual_scout(H, E, D, layers, seed=7 + layers)
    x = make_hidden(T, H, dtype, seed=84 + T)
    want = _residual_oracle(mod, x.float().numpy())
    mod = mod.to(device)
    fused = fused_scout(mod, x.to(device))
    assert isinstance(fused, FusedResidualScout) and fused_scout(mod, x.to(device)) is fused
    pred = fused(x.to(device))
    assert pred.dtype == torch.float32 and tuple(pred.shape) == (T, E)
    torch.testing.assert_close(pred.cpu(), torch.from_numpy(want), rtol=1e-3, atol=1e-7)
    torch.testing.assert_close(pred.sum(-1), torch.ones(T, device=device), rtol=1e-5, atol=1e-5)
    with torch.no_grad():
        torch.testing.assert_close(pred, mod(x.to(device).float()), rtol=1e-3, atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("residual", [False, True])
@pytest.mark.parametrize("T", [5, 70])
def test_rs_predictors_that_read_the_routing(device, dtype, residual, T):
    """``feature_mode = hidden_router_topk``: one launch lays out [x | routing-weight columns | padding]
    (bit-exact against the oracle's feature rows: E = 60 makes the row length 572, padded to 576), and the
    predictors run on those rows; against the oracle fed the oracle's own concatenation."""
    from oracle import ref_rs
    from sparse_amd.rs import RoutingScoutMLP, fused_scout
    ops = _ops()
    H, E, K, D = 512, 60, 4, 128
    x = make_hidden(T, H, dtype, seed=90 + T)
    g = torch.Generator().manual_seed(91 + T)
    topi = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    topv = torch.rand((T, K), generator=g).to(dtype)
    if T > 1:
        topv[1].zero_()                                             # a row whose weights sum to zero
    feat = ref_rs.router_topk_feature(topi.numpy(), topv.float().numpy(), E)
    rows = np.concatenate([x.float().numpy(), feat], axis=1)
    got_rows = ops.rs_features(x.to(device), topi.to(device), topv.to(device), E)
    assert tuple(got_rows.shape) == (T, 576)
    assert np.array_equal(got_rows[:, :H + E].cpu().numpy(), rows) and not bool(got_rows[:, H + E:].any())
    if residual:
        mod = _residual_scout(H + E, E, D, 2, seed=12)
        want = _residual_oracle(mod, rows)
    else:
        torch.manual_seed(13)
        mod = RoutingScoutMLP(H + E, E, hidden_dim=D).eval()
        bn = mod.mlp[1]
        n = lambda t: t.detach().numpy()
        want = ref_rs.routing_scout_forward(rows, n(mod.mlp[0].weight), n(mod.mlp[0].bias), n(bn.weight), n(bn.bias),
                                            n(bn.running_mean), n(bn.running_var), n(mod.mlp[4].weight),
                                            n(mod.mlp[4].bias), eps=bn.eps)
    mod = mod.to(device)
    assert fused_scout(mod, x.to(device)) is None                   # the wrong input kind for this module
    fused = fused_scout(mod, x.to(device), "hidden_router_topk", E)
    assert fused is not None
    pred = fused(got_rows)
    torch.testing.assert_close(pred.cpu(), torch.from_numpy(want), rtol=1e-3, atol=1e-7)


def test_rs_building_blocks_reject_bad_arguments(device):
    ops = _ops()
    x = torch.zeros((4, 64), device=device)
    w, b = torch.zeros((16, 64), device=device), torch.zeros(16, device=device)
    with pytest.raises(Exception):
        ops.rs_dense(x[:, :60].contiguous(), w[:, :60].contiguous(), b)          # width off the 8-grid
    with pytest.raises(Exception):
        ops.rs_dense(x, w, b, act="tanh")
    with pytest.raises(Exception):
        ops.rs_layernorm(x, torch.ones(64, device=device), torch.zeros(64, device=device), -1.0)
    with pytest.raises(Exception):
        ops.rs_layernorm(x, torch.ones(64, device=device), torch.zeros(64, device=device), 1e-5,
                         out=torch.empty((4, 32), device=device))               # rows shorter than the width
    with pytest.raises(Exception):
        ops.rs_softmax(torch.zeros((2, 300), device=device))                    # more than 256 experts
    with pytest.raises(Exception):
        ops.rs_features(x.bfloat16(), torch.zeros((4, 2), device=device, dtype=torch.int64),
                        torch.zeros((4, 2), device=device, dtype=torch.bfloat16), 300)


@pytest.mark.parametrize("T,decode", [(8, True), (128, False)])
def test_ffn_fp32_matches_oracle(device, T, decode):
    ops = _ops()
    layer = make_layer(256, 10, 128, 3, dtype=torch.float32, seed=41, std=0.05)
    x = make_hidden(T, 256, torch.float32, seed=42)
    topv, topi = _routing(layer, x)
    out, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=decode)
    ref = ref_moe.experts_world1_exact(x, topi, topv, layer["experts"])
    torch.testing.assert_close(out, ref, **F32_TOL)


def test_segment_order_changes_nothing(device):
    """EPIPE reorders expert execution; values must not move (host-ordered segment list)."""
    ops = _ops()
    layer = make_layer(512, 12, 256, 4, dtype=torch.bfloat16, seed=51, std=0.05)
    x = make_hidden(16, 512, torch.bfloat16, seed=52)
    topv, topi = _routing(layer, x)
    base, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=True)
    active = sorted(set(topi.reshape(-1).tolist()))
    shuffled = list(reversed(active))
    other, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=True, order=shuffled)
    assert torch.equal(base, other)
    pre, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=False, order=shuffled)
    pre2, _, _ = _run_routed(ops, layer, x, topv, topi, device, decode=False)
    assert torch.equal(pre, pre2)


# ------------------------------------------------------------------ weight layout
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_tile_weight_kernel_matches_host_packing(device, dtype):
    from sparse_amd import _lib, ops
    from sparse_amd.weights import tile_weight, untile_weight
    w = torch.randn(48, 192).to(dtype)
    ref = tile_weight(w)
    assert torch.equal(untile_weight(ref, 48, 192), w)
    src = w.to(device)
    dst = torch.empty(48 * 192, device=device, dtype=dtype)
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.sparse_hip_tile_weight(src.data_ptr(), dst.data_ptr(), 48, 192, ops.dtype_code(dtype), 1, stream),
               "tile")
    assert torch.equal(dst.cpu(), ref)
    back = torch.empty_like(src)
    _lib.check(lib.sparse_hip_tile_weight(dst.data_ptr(), back.data_ptr(), 48, 192, ops.dtype_code(dtype), 0, stream),
               "untile")
    assert torch.equal(back.cpu(), w)
    with pytest.raises(ValueError):
        _lib.check(lib.sparse_hip_tile_weight(src.data_ptr(), dst.data_ptr(), 40, 192, ops.dtype_code(dtype), 1,
                                              stream), "tile")


# ------------------------------------------------------------------ shared expert + combine

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("H,E,I,K,Is,T,gated", [
    (512, 12, 256, 4, 384, 300, True),        # 8 / 4 / 6 k slabs, ragged segments
    (2048, 60, 1408, 4, 5632, 700, True),     # the Qwen shape
    (2048, 64, 1408, 6, 2816, 1100, False),   # the DeepSeek shape: more tiles than one round of the grid
    (320, 6, 192, 2, 448, 200, False),        # odd slab counts (5, 3, 7), column tiles that end inside a group
    (64, 3, 64, 1, 64, 129, True),            # one slab, one column tile, K = 1
])
def test_merged_prefill_equals_the_separate_calls(device, dtype, H, E, I, K, Is, T, gated):
    """Routed experts and shared expert of a prefill-size call as one launch per projection
    (``sparse_hip_moe_ffn_prefill``) against ``grouped_swiglu`` + ``shared_expert``: the same bits in the
    routed rows, the routed intermediate, the shared intermediate and the shared output; with the routed
    experts alone and with the shared expert alone; counted waits against full drains."""
    from sparse_amd import _lib
    from sparse_amd.weights import ExpertSlab, tile_weight
    ops = _ops()
    lib = _lib.load()
    layer = make_layer(H, E, I, K, Is=Is, shared_gate=gated, dtype=dtype, seed=71 + H, std=0.05)
    x = make_hidden(T, H, dtype, seed=72 + T)
    g = torch.Generator().manual_seed(73)
    popularity = 1.0 / torch.arange(1, E + 1, dtype=torch.float32) ** 1.1
    if E > 3:
        popularity[E - 1] = 0.0                                               # an expert nobody routes to
    topi = torch.multinomial(popularity.expand(T, E), K, replacement=False, generator=g)
    topv = torch.rand(T, K, generator=g).to(dtype)
    slab = ExpertSlab.resident(layer["experts"], H, I, dtype, device)
    ex = ops.make_experts(slab.data, slab.expert_slot, E, H, I)
    xd, tvd = x.to(device), topv.to(device)
    perm = ops.permute_build(topi.to(device), E)
    segs = ops.seglist_device(perm, min(E, T * K))
    gw, uw, dw = (tile_weight(t.to(device)).reshape(t.shape).contiguous() for t in layer["shared"])
    sg = None
    if gated:
        sg = torch.nn.functional.linear(x.float(), layer["shared_gate_w"].float().reshape(1, -1)).reshape(-1)
        sg = sg.to(dtype).to(device)

    def fresh():
        return (torch.zeros((T * K, I), device=device, dtype=dtype), torch.zeros((T * K, H), device=device, dtype=dtype),
                torch.zeros((T, Is), device=device, dtype=dtype), torch.zeros((T, H), device=device, dtype=dtype))

    want = fresh()
    ops.grouped_swiglu(ex, xd, tvd, perm, segs, want[0], want[1], decode=False)
    ops.shared_expert(xd, gw, uw, dw, sg, want[2], want[3])
    names = ("routed intermediate", "routed rows", "shared intermediate", "shared output")

    def merged(shared=True, routed=True):
        got = fresh()
        ops.moe_ffn_prefill(ex, xd, tvd, perm, segs if routed else ops.seglist_host([], []), got[0], got[1],
                            (gw, uw, dw) if shared else None, sg, got[2] if shared else None,
                            got[3] if shared else None)
        torch.cuda.synchronize()
        return got

    got = merged()
    for a, b, what in zip(got, want, names):
        assert torch.equal(a, b), what
    assert float(got[1].float().abs().max()) > 0 and float(got[3].float().abs().max()) > 0
    only_routed = merged(shared=False)
    assert torch.equal(only_routed[0], want[0]) and torch.equal(only_routed[1], want[1])
    assert int(only_routed[3].abs().sum()) == 0
    only_shared = merged(routed=False)
    assert torch.equal(only_shared[2], want[2]) and torch.equal(only_shared[3], want[3])
    assert int(only_shared[1].abs().sum()) == 0
    assert lib.sparse_hip_prefill_drain_waits(1) == 0
    try:
        safe = merged()
    finally:
        assert lib.sparse_hip_prefill_drain_waits(0) == 1
    for a, b, what in zip(safe, want, names):
        assert torch.equal(a, b), f"{what}: counted waits and full drains differ"


def test_merged_prefill_rejects_bad_arguments(device):
    ops = _ops()
    from sparse_amd._lib import SparseHipError
    from sparse_amd.weights import ExpertSlab
    layer = make_layer(128, 4, 64, 2, Is=64, dtype=torch.float32, seed=5)
    slab = ExpertSlab.resident(layer["experts"], 128, 64, torch.float32, device)
    ex = ops.make_experts(slab.data, slab.expert_slot, 4, 128, 64)
    x = make_hidden(40, 128, torch.float32).to(device)
    with pytest.raises((SparseHipError, ValueError)):       # fp32 takes the separate entry points
        perm = ops.permute_build(torch.zeros((40, 2), dtype=torch.int64, device=device), 4)
        ops.moe_ffn_prefill(ex, x, torch.ones((40, 2), device=device), perm, ops.seglist_device(perm, 4),
                            torch.zeros((80, 64), device=device), torch.zeros((80, 128), device=device))

@pytest.mark.parametrize("dtype,T", [(torch.bfloat16, 8), (torch.bfloat16, 32), (torch.bfloat16, 200),
                                     (torch.bfloat16, 2048), (torch.bfloat16, 2500),   # XCDs own bands of M-tiles
                                     (torch.float32, 8), (torch.float32, 100)])
@pytest.mark.parametrize("gated", [True, False])
def test_shared_expert(device, dtype, T, gated):
    ops = _ops()
    layer = make_layer(512, 4, 64, 2, Is=384, shared_gate=gated, dtype=dtype, seed=61, std=0.05)
    x = make_hidden(T, 512, dtype, seed=62)
    ref = ref_moe.shared_expert_forward(x, layer["shared"], layer["shared_gate_w"])
    xd = x.to(device)
    sg = None
    if gated:
        _, sg = ops.router_logits(xd, layer["gate_w"].to(device), layer["shared_gate_w"].to(device))
    from sparse_amd.weights import tile_weight
    gw, uw, dw = (tile_weight(t).reshape(t.shape).contiguous().to(device) for t in layer["shared"])
    inter = torch.empty((T, 384), device=device, dtype=dtype)
    out = torch.empty((T, 512), device=device, dtype=dtype)
    ops.shared_expert(xd, gw, uw, dw, sg, inter, out)
    torch.testing.assert_close(out.cpu().float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("T", [1, 8, 17, 32])
@pytest.mark.parametrize("gated", [True, False])
def test_fused_decode_with_the_shared_reduction_split(device, T, gated):
    """The fused decode launch pair with the workspace that spreads the shared expert's long
    down-projection reduction over four workgroups per tile, finished by combine_split: routed
    parts bit for bit those of the one-workgroup form, the layer output within one bf16
    rounding of combine() on that form (the fp32 sum is grouped differently) and within
    tolerance of the oracle, the same bits call after call, also when the two forms alternate."""
    ops = _ops()
    from sparse_amd.weights import ExpertSlab, tile_weight
    H, E, I, K, Is = 512, 8, 128, 2, 1024
    dtype = torch.bfloat16
    layer = make_layer(H, E, I, K, Is=Is, shared_gate=gated, dtype=dtype, seed=81, std=0.05)
    xc = make_hidden(T, H, dtype, seed=82)
    x = xc.to(device)
    slab = ExpertSlab.resident(layer["experts"], H, I, dtype, device)
    experts = ops.make_experts(slab.data, slab.expert_slot, E, H, I)
    logits, sg = ops.router_logits(x, layer["gate_w"].to(device), layer["shared_gate_w"].to(device) if gated else None)
    topv, topi = ops.gate_topk(logits, K, out_dtype=dtype)
    perm = ops.permute_build(topi, E)
    segs = ops.seglist_device(perm, min(E, T * K))
    sw = tuple(tile_weight(t).reshape(t.shape).contiguous().to(device) for t in layer["shared"])
    nparts = ops.decode_split_parts(Is)
    assert nparts == 4 and ops.decode_split_parts(64 * 7) == 1
    ws = ops.decode_split_workspace(T, H, device)

    def run(split):
        inter = torch.empty((T * K, I), device=device, dtype=dtype)
        parts = torch.empty((T * K, H), device=device, dtype=dtype)
        sh_inter = torch.empty((T, Is), device=device, dtype=dtype)
        sh_out = torch.full((T, H), float("nan"), device=device, dtype=dtype)
        out = torch.empty((T, H), device=device, dtype=dtype)
        ws.fill_(float("nan"))
        ops.moe_ffn_decode(experts, x, topv, perm, segs, inter, parts, sw, sg if gated else None, sh_inter, sh_out,
                           ws if split else None)
        if split:
            assert torch.isnan(sh_out.float()).all()            # left to combine_split
            ops.combine_split(parts, perm, ws, nparts, sg if gated else None, T, K, out)
        else:
            ops.combine(parts, perm, sh_out, T, K, out)
        torch.cuda.synchronize()
        return parts, out

    parts0, out0 = run(False)
    ref, _, _, _ = ref_moe.moe_forward(xc, layer["gate_w"], layer["experts"], K, layer["shared"], layer["shared_gate_w"],
                                       router_logits=logits.cpu())
    first = None
    for split in (True, False, True, True):
        parts1, out1 = run(split)
        assert torch.equal(parts1, parts0)
        if not split:
            assert torch.equal(out1, out0)
            continue
        first = out1 if first is None else first
        assert torch.equal(out1, first) and not torch.isnan(out1.float()).any()
        torch.testing.assert_close(out1.float(), out0.float(), rtol=1.6e-2, atol=1e-6)   # two bf16 roundings apart at most
        torch.testing.assert_close(out1.cpu().float(), ref.float(), **tol(dtype))
    assert (first == out0).float().mean() > 0.9                      # most sums round the same way


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_combine_is_ordered_sum(device, dtype):
    ops = _ops()
    T, K, H, E = 37, 4, 256, 20
    g = torch.Generator().manual_seed(71)
    scores = torch.rand(T, E, generator=g)
    topi = torch.topk(scores, K, dim=1).indices.to(torch.int64)
    parts_tkh = (torch.randn(T, K, H, generator=g) * 3).to(dtype)
    shared = torch.randn(T, H, generator=g).to(dtype)
    ref = ref_moe.combine_expert_outputs(parts_tkh, topi) + shared
    p = ops.permute_build(topi.to(device), E)
    perm = p.perm.cpu().long()
    parts_sorted = parts_tkh.reshape(T * K, H)[perm].contiguous().to(device)
    out = torch.empty((T, H), device=device, dtype=dtype)
    ops.combine(parts_sorted, p, shared.to(device), T, K, out)
    # same adds in the same order: bit-exact
    assert torch.equal(out.cpu(), ref)
