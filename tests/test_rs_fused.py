"""The folded form of the routing-scout MLP (what the HIP predictor kernel is fed), checked on the host:
BatchNorm in eval mode is a per-row scale and shift of the first Linear, Dropout is the identity."""
import torch

import numpy as np

from oracle import ref_rs
from sparse_amd.rs import FusedResidualScout, FusedScout, RoutingScoutMLP, RoutingScoutResidualMLP, fused_scout


def _module(H=96, E=12, D=40, seed=3):
    torch.manual_seed(seed)
    mod = RoutingScoutMLP(H, E, hidden_dim=D)
    bn = mod.mlp[1]
    with torch.no_grad():
        bn.running_mean.copy_(torch.randn(D) * 0.4)
        bn.running_var.copy_(torch.rand(D) * 3 + 0.1)
        bn.weight.copy_(torch.rand(D) + 0.5)
        bn.bias.copy_(torch.randn(D) * 0.3)
    return mod.eval()


def test_folded_parameters_reproduce_the_module():
    mod = _module()
    f = FusedScout(mod)
    assert (f.input_dim, f.hidden_dim, f.num_experts) == (96, 40, 12)
    x = torch.randn(7, 96)
    with torch.no_grad():
        want = mod(x)
    hidden = torch.relu(x @ f.w1.T + f.b1)
    got = torch.softmax(hidden @ f.w2.T + f.b2, dim=-1)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-7)
    # the fold is not a no-op: without it the answer differs
    plain = torch.softmax(torch.relu(x @ mod.mlp[0].weight.T + mod.mlp[0].bias) @ f.w2.T + f.b2, dim=-1)
    assert (plain - want).abs().max() > 1e-3


def test_host_tensors_and_other_predictors_keep_the_module_path():
    mod = _module()
    assert fused_scout(mod, torch.randn(4, 96)) is None                 # host tensor: no HIP predictor
    assert fused_scout(torch.nn.Linear(96, 12), torch.randn(4, 96)) is None


def _residual_module(H=96, E=12, D=40, layers=2, seed=4):
    torch.manual_seed(seed)
    mod = RoutingScoutResidualMLP(H, E, hidden_dim=D, num_hidden_layers=layers)
    with torch.no_grad():
        for m in mod.modules():
            if isinstance(m, torch.nn.LayerNorm):          # not the identity affine
                m.weight.copy_(torch.rand_like(m.weight) + 0.5)
                m.bias.copy_(torch.randn_like(m.bias) * 0.3)
        mod.head.weight.mul_(4.0)
    return mod.eval()


def _oracle_args(mod):
    n = lambda t: t.detach().numpy()
    stem = (n(mod.input[0].weight), n(mod.input[0].bias), n(mod.input[1].weight), n(mod.input[1].bias))
    units = [(n(u.net[0].weight), n(u.net[0].bias), n(u.net[1].weight), n(u.net[1].bias), n(u.net[4].weight),
              n(u.net[4].bias)) for u in mod.blocks]
    return stem, units, (n(mod.out_norm.weight), n(mod.out_norm.bias)), (n(mod.head.weight), n(mod.head.bias))


def test_residual_oracle_matches_torch_layers_and_hand_made_cases():
    """The numpy restatement of the residual predictor against ``torch.nn`` layers holding the same
    parameters (LayerNorm, exact GELU and Linear are library routines there), for zero, one and three
    units; plus two cases fixed by the mathematics."""
    for layers in (0, 1, 3):
        mod = _residual_module(layers=layers, seed=10 + layers)
        x = torch.randn(9, 96) * 2 + 0.5
        with torch.no_grad():
            want = mod(x).numpy()
        got = ref_rs.routing_scout_residual_forward(x.numpy(), *_oracle_args(mod))
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-7)
        np.testing.assert_allclose(got.sum(-1), 1.0, rtol=1e-5)
    # a unit whose second Linear is zero adds nothing: the answer equals the model without units
    mod = _residual_module(layers=1, seed=20)
    stem, units, out_norm, head = _oracle_args(mod)
    dead = [(u[0], u[1], u[2], u[3], np.zeros_like(u[4]), np.zeros_like(u[5])) for u in units]
    x = np.random.default_rng(0).standard_normal((5, 96)).astype(np.float32)
    np.testing.assert_array_equal(ref_rs.routing_scout_residual_forward(x, stem, dead, out_norm, head),
                                  ref_rs.routing_scout_residual_forward(x, stem, [], out_norm, head))
    assert np.abs(ref_rs.routing_scout_residual_forward(x, stem, units, out_norm, head)
                  - ref_rs.routing_scout_residual_forward(x, stem, [], out_norm, head)).max() > 1e-4
    # rows that are constant normalise to the LayerNorm's bias, whatever the constant
    a = ref_rs.routing_scout_residual_forward(np.full((2, 96), 3.0, np.float32), stem, units, out_norm, head)
    b = ref_rs.routing_scout_residual_forward(np.full((2, 96), -7.5, np.float32), stem, units, out_norm, head)
    np.testing.assert_allclose(a, b, rtol=1e-6)


def test_residual_fused_parameters_follow_the_module():
    mod = _residual_module(H=100, layers=2)                     # 100 is not a multiple of 8: padded columns
    f = FusedResidualScout(mod)
    assert (f.input_dim, f.hidden_dim, f.num_experts) == (100, 40, 12)
    assert f.stem[3].shape == (40, 104) and bool((f.stem[3][:, 100:] == 0).all())
    assert torch.equal(f.stem[3][:, :100], mod.input[1].weight)
    assert len(f.units) == 2 and f.units[1][3].shape == (80, 40) and f.units[1][5].shape == (40, 80)
    assert fused_scout(mod, torch.randn(4, 100)) is None          # host tensor
    assert fused_scout(mod, torch.randn(4, 100), mode="other") is None
