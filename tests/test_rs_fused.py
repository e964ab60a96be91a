"""The folded form of the routing-scout MLP (what the HIP predictor kernel is fed), checked on the host:
BatchNorm in eval mode is a per-row scale and shift of the first Linear, Dropout is the identity."""
import torch

from sparse_amd.rs import FusedScout, RoutingScoutMLP, fused_scout


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
