"""RS (routing scout) predictors: small per-layer MLPs that guess the next layer's experts.

``RoutingScoutMLP`` has the layer stack and parameter names of the reference's module of
the same name (utils/eval_core.py:3402-3417: Linear, BatchNorm1d, ReLU, Dropout(0.1),
Linear, Softmax), so a bank trained for the reference (``rs_l{L}_inL{L-1}.pth`` payloads
with a ``state_dict``, :3490-3550) loads into it unchanged.  Prediction runs on the device
in fp32 through PyTorch; only its top-k leaves the device.
"""
from __future__ import annotations

from typing import List, Optional

import torch
from torch import nn


class RoutingScoutMLP(nn.Module):
    def __init__(self, input_dim: int, num_experts: int, hidden_dim: int = 1024) -> None:
        super().__init__()
        layers = [
            nn.Linear(input_dim, hidden_dim),
            nn.BatchNorm1d(hidden_dim),
            nn.ReLU(),
            nn.Dropout(0.1),
            nn.Linear(hidden_dim, num_experts),
            nn.Softmax(dim=-1),
        ]
        self.mlp = nn.Sequential(*layers)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.mlp(x.reshape(-1, x.shape[-1]))


def random_init_bank(num_layers: int, hidden: int, num_experts: int, hidden_dim: int = 512, seed: int = 0,
                     device: Optional[torch.device] = None) -> List[Optional[nn.Module]]:
    """One seeded random-init predictor per target layer ``1 .. num_layers-1`` (entry 0 is
    None: nothing predicts the first layer), in eval mode."""
    bank: List[Optional[nn.Module]] = [None]
    for layer in range(1, num_layers):
        torch.manual_seed(seed + layer)
        module = RoutingScoutMLP(hidden, num_experts, hidden_dim=hidden_dim).eval()
        if device is not None:
            module = module.to(device)
        for p in module.parameters():
            p.requires_grad_(False)
        bank.append(module)
    return bank


def load_rs_payload(path: str, device: Optional[torch.device] = None) -> nn.Module:
    """Load one ``rs_l{L}_inL{L-1}.pth`` payload (dict with ``input_dim``, ``hidden_dim``,
    ``state_dict`` and the expert count implied by the last Linear)."""
    payload = torch.load(path, map_location="cpu", weights_only=True)
    state = payload["state_dict"]
    num_experts = int(state["mlp.4.weight"].shape[0])
    module = RoutingScoutMLP(int(payload["input_dim"]), num_experts, hidden_dim=int(payload["hidden_dim"]))
    module.load_state_dict(state)
    module.eval()
    return module.to(device) if device is not None else module


def informed_bank(gate_weights: List[Optional[torch.Tensor]], hidden_dim: int = 512,
                  device: Optional[torch.device] = None) -> List[Optional[nn.Module]]:
    """Predictors that reproduce a given router: entry l is built from ``gate_weights[l]``
    ([E,H], the gate of layer l) so that ``RS_l(x) = softmax(gate_l x)``.  The hidden layer
    holds +gate and -gate rows (ReLU(a) - ReLU(-a) = a), BatchNorm is the identity in eval
    mode.  Useful where every layer of a synthetic stack reads the same hidden state, so the
    next layer's routing is predictable from the current layer's input."""
    bank: List[Optional[nn.Module]] = []
    for gw in gate_weights:
        if gw is None:
            bank.append(None)
            continue
        E, H = gw.shape
        if 2 * E > hidden_dim:
            raise ValueError("hidden_dim must be at least twice the number of experts")
        module = RoutingScoutMLP(H, E, hidden_dim=hidden_dim).eval()
        lin1, bn, lin2 = module.mlp[0], module.mlp[1], module.mlp[4]
        with torch.no_grad():
            lin1.weight.zero_()
            lin1.bias.zero_()
            lin1.weight[:E] = gw.float().cpu()
            lin1.weight[E:2 * E] = -gw.float().cpu()
            bn.weight.fill_(1.0)
            bn.bias.zero_()
            bn.running_mean.zero_()
            bn.running_var.fill_(1.0)
            lin2.weight.zero_()
            lin2.bias.zero_()
            idx = torch.arange(E)
            lin2.weight[idx, idx] = 1.0
            lin2.weight[idx, E + idx] = -1.0
        for p in module.parameters():
            p.requires_grad_(False)
        bank.append(module.to(device) if device is not None else module)
    return bank
