"""RS (routing scout) predictors: small per-layer MLPs that guess the next layer's experts.

``RoutingScoutMLP`` has the layer stack and parameter names of the reference's module of
the same name (utils/eval_core.py:3402-3417: Linear, BatchNorm1d, ReLU, Dropout(0.1),
Linear, Softmax), so a bank trained for the reference (``rs_l{L}_inL{L-1}.pth`` payloads
with a ``state_dict``, :3490-3550) loads into it unchanged.  Prediction runs on the device
in fp32 through the HIP predictor kernels, at any token count: the plain MLP in two launches
(``FusedScout``, ``sparse_hip_rs_predict``), the residual predictor as a chain of LayerNorm and dense
launches (``FusedResidualScout``), predictors that also read the routing after one launch that lays
their input rows out; only the top-k leaves the device.  The ``nn.Module`` classes hold the parameters
(and run on host tensors, in training, and for shapes the kernels do not take).
"""
from __future__ import annotations

import os
import re
from typing import Any, Dict, List, Optional, Tuple

import torch
from torch import nn

from . import _lib


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


def _padded_columns(w: torch.Tensor) -> torch.Tensor:
    """``w [D, H]`` as fp32 with zero columns appended up to a multiple of 8 (the dense kernel reads rows
    eight values at a time; an input row padded with zeros the same way gives the same products)."""
    w = w.detach().float()
    pad = -w.shape[1] % 8
    if pad:
        w = torch.cat([w, w.new_zeros((w.shape[0], pad))], dim=1)
    return w.contiguous()


class FusedScout:
    """The parameters of a ``RoutingScoutMLP`` in eval mode as the HIP predictor kernel takes them: fp32,
    row-major, the BatchNorm's running statistics and affine folded into the first Linear (eval mode makes
    it a per-row scale and shift).  Built once per module (``fused_scout``); a module that is retrained or
    moved afterwards must be fused again."""

    def __init__(self, module: "RoutingScoutMLP") -> None:
        lin1, bn, lin2 = module.mlp[0], module.mlp[1], module.mlp[4]
        with torch.no_grad():
            scale = bn.weight.float() / torch.sqrt(bn.running_var.float() + bn.eps)
            self.w1 = _padded_columns(lin1.weight.float() * scale[:, None])
            self.b1 = ((lin1.bias.float() - bn.running_mean.float()) * scale + bn.bias.float()).contiguous()
            self.w2 = lin2.weight.float().contiguous()
            self.b2 = lin2.bias.float().contiguous()
        self.input_dim, self.hidden_dim, self.num_experts = lin1.in_features, self.w1.shape[0], self.w2.shape[0]
        self.device = self.w1.device

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        """``x [T, input_dim rounded up to a multiple of 8]``, in the activations' dtype or fp32."""
        from . import ops
        return ops.rs_predict(x, self.w1, self.b1, self.w2, self.b2)


class FusedResidualScout:
    """The parameters of a ``RoutingScoutResidualMLP`` in eval mode (Dropout is the identity) as the HIP
    kernels take them, and the launch chain: LayerNorm, dense + GELU; per unit LayerNorm, dense + GELU,
    dense + residual; LayerNorm, dense, softmax."""

    def __init__(self, module: "RoutingScoutResidualMLP") -> None:
        f = lambda t: t.detach().float().contiguous()
        norm, lin = module.input[0], module.input[1]
        self.stem = (f(norm.weight), f(norm.bias), float(norm.eps), _padded_columns(lin.weight), f(lin.bias))
        self.units = []
        for unit in module.blocks:
            n, up, down = unit.net[0], unit.net[1], unit.net[4]
            self.units.append((f(n.weight), f(n.bias), float(n.eps), f(up.weight), f(up.bias), f(down.weight),
                               f(down.bias)))
        self.out_norm = (f(module.out_norm.weight), f(module.out_norm.bias), float(module.out_norm.eps))
        self.head = (f(module.head.weight), f(module.head.bias))
        self.input_dim, self.hidden_dim, self.num_experts = lin.in_features, lin.out_features, module.head.out_features
        self.device = self.head[0].device

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        """``x [T, input_dim rounded up to a multiple of 8]``, in the activations' dtype or fp32."""
        from . import ops
        T = x.shape[0]
        gamma, beta, eps, w, b = self.stem
        new = lambda width: torch.empty((T, width), device=x.device, dtype=torch.float32)
        normed = ops.rs_layernorm(x, gamma, beta, eps, width=self.input_dim)
        h = ops.rs_dense(normed, w, b, act="gelu")
        if self.units:
            normed, wide, other = new(self.hidden_dim), new(2 * self.hidden_dim), new(self.hidden_dim)
        for gamma, beta, eps, w_up, b_up, w_down, b_down in self.units:
            ops.rs_layernorm(h, gamma, beta, eps, out=normed)
            ops.rs_dense(normed, w_up, b_up, act="gelu", out=wide)
            ops.rs_dense(wide, w_down, b_down, residual=h, out=other)
            h, other = other, h
        gamma, beta, eps = self.out_norm
        normed = ops.rs_layernorm(h, gamma, beta, eps)
        return ops.rs_softmax(ops.rs_dense(normed, self.head[0], self.head[1]))


def fused_scout(module: Any, x: torch.Tensor, mode: str = "hidden", num_experts: int = 0):
    """The HIP form of the predictor ``module`` for a call on ``x [T, H]`` with input kind ``mode``
    (``hidden``: the token rows; ``hidden_router_topk``: the token rows followed by ``num_experts``
    routing-weight columns), or None where the kernels do not apply (another class, training mode, host
    tensors, parameters on another device, widths the kernels do not take); cached on the module."""
    if not (isinstance(module, (RoutingScoutMLP, RoutingScoutResidualMLP)) and not module.training
            and x.is_cuda and x.dim() == 2 and x.shape[0] >= 1):
        return None
    if mode == "hidden":
        width = x.shape[1]
        if width % 8:
            return None
    elif mode == "hidden_router_topk":
        width = x.shape[1] + int(num_experts)
        if not 1 <= int(num_experts) <= _lib.MAX_EXPERTS:
            return None
    else:
        return None
    fused = getattr(module, "_sparse_fused", None)
    if fused is None or fused.device != x.device:
        plain = isinstance(module, RoutingScoutMLP)
        first = module.mlp[0] if plain else module.input[1]
        last = module.mlp[4] if plain else module.head
        if first.weight.device != x.device or last.out_features > _lib.MAX_EXPERTS:
            return None
        if plain and first.out_features % 4:
            return None
        if not plain and first.out_features % 8:
            return None
        fused = FusedScout(module) if plain else FusedResidualScout(module)
        object.__setattr__(module, "_sparse_fused", fused)
    return fused if fused.input_dim == width else None


class _ResidualUnit(nn.Module):
    def __init__(self, width: int, dropout: float) -> None:
        super().__init__()
        self.net = nn.Sequential(
            nn.LayerNorm(width), nn.Linear(width, 2 * width), nn.GELU(), nn.Dropout(dropout),
            nn.Linear(2 * width, width), nn.Dropout(dropout))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return x + self.net(x)


class RoutingScoutResidualMLP(nn.Module):
    """The deeper predictor (``model_type = next_layer_residual_logits_rs``): LayerNorm +
    Linear + GELU stem, pre-norm residual units twice as wide inside, LayerNorm, Linear head,
    softmax.  Submodule names (``input``, ``blocks.N.net``, ``out_norm``, ``head``) follow
    utils/eval_core.py:3419-3464 so that its checkpoints load by key."""

    def __init__(self, input_dim: int, num_experts: int, hidden_dim: int = 1024, num_hidden_layers: int = 3,
                 dropout: float = 0.05) -> None:
        super().__init__()
        self.input = nn.Sequential(nn.LayerNorm(input_dim), nn.Linear(input_dim, hidden_dim), nn.GELU(),
                                   nn.Dropout(dropout))
        self.blocks = nn.Sequential(*[_ResidualUnit(hidden_dim, dropout) for _ in range(max(0, int(num_hidden_layers)))])
        self.out_norm = nn.LayerNorm(hidden_dim)
        self.head = nn.Linear(hidden_dim, num_experts)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        h = self.blocks(self.input(x.reshape(-1, x.shape[-1])))
        return torch.softmax(self.head(self.out_norm(h)), dim=-1)


def topk_for_planning(pred: torch.Tensor, pred_k: int, norm_topk_prob: bool, dtype: torch.dtype):
    """What the prefetch planner is fed from a predictor output ``pred [T,E]`` (fp32): the top
    ``pred_k`` experts per token, renormalised only for models that renormalise their router,
    with the probabilities rounded to the activation dtype and widened again
    (utils/eval_core.py:10985-10996).  Returns ``(topi int64 [T,k], topv float32 [T,k])``."""
    pred_k = min(int(pred.shape[-1]), int(pred_k))
    topv, topi = stable_topk(pred.to(torch.float32), pred_k)
    if norm_topk_prob:
        topv = topv / topv.sum(dim=-1, keepdim=True).clamp_min(1e-12)
    return topi.to(torch.long), topv.to(dtype).to(torch.float32)


def stable_topk(values: torch.Tensor, k: int):
    """Top-k of fp32 rows, descending, equal values in ascending index order (``torch.topk``
    leaves that order open, and the planner's candidate order depends on it).  Device rows go
    through the HIP top-k kernel; rows wider than the kernel takes, more than its 16
    selections, or host tensors (planner logic exercised without a device) are ranked by a
    stable sort."""
    if values.is_cuda and k <= _lib.MAX_TOPK and values.shape[-1] <= _lib.MAX_EXPERTS and values.dim() == 2:
        from . import ops
        return ops.topk_values(values.contiguous(), k)
    order = torch.sort(values, dim=-1, descending=True, stable=True)
    return order.values[..., :k].contiguous(), order.indices[..., :k].contiguous()


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


# ---- checkpoint directories -------------------------------------------------------------
_CKPT_NAME = re.compile(r"(rs|cv)_l(\d+)_inL(-?\d+)\.pth")


def _state_dict_of(payload: Any) -> Dict[str, torch.Tensor]:
    if isinstance(payload, dict):
        for key in ("state_dict", "model_state_dict"):
            if isinstance(payload.get(key), dict):
                return payload[key]
        if payload and all(torch.is_tensor(v) for v in payload.values()):
            return payload
    raise RuntimeError(f"Cannot extract state_dict from payload type={type(payload)}")


def module_from_payload(payload: Any, fallback_input_dim: int, fallback_num_experts: int) -> nn.Module:
    """Build the predictor a checkpoint payload describes (utils/eval_core.py:3490-3550):
    ``model_type`` picks the class, a bare state dict is a 1024-wide ``RoutingScoutMLP``.
    Only predictors of routing probabilities are built; cache-value checkpoints raise.  The
    checkpoint's ``feature_mode`` is left on the module as ``rs_feature_mode`` (``hidden``: the
    layer's hidden state; ``hidden_router_topk``: that plus ``router_topk_feature`` of the
    source layer's own routing), as the reference does (:3522, :3539)."""
    meta = payload if isinstance(payload, dict) else {}
    if meta.get("task", "") == "cache_value_rs":
        raise NotImplementedError("cache_value_rs checkpoints are not supported")
    feature = str(meta.get("feature_mode", "hidden"))
    kind = meta.get("model_type", "")
    input_dim = int(meta.get("input_dim", fallback_input_dim))
    num_experts = int(meta.get("num_experts", fallback_num_experts))
    hidden_dim = int(meta.get("hidden_dim", 1024))
    if kind == "next_layer_residual_logits_rs":
        module: nn.Module = RoutingScoutResidualMLP(input_dim, num_experts, hidden_dim=hidden_dim,
                                                    num_hidden_layers=int(meta.get("num_hidden_layers", 3)))
    elif kind == "independent_light_logits_rs":
        module = RoutingScoutMLP(input_dim, num_experts, hidden_dim=hidden_dim)
    else:
        module = RoutingScoutMLP(fallback_input_dim, fallback_num_experts, hidden_dim=1024)
    module.load_state_dict(_state_dict_of(payload), strict=True)
    if kind in ("next_layer_residual_logits_rs", "independent_light_logits_rs"):
        module.rs_feature_mode = feature
    return module


def router_topk_feature(idx: torch.Tensor, w: torch.Tensor, num_experts: int) -> torch.Tensor:
    """Dense ``[T, E]`` fp32 rows holding each token's routing weights, renormalised to sum 1,
    at its chosen experts (utils/eval_core.py:10903-10908)."""
    feat = torch.zeros((idx.shape[0], int(num_experts)), device=idx.device, dtype=torch.float32)
    ww = w.float()
    ww = ww / ww.sum(dim=-1, keepdim=True).clamp_min(1e-12)
    feat.scatter_add_(1, idx.to(torch.long), ww)
    return feat


def load_rs_bank(rs_dir: str, num_layers: int, hidden_dim: int, num_experts: int,
                 device: Optional[torch.device] = None,
                 require_complete: bool = True) -> Tuple[List[nn.Module], List[int], List[str]]:
    """Load a directory of next-layer predictors, ``rs_l{L}_inL{L-1}.pth`` for target layer L
    (utils/eval_core.py:3553-3658).  Returns ``(modules, source_layers, missing)`` with one
    module per layer.  Layers below the first target present are never predicted, so their
    absence is not an error and they get an untrained placeholder, as do other absent layers
    when ``require_complete`` is false; with it true an absent layer raises.  Files are read
    with ``weights_only=True``."""
    names = {}
    for name in sorted(os.listdir(rs_dir)):
        m = _CKPT_NAME.fullmatch(name)
        if m and int(m.group(2)) == int(m.group(3)) + 1:
            names.setdefault(int(m.group(2)), {})[m.group(1)] = name
    if not names:
        raise NotImplementedError(f"{rs_dir} holds no next-layer predictors (rs_l{{L}}_inL{{L-1}}.pth)")
    first_target = min(names)
    modules: List[nn.Module] = []
    sources: List[int] = []
    missing: List[str] = []
    for layer in range(int(num_layers)):
        found = names.get(layer, {})
        name = found.get("cv") or found.get("rs")
        if name is None:
            if layer >= first_target:
                missing.append(f"[L{layer}] tried: cv_l{layer}_inL{layer - 1}.pth, rs_l{layer}_inL{layer - 1}.pth")
            module: nn.Module = RoutingScoutMLP(hidden_dim, num_experts, hidden_dim=1024)
            source = layer - 1
        else:
            payload = torch.load(os.path.join(rs_dir, name), map_location="cpu", weights_only=True)
            module = module_from_payload(payload, hidden_dim, num_experts)
            source = int(payload.get("source_layer", layer - 1)) if isinstance(payload, dict) else layer - 1
        module = module.to(torch.float32).eval()
        for p in module.parameters():
            p.requires_grad_(False)
        modules.append(module.to(device) if device is not None else module)
        sources.append(source)
    if require_complete and missing:
        raise RuntimeError("RS checkpoint set incomplete:\n" + "\n".join(missing[:32]))
    return modules, sources, missing
