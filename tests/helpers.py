"""Seeded synthetic MoE layers shared by the tests (weights ~N(0, 0.02), hidden ~N(0, 1))."""
from __future__ import annotations

import torch

Q_SHAPE = dict(H=2048, E=60, I=1408, K=4, Is=5632, shared_gate=True)
D_SHAPE = dict(H=2048, E=64, I=1408, K=6, Is=2816, shared_gate=False)


def make_layer(H, E, I, K, Is=0, shared_gate=False, dtype=torch.float32, seed=0, std=0.02):
    g = torch.Generator().manual_seed(seed)

    def w(*shape):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    layer = dict(H=H, E=E, I=I, K=K, Is=Is, dtype=dtype)
    layer["gate_w"] = w(E, H)
    layer["experts"] = [(w(I, H), w(I, H), w(H, I)) for _ in range(E)]
    layer["shared"] = (w(Is, H), w(Is, H), w(H, Is)) if Is else None
    layer["shared_gate_w"] = w(H) if (Is and shared_gate) else None
    return layer


def make_hidden(T, H, dtype=torch.float32, seed=1000):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(T, H, generator=g).to(dtype)


def oracle_layer(mlp_block):
    """CPU tensors of a duck-typed ``mlp_block`` in the oracle's argument format."""
    def cpu(t):
        return t.detach().cpu()

    def triple(m):
        return (cpu(m.gate_proj.weight), cpu(m.up_proj.weight), cpu(m.down_proj.weight))

    experts = mlp_block.experts
    if hasattr(experts, "gate_up_proj"):
        gu, dn = cpu(experts.gate_up_proj), cpu(experts.down_proj)
        inter = gu.shape[1] // 2
        ex = [(gu[e, :inter].contiguous(), gu[e, inter:].contiguous(), dn[e].contiguous()) for e in range(gu.shape[0])]
    else:
        ex = [triple(m) for m in experts]
    shared_mod = getattr(mlp_block, "shared_expert", None) or getattr(mlp_block, "shared_experts", None)
    sg = getattr(mlp_block, "shared_expert_gate", None)
    return dict(
        gate_w=cpu(mlp_block.gate.weight),
        experts=ex,
        shared=triple(shared_mod) if shared_mod is not None else None,
        shared_gate_w=cpu(sg.weight).reshape(-1) if sg is not None else None,
        family="qwen_shared" if hasattr(mlp_block, "shared_expert") else "deepseek_shared",
    )


def copy_is_late(seed: int, layer: int, step: int, eid: int, rate: float) -> bool:
    """Whether the prefetch copy of expert ``eid`` admitted at ``step`` into ``layer`` is still
    in flight the first time anyone asks (a pure function of its arguments, so that traces
    recorded from different implementations agree on it whatever order they ask in)."""
    import zlib
    return (zlib.crc32(f"{seed}:{layer}:{step}:{eid}".encode()) % 10000) < int(rate * 10000)


def seeded_moe_layer(shape, T, dtype, seed, shared_gate=True, std=None):
    """Inputs of one small layer call, a pure function of its arguments: ``shape`` is
    ``(H, E, I, K, Is)``.  Used where a fixture stores only outputs: the script that records
    them and the test that replays them both build the inputs here; ``checksum`` guards
    against the generator ever producing other numbers.  The default weight scale gives
    these narrow layers the activation scale of the full-size configurations (weights of
    std 0.02 at a hidden size of 2048: pre-activations of std ~0.9, layer outputs of a few
    tenths), so the absolute tolerances stated for those apply unchanged."""
    H, E, I, _K, Is = shape
    if std is None:
        std = 0.02 * (2048.0 / H) ** 0.5
    g = torch.Generator().manual_seed(seed)

    def w(*dims):
        return (torch.randn(*dims, generator=g) * std).to(dtype)

    out = dict(x=torch.randn(T, H, generator=g).to(dtype), gate_w=w(E, H),
               experts=[(w(I, H), w(I, H), w(H, I)) for _ in range(E)],
               shared=(w(Is, H), w(Is, H), w(H, Is)) if Is else None,
               shared_gate_w=w(H) if (Is and shared_gate) else None)
    total = out["x"].double().abs().sum() + out["gate_w"].double().abs().sum()
    for triple in out["experts"] + ([out["shared"]] if Is else []):
        total = total + sum(t.double().abs().sum() for t in triple)
    out["checksum"] = float(total)
    return out


def seeded_prediction(seed: int, step: int, layer: int, T: int, E: int) -> "torch.Tensor":
    """Dense predictor output ``[T, E]`` (rows sum to one) for the prefetch planned at ``step``
    by ``layer`` for the next one; a pure function of its arguments."""
    g = torch.Generator().manual_seed(1000003 * seed + 1009 * step + layer)
    return torch.softmax(torch.randn(T, E, generator=g) * 2.0, dim=-1)
