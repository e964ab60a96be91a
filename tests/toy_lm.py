"""A tiny attention-free causal LM with the Hugging Face call convention, for harness tests:
embedding -> layers of ``x + mlp(rmsnorm(x))`` -> lm_head.  ``mlp`` is any module taking
``[B,S,H]``; a tuple return (Qwen family: ``(hidden, router_logits)``) is unpacked the way
the Hugging Face decoder layers do."""
from types import SimpleNamespace

import torch
from torch import nn


class ToyLayer(nn.Module):
    def __init__(self, mlp):
        super().__init__()
        self.mlp = mlp

    def forward(self, x):
        h = x.float()
        h = (h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6)).to(x.dtype)
        y = self.mlp(h)
        if isinstance(y, tuple):
            y = y[0]
        return x + y


class ToyDecoder(nn.Module):
    def __init__(self, vocab, hidden, mlps, dtype, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.embed = nn.Parameter(torch.randn(vocab, hidden, generator=g).to(dtype), requires_grad=False)
        self.layers = nn.ModuleList([ToyLayer(m) for m in mlps])


class ToyCausalLM(nn.Module):
    def __init__(self, vocab, hidden, mlps, dtype=torch.float32, seed=0):
        super().__init__()
        self.model = ToyDecoder(vocab, hidden, mlps, dtype, seed)
        g = torch.Generator().manual_seed(seed + 1)
        self.lm_head = nn.Parameter((torch.randn(vocab, hidden, generator=g) * 0.05).to(dtype), requires_grad=False)
        self.calls = []

    def forward(self, input_ids, attention_mask=None, use_cache=True, past_key_values=None, return_dict=True):
        from sparse_amd.context import SparseContext
        self.calls.append((SparseContext.current_phase, SparseContext.runtime_call_id, tuple(input_ids.shape),
                           None if attention_mask is None else int(attention_mask.shape[1]),
                           past_key_values is not None))
        x = self.model.embed[input_ids]
        for layer in self.model.layers:
            x = layer(x)
        logits = torch.nn.functional.linear(x, self.lm_head).float()
        seen = (past_key_values or 0) + int(input_ids.shape[1])
        return SimpleNamespace(logits=logits, past_key_values=seen)


class OracleMoe(nn.Module):
    """CPU stand-in for a sparse MLP: keeps the duck-typed weights and evaluates them with
    the oracle's layer forward."""

    def __init__(self, mlp_block, top_k):
        super().__init__()
        self.block = mlp_block
        self.top_k = top_k

    def forward(self, x):
        from oracle import ref_moe
        from tests.helpers import oracle_layer
        lay = oracle_layer(self.block)
        B, S, H = x.shape
        out, _, _, _ = ref_moe.moe_forward(x.reshape(-1, H).cpu(), lay["gate_w"], lay["experts"], self.top_k,
                                           lay["shared"], lay["shared_gate_w"], family=lay["family"])
        return out.view(B, S, H).to(x.device)
