#!/usr/bin/env python3
"""Benchmark of the MI355X MoE-layer path.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of a decode batch (8 tokens) through the 24 MoE layers of the
Qwen1.5-MoE-A2.7B-shaped stack (hidden 2048, 60 experts x 1408, top-4, shared expert 5632
with sigmoid gate), bf16, random-init weights ~N(0, 0.02) seeded per layer, all experts
resident in HBM.  Inputs are resident in HBM before the timed region; every layer of a
step consumes that step's hidden state ~N(0, 1) (seed 1000 + step).  The step is captured
once in a HIP graph and replayed.  One JSON line is printed with the whole-job tokens/s,
the HBM roofline of the dominant kernel (the fused gate/up projection), measured with HIP
events in an instrumented eager pass over the same steps, and a CPU baseline: the CPU
oracle of the same layer timed on the host cores of this box on a bounded sample.

Extra workloads (reported under "extra"): decode at batch 1 and 32, and the
DeepSeek-V2-Lite-shaped 4096-token prefill (hidden 2048, 64 experts x 1408, top-6,
shared MLP 2816, 26 layers) with its MFMA roofline.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def build_stack(shape, dtype, device, offload="gpu", seed0=0, **kw):
    from sparse_amd.block import DistributedSparseMoeBlock
    from sparse_amd.context import DistEnv, SparseContext
    from sparse_amd.synthetic import make_mlp_block
    SparseContext.reset()
    env = DistEnv(0, 1, 0, device)
    blocks = []
    for layer in range(shape["num_layers"]):
        mlp = make_mlp_block(shape, dtype=dtype, seed=seed0 + layer, device=device, fused=True)
        blocks.append(DistributedSparseMoeBlock(
            layer, mlp, None, env, num_layers=shape["num_layers"], num_experts=shape["num_experts"],
            top_k=shape["top_k"], dtype=dtype, expert_offload=offload, **kw))
        del mlp
    return blocks


def stack_step(blocks, hidden):
    outs = []
    for blk in blocks:
        ret = blk(hidden)
        outs.append(ret[0] if isinstance(ret, tuple) else ret)
    return outs


def make_inputs(shape, batch, seq, n, dtype, device):
    from sparse_amd.synthetic import make_hidden
    return [make_hidden(batch * seq, shape["hidden"], dtype, seed=1000 + i, device=device).view(batch, seq, -1)
            for i in range(n)]


def time_steps(blocks, inputs, warmup, steps, use_graph):
    """Wall time of exactly ``steps`` steps, inputs already on the device."""
    static_in = inputs[0].clone()
    graph = None
    if use_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            stack_step(blocks, static_in)  # allocate workspaces outside capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            keep = stack_step(blocks, static_in)

    def one(i):
        static_in.copy_(inputs[i % len(inputs)])
        if graph is not None:
            graph.replay()
        else:
            stack_step(blocks, static_in)

    for i in range(warmup):
        one(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        one(warmup + i)
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def instrumented_pass(blocks, inputs, steps):
    """Eager pass with HIP events around every kernel launch; also counts the distinct
    routed experts of every layer call.  Returns (per-kernel stats, mean distinct experts)."""
    from sparse_amd import ops
    ops.profile_reset()
    ops.profile_enable(True)
    distinct = []
    try:
        for i in range(steps):
            x = inputs[i % len(inputs)]
            for blk in blocks:
                blk(x)
                ws = blk._workspace(x.shape[0] * x.shape[1])
                distinct.append(int(ws.perm.n_active.item()))
        torch.cuda.synchronize()
        stats = ops.profile_read()
    finally:
        ops.profile_enable(False)
        ops.profile_reset()
    return stats, sum(distinct) / max(1, len(distinct))


def decode_workload(blocks, shape, batch, steps, warmup, dtype, device, use_graph=True):
    inputs = make_inputs(shape, batch, 1, max(8, min(64, warmup + steps)), dtype, device)
    wall = time_steps(blocks, inputs, warmup, steps, use_graph)
    stats, mean_u = instrumented_pass(blocks, inputs, min(steps, 16))
    H, I, Is, K = shape["hidden"], shape["inter"], shape["shared_inter"], shape["top_k"]
    es = 2
    # algorithmic bytes of one fused gate/up launch: the gate and up matrices of every
    # distinct routed expert and of the shared expert, the token rows in, the products out
    gu_bytes = mean_u * 2 * I * H * es + 2 * Is * H * es + batch * H * es + batch * K * I * es + batch * Is * es
    dn_bytes = mean_u * I * H * es + Is * H * es + batch * K * I * es + batch * Is * es + (batch * K + batch) * H * es
    gu_ms, gu_n, gu_name = stats["decode_gateup"]
    dn_ms, dn_n, _ = stats["decode_down"]
    gu_avg_s = gu_ms / max(1, gu_n) / 1e3
    dn_avg_s = dn_ms / max(1, dn_n) / 1e3
    layer_bytes = mean_u * 3 * I * H * es + 3 * Is * H * es + shape["num_experts"] * H * es + H * es + \
        2 * batch * H * es
    ms_per_step = wall / steps * 1e3
    return dict(
        batch=batch, ms_per_step=ms_per_step, tokens_per_s=batch * steps / wall, mean_distinct_experts=mean_u,
        step_hbm_gbps=layer_bytes * len(blocks) / (ms_per_step / 1e3) / 1e9,
        step_hbm_frac=layer_bytes * len(blocks) / (ms_per_step / 1e3) / 1e9 / HBM_PEAK_GBPS,
        gateup=dict(kernel=gu_name, launches=gu_n, avg_us=gu_avg_s * 1e6, bytes_per_launch=gu_bytes,
                    gbps=gu_bytes / gu_avg_s / 1e9 if gu_avg_s else 0.0),
        down=dict(launches=dn_n, avg_us=dn_avg_s * 1e6, bytes_per_launch=dn_bytes,
                  gbps=dn_bytes / dn_avg_s / 1e9 if dn_avg_s else 0.0),
        kernels_us={k: (v[0] / max(1, v[1]) * 1e3) for k, v in stats.items() if v[1]},
        graph=bool(use_graph),
    )


def prefill_workload(shape, tokens, steps, warmup, dtype, device):
    blocks = build_stack(shape, dtype, device)
    inputs = make_inputs(shape, 1, tokens, 2, dtype, device)
    wall = time_steps(blocks, inputs, warmup, steps, use_graph=False)
    stats, _ = instrumented_pass(blocks, inputs, min(steps, 2))
    H, I, Is, K, E = shape["hidden"], shape["inter"], shape["shared_inter"], shape["top_k"], shape["num_experts"]
    flops_layer = 2.0 * tokens * K * 3 * H * I + 2.0 * tokens * 3 * H * Is + 2.0 * tokens * H * E
    gu_ms, gu_n, gu_name = stats["prefill_gateup"]
    # one routed gate/up launch: 2 * (T*K) * H * 2I flops
    gu_flops = 2.0 * tokens * K * H * 2 * I
    # launches alternate shared / routed; split the time by flops share
    routed_share = (tokens * K * I) / (tokens * K * I + tokens * Is)
    gu_routed_s = gu_ms / 1e3 * routed_share / max(1, gu_n // 2)
    ms_per_step = wall / steps * 1e3
    out = dict(
        tokens=tokens, ms_per_step=ms_per_step, tokens_per_s=tokens * steps / wall,
        layer_tflops=flops_layer * len(blocks) / (ms_per_step / 1e3) / 1e12,
        mfma_frac=flops_layer * len(blocks) / (ms_per_step / 1e3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        gateup=dict(kernel=gu_name, launches=gu_n, est_routed_avg_us=gu_routed_s * 1e6,
                    tflops=gu_flops / gu_routed_s / 1e12 if gu_routed_s else 0.0),
        kernels_us={k: (v[0] / max(1, v[1]) * 1e3) for k, v in stats.items() if v[1]},
    )
    del blocks
    torch.cuda.empty_cache()
    return out


def cpu_baseline(shape, batch, dtype, device, budget_s=12.0):
    """The CPU oracle of one layer of the same workload on this box's host cores."""
    from oracle import ref_moe
    from sparse_amd.synthetic import make_hidden, make_mlp_block
    cores = min(16, os.cpu_count() or 1)
    torch.set_num_threads(cores)
    mlp = make_mlp_block(shape, dtype=dtype, seed=0, device=device, fused=True)
    gu, dn = mlp.experts.gate_up_proj.cpu(), mlp.experts.down_proj.cpu()
    I = shape["inter"]
    experts = [(gu[e, :I].contiguous(), gu[e, I:].contiguous(), dn[e].contiguous()) for e in range(gu.shape[0])]
    sh = mlp.shared_expert
    shared = (sh.gate_proj.weight.cpu(), sh.up_proj.weight.cpu(), sh.down_proj.weight.cpu())
    gate_w, sgw = mlp.gate.weight.cpu(), mlp.shared_expert_gate.weight.cpu().reshape(-1)
    del mlp
    n = 0
    t0 = time.perf_counter()
    while True:
        x = make_hidden(batch, shape["hidden"], dtype, seed=1000 + n)
        ref_moe.moe_forward(x, gate_w, experts, shape["top_k"], shared, sgw)
        n += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or n >= 200:
            break
    per_layer = dt / n
    return dict(value=batch / (per_layer * shape["num_layers"]), unit="tokens/s", cores=cores, kind="port",
                sample=f"{n} decode layer-calls (batch {batch}, 1 of {shape['num_layers']} layers, bf16) of the "
                       f"CPU oracle in {dt:.1f} s, scaled linearly to {shape['num_layers']} layers")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip batch 1/32 decode and the prefill workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only-prefill", action="store_true", help="run just the prefill workload (for profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    from sparse_amd import _lib
    from sparse_amd.synthetic import DEEPSEEK, QWEN
    _lib.load()
    device = torch.device("cuda:0")
    dtype = torch.bfloat16

    if args.only_prefill:
        print(json.dumps(prefill_workload(DEEPSEEK, 4096, max(2, args.steps), args.warmup, dtype, device)))
        return
    blocks = build_stack(QWEN, dtype, device)
    main_res = decode_workload(blocks, QWEN, 8, args.steps, args.warmup, dtype, device, not args.no_graph)
    extra = {}
    if not args.no_extra:
        for b in (1, 32):
            extra[f"decode_b{b}"] = decode_workload(blocks, QWEN, b, max(10, args.steps // 2), args.warmup, dtype,
                                                    device, not args.no_graph)
    del blocks
    from sparse_amd.block import _Workspace
    _Workspace._cache.clear()
    torch.cuda.empty_cache()
    if not args.no_extra:
        extra["prefill_4k_deepseek"] = prefill_workload(DEEPSEEK, 4096, max(2, min(10, args.steps // 10)), 1, dtype,
                                                        device)
    cpu = None if args.no_cpu_baseline else cpu_baseline(QWEN, 8, dtype, device)

    gu = main_res["gateup"]
    line = {
        "metric": "MoE-layer tokens/s (decode b=8, prefill 4k) + % of MFMA/HBM/H2D roofline",
        "value": main_res["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "qwen1.5-moe-a2.7b-shaped MoE stack, decode batch 8, 24 layers, all 60 experts resident "
                        "(BASELINE configs[1])",
            "hidden": QWEN["hidden"], "experts": QWEN["num_experts"], "inter": QWEN["inter"],
            "top_k": QWEN["top_k"], "shared_inter": QWEN["shared_inter"], "layers": QWEN["num_layers"],
            "batch": 8, "hip_graph": main_res["graph"],
        },
        "roofline": {
            "bound": "hbm", "achieved": gu["gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": gu["gbps"] / HBM_PEAK_GBPS, "traffic": None, "kernel": gu["kernel"],
            "bytes_per_launch": gu["bytes_per_launch"], "avg_launch_us": gu["avg_us"], "launches": gu["launches"],
            "mean_distinct_experts": main_res["mean_distinct_experts"],
        },
        "cpu_baseline": cpu,
        "step_hbm_frac": main_res["step_hbm_frac"],
        "kernels_us": main_res["kernels_us"],
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
