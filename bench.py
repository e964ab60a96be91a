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

Extra workloads (reported under "extra"): decode at batch 1 and 32, the
DeepSeek-V2-Lite-shaped 4096-token prefill (hidden 2048, 64 experts x 1408, top-6,
shared MLP 2816, 26 layers) with its MFMA roofline, and the two offloaded configurations
(expert-cache decode rr vs rs, readiness-aware chunked prefill rr vs rs-epipe vs sparse)
with hit rates, stall and host-link rates; ``--cached-decode N`` / ``--epipe-prefill`` run
those two alone at full length.
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import tempfile
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_PEAK_CLOCK_MHZ = 2400.0   # the clock the published MFMA rate is quoted at


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


SETTLE_SECONDS = 0.25


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

    # Before the warm-up steps proper the device is brought out of its idle power state: untimed steps for a
    # quarter of a second (the clocks of an idle part take tens of milliseconds to settle, more than a handful
    # of 2 ms warm-up steps lasts; a 20-step measurement started cold reads 1-3 % slow and varies run to run).
    settle_until = time.perf_counter() + SETTLE_SECONDS
    n_settle = 0
    while time.perf_counter() < settle_until and n_settle < 2000:
        one(n_settle)
        n_settle += 1
        if n_settle % 8 == 0:
            torch.cuda.synchronize()
    for i in range(warmup):
        one(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        one(warmup + i)
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def instrumented_pass(blocks, inputs, steps, per_step=False):
    """Eager pass with HIP events around every kernel launch; also counts the distinct
    routed experts of every layer call.  Returns (per-kernel stats, mean distinct experts), and with
    ``per_step`` also the mean over the layers for each step."""
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
    mean = sum(distinct) / max(1, len(distinct))
    if not per_step:
        return stats, mean
    n = len(blocks)
    return stats, mean, [sum(distinct[i * n:(i + 1) * n]) / n for i in range(steps)]


def decode_workload(blocks, shape, batch, steps, warmup, dtype, device, use_graph=True):
    inputs = make_inputs(shape, batch, 1, max(8, min(64, warmup + steps)), dtype, device)
    wall = time_steps(blocks, inputs, warmup, steps, use_graph)
    # per-kernel times and the number of distinct routed experts, on the very inputs the timed steps ran
    # (the algorithmic bytes of a step depend on how many experts its tokens hit): timed step i read input
    # (warmup + i) mod len(inputs), so every input is instrumented once and weighted by how often it was timed
    used = [(warmup + i) % len(inputs) for i in range(steps)]
    order = sorted(set(used))
    stats, _mean, per_input = instrumented_pass(blocks, [inputs[j] for j in order], len(order), per_step=True)
    weight = {j: used.count(j) for j in order}
    mean_u = sum(per_input[n] * weight[j] for n, j in enumerate(order)) / len(used)
    H, I, Is, K = shape["hidden"], shape["inter"], shape["shared_inter"], shape["top_k"]
    es = 2
    from sparse_amd import ops
    # calls of up to 16 tokens compute the shared expert's gate and up projections inside the
    # routing launch; larger ones inside the gate/up launch
    shared_in_route = bool(blocks[0].route_with_shared and blocks[0].gate_packed is not None
                           and batch <= ops.ROUTE_PACKED_MAX_TOKENS and Is % 32 == 0)
    shared_up_bytes = 2 * Is * H * es + batch * Is * es
    # algorithmic bytes of one gate/up launch: the gate and up matrices of every distinct routed
    # expert (and of the shared expert when they run here), the token rows in, the products out
    gu_bytes = mean_u * 2 * I * H * es + batch * H * es + batch * K * I * es + (0 if shared_in_route else shared_up_bytes)
    rt_bytes = 64 * H * es + batch * H * es + (shared_up_bytes if shared_in_route else 0)
    dn_bytes = mean_u * I * H * es + Is * H * es + batch * K * I * es + batch * Is * es + (batch * K + batch) * H * es
    gu_ms, gu_n, gu_name = stats["decode_gateup"]
    dn_ms, dn_n, _ = stats["decode_down"]
    rt_ms, rt_n, _ = stats.get("route_decode", (0.0, 0, ""))
    gu_avg_s = gu_ms / max(1, gu_n) / 1e3
    dn_avg_s = dn_ms / max(1, dn_n) / 1e3
    rt_avg_s = rt_ms / max(1, rt_n) / 1e3
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
        route=dict(launches=rt_n, avg_us=rt_avg_s * 1e6, bytes_per_launch=rt_bytes,
                   gbps=rt_bytes / rt_avg_s / 1e9 if rt_avg_s else 0.0, shared_gate_up_inside=shared_in_route),
        kernels_us={k: (v[0] / max(1, v[1]) * 1e3) for k, v in stats.items() if v[1]},
        graph=bool(use_graph),
    )


class GpuTelemetry:
    """Socket power and shader clock of the GPU in use, sampled from host threads while a workload runs.
    Power: the amdgpu driver's hwmon file (power1_average or power1_input, with power1_cap) every
    ``period`` seconds.  Clock: hwmon freq1_input where the driver has it, else one `amd-smi metric` child
    process per sample (a few a second; it also gives the power where the sysfs file is missing), averaged
    over the XCDs.  What the box does not expose to this user is reported as missing, without figures."""

    enabled = True      # --no-telemetry: no sampling threads and no child processes (runs under a profiler)

    def __init__(self, device_index=0, period=0.01):
        import glob
        self.period, self.power, self.clock, self.note = period, [], [], None
        self._stop, self._threads = None, []
        self.hwmon = None
        if not GpuTelemetry.enabled:
            self.note = "switched off (--no-telemetry)"
            self.power_file = self.freq_file = self.smi = self.cap_w = None
            return
        want = None
        try:
            p = torch.cuda.get_device_properties(device_index)
            want = f"{p.pci_domain_id:04x}:{p.pci_bus_id:02x}:{p.pci_device_id:02x}"
        except Exception:  # noqa: BLE001
            pass
        cards = []
        for card in sorted(glob.glob("/sys/class/drm/card[0-9]*")):
            if "-" in os.path.basename(card):
                continue
            hw = sorted(glob.glob(os.path.join(card, "device", "hwmon", "hwmon*")))
            if hw:
                cards.append((hw[0], os.path.realpath(os.path.join(card, "device"))))
        match = [c for c in cards if want and want in c[1]]
        pick = match[0] if match else (cards[0] if len(cards) == 1 else None)
        if pick is not None:
            self.hwmon = pick[0]
        self.power_file = next((f for f in ("power1_average", "power1_input")
                                if self.hwmon and (self._read(f) or "").isdigit()), None)
        self.freq_file = "freq1_input" if self.hwmon and (self._read("freq1_input") or "").isdigit() else None
        cap = self._read("power1_cap") if self.hwmon else None
        self.cap_w = int(cap) / 1e6 if cap and cap.isdigit() else None
        self.smi = None
        if self.power_file is None or self.freq_file is None:
            self.smi = self._amd_smi()
        self.power_source = (f"sysfs {self.power_file}" if self.power_file
                             else "amd-smi socket_power" if self.smi and self.smi[0] is not None else None)
        self.clock_source = ("sysfs freq1_input" if self.freq_file
                             else "amd-smi gfx clk, mean over XCDs" if self.smi and self.smi[1] is not None else None)
        if not (self.power_source or self.clock_source):
            self.note = (f"no readable power / clock source: {len(cards)} drm cards with hwmon, wanted PCI {want}, "
                         "amd-smi metric gave nothing")

    def _read(self, name):
        try:
            with open(os.path.join(self.hwmon, name)) as f:
                return f.read().strip()
        except OSError:
            return None

    @staticmethod
    def _amd_smi():
        import subprocess
        try:
            raw = subprocess.run(["amd-smi", "metric", "--power", "--clock", "--json"], capture_output=True,
                                 text=True, timeout=10).stdout
            data = json.loads(raw)
        except Exception:  # noqa: BLE001
            return None
        if isinstance(data, dict):
            data = data.get("gpu_data")
        entry = data[0] if isinstance(data, list) and data else None
        if not isinstance(entry, dict):
            return None

        def number(node):
            node = node.get("value") if isinstance(node, dict) else node
            return float(node) if isinstance(node, (int, float)) else None

        power = number((entry.get("power") or {}).get("socket_power"))
        gfx = [number(v.get("clk")) for k, v in (entry.get("clock") or {}).items()
               if k.startswith("gfx") and isinstance(v, dict)]
        gfx = [v for v in gfx if v is not None]
        if power is None and not gfx:
            return None
        return (power, sum(gfx) / len(gfx) if gfx else None)

    def __enter__(self):
        import threading
        if self.note:
            return self
        self._stop = threading.Event()

        def sysfs_loop():
            while not self._stop.is_set():
                if self.power_file:
                    v = self._read(self.power_file)
                    if v and v.isdigit():
                        self.power.append(int(v) / 1e6)
                if self.freq_file:
                    v = self._read(self.freq_file)
                    if v and v.isdigit():
                        self.clock.append(int(v) / 1e6)
                self._stop.wait(self.period)

        def smi_loop():
            while not self._stop.is_set():
                got = self._amd_smi()
                if got is not None:
                    if self.power_file is None and got[0] is not None:
                        self.power.append(got[0])
                    if self.freq_file is None and got[1] is not None:
                        self.clock.append(got[1])
                self._stop.wait(0.05)

        loops = ([sysfs_loop] if (self.power_file or self.freq_file) else []) + ([smi_loop] if self.smi else [])
        for fn in loops:
            t = threading.Thread(target=fn, daemon=True)
            t.start()
            self._threads.append(t)
        return self

    def __exit__(self, *exc):
        if self._stop is not None:
            self._stop.set()
        for t in self._threads:
            t.join(timeout=15)
        return False

    def summary(self):
        if self.note:
            return {"available": False, "note": self.note}
        stat = lambda v: ({"mean": sum(v) / len(v), "min": min(v), "max": max(v), "samples": len(v)} if v else None)
        return {"available": True, "power_source": self.power_source, "clock_source": self.clock_source,
                "power_w": stat(self.power), "power_cap_w": self.cap_w, "sclk_mhz": stat(self.clock)}


def prefill_workload(shape, tokens, steps, warmup, dtype, device):
    blocks = build_stack(shape, dtype, device)
    inputs = make_inputs(shape, 1, tokens, 2, dtype, device)
    wall = time_steps(blocks, inputs, warmup, steps, use_graph=False)
    # per-kernel durations, launches in one stream (the default form: routed and shared tiles in one
    # launch per projection)
    stats, _ = instrumented_pass(blocks, inputs, min(steps, 2))
    # the clock the compute units really run at under this load (each workgroup of the FFN kernel
    # reads the shader clock and the constant 100 MHz clock at its first and last instruction)
    from sparse_amd import ops
    clk = torch.zeros(2, dtype=torch.int64, device=device)
    ops.prefill_clock_probe(clk)
    try:
        time_steps(blocks, inputs, 0, 2, use_graph=False)
    finally:
        ops.prefill_clock_probe(None)
    clock_mhz = ops.prefill_shader_clock_mhz(clk)
    # the other form, same bits: routed and shared expert in separate launches, the shared expert's on a
    # second stream beside routing and routed tiles
    merged = bool(blocks[0].merged_prefill)
    for blk in blocks:
        blk.merged_prefill = not merged
    wall_other = time_steps(blocks, inputs, 1, steps, use_graph=False)
    for blk in blocks:
        blk.merged_prefill = merged
    # socket power and shader clock as the driver reports them, sampled from a host thread during a pass
    # of its own (at least about a second of steps), so that the sampling cannot touch the timed figure
    telemetry = GpuTelemetry().summary()
    if GpuTelemetry.enabled:
        tele_steps = max(steps, int(3.0 / max(wall / steps, 1e-4)))
        with GpuTelemetry() as tele:
            wall_tele = time_steps(blocks, inputs, 0, tele_steps, use_graph=False)
        telemetry = tele.summary()
        telemetry["ms_per_step_while_sampling"] = wall_tele / tele_steps * 1e3
    # what the matrix cores sustain on this box with nothing but the kernel's wavefront tile going on:
    # operands in registers, and with the activation fragments read from LDS every k step
    probe = {}
    for name, from_lds in (("registers", False), ("lds_fragments", True)):
        with GpuTelemetry() as tele:
            # about two seconds of back-to-back probe launches while the power and clock are sampled
            until = time.perf_counter() + (2.0 if GpuTelemetry.enabled else 0.0)
            while True:
                tf, mhz = ops.mfma_probe(from_lds, device=device)
                if time.perf_counter() >= until:
                    break
        probe[name] = {"tflops": tf, "clock_mhz": mhz, "frac_of_peak": tf / MFMA_BF16_PEAK_TFLOPS,
                       "telemetry": tele.summary()}
    H, I, Is, K, E = shape["hidden"], shape["inter"], shape["shared_inter"], shape["top_k"], shape["num_experts"]
    flops_layer = 2.0 * tokens * K * 3 * H * I + 2.0 * tokens * 3 * H * Is + 2.0 * tokens * H * E
    gu_ms, gu_n, gu_name = stats["prefill_gateup"]
    dn_ms, dn_n, _ = stats["prefill_down"]
    # flops of the gate/up and of the down launches of one layer call (routed + shared)
    gu_flops = 2.0 * tokens * H * 2 * (K * I + Is)
    dn_flops = gu_flops / 2
    per_call = 1 if merged else 2          # launches of each projection per layer call
    gu_s = gu_ms / 1e3 / max(1, gu_n) * per_call
    dn_s = dn_ms / 1e3 / max(1, dn_n) * per_call
    ms_per_step = wall / steps * 1e3
    out = dict(
        tokens=tokens, steps=steps, ms_per_step=ms_per_step, tokens_per_s=tokens * steps / wall,
        form="merged launches" if merged else "separate launches, shared expert on a second stream",
        ms_per_step_other_form=wall_other / steps * 1e3,
        layer_tflops=flops_layer * len(blocks) / (ms_per_step / 1e3) / 1e12,
        mfma_frac=flops_layer * len(blocks) / (ms_per_step / 1e3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        # busy compute units' average shader clock during the FFN launches, and the fraction of the
        # MFMA rate that clock allows (the published peak assumes MFMA_PEAK_CLOCK_MHZ)
        ffn_shader_clock_mhz=clock_mhz,
        telemetry=telemetry,
        mfma_frac_at_clock=(flops_layer * len(blocks) / (ms_per_step / 1e3) / 1e12
                            / (MFMA_BF16_PEAK_TFLOPS * clock_mhz / MFMA_PEAK_CLOCK_MHZ)) if clock_mhz else None,
        # a loop of the same MFMAs on the same wavefront tile and nothing else (sparse_hip_mfma_probe)
        mfma_probe=probe,
        gateup=dict(kernel=gu_name, launches=gu_n, us_per_layer_call=gu_s * 1e6,
                    tflops=gu_flops / gu_s / 1e12 if gu_s else 0.0,
                    mfma_frac=gu_flops / gu_s / 1e12 / MFMA_BF16_PEAK_TFLOPS if gu_s else 0.0),
        down=dict(launches=dn_n, us_per_layer_call=dn_s * 1e6, tflops=dn_flops / dn_s / 1e12 if dn_s else 0.0,
                  mfma_frac=dn_flops / dn_s / 1e12 / MFMA_BF16_PEAK_TFLOPS if dn_s else 0.0),
        kernels_us={k: (v[0] / max(1, v[1]) * 1e3) for k, v in stats.items() if v[1]},
    )
    del blocks
    torch.cuda.empty_cache()
    return out


def build_offload_stack(shape, dtype, device, method, capacity, top_m, rs_kind="random", offload="cpu",
                        **overrides):
    """A stack whose routing is skewed (Zipf popularity + co-activating clusters of 4) and whose
    routed experts live in pinned host memory behind an HBM cache of ``capacity`` slots."""
    from sparse_amd.block import DistributedSparseMoeBlock
    from sparse_amd.context import DistEnv, Metrics, SparseContext
    from sparse_amd.methods import method_settings, residency_config
    from sparse_amd.rs import informed_bank, random_init_bank
    from sparse_amd.synthetic import add_routing_structure, make_mlp_block
    SparseContext.reset()
    metrics = Metrics()
    metrics.time_copies = True
    kw = method_settings(method)["kwargs"]
    env = DistEnv(0, 1, 0, device)
    blocks, gates, structure = [], [], None
    for layer in range(shape["num_layers"]):
        mlp = make_mlp_block(shape, dtype=dtype, seed=layer, device=device, fused=True)
        structure = add_routing_structure(mlp, shape["num_experts"], seed=layer)
        gates.append(mlp.gate.weight.detach().clone() if layer > 0 else None)
        cfg = residency_config(method, capacity, top_m, **overrides) if offload == "cpu" else None
        blocks.append(DistributedSparseMoeBlock(
            layer, mlp, None, env, num_layers=shape["num_layers"], num_experts=shape["num_experts"],
            top_k=shape["top_k"], dtype=dtype, expert_offload=offload, expert_cache=capacity,
            planner_mode=kw["planner_mode"] if offload == "cpu" else "none", prefetch_top_m=top_m,
            placement_mode=kw["placement_mode"], metrics=metrics, residency_config=cfg))
        del mlp
    if offload == "cpu" and kw["planner_mode"] == "rs_prefetch":
        if rs_kind == "informed":
            bank = informed_bank(gates, hidden_dim=512, device=device)
        else:
            bank = random_init_bank(shape["num_layers"], shape["hidden"], shape["num_experts"], hidden_dim=512,
                                    seed=0, device=device)
        SparseContext.set_rs_bank(bank)
    return blocks, metrics, structure


def release_stack():
    """Drop a stack the caller has let go of: the layer registry and the block <-> backend
    cycle keep it alive until a collection, and with it its HBM slab and pinned arena."""
    from sparse_amd.block import _Workspace
    from sparse_amd.context import SparseContext
    SparseContext.reset()
    _Workspace._cache.clear()
    gc.collect()
    torch.cuda.empty_cache()


def run_phase_steps(blocks, inputs, phase, first_call=0):
    """Drive the stack as the reference's decode loop does: phase and call id before every
    pass over the layers.  Returns the wall time with the device drained on both sides."""
    from sparse_amd.context import SparseContext
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i, x in enumerate(inputs):
        SparseContext.current_phase = phase
        SparseContext.begin_runtime_call(first_call + i)
        for blk in blocks:
            blk(x)
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def offload_report(metrics, blocks, wall, n_steps, tokens_per_step, resident_ms):
    lanes = dict(metrics.harvest_timings())
    counts = dict(metrics.timings_n)
    eb = blocks[0].arena.expert_bytes
    demand_bytes, pf_bytes = metrics.demand_h2d_bytes, metrics.prefetch_h2d_bytes
    total_bytes = demand_bytes + pf_bytes
    n_copies = total_bytes // eb
    timed_n = sum(counts.values())
    timed_ms = sum(lanes.values())
    # only the first 100 000 copies carry an event pair; scale lane times to all copies
    scale = n_copies / timed_n if timed_n else 0.0
    accesses = metrics.cache_hit_count + metrics.prefetch_hit_count + metrics.cache_miss_count
    ms_step = wall / n_steps * 1e3
    return dict(
        ms_per_step=ms_step, tokens_per_s=tokens_per_step * n_steps / wall,
        ratio_to_resident=ms_step / resident_ms if resident_ms else None,
        hit_rate=metrics.hit_rate(), accesses=accesses, misses=metrics.cache_miss_count,
        prefetch_hits=metrics.prefetch_hit_count, prefetch_admitted=metrics.prefetch_admitted_count,
        prefetch_wasted=metrics.prefetch_wasted_count,
        h2d_gb=total_bytes / 1e9, demand_h2d_gb=demand_bytes / 1e9, prefetch_h2d_gb=pf_bytes / 1e9,
        copies=int(n_copies), copies_timed=int(timed_n),
        # copies on the compute lane are the exposed stall (the reference's demand-H2D window)
        exposed_demand_copy_ms_per_step=lanes.get("compute_h2d_ms", 0.0) * scale / n_steps,
        side_copy_ms_per_step=(lanes.get("prefetch_h2d_ms", 0.0) + lanes.get("epipe_h2d_ms", 0.0)) * scale / n_steps,
        stall_ms_per_step=max(0.0, ms_step - resident_ms) if resident_ms else None,
        # one copy's bytes over its own event-pair time (copies on two lanes share the link)
        h2d_gbps_per_copy=timed_n * eb / (timed_ms / 1e3) / 1e9 if timed_ms else 0.0,
        h2d_gbps_over_wall=total_bytes / wall / 1e9,
        expert_bytes=eb,
    )


class PolicyCallLog:
    """Records the calls a stack's blocks make into their residency policy (prefetch budget, plan, execute),
    in order, with the phase / call id / stage each was made under, so that the same run can be replayed
    through the CPU oracle of the policy afterwards.  A check beside the measurement, not part of it: the
    wrappers append to a list and call through."""

    NAMES = ("prefetch_budget", "schedule_prefetch", "execute")

    def __init__(self, blocks):
        self.calls = []
        for blk in blocks:
            res = blk.residency
            for name in self.NAMES:
                setattr(res, name, self._wrap(res, name, getattr(res, name)))

    def _wrap(self, res, name, inner):
        def call(*args):
            self.calls.append((res.layer_idx, name, tuple(list(a) if isinstance(a, list) else a for a in args),
                               (res.phase, res.call_id, getattr(res, "stage", "decode"))))
            return inner(*args)
        return call

    def oracle_misses(self, cfg, num_layers, num_experts, top_k):
        """Demand misses the oracle's state machine counts when fed the recorded calls (every copy taken
        as complete when asked: which copies are late changes waits, not residency, without EPIPE)."""
        from oracle.ref_layer import RefConfig, RefLayer
        ref_cfg = RefConfig(**{n: getattr(cfg, n) for n in vars(RefConfig()) if hasattr(cfg, n)})
        layers = [RefLayer(l, num_experts, top_k, ref_cfg) for l in range(num_layers)]
        for layer, name, args, (phase, call_id, stage) in self.calls:
            lay = layers[layer]
            lay.phase, lay.call_id, lay.stage = phase, call_id, stage
            getattr(lay, name)(*args)
        return sum(1 for lay in layers for t in lay.trace if t[0] == "miss")


def cached_decode_workload(dtype, device, steps, batch=8, capacity=15, top_m=8, short_steps=None, variants=None):
    """BASELINE configs[3]: Qwen shape, HBM cache of 25 % of each layer's experts, the rest in
    pinned host memory, skewed co-activating routing, rr vs rs (random-init predictor, as the
    config says, and a predictor that reproduces the next layer's router)."""
    from sparse_amd.block import _Workspace
    from sparse_amd.synthetic import QWEN, make_structured_hidden
    shape = QWEN
    n_clusters = shape["num_experts"] // 4
    # The configuration states 512 decode steps and names two methods, rr and rs with a
    # random-init predictor: those run `steps` steps.  The other variants (predictors that
    # reproduce the next router, EPIPE, the cost-aware policy, the staging engine) are this
    # build's additions and run `short_steps` steps; every entry says how many it ran.
    short_steps = steps if short_steps is None else min(steps, short_steps)
    out = {"steps": steps, "config_steps": 512, "batch": batch, "capacity": capacity, "experts": shape["num_experts"],
           "top_m": top_m}

    def inputs_for(structure):
        return [make_structured_hidden(batch, shape["hidden"], n_clusters, structure["cluster_prob"], dtype,
                                       seed=5000 + i, device=device).view(batch, 1, -1) for i in range(steps)]

    blocks, _m, structure = build_offload_stack(shape, dtype, device, "rr", capacity, top_m, offload="gpu")
    inputs = inputs_for(structure)
    run_phase_steps(blocks, inputs[:8], "decode")
    wall = run_phase_steps(blocks, inputs[:short_steps], "decode")
    resident_ms = wall / short_steps * 1e3
    out["resident_eager_ms_per_step"] = resident_ms
    # cost table for the cost-aware local policy, measured on this GPU with the resident layer 0
    from sparse_amd.local_policy import CostProfile, install_lightweight_policies, measure_costs, write_profile
    costs = measure_costs(blocks[0])
    out["measured_costs"] = {k: round(v, 6) for k, v in costs.items()}
    profile_path = os.path.join(tempfile.gettempdir(), f"sparse_costs_{os.getpid()}.json")
    write_profile(profile_path, costs, calibrated=True, provenance="bench.py measure_costs on the running GPU")
    del blocks
    release_stack()
    all_variants = (("rr", "rr", "random"), ("rs_random_init", "rs", "random"),
                    ("rs_informed", "rs", "informed"), ("rs-epipe_informed", "rs-epipe", "informed"),
                    ("rs-epipe_light_informed", "rs-epipe", "informed"),
                    ("rs-epipe_staged_informed", "rs-epipe", "informed"))
    for name, method, rs_kind in all_variants:
        if variants is not None and name not in variants:
            continue
        n_steps = steps if name in ("rr", "rs_random_init") else short_steps
        print(f"[bench] cached decode: {name}, {n_steps} steps", file=sys.stderr, flush=True)
        staged = "staged" in name
        kw = dict(staging_pool_slots=4) if staged else {}
        blocks, metrics, _ = build_offload_stack(shape, dtype, device, method, capacity, top_m, rs_kind=rs_kind,
                                                 **kw)
        policies = install_lightweight_policies(CostProfile(profile_path, 1)) if "light" in name else []
        engine = None
        if staged:
            # the bounded staging engine instead of the in-line planner: graph-captured predictor,
            # worker-thread publication into a per-layer pool of 4 slots
            from sparse_amd.context import SparseContext
            from sparse_amd.staging import BoundedRS
            engine = BoundedRS(slots=4)
            engine.prepare({b.layer_idx: b for b in blocks}, SparseContext.rs_bank, batch=batch, dtype=dtype)
            engine.install()
            engine.begin(name)
        # the two methods the configuration names also record their policy calls, replayed through the CPU
        # oracle after the timed region: its miss count for the same routing goes beside the product's
        log = PolicyCallLog(blocks) if name in ("rr", "rs_random_init") else None
        wall = run_phase_steps(blocks, inputs[:n_steps], "decode")   # cold cache, all steps timed
        out[name] = offload_report(metrics, blocks, wall, n_steps, batch, resident_ms)
        out[name]["steps"] = n_steps
        out[name]["shortened"] = n_steps < 512
        if log is not None:
            out[name]["oracle_misses"] = log.oracle_misses(blocks[0].residency.cfg, len(blocks),
                                                           shape["num_experts"], shape["top_k"])
            print(f"[bench] cached decode: {name}: misses {out[name]['misses']}, oracle on the same routing "
                  f"{out[name]['oracle_misses']}", file=sys.stderr, flush=True)
            del log
        if policies:
            out[name]["policy"] = {k: sum(p.stats[k] for p in policies)
                                   for k in ("prefetch_calls", "candidate_scores", "feedback_updates",
                                             "residual_calls")}
        if engine is not None:
            st = engine.finish()
            engine.restore()
            engine.shutdown()
            out[name]["staging"] = {k: st[k] for k in ("predictions", "issued", "used", "wasted", "retained",
                                                        "skipped_slots", "closed_before_publish")}
            del engine
        del blocks, metrics
        release_stack()
    return out


def epipe_prefill_workload(dtype, device, tokens=4096, chunk=2048, capacity=19, top_m=8):
    """BASELINE configs[4]: DeepSeek shape, 4096-token prefill as two 2048-token prefill-phase
    calls, HBM cache of 30 % of the routed experts, rr vs rs-epipe vs sparse with the EPIPE
    prefill stage on."""
    from sparse_amd.block import _Workspace
    from sparse_amd.synthetic import DEEPSEEK, make_structured_hidden
    shape = DEEPSEEK
    n_clusters = shape["num_experts"] // 4
    n_chunks = tokens // chunk
    out = {"tokens": tokens, "chunk": chunk, "capacity": capacity, "experts": shape["num_experts"]}

    def inputs_for(structure, seed0):
        return [make_structured_hidden(chunk, shape["hidden"], n_clusters, structure["cluster_prob"], dtype,
                                       seed=seed0 + i, device=device).view(1, chunk, -1) for i in range(n_chunks)]

    blocks, _m, structure = build_offload_stack(shape, dtype, device, "rr", capacity, top_m, offload="gpu")
    warm, inputs = inputs_for(structure, 7000), inputs_for(structure, 7100)
    run_phase_steps(blocks, warm, "prefill")
    wall = run_phase_steps(blocks, inputs, "prefill")
    resident_ms = wall * 1e3
    out["resident_ms_per_request"] = resident_ms
    del blocks
    release_stack()
    # rr / rs-epipe / sparse as the configuration names them (the reference stages one missing
    # expert per call beside the resident work), then the same with every missing expert
    # streamed on the EPIPE lane (this build's stream-all ordering)
    for name, method, extra_kw in (("rr", "rr", {}), ("rs-epipe", "rs-epipe", {}), ("sparse", "sparse", {}),
                                   ("rs-epipe_stream_all", "rs-epipe", dict(epipe_stream_all=True))):
        print(f"[bench] chunked prefill: {name}", file=sys.stderr, flush=True)
        # rr is the plain baseline: demand copies on the compute lane, no EPIPE stage in prefill
        blocks, metrics, _ = build_offload_stack(shape, dtype, device, method, capacity, top_m, rs_kind="informed",
                                                 epipe_prefill_enable=method != "rr", **extra_kw)
        wall = run_phase_steps(blocks, inputs, "prefill")   # cold cache
        rep = offload_report(metrics, blocks, wall, 1, tokens, resident_ms)
        rep["ms_per_request"] = rep.pop("ms_per_step")
        out[name] = rep
        del blocks, metrics
        release_stack()
    return out


def measured_traffic_ratio(kernel="decode_gateup"):
    """HBM bytes per launch over algorithmic bytes per launch for the dominant kernel, as
    measured with hardware counters (two profiler runs, scaled by a plain copy) and recorded
    in the committed summary; None when there is no summary."""
    path = os.path.join(ROOT, "profiles", "decode_b8_qwen_hbm_traffic.txt")
    try:
        for line in open(path):
            parts = line.split()
            if len(parts) == 3 and parts[0] == "traffic_over_algorithmic" and parts[1] == kernel:
                return float(parts[2])
    except OSError:
        pass
    return None


def usable_cores():
    """Host cores this process may use: the scheduler affinity, cut down by the cgroup's CPU
    quota and by the thread share the machine's operator exports (OMP_NUM_THREADS) where
    those are set.  Returns (count, how it was derived)."""
    total = os.cpu_count() or 1
    try:
        n = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        n = total
    note = [f"os.cpu_count()={total}", f"affinity={n}"]
    try:
        quota, period = open("/sys/fs/cgroup/cpu.max").read().split()[:2]
        if quota != "max":
            q = max(1, int(int(quota) / int(period)))
            note.append(f"cgroup quota={q}")
            n = min(n, q)
    except (OSError, ValueError):
        pass
    env = os.environ.get("OMP_NUM_THREADS", "").strip()
    if env.isdigit() and int(env) > 0:
        note.append(f"OMP_NUM_THREADS={env}")
        n = min(n, int(env))
    return max(1, n), ", ".join(note)


def _cpu_layer(shape, dtype, device):
    """CPU weights of layer 0 of a stack and a function that runs the CPU oracle on a token batch."""
    from oracle import ref_moe
    from sparse_amd.synthetic import make_mlp_block
    mlp = make_mlp_block(shape, dtype=dtype, seed=0, device=device, fused=True)
    gu, dn = mlp.experts.gate_up_proj.cpu(), mlp.experts.down_proj.cpu()
    I = shape["inter"]
    experts = [(gu[e, :I].contiguous(), gu[e, I:].contiguous(), dn[e].contiguous()) for e in range(gu.shape[0])]
    sh = getattr(mlp, "shared_expert", None) or getattr(mlp, "shared_experts", None)
    shared = (sh.gate_proj.weight.cpu(), sh.up_proj.weight.cpu(), sh.down_proj.weight.cpu())
    sg = getattr(mlp, "shared_expert_gate", None)
    sgw = sg.weight.cpu().reshape(-1) if sg is not None else None
    gate_w = mlp.gate.weight.cpu()
    family = shape["family"]
    del mlp

    def run(x):
        return ref_moe.moe_forward(x, gate_w, experts, shape["top_k"], shared, sgw, family=family)

    return run


def _time_cpu(run, tokens, hidden, dtype, threads, budget_s, max_calls=5000):
    from sparse_amd.synthetic import make_hidden
    torch.set_num_threads(threads)
    n = 0
    t0 = time.perf_counter()
    while True:
        run(make_hidden(tokens, hidden, dtype, seed=1000 + n))
        n += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or n >= max_calls:
            return n, dt


def cpu_baseline(shape, batch, dtype, device, budget_s=12.0):
    """The CPU oracle of one layer of the same workload on this box's host cores."""
    cores, core_note = usable_cores()
    run = _cpu_layer(shape, dtype, device)
    n, dt = _time_cpu(run, batch, shape["hidden"], dtype, cores, budget_s * 0.6)
    n1, dt1 = _time_cpu(run, batch, shape["hidden"], dtype, 1, budget_s * 0.4)  # the reference serves with OMP_NUM_THREADS=1 (run_case.sh:229)
    torch.set_num_threads(cores)
    layers = shape["num_layers"]
    return dict(value=batch / (dt / n * layers), unit="tokens/s", cores=cores, kind="port",
                value_1_thread=batch / (dt1 / n1 * layers), host_cpu_count=os.cpu_count(), cores_note=core_note,
                sample=f"{n} decode layer-calls (batch {batch}, 1 of {layers} layers, bf16) of the CPU oracle in "
                       f"{dt:.1f} s on {cores} threads, and {n1} in {dt1:.1f} s on 1 thread, each scaled linearly "
                       f"to {layers} layers")


def cpu_baseline_prefill(shape, tokens, sample_tokens, dtype, device, budget_s=8.0):
    """The CPU oracle beside the prefill figure: one layer of the DeepSeek-shaped stack on a
    ``sample_tokens``-token batch (bf16), scaled linearly to ``tokens`` tokens through all layers."""
    cores, _ = usable_cores()
    run = _cpu_layer(shape, dtype, device)
    n, dt = _time_cpu(run, sample_tokens, shape["hidden"], dtype, cores, budget_s * 0.5, max_calls=50)
    n1, dt1 = _time_cpu(run, sample_tokens, shape["hidden"], dtype, 1, budget_s * 0.5, max_calls=20)
    torch.set_num_threads(cores)
    layers = shape["num_layers"]
    return dict(value=sample_tokens / (dt / n * layers), unit="tokens/s", cores=cores, kind="port",
                value_1_thread=sample_tokens / (dt1 / n1 * layers),
                sample=f"{n} layer-calls of {sample_tokens} tokens (1 of {layers} layers, bf16, DeepSeek-V2-Lite shape) "
                       f"of the CPU oracle in {dt:.1f} s on {cores} threads, and {n1} in {dt1:.1f} s on 1 thread; "
                       f"tokens/s through {layers} layers, i.e. comparable with prefill_4k.tokens_per_s")


def cpu_baseline_config1(shape, device, budget_s=6.0):
    """BASELINE configs[0] exactly: one Qwen-shaped layer in fp32, 128 tokens, on the host cores."""
    cores, _ = usable_cores()
    run = _cpu_layer(shape, torch.float32, device)
    n, dt = _time_cpu(run, 128, shape["hidden"], torch.float32, cores, budget_s * 0.5, max_calls=200)
    n1, dt1 = _time_cpu(run, 128, shape["hidden"], torch.float32, 1, budget_s * 0.5, max_calls=50)
    torch.set_num_threads(cores)
    return dict(value=128 / (dt / n), unit="tokens/s (one layer)", cores=cores, kind="port",
                value_1_thread=128 / (dt1 / n1), ms_per_layer_call=dt / n * 1e3, ms_per_layer_call_1_thread=dt1 / n1 * 1e3,
                sample=f"{n} calls of one fp32 Qwen-shaped layer on 128 tokens in {dt:.1f} s on {cores} threads, "
                       f"{n1} in {dt1:.1f} s on 1 thread (BASELINE configs[0])")


def routing_launch_probe(dtype, device, batch=8, replays=50):
    """The decode routing launch taken apart: the router's workgroup alone (every layer's own gate matrix, and
    one gate matrix for all layers, i.e. cached), the shared expert's gate/up projections alone, and both in
    one launch as the block runs them; each as a HIP graph over the stack's layers, microseconds per layer."""
    from sparse_amd import ops
    from sparse_amd.synthetic import QWEN
    blocks = build_stack(QWEN, dtype, device)
    x = make_inputs(QWEN, batch, 1, 1, dtype, device)[0].view(batch, -1).contiguous()
    spaces = [b._workspace(batch) for b in blocks]
    logits = torch.empty((batch, QWEN["num_experts"]), device=device, dtype=blocks[0].logits_dtype)

    def router(blk, ws, shared_up=None):
        ops.route_decode_packed(x, blk.gate_packed, blk.num_experts, blk.shared_gate_weight is not None, blk.top_k,
                                blk.norm_topk_prob, logits, ws.shared_gate, ws.topv, ws.topi, ws.perm,
                                shared_up=shared_up)

    forms = {
        "router_alone_us": lambda: [router(b, ws) for b, ws in zip(blocks, spaces)],
        "router_alone_one_gate_matrix_us": lambda: [router(blocks[0], spaces[0]) for _ in blocks],
        "shared_gate_up_alone_us": lambda: [ops.shared_gate_up(x, b.shared_weights[0], b.shared_weights[1],
                                                               ws.shared_inter) for b, ws in zip(blocks, spaces)],
        "router_and_shared_gate_up_us": lambda: [router(b, ws, (b.shared_weights[0], b.shared_weights[1],
                                                                ws.shared_inter)) for b, ws in zip(blocks, spaces)],
    }
    out = {"batch": batch, "layers": len(blocks), "replays": replays}
    for name, fn in forms.items():
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        out[name] = (time.perf_counter() - t0) / replays / len(blocks) * 1e6
        del graph
    del blocks
    release_stack()
    return out


def library_gemms(device, dtype=torch.bfloat16, runs=20):
    """Plain GEMMs of the vendor library through torch at the prefill workload's shapes (no gather, no
    SwiGLU epilogue, no routing weights): a reference point for the grouped kernels' launch times, not
    part of any step."""
    cases = (("dense [4096x2048]x[2048x5632] (shared gate+up as one GEMM)", None, 4096, 2048, 5632),
             ("dense [4096x2816]x[2816x2048] (shared down)", None, 4096, 2816, 2048),
             ("bmm 64x[384x2048]x[2048x2816] (routed gate+up, even segments)", 64, 384, 2048, 2816),
             ("bmm 64x[384x1408]x[1408x2048] (routed down, even segments)", 64, 384, 1408, 2048),
             ("dense 8192^3", None, 8192, 8192, 8192))
    out = []
    for name, batch, m, k, n in cases:
        lead = (batch,) if batch else ()
        a = torch.randn(*lead, m, k, device=device, dtype=torch.float32).to(dtype)
        b = torch.randn(*lead, k, n, device=device, dtype=torch.float32).to(dtype)
        for _ in range(3):
            torch.matmul(a, b)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(runs):
            torch.matmul(a, b)
        stop.record()
        torch.cuda.synchronize()
        us = start.elapsed_time(stop) * 1e3 / runs
        flops = 2.0 * (batch or 1) * m * k * n
        out.append({"gemm": name, "us": us, "tflops": flops / us / 1e6,
                    "frac_of_peak": flops / us / 1e6 / MFMA_BF16_PEAK_TFLOPS})
        del a, b
    return out


def compact_prefill(r):
    """The handful of prefill figures that travel inside ``roofline``."""
    if not r:
        return None
    return {"bound": "mfma", "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "achieved": r["layer_tflops"],
            "frac": r["mfma_frac"], "ms_per_step": r["ms_per_step"], "tokens_per_s": r["tokens_per_s"],
            "steps": r["steps"], "form": r["form"], "ms_per_step_other_form": r["ms_per_step_other_form"],
            "gateup_us_per_layer_call": r["gateup"]["us_per_layer_call"], "gateup_mfma_frac": r["gateup"]["mfma_frac"],
            "down_us_per_layer_call": r["down"]["us_per_layer_call"], "down_mfma_frac": r["down"]["mfma_frac"],
            "ffn_shader_clock_mhz": r["ffn_shader_clock_mhz"], "mfma_frac_at_clock": r["mfma_frac_at_clock"],
            "mfma_probe_lds_fragments_frac": r["mfma_probe"]["lds_fragments"]["frac_of_peak"],
            # socket power / shader clock the driver reported during a pass of the same steps, and during
            # the probe loop (None where the box exposes neither sysfs files nor amd-smi to this user)
            "telemetry": _compact_telemetry(r.get("telemetry")),
            "mfma_probe_telemetry": _compact_telemetry(r["mfma_probe"]["lds_fragments"].get("telemetry"))}


def _compact_telemetry(t):
    if not t or not t.get("available"):
        return {"available": False, "note": (t or {}).get("note")}
    p, c = t.get("power_w") or {}, t.get("sclk_mhz") or {}
    return {"available": True, "power_source": t["power_source"], "clock_source": t["clock_source"],
            "power_samples": p.get("samples"), "power_w_mean": p.get("mean"), "power_w_max": p.get("max"),
            "power_cap_w": t.get("power_cap_w"), "sclk_samples": c.get("samples"), "sclk_mhz_mean": c.get("mean"),
            "sclk_mhz_min": c.get("min"), "sclk_mhz_max": c.get("max")}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip batch 1/32 decode and the prefill workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-offload", action="store_true", help="skip the two offloaded workloads (the long legs)")
    ap.add_argument("--only-prefill", action="store_true", help="run just the prefill workload (for profiling)")
    ap.add_argument("--only-decode", type=int, default=0, metavar="BATCH",
                    help="run just the all-resident decode workload at this batch size (for profiling)")
    ap.add_argument("--no-telemetry", action="store_true",
                    help="do not sample power and clock (no sampling threads, no amd-smi child processes)")
    ap.add_argument("--routing-launch-probe", action="store_true",
                    help="time the decode routing launch's parts (router alone, shared gate/up alone, both) and exit")
    ap.add_argument("--library-gemms", action="store_true",
                    help="time plain vendor-library GEMMs at the prefill shapes (a reference point) and exit")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch a 256 MiB plain copy kernel a few times (yardstick for --pmc byte counters)")
    ap.add_argument("--cached-decode", type=int, default=0, metavar="STEPS",
                    help="run just the expert-cache decode comparison (rr vs rs) for STEPS decode steps")
    ap.add_argument("--epipe-prefill", action="store_true",
                    help="run just the readiness-aware chunked prefill comparison (rr vs rs-epipe vs sparse)")
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

    GpuTelemetry.enabled = not args.no_telemetry
    if args.library_gemms:
        print(json.dumps({"library_gemms": library_gemms(device)}))
        return
    if args.routing_launch_probe:
        print(json.dumps({"routing_launch_probe": routing_launch_probe(dtype, device)}))
        return
    if args.calib_copy:
        from sparse_amd import ops
        src = torch.empty(256 << 20, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(4):
            ops.calib_copy(src, dst)
        torch.cuda.synchronize()
        del src, dst
    if args.only_prefill:
        print(json.dumps(prefill_workload(DEEPSEEK, 4096, max(2, args.steps), args.warmup, dtype, device)))
        return
    if args.only_decode:
        blocks = build_stack(QWEN, dtype, device)
        print(json.dumps(decode_workload(blocks, QWEN, args.only_decode, args.steps, args.warmup, dtype, device,
                                         not args.no_graph)))
        return
    if args.cached_decode:
        print(json.dumps({"cached_decode_qwen": cached_decode_workload(dtype, device, args.cached_decode)}))
        return
    if args.epipe_prefill:
        print(json.dumps({"epipe_prefill_deepseek": epipe_prefill_workload(dtype, device)}))
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
        extra["prefill_4k_deepseek"] = prefill_workload(DEEPSEEK, 4096, max(10, min(50, args.steps // 2)), 2, dtype,
                                                        device)
    if not args.no_extra:
        # the same stack and step in fp16, the dtype of the reference's formal runs
        blocks16 = build_stack(QWEN, torch.float16, device)
        extra["decode_b8_fp16"] = decode_workload(blocks16, QWEN, 8, max(20, args.steps // 2), args.warmup,
                                                  torch.float16, device, not args.no_graph)
        del blocks16
        _Workspace._cache.clear()
        torch.cuda.empty_cache()
    if not args.no_extra and not args.no_offload:
        # the offloaded configurations: rr and rs as the configuration states them (512 decode steps
        # from a cold cache), this build's other variants at 64 steps and labelled so; a failure
        # here (e.g. no pinned memory to be had) must not cost the main line
        for name, leg in (("cached_decode_qwen", lambda: cached_decode_workload(dtype, device, 512, short_steps=64)),
                          ("epipe_prefill_deepseek", lambda: epipe_prefill_workload(dtype, device))):
            try:
                extra[name] = leg()
            except Exception as exc:  # noqa: BLE001
                extra[name] = {"error": repr(exc)[:300]}
            release_stack()
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(QWEN, 8, dtype, device)
        # the CPU oracle beside the other half of the metric and on the reference's own CPU-runnable case
        for key, leg in (("prefill", lambda: cpu_baseline_prefill(DEEPSEEK, 4096, 512, dtype, device)),
                         ("config1", lambda: cpu_baseline_config1(QWEN, device))):
            try:
                cpu[key] = leg()
            except Exception as exc:  # noqa: BLE001
                cpu[key] = {"error": repr(exc)[:300]}

    if cpu is not None and isinstance(extra.get("cached_decode_qwen"), dict):
        # the residency policy's CPU oracle replayed on the routing of the two methods the configuration
        # names: its demand-miss count beside the product's
        cpu["policy_oracle"] = {name: {"misses": leg.get("misses"), "oracle_misses": leg.get("oracle_misses"),
                                       "steps": leg.get("steps")}
                                for name, leg in extra["cached_decode_qwen"].items()
                                if isinstance(leg, dict) and "oracle_misses" in leg}
    gu = main_res["gateup"]
    ratio = measured_traffic_ratio()
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
            "frac": gu["gbps"] / HBM_PEAK_GBPS,
            # HBM bytes per launch: NOT measured in this run (counters need the profiler); the ratio
            # recorded in profiles/ (FETCH_SIZE + WRITE_SIZE runs scaled by a plain copy) applied to
            # this run's algorithmic bytes
            "traffic": (gu["bytes_per_launch"] * ratio) if ratio else None,
            "traffic_source": ("recorded: profiles/decode_b8_qwen_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / "
                               "WRITE_SIZE, scaled by a plain copy kernel) x this run's algorithmic bytes"
                               if ratio else None),
            "traffic_over_algorithmic": ratio, "kernel": gu["kernel"],
            "bytes_per_launch": gu["bytes_per_launch"], "avg_launch_us": gu["avg_us"], "launches": gu["launches"],
            "mean_distinct_experts": main_res["mean_distinct_experts"],
            # the whole step against the HBM roofline (the figure the 0.70 target is stated on); the
            # dominant kernel's own fraction is `frac` above
            "step_hbm_frac": main_res["step_hbm_frac"],
            "step_hbm_gbps": main_res["step_hbm_gbps"],
            # the other half of the metric: the DeepSeek-V2-Lite-shaped 4096-token prefill (BASELINE
            # configs[2]) against the bf16 MFMA peak, and the same decode step in fp16
            "prefill_4k": compact_prefill(extra.get("prefill_4k_deepseek")),
            "decode_b8_fp16": ({"ms_per_step": extra["decode_b8_fp16"]["ms_per_step"],
                                "step_hbm_frac": extra["decode_b8_fp16"]["step_hbm_frac"]}
                               if "decode_b8_fp16" in extra else None),
            "decode_b1_step_hbm_frac": extra["decode_b1"]["step_hbm_frac"] if "decode_b1" in extra else None,
            "decode_b32_step_hbm_frac": extra["decode_b32"]["step_hbm_frac"] if "decode_b32" in extra else None,
        },
        "cpu_baseline": cpu,
        "step_hbm_frac": main_res["step_hbm_frac"],
        "kernels_us": main_res["kernels_us"],
        "launches": {"gateup": main_res["gateup"], "down": main_res["down"], "route": main_res["route"]},
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
