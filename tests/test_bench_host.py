"""Host-side pieces of bench.py that need no GPU: the power / clock sampler on a stand-in sysfs tree and
on `amd-smi`'s JSON, the policy call log replayed through the oracle, and the command-line contract."""
import json
import subprocess
import sys
import time
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))
import bench  # noqa: E402


SMI = {"gpu_data": [{"gpu": 0,
                     "power": {"socket_power": {"value": 1377, "unit": "W"}, "gfx_voltage": "N/A"},
                     "clock": {"gfx_0": {"clk": {"value": 1800, "unit": "MHz"}, "max_clk": {"value": 2400, "unit": "MHz"}},
                               "gfx_1": {"clk": {"value": 1900, "unit": "MHz"}},
                               "mem_0": {"clk": {"value": 2000, "unit": "MHz"}}}}]}


def test_amd_smi_json_is_reduced_to_power_and_mean_gfx_clock(monkeypatch):
    def fake_run(cmd, **kw):
        assert cmd[:2] == ["amd-smi", "metric"]
        return subprocess.CompletedProcess(cmd, 0, stdout=json.dumps(SMI), stderr="")
    monkeypatch.setattr(subprocess, "run", fake_run)
    assert bench.GpuTelemetry._amd_smi() == (1377.0, 1850.0)
    monkeypatch.setattr(subprocess, "run", lambda cmd, **kw: subprocess.CompletedProcess(cmd, 0, stdout="N/A", stderr=""))
    assert bench.GpuTelemetry._amd_smi() is None


def test_sampler_reads_a_hwmon_directory_and_summarises(tmp_path, monkeypatch):
    hw = tmp_path / "hwmon3"
    hw.mkdir()
    (hw / "power1_input").write_text("1250000000\n")
    (hw / "power1_cap").write_text("1400000000\n")
    (hw / "freq1_input").write_text("1900000000\n")
    monkeypatch.setattr(bench.GpuTelemetry, "enabled", False)
    t = bench.GpuTelemetry(period=0.005)           # built switched off, then pointed at the stand-in tree
    assert t.summary() == {"available": False, "note": "switched off (--no-telemetry)"}
    t.note, t.hwmon, t.power_file, t.freq_file, t.cap_w = None, str(hw), "power1_input", "freq1_input", 1400.0
    t.power_source, t.clock_source = "sysfs power1_input", "sysfs freq1_input"
    with t:
        time.sleep(0.05)
        (hw / "power1_input").write_text("1350000000\n")
        time.sleep(0.05)
    s = t.summary()
    assert s["available"] and s["power_cap_w"] == 1400.0
    assert s["power_w"]["min"] == 1250.0 and s["power_w"]["max"] == 1350.0 and s["power_w"]["samples"] >= 4
    assert s["sclk_mhz"]["mean"] == 1900.0
    c = bench._compact_telemetry(s)
    assert c["power_w_max"] == 1350.0 and c["sclk_mhz_mean"] == 1900.0 and c["power_cap_w"] == 1400.0
    assert bench._compact_telemetry(None) == {"available": False, "note": None}


def test_policy_call_log_replays_through_the_oracle():
    """The wrappers record budget / plan / execute calls with the phase they were made under and call through;
    the oracle fed the record counts the misses the product counted."""
    from sparse_amd.methods import residency_config
    from tests.test_residency import RoutingModel, product_layer
    cfg = residency_config("rs", 4, 3)
    E, K, layers = 16, 2, 3
    made = [product_layer(cfg, E=E, K=K, layer=l) for l in range(layers)]

    class Blk:
        def __init__(self, res):
            self.residency = res
    log = bench.PolicyCallLog([Blk(m[0]) for m in made])
    model = RoutingModel(E, K, 4, seed=5)
    for step in range(40):
        routes = [model.route() for _ in range(layers)]
        for l in range(layers):
            if l + 1 < layers:
                tgt = made[l + 1][0]
                tgt.phase, tgt.call_id = "decode", step
                budget = tgt.prefetch_budget(("next_layer_rs", "decode", step, l, l + 1))
                if budget > 0:
                    ids, probs = model.predict(routes[l + 1], tgt.predict_topk())
                    tgt.schedule_prefetch(ids, probs, budget)
            lay = made[l][0]
            lay.phase, lay.call_id, lay.stage = "decode", step, "decode"
            lay.execute(routes[l])
    names = {c[1] for c in log.calls}
    assert names == {"prefetch_budget", "schedule_prefetch", "execute"}
    product_misses = sum(1 for m in made for kind, _l, _e in m[2].events if kind == "miss")
    assert product_misses > 0
    assert log.oracle_misses(cfg, layers, E, K) == product_misses


def test_more_than_one_gpu_is_refused():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode == 2
    assert "one GPU" in proc.stderr
