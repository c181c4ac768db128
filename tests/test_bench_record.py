"""The benchmark's last stdout line must stay small enough for any harness to lift it:
build it from stub measurements and check its size, its keys and that it round-trips."""
import json

import bench


def _row(name, with_cold=True):
    r = {
        "workload": f"{name} fwd+bwd fp32 some rather long description of the workload (informational)",
        "algorithmic_bytes": {"fwd": 134217728, "bwd": 201326592},
        "ms_per_step": 0.050688199999626704, "gbs": 6619.771860166096,
        "frac_of_hbm_peak": 0.8274714825207621, "samples_per_s": 10100970.24561477,
        "fwd_ms": 0.022737499326467514, "bwd_ms": 0.032495999708771706,
        "fwd_ms_min": 0.0219, "bwd_ms_min": 0.0317, "fwd_ms_mean": 0.0229, "bwd_ms_mean": 0.0326,
        "fwd_gbs": 5902.9238911846505, "bwd_gbs": 6195.426938831968,
        "bwd_back_to_back_ms": 0.030069780349731446, "event_pair_ms": 0.005178999854251742,
        "graph_replay": {"ms_per_step": 0.0504, "gbs": 6651.2, "frac_of_hbm_peak": 0.8314},
        "cpu": {"fwd_ms": 2.9, "bwd_ms": 3.2, "gbs": 55.02692191196601, "samples_per_s": 83964.4, "threads": 16,
                "warmups": 3, "reps": 5, "seconds": 0.05, "env": dict(bench.CPU_ENV)},
    }
    if with_cold:
        r["cold"] = {"copies": 4, "ms_per_step": 0.0592, "gbs": 5662.7, "frac_of_hbm_peak": 0.7078423040307945}
    return r


def _stub_results():
    names = ["cfg2_softmax", "cfg2_log_softmax", "cfg1_layer_norm", "cfg3_batch_norm", "cfg4_layer_norm_f16",
             "cfg5a_channelwise_softmax", "cfg5b_wide_softmax"] + [f"extra_row_number_{i}" for i in range(40)]
    return {n: _row(n, with_cold=(i % 2 == 0)) for i, n in enumerate(names)}


def test_record_is_small_and_round_trips():
    yard = {"tensor_bytes": 67108864, "copy_gbs": 5102.123456789, "copy_frac": 0.6378,
            "add_gbs": 5523.123456789, "add_frac": 0.6904}
    committed = {"traffic_bytes_per_launch": 201444266.58761224, "rocprof_avg_us": 30.011206451612903}
    out = bench.build_record(_stub_results(), "cfg2_softmax", 20, 5, yard, committed)
    line = json.dumps(out)
    assert len(line) < 4096, len(line)
    assert json.loads(line) == out
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in out, key
    assert "layers" not in out
    assert set(out["config"]["per_config"]) == {n for n in _stub_results() if n.startswith("cfg")}
    assert out["config"]["workload"].startswith("cfg2_softmax")
    rf = out["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in rf, key
    cb = out["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] == 16 and "3 warm-ups" in cb["sample"]


def test_roofline_fraction_is_this_runs_measurement():
    res = _stub_results()
    committed = {"traffic_bytes_per_launch": 2.0e8, "rocprof_avg_us": 30.0}
    a = bench.build_record(res, "cfg2_softmax", 20, 5, None, committed)["roofline"]
    assert a["agrees_with_rocprof"] is True
    assert abs(a["achieved"] - 201326592 / (res["cfg2_softmax"]["bwd_back_to_back_ms"] * 1e-3) / 1e9) < 1e-6
    # a slower kernel moves the fraction, whatever the committed trace says
    res["cfg2_softmax"]["bwd_back_to_back_ms"] = 0.034
    b = bench.build_record(res, "cfg2_softmax", 20, 5, None, committed)["roofline"]
    assert b["frac"] < a["frac"] and b["agrees_with_rocprof"] is False
    assert abs(b["frac"] - 201326592 / 0.034e-3 / 1e9 / 8000.0) < 1e-9
    c = bench.build_record(res, "cfg2_softmax", 20, 5, None, None)["roofline"]
    assert c["traffic"] is None and c["agrees_with_rocprof"] is None


def test_more_than_one_gpu_is_refused():
    import subprocess
    import sys
    p = subprocess.run([sys.executable, bench.__file__, "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode == 2 and "one GPU" in p.stderr
