"""bench.py's command-line contract and the byte model behind its roofline figures."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")
sys.path.insert(0, ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_algorithmic_bytes_per_parameter():
    """Every stream read once and / or written once: the per-rule figures the roofline uses."""
    import bench
    assert bench.BYTES_PER_PARAM == {"sgd": 20, "adam": 28, "rmsprop": 20, "adagrad": 20, "adadelta": 28,
                                     "nadam": 28, "adam_amp": 28}
    # L-BFGS: update pass alone when no pair is valid; 32 + 32 c with c valid pairs
    assert bench.lbfgs_bytes_per_param(0) == 28
    assert [bench.lbfgs_bytes_per_param(c) for c in (1, 2, 10)] == [64, 96, 352]


REQUIRED = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
            "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline")


def check_default_line(line, steps, warmup):
    """What the driver needs of the LAST line of the default run: short enough to survive its capture, valid JSON,
    the headline record with roofline and CPU baseline, every other configuration's figures."""
    import bench
    assert len(line) < 2048, len(line)
    j = json.loads(line)
    for key in REQUIRED:
        assert key in j, key
    assert j["n_gpus"] == 1 and j["steps"] == steps and j["warmup"] == warmup and j["vs_baseline"] is None
    assert j["dtype"] == "f32" and j["unit"] == "params/s" and j["higher_is_better"] is True
    assert "config5" in j["config"]["workload"] and j["config"]["params"] == 1_012_301_824 and "model" not in j["config"]
    roof = j["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "kernel_ms", "bytes_per_param"):
        assert key in roof, key
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["bytes_per_param"] == 28
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-4
    # the line's own figures agree with each other: value = params / ms_per_step, achieved = 28 B x params / kernel_ms
    assert abs(j["value"] - j["config"]["params"] / (j["ms_per_step"] * 1e-3)) / j["value"] < 1e-4
    assert abs(roof["achieved"] - 28 * j["config"]["params"] / (roof["kernel_ms"] * 1e-3) / 1e9) / roof["achieved"] < 1e-4
    cpu = j["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    amp = j["amp"]
    assert amp["default"] in ("in_place", "one_pass")
    for form in ("in_place", "one_pass"):
        assert 0 < amp[form]["frac"] < 1 and amp[form]["ms_per_step"] > 0
    assert sorted(j["configs"]) == sorted(n for n in bench.BASELINE_CONFIGS if n != "c5")
    for name, c in j["configs"].items():
        for key in ("ms_per_step", "steps", "value", "frac", "kernel_ms", "cpu"):
            assert key in c, (name, key)
        if name.startswith("c3-"):
            assert 0 < c["frac_hbm"] < 1
    assert j["configs"]["c4"]["frac_one_pass"] > 0
    assert j["records"].endswith("bench_configs.json")
    return j


def synthetic_records():
    """Records shaped like the ones the single-workload runs print, with figures of full double precision and prose
    fields longer than the real ones."""
    import bench
    prose = "a sentence that goes on and on about how this figure was taken, " * 8
    roof = lambda k: {"bound": "hbm", "achieved": 6587.123456789012 + k, "peak": 8000.0, "unit": "GB/s",
                      "frac": (6587.123456789012 + k) / 8000.0, "traffic": 2.8359e10, "traffic_source": prose,
                      "kernel": "multi_tensor_update_kernel<adam>", "bytes_per_param": 28,
                      "kernel_ms": 4.302727222442627, "kernel_ms_median": 4.3, "kernel_ms_min": 4.29,
                      "copy_kernel_gbs": 6617.441724517294, "frac_of_copy_kernel": 0.9872677298195458, "note": prose,
                      "frac_hbm": 0.7912345678, "achieved_hbm": 6329.87654321, "footprint_bytes": 400000000}
    cpu = {"value": 5644320252.590273, "unit": "params/s", "cores": 16, "kind": "port", "sample": prose,
           "sample_params": 95543296, "sample_steps": 740, "sample_seconds": 12.04567}
    form = lambda k: {"value": 213929119892.47342, "unit": "params/s", "ms_per_step": 4.731949650000011, "dtype": prose[:60],
                      "skipped_steps": 0, "roofline": roof(k), "form": prose,
                      "async": {"value": 2.1e11, "ms_per_step": 4.718167249999983, "kernel_ms": 4.712443923950195,
                                "achieved": 6014.8092007937, "frac": 0.7518511500992126, "note": prose}}
    records = {}
    for name in bench.BASELINE_CONFIGS:
        params = 1_012_301_824
        wall = 4.302727222442627 * 1.0007
        if name in ("c1", "c2-sgd", "c2-adam", "c3-rmsprop"):      # microsecond steps print longer
            wall *= 1.0123e-3
        r = {"metric": "params updated/sec (Adam fp32 multi-tensor step) + achieved HBM GB/s (% of peak)",
             "value": params / (wall * 1e-3), "unit": "params/s", "n_gpus": 1,
             "steps": 20 if name == "c5" else 200, "warmup": 5 if name == "c5" else 300, "ms_per_step": wall,
             "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
             "config": {"workload": bench.WORKLOADS[name][0], "tensors": 400, "params": params, "rule": "adam",
                        "hyper": {"lr": 0.001}, "launch": {"chunk": "auto"}, "state_placement": prose},
             "roofline": roof(0), "cpu_baseline": cpu}
        r["roofline"]["kernel_ms"] = wall / 1.0007
        if not name.startswith("c3-"):
            for key in ("frac_hbm", "achieved_hbm"):
                del r["roofline"][key]
        r["roofline"]["achieved"] = 28 * params / (r["roofline"]["kernel_ms"] * 1e-3) / 1e9
        r["roofline"]["frac"] = r["roofline"]["achieved"] / 8000.0
        if name == "c5":
            r["amp"] = {"default_form": "in_place", "in_place": form(1), "one_pass": form(2), "cpu_baseline": cpu}
        if name == "c4":
            r.update({"in_place": form(1), "one_pass": form(2), "fp32_adam": {"roofline": roof(3)}, "form": prose})
        records[name] = r
    return records


def test_the_default_runs_last_line_is_short_and_complete():
    """The final line of the default run is assembled by compact_line from the per-configuration records: under
    2 KB however long the records' prose, parseable, with every field the driver's record needs."""
    import bench
    line = bench.compact_line(synthetic_records(), "gpurun_out/bench_configs.json")
    assert "\n" not in line
    j = check_default_line(line, 20, 5)
    assert "note" not in j["roofline"] and "sentence" not in json.dumps(j["configs"])
    # without the CPU leg the line still parses and says so
    records = synthetic_records()
    for r in records.values():
        r["cpu_baseline"] = None
    j = json.loads(bench.compact_line(records, "x/bench_configs.json"))
    assert j["cpu_baseline"] is None and all(c["cpu"] is None for c in j["configs"].values())


def test_the_line_limit_holds_by_construction(monkeypatch):
    """If the figures ever print longer than expected, compact_line drops the least needed per-configuration fields
    rather than exceed the limit; the headline record keeps every required field."""
    import bench
    monkeypatch.setattr(bench, "LINE_LIMIT", 1650)
    line = bench.compact_line(synthetic_records(), "gpurun_out/bench_configs.json")
    assert len(line) <= 1650
    j = json.loads(line)
    for key in REQUIRED + ("amp", "configs"):
        assert key in j, key
    assert all("frac" in c and "ms_per_step" in c and "value" in c for c in j["configs"].values())


def test_workload_lists_match_the_configurations():
    from workloads import amp_125m_sizes, cnn_sizes, ragged_sizes, transformer_block_sizes
    assert sum(cnn_sizes()) == 1_143_690 and len(cnn_sizes()) == 16
    assert sum(ragged_sizes()) == 25_000_000 and len(ragged_sizes()) == 160
    assert min(ragged_sizes()) >= 64 and max(ragged_sizes()) <= 4 * 1024 * 1024
    assert sum(amp_125m_sizes()) == 125_000_000 and len(amp_125m_sizes()) == 60
    t = transformer_block_sizes()
    assert sum(t) == 1_012_301_824 and len(t) == 400
    assert t.count(4096 * 4096) == 28 and t.count(4096 * 11008) == 12 and t.count(4096) == 360


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    """A short run of a small workload prints exactly one line of JSON with the fields the driver reads."""
    r = subprocess.run([sys.executable, BENCH, "--workload", "c2-adam", "--steps", "5", "--warmup", "2", "--cpu-seconds", "2"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    j = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in j, key
    assert j["n_gpus"] == 1 and j["steps"] == 5 and j["warmup"] == 2 and j["vs_baseline"] is None
    assert "workload" in j["config"] and "model" not in j["config"]
    roof = j["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-12
    assert "traffic" in roof and "not measured" in roof["traffic_source"]
    assert j["amp"]["default_form"] == "in_place" and {"in_place", "one_pass"} <= set(j["amp"])
    cpu = j["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]


@pytest.mark.gpu
def test_default_run_ends_with_one_short_line_the_driver_can_parse():
    """The command the driver runs (no workload named), shortened: every configuration in a process of its own,
    the full records in the file the line names, and stdout = ONE line under 2 KB."""
    r = subprocess.run([sys.executable, BENCH, "--gpus", "1", "--steps", "2", "--warmup", "1", "--cpu-seconds", "0.3"],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, [len(l) for l in lines]
    j = check_default_line(lines[-1], 2, 1)
    full = json.load(open(os.path.join(ROOT, j["records"])))
    assert sorted(full) == sorted(["c5"] + list(j["configs"]))
    for name, rec in full.items():
        assert "roofline" in rec and "cpu_baseline" in rec, name
    assert full["c5"]["amp"]["default_form"] == j["amp"]["default"]
    for name in ("c3-rmsprop", "c3-adagrad", "c3-adadelta", "c3-nadam"):
        roof = full[name]["roofline"]
        assert roof["rotated"]["footprint_bytes"] > 1 << 30 and roof["frac_of_copy_kernel"] <= 1.0, (name, roof)


@pytest.mark.gpu
def test_placement_workload_prints_both_placements_for_every_layout():
    """The command behind profiles/adam_c5_1b_state_placement.md runs and reports the step with the state buffers
    wherever the allocator puts them and at the optimizers' phases, in each layout of device memory."""
    r = subprocess.run([sys.executable, BENCH, "--workload", "placement", "--steps", "2", "--warmup", "1"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    j = json.loads(lines[0])
    assert len(j["layouts"]) == 6 and j["config"]["state_phases"] == [512 << 10, 1536 << 10]
    for row in j["layouts"]:
        for key in ("plain", "placed", "plain_again", "placed_again"):
            assert 0.3 < row[key]["frac"] < 1.0, (row["spacer_bytes"], key, row[key])
    assert j["plain_range"][0] <= j["plain_mean"] <= j["plain_range"][1]
    assert j["placed_range"][0] <= j["placed_mean"] <= j["placed_range"][1]
