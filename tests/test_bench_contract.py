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
    cpu = j["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]


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
