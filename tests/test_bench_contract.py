"""bench.py's command-line contract: what can be checked without a GPU, and
(marked gpu) that the default-shaped run prints one JSON line with the fields
the harness reads."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_unknown_workload_is_refused():
    r = subprocess.run([sys.executable, BENCH, "--workload", "nope"], capture_output=True, text=True)
    assert r.returncode != 0 and "unknown workload" in r.stderr


def test_parameter_server_round_trip_mode_runs_on_the_host():
    r = subprocess.run([sys.executable, BENCH, "--ps-roundtrip"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["metric"] == "ps_round_trip_us"
    for d in ("100", "512", "1001", "16385"):
        for mode in ("dense", "packed"):
            assert out["widths"][d][mode]["read_us"] > 0
            assert out["widths"][d][mode]["bupdate_us"] > 0


def test_traffic_table_names_known_workloads_and_committed_summaries():
    sys.path.insert(0, ROOT)
    import bench
    from paracel_amd.datagen import gen

    cfgs = gen.configs()
    for name, (rows, kernel, nbytes, src) in bench.MEASURED_TRAFFIC.items():
        assert name in cfgs and cfgs[name].n == rows
        assert os.path.exists(os.path.join(ROOT, src)), src
        # counter traffic can only exceed the algorithmic bytes, and not by much; a shard
        # whose constant first column stays on the host reads one column less than the
        # reference's row has
        stored = cfgs[name].algorithmic_bytes() - (8 * rows if cfgs[name].bias_first else 0)
        assert 1.0 <= nbytes / stored < 1.1
        # a figure measured with another kernel or another shard size is not reported
        assert bench.measured_traffic(cfgs[name], kernel) == (nbytes, src)
        assert bench.measured_traffic(cfgs[name], kernel + " ") == (None, None)
        assert bench.measured_traffic(cfgs[name].scaled(rows // 2), kernel) == (None, None)
    for name in bench.PER_CONFIG:
        assert name in cfgs


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    r = subprocess.run([sys.executable, BENCH, "--workload", "c2_headline_1m_x_1000", "--rows",
                        "200000", "--steps", "5", "--warmup", "1", "--cpu-sample-rows", "20000"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
                "roofline", "cpu_baseline"):
        assert key in out
    assert out["n_gpus"] == 1 and out["steps"] == 5 and out["dtype"] == "f64"
    assert out["vs_baseline"] is None and out["data"] == "synthetic"
    assert "workload" in out["config"] and "model" not in out["config"]
    rf = out["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s"
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-12
    assert 0.3 < rf["frac"] < 1.0
    assert rf["traffic"] is None          # 200 000 rows: not the shard the counters were read on
    assert abs(rf["whole_step_frac"] - rf["whole_step_gbs"] / rf["peak"]) < 1e-12
    assert rf["read_probe_gbs"] > 0 and rf["copy_probe_gbs"] > 0
    assert out["config"]["kernel"].startswith("shard_pass<8,4,1,4")
    cb = out["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and cb["sample"]
    assert cb["cores"] <= cb["host_cpu_count"] and cb["cores"] <= 16


@pytest.mark.gpu
def test_the_default_run_fits_what_the_harness_keeps():
    # the default run: headline + the other configurations, config 5 through the parameter
    # server with 1, 2 and 4 workers, the loader, the other shapes -- ONE line, short enough
    # that nothing falls off the front of a log that keeps its last few KB
    r = subprocess.run([sys.executable, BENCH, "--steps", "3", "--warmup", "1"],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-3000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    assert len(lines[0]) < 6144, len(lines[0])
    out = json.loads(lines[0])
    assert out["config"]["workload"] == "c2_headline_1m_x_1000" and out["steps"] == 3
    cols = out["row_cols"]
    for name in ("c1_dense_100k_x_100", "c3_tall_10m_x_256", "c4_wide_200k_x_16384",
                 "c4b_wide_200k_x_16385", "c5_e2e_2m_x_512"):
        row = out["per_config"][name]
        assert len(row) == len(cols) and row[cols.index("kernel_ms")] > 0, (name, row)
        assert row[cols.index("cpu_steps_per_s_16")] > 0
    for name, row in out["other_shapes"].items():
        assert len(row) == len(cols) and 0.3 < row[cols.index("frac")] < 1.0, (name, row)
    assert "x_wide_75k_x_20000" in out["other_shapes"]
    ps = out["c5_via_ps"]
    assert [r[0] for r in ps["rows"]] == [1, 2, 4]
    for r_ in ps["rows"]:
        assert r_[1] > 0 and r_[4] <= 1e-8, r_
        # worker 0's round in its six phases: they add up to the round
        assert len(r_[5]) == 6 and abs(sum(r_[5]) - r_[2]) < 0.1 * r_[2], r_
    assert out["c1_latency_us"]["train_dgd_per_round"] > 0
    assert out["c5_text_to_shard"]["text_gb_per_s"] > 0
