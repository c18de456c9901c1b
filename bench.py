#!/usr/bin/env python3
"""Benchmark of the worker-side logistic-regression gradient step on one MI355X.

A step is one fused loss+gradient pass (plr_loss_grad through the C ABI) over a
synthetic shard that is already resident in HBM: theta goes in from the host,
the gradient sum and the loss come back to the host.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps 50] [--warmup 5] [--workload NAME]
                    [--no-cpu-baseline] [--rows N] [--headline-only]

The line is the headline configuration (1M x 1000).  Unless --workload or
--headline-only is given, the other configurations (c1, c3, c4, c4b, c5 bare and
c5 end to end through the parameter server) are timed in the same run, with the
same steps, and reported under "per_config".  The headline does exactly --warmup
untimed steps (default 5); every other workload, unless --warmup is given, keeps
warming up until 60 ms have passed and reports how many steps that took: after an
idle spell (generating and uploading a shard) the device needs 20-40 ms to be
back at its clocks, which the latency-sensitive kernels show and the headline
kernel does not.

roofline.achieved = algorithmic bytes per step (X once + y + theta + gradient +
loss = 8nd + 8n + 16d + 8) / average duration of the streaming kernel, measured
with HIP events recorded on the library's own stream around that launch.
cpu_baseline times the CPU oracle's restatement of the reference traversal
(lr.cpp:132-138, reference data layout) on the host cores of this box, on a
bounded row sample, scaled linearly in n to the full shard.
"""
import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, vendor figure

# HBM bytes per launch of the streaming kernel from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs (scaled by what the same counters read for a copy kernel of
# known size): workload -> (rows, kernel description the figure was measured with,
# bytes, summary file).  Reported only when rows and kernel match what this run
# uses, so a changed variant choice yields null instead of a stale figure.
MEASURED_TRAFFIC = {
    "c1_dense_100k_x_100": (
        100000,
        "shard_pass<NCH=1,R=16,WCOL=1,WROW=4,ALLCH=1,TL=0> nch_rt=1 tail=0 pitch=100 "
        "grid=512 x 256 threads (occupancy 2 blocks/CU, 256 CUs)",
        82217759, "profiles/shard_pass_c1_dense_100k_x_100.md"),
    "c2_headline_1m_x_1000": (
        1000000,
        "shard_pass<NCH=8,R=4,WCOL=1,WROW=4,ALLCH=1,TL=0> nch_rt=8 tail=0 pitch=1000 "
        "grid=256 x 256 threads (occupancy 1 blocks/CU, 256 CUs)",
        8055154154, "profiles/shard_pass_c2_headline_1m_x_1000.md"),
    "c3_tall_10m_x_256": (
        10000000,
        "shard_pass<NCH=2,R=32,WCOL=1,WROW=4,ALLCH=1,TL=0> nch_rt=2 tail=0 pitch=256 "
        "grid=256 x 256 threads (occupancy 1 blocks/CU, 256 CUs)",
        20560483722, "profiles/shard_pass_c3_tall_10m_x_256.md"),
    "c4_wide_200k_x_16384": (
        200000,
        "shard_pass<NCH=16,R=1,WCOL=8,WROW=1,ALLCH=1,TL=0> nch_rt=16 tail=0 pitch=16384 "
        "grid=256 x 512 threads (occupancy 1 blocks/CU, 256 CUs)",
        26261494888, "profiles/shard_pass_c4_wide_200k_x_16384.md"),
    "c4b_wide_200k_x_16385": (
        200000,
        "shard_pass<NCH=16,R=1,WCOL=8,WROW=1,ALLCH=1,TL=1> nch_rt=16 tail=16 pitch=16400 "
        "grid=256 x 512 threads (occupancy 1 blocks/CU, 256 CUs)",
        26287135754, "profiles/shard_pass_c4b_wide_200k_x_16385.md"),
    "c5_e2e_2m_x_512": (
        2000000,
        "shard_pass<NCH=4,R=16,WCOL=1,WROW=2,ALLCH=1,TL=0> nch_rt=4 tail=0 pitch=512 "
        "grid=512 x 128 threads (occupancy 2 blocks/CU, 256 CUs)",
        8210240021, "profiles/shard_pass_c5_e2e_2m_x_512.md"),
    "x_narrow_100m_x_2": (
        100000000,
        "lane_pass<NP=1,U=4,WROW=4> row-tiled layout, pitch=2, 256 rows per group, "
        "grid=768 x 256 threads (occupancy 3 blocks/CU, 256 CUs)",
        2400596292, "profiles/lane_pass_x_narrow_100m_x_2.md"),
    "x_narrow_30m_x_16": (
        30000000,
        "lane_pass<NP=8,U=1,WROW=4> row-tiled layout, pitch=16, 64 rows per group, "
        "grid=512 x 256 threads (occupancy 2 blocks/CU, 256 CUs)",
        4080835977, "profiles/lane_pass_x_narrow_30m_x_16.md"),
    "x_narrow_10m_x_41": (
        10000000,
        "lane2_pass<NP=21,U=2,WROW=1> row-tiled layout, pitch=42, 128 rows per group, "
        "grid=1024 x 128 threads (occupancy 4 blocks/CU, 256 CUs)",
        3440526459, "profiles/lane2_pass_x_narrow_10m_x_41.md"),
    "x_short_30m_x_66": (
        30000000,
        "pair_pass<G=8,WROW=4> pitch=66, 16 rows per tile, grid=512 x 256 threads "
        "(occupancy 2 blocks/CU, 256 CUs)",
        16138109813, "profiles/pair_pass_x_short_30m_x_66.md"),
    "x_short_30m_x_72": (
        30000000,
        "pair_pass<G=8,WROW=4> pitch=72, 16 rows per tile, grid=512 x 256 threads "
        "(occupancy 2 blocks/CU, 256 CUs)",
        17578887363, "profiles/pair_pass_x_short_30m_x_72.md"),
    "x_c1shape_20m_x_100": (
        20000000,
        "shard_pass<NCH=1,R=32,WCOL=1,WROW=4,ALLCH=1,TL=0> nch_rt=1 tail=0 pitch=100 "
        "grid=256 x 256 threads (occupancy 1 blocks/CU, 256 CUs)",
        16356598780, "profiles/shard_pass_x_c1shape_20m_x_100.md"),
    "x_bias_10m_x_257": (
        10000000,
        "shard_pass<NCH=2,R=32,WCOL=1,WROW=4,ALLCH=1,TL=0> nch_rt=2 tail=0 pitch=256 "
        "grid=256 x 256 threads (occupancy 1 blocks/CU, 256 CUs); first column constant "
        "1, not stored",
        20560493013, "profiles/shard_pass_x_bias_10m_x_257.md"),
    "x_bias_1m_x_2049": (
        1000000,
        "shard_pass<NCH=16,R=2,WCOL=1,WROW=4,ALLCH=1,TL=0> nch_rt=16 tail=0 pitch=2048 "
        "grid=256 x 256 threads (occupancy 1 blocks/CU, 256 CUs); first column constant "
        "1, not stored",
        16404232399, "profiles/shard_pass_x_bias_1m_x_2049.md"),
    "x_wide_250k_x_9000": (
        250000,
        "shard_pass<NCH=9,R=2,WCOL=8,WROW=1,ALLCH=0,TL=0> nch_rt=9 tail=0 pitch=9008 "
        "grid=256 x 512 threads (occupancy 1 blocks/CU, 256 CUs)",
        18190815746, "profiles/shard_pass_x_wide_250k_x_9000.md"),
    "x_wide_75k_x_20000": (
        75000,
        "team_pass<NCH=7,LAG=1> 3 column blocks of 52- chunks, 85 teams, pitch=20000 "
        "grid=255 x 512 threads (occupancy 1 blocks/CU, 256 CUs)",
        12149365862, "profiles/team_pass_x_wide_75k_x_20000.md"),
    "x_verywide_100k_x_32768": (
        100000,
        "team_pass<NCH=8,LAG=1> 4 column blocks of 64 chunks, 64 teams, pitch=32768 "
        "grid=256 x 512 threads (occupancy 1 blocks/CU, 256 CUs)",
        26348055385, "profiles/team_pass_x_verywide_100k_x_32768.md"),
    "x_wide_30k_x_50000": (
        30000,
        "team_pass<NCH=7,LAG=2> 7 column blocks of 55- chunks, 36 teams, pitch=50000 "
        "grid=252 x 512 threads (occupancy 1 blocks/CU, 256 CUs)",
        12111127486, "profiles/team_pass_x_wide_30k_x_50000.md"),
}

# The other configurations a default run times after the headline.
PER_CONFIG = ["c1_dense_100k_x_100", "c3_tall_10m_x_256", "c4_wide_200k_x_16384",
              "c4b_wide_200k_x_16385", "c5_e2e_2m_x_512"]

# Shapes beyond the five configurations, one per kernel family and layout, timed last in
# a default run (GPU only) and reported under other_shapes.
OTHER_SHAPES = ["x_narrow_100m_x_2", "x_narrow_30m_x_16", "x_narrow_10m_x_41", "x_short_30m_x_66",
                "x_c1shape_20m_x_100", "x_bias_10m_x_257", "x_wide_250k_x_9000",
                "x_wide_75k_x_20000", "x_verywide_100k_x_32768", "x_wide_30k_x_50000"]

# A one-GPU box gives a job 16 CPUs whatever os.cpu_count() shows there.
CPU_SHARE = 16

KEEP_BIAS_COLUMN = False  # --keep-bias-column


def measured_traffic(cfg, kernel_info):
    ent = MEASURED_TRAFFIC.get(cfg.name)
    if not ent or ent[0] != cfg.n or ent[1] != kernel_info:
        return None, None
    return ent[2], ent[3]


def cpu_threads():
    return max(1, min(CPU_SHARE, os.cpu_count() or 1))


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=int(os.environ.get("WORLD_SIZE", "1")))
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed warm-up steps (default 5).  The headline workload does exactly "
                         "these; the other workloads, when --warmup is not given, go on warming "
                         "up until 60 ms have passed: after an idle spell the device needs 20-40 "
                         "ms to reach its clocks, which the latency-bound kernels (narrow and "
                         "very wide rows) feel and the headline kernel does not")
    ap.add_argument("--workload", default=None,
                    help="time only this workload (default: the headline c2_headline_1m_x_1000 "
                         "plus the other configurations under per_config)")
    ap.add_argument("--keep-bias-column", action="store_true",
                    help="workloads whose first column is the constant bias: store it in HBM "
                         "like any other column (default: it stays on the host)")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip the per_config and other_shapes sections of a default run")
    ap.add_argument("--rows", type=int, default=0, help="override n (debugging)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-rows", type=int, default=0)
    ap.add_argument("--train", action="store_true",
                    help="device-resident training rounds (plr_train_dgd, theta stays in HBM) "
                         "with the final theta checked against the CPU oracle")
    ap.add_argument("--e2e", action="store_true",
                    help="end-to-end rounds through the host parameter server (C++ worker + "
                         "plr_ps_server over ZeroMQ) instead of the bare gradient step")
    ap.add_argument("--workers", type=int, default=1,
                    help="with --e2e: worker processes sharing the GPU, each with n / W rows")
    ap.add_argument("--no-dense-ps", action="store_true",
                    help="with --e2e: start the server with its dense-vector fast path off")
    ap.add_argument("--parse", action="store_true",
                    help="the loader instead of the gradient step: sample text -> resident shard "
                         "on the device (plr_set_data_csv) against the host's parsers")
    ap.add_argument("--parse-format", default="%.6f",
                    help="with --parse: the printf format of the sample text's fields "
                         "(e.g. %%.17g for full-precision spellings)")
    ap.add_argument("--ps-roundtrip", action="store_true",
                    help="host only: microseconds per paracel_read / paracel_bupdate round trip "
                         "against plr_ps_server, dense fast path on and off")
    a = ap.parse_args()
    # an explicit --warmup is taken literally everywhere
    a.settle_ms = 60.0 if a.warmup is None else 0.0
    if a.warmup is None:
        a.warmup = 5
    return a


def upload(ctx, cfg, chunk_bytes=1 << 30, keep_rows=0):
    """Generate the shard on the host in row chunks and stream it to HBM.
    Returns the first keep_rows rows (for the CPU baseline sample)."""
    import numpy as np

    # a shard as the file path builds it starts every row with the bias 1.0: say so, and
    # the library keeps that column out of HBM (--keep-bias-column stores it, for comparison)
    ctx.set_option("first_column_is_one", 1 if (cfg.bias_first and not KEEP_BIAS_COLUMN) else 0)
    ctx.alloc_data(cfg.n, cfg.d)
    chunk_rows = max(1, chunk_bytes // (8 * cfg.d))
    keepX, keepy = [], []
    kept = 0
    buf = np.empty((min(chunk_rows, cfg.n), cfg.d))  # reused: first touch of fresh pages is slow
    for lo in range(0, cfg.n, chunk_rows):
        m = min(chunk_rows, cfg.n - lo)
        X, y = cfg.rows(lo, m, out=buf[:m])
        ctx.set_data_chunk(lo, X, y)
        if kept < keep_rows:
            t = min(m, keep_rows - kept)
            keepX.append(X[:t].copy())
            keepy.append(y[:t].copy())
            kept += t
    if keep_rows:
        return np.concatenate(keepX), np.concatenate(keepy)
    return None, None


def reference_build_status():
    """The reference's own lr_serial needs Boost, Eigen3, msgpack-c and gflags headers
    (include/ps.hpp); say whether this box has them (it is timed only if it can be built)."""
    need = {"boost": ["boost/version.hpp"], "eigen3": ["eigen3/Eigen/Dense", "Eigen/Dense"],
            "msgpack-c": ["msgpack.hpp"], "gflags": ["gflags/gflags.h"]}
    roots = ["/usr/include", "/usr/local/include", "/opt/conda/include"]
    missing = [k for k, hs in need.items()
               if not any(os.path.exists(os.path.join(r, h)) for r in roots for h in hs)]
    if missing:
        return "reference not buildable here: no " + ", ".join(missing)
    return "reference dependencies present (reference binary not timed by this script)"


def cpu_model_name():
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.startswith("model name"):
                    return ln.split(":", 1)[1].strip()
    except OSError:
        pass
    return ""


def cpu_baseline(cfg, Xs, ys, theta, reps1=4, repsp=20):
    """Reference traversal on the host cores: 1 core (tool/lr_serial, prun.py -w 1)
    and P local workers (mpirun -n P bin/lr), on the row sample, scaled to n."""
    from oracle import oracle

    m = Xs.shape[0]
    cores = cpu_threads()
    t1, _, tl1, _ = oracle.baseline_time(Xs, ys, theta, cfg.alpha, cfg.beta, threads=1, reps=reps1)
    tp, _, tlp, _ = oracle.baseline_time(Xs, ys, theta, cfg.alpha, cfg.beta, threads=cores,
                                         reps=repsp)
    scale = cfg.n / float(m)
    whole = "all %d rows" % m if m == cfg.n else \
        "first %d of %d rows, time scaled linearly in n" % (m, cfg.n)
    return {
        "value": 1.0 / (tp * scale),
        "unit": "steps/s",
        "cores": cores,
        "host_cpu_count": os.cpu_count(),
        "kind": "port",
        "sample": "%s (d=%d), gradient traversal lr.cpp:132-138 in the reference's "
                  "vector<vector<double>> layout, g++ -O3, %d threads as local workers (a "
                  "one-GPU box gives a job %d CPUs)" % (whole, cfg.d, cores, CPU_SHARE),
        "value_1core": 1.0 / (t1 * scale),
        "loss_pass_seconds_1core_scaled": tl1 * scale,
        "loss_pass_seconds_pcore_scaled": tlp * scale,
        "cpu_model": cpu_model_name(),
        "reference_build": reference_build_status(),
    }


def run_train(a, cfg):
    """steps rounds of delta + theta += delta on the device (tool/lr_serial.cpp:95-110)."""
    import numpy as np

    from paracel_amd import Plr

    ctx = Plr(0)
    X, y = cfg.rows(0, cfg.n)
    ctx.set_data(X, y)
    theta0 = np.zeros(cfg.d)
    ctx.train_dgd(theta0, cfg.alpha, cfg.beta, max(1, a.warmup))
    t0 = time.perf_counter()
    theta = ctx.train_dgd(theta0, cfg.alpha, cfg.beta, a.steps)
    sec = time.perf_counter() - t0
    out = {
        "metric": "lr_train_iters_per_sec", "value": a.steps / sec, "unit": "iters/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": 1e3 * sec / a.steps,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f64",
        "data": "synthetic",
        "config": {"workload": cfg.name + " device-resident training", "n": cfg.n, "d": cfg.d,
                   "step": "plr_train_dgd: delta at theta (fused pass) + theta += delta, theta "
                           "kept in HBM for all rounds", "alpha": cfg.alpha, "beta": cfg.beta,
                   "kernel": ctx.kernel_info()},
        "theta_rel_err_vs_cpu": None,
    }
    if not a.no_cpu_baseline:
        from oracle import oracle

        t0 = time.perf_counter()
        theta_cpu = oracle.train_dgd(X, y, theta0, cfg.alpha, cfg.beta, a.steps)
        sec_cpu = time.perf_counter() - t0
        out["theta_rel_err_vs_cpu"] = float(np.linalg.norm(theta - theta_cpu) /
                                            np.linalg.norm(theta_cpu))
        out["cpu_baseline"] = {"value": a.steps / sec_cpu, "unit": "iters/s", "cores": 1,
                               "kind": "port",
                               "sample": "all %d rounds on the full shard, 1 core "
                                         "(tool/lr_serial.cpp learning loop restated)" % a.steps}
    ctx.close()
    print(json.dumps(out), flush=True)


def run_e2e(a, cfg, rounds=None, workers=1, theta_cpu=None):
    """steps rounds of read theta -> GPU delta -> bupdate against a real server
    process, by `workers` worker processes that share the GPU (each with its n / workers
    rows of the shard); final theta against the CPU oracle's multi-worker training."""
    import subprocess
    import tempfile

    import numpy as np

    rounds = rounds or a.steps

    pkg = os.path.join(ROOT, "paracel_amd")
    if cfg.spec.kind != 0 or cfg.spec.zero_prob != 0.0 or cfg.spec.outlier_mod != 0:
        raise SystemExit("bench.py --e2e: the worker's --synthetic mode generates plain normal "
                         "shards only (c1, c2, c5)")
    srv = subprocess.Popen([os.path.join(pkg, "plr_ps_server")] +
                           (["--no-dense"] if a.no_dense_ps else []),
                           stdout=subprocess.PIPE, text=True)
    try:
        info = srv.stdout.readline().strip()
        with tempfile.TemporaryDirectory() as td:
            tout = os.path.join(td, "theta.bin")
            procs = []
            for r in range(workers):
                cmd = [os.path.join(pkg, "plr_lr_worker"), "--server_info", info,
                       "--synthetic", "%x,%d,%d,%.17g" % (cfg.seed, cfg.n, cfg.d, cfg.spec.scale),
                       "--rounds", str(rounds), "--alpha", "%.17g" % cfg.alpha,
                       "--beta", "%.17g" % cfg.beta, "--theta0", "zero",
                       "--update_file", os.path.join(pkg, "liblr_update.so"), "--theta_out", tout,
                       "--worker_id", str(r), "--worker_sz", str(workers)]
                procs.append(subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                                              text=True))
            reps = []
            for p in procs:
                o, e = p.communicate()
                if p.returncode != 0:
                    for q in procs:
                        q.kill()
                    raise RuntimeError("worker failed: " + e)
                reps.append(json.loads(o.strip().splitlines()[-1]))
                # "workerR ms per round: read theta a, wait for the GPU b, pass c, barrier d,
                # bupdate e, barrier f"
                for ln in o.splitlines():
                    if " ms per round: " in ln:
                        reps[-1]["phases_ms"] = [float(t.rsplit(" ", 1)[1])
                                                 for t in ln.split(": ", 1)[1].split(", ")]
            theta_gpu = np.fromfile(tout)
    finally:
        srv.kill()
        srv.wait()
    # the workers leave every round through the same barrier: the slowest one's clock
    sec = max(r["seconds"] for r in reps)
    kern_ms = sum(r["gpu_kernel_ms_per_iter"] for r in reps)  # the GPU runs them one after another
    out = {
        "metric": "lr_e2e_iters_per_sec", "value": rounds / sec, "unit": "iters/s",
        "n_gpus": 1, "steps": rounds, "warmup": 0,
        "ms_per_step": 1e3 * sec / rounds, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": cfg.name + " via parameter server", "n": cfg.n, "d": cfg.d,
                   "workers": workers,
                   "step": "paracel_read theta -> plr_dgd_delta -> paracel_bupdate delta "
                           "(ZeroMQ REQ/REP, msgpack, dlopen'ed lr_theta_update)",
                   "ps_dense_fast_path": not a.no_dense_ps,
                   "alpha": cfg.alpha, "beta": cfg.beta},
        "gpu_only_iters_per_sec": 1e3 / kern_ms,
        "gpu_kernel_ms_per_iter": kern_ms,
        "final_loss": reps[0]["final_loss"],
        "theta_rel_err_vs_cpu": None,
        # worker 0's round: read theta, wait for the GPU, pass, barrier, bupdate, barrier
        "worker0_phases_ms": reps[0].get("phases_ms"),
    }
    if theta_cpu is None and not a.no_cpu_baseline:
        from oracle import oracle

        cores = cpu_threads()
        X = np.empty((cfg.n, cfg.d))
        y = np.empty(cfg.n)
        step = 262144
        for lo in range(0, cfg.n, step):
            m = min(step, cfg.n - lo)
            _, y[lo:lo + m] = cfg.rows(lo, m, out=X[lo:lo + m])
        t0 = time.time()
        theta_cpu = oracle.train_dgd_workers(X, y, np.zeros(cfg.d), cfg.alpha, cfg.beta,
                                             rounds, cores)
        sec = time.time() - t0
        out["cpu_baseline"] = {"value": rounds / sec, "unit": "iters/s", "cores": cores,
                               "host_cpu_count": os.cpu_count(), "kind": "port",
                               "sample": "all %d rounds on the full shard, %d local workers "
                                         "(threads), in-process server add" % (rounds, cores)}
    if theta_cpu is not None:
        out["theta_rel_err_vs_cpu"] = float(np.linalg.norm(theta_gpu - theta_cpu) /
                                            np.linalg.norm(theta_cpu))
        out["theta_cpu"] = theta_cpu
    return out


def run_ps_roundtrip(a):
    """Host only: what a DGD round costs besides the gradient -- the two
    parameter-server calls, timed by plr_ps_roundtrip with the server's dense
    fast path on and off."""
    import subprocess

    pkg = os.path.join(ROOT, "paracel_amd")
    out = {"metric": "ps_round_trip_us", "unit": "us", "widths": {}, "iters": 2000}
    for mode in ("dense", "packed"):
        srv = subprocess.Popen([os.path.join(pkg, "plr_ps_server")] +
                               ([] if mode == "dense" else ["--no-dense"]),
                               stdout=subprocess.PIPE, text=True)
        try:
            info = srv.stdout.readline().strip()
            r = subprocess.run([os.path.join(pkg, "plr_ps_roundtrip"), "--server_info", info,
                                "--update_file", os.path.join(pkg, "liblr_update.so"),
                                "--d", "100,512,1001,16385", "--iters", "2000"],
                               capture_output=True, text=True, check=True)
        finally:
            srv.kill()
            srv.wait()
        for line in r.stdout.strip().splitlines():
            rec = json.loads(line)
            out["widths"].setdefault(str(rec["d"]), {})[mode] = {
                "read_us": rec["read_us"], "bupdate_us": rec["bupdate_us"]}
    print(json.dumps(out), flush=True)


def run_step(a, cfg, with_cpu, full_cpu_sample=False, cpu_reps=(4, 20), settle_ms=0.0):
    """The bare gradient step on one workload: upload, warm up, time a.steps calls of
    plr_loss_grad; returns the result record (contract keys + roofline + cpu_baseline)."""
    from paracel_amd import Plr

    theta = cfg.theta()
    sample_rows = 0
    if with_cpu:
        # bounded CPU leg: ~2 GB of rows (a few seconds per traversal on one core), or
        # the whole shard where asked (the headline: 8 GB fit the host)
        sample_rows = a.cpu_sample_rows or (
            cfg.n if full_cpu_sample else max(1, min(cfg.n, int(2.0e9 // (8 * cfg.d)))))

    ctx = Plr(0)
    t0 = time.time()
    Xs, ys = upload(ctx, cfg, keep_rows=sample_rows)
    t_up = time.time() - t0
    info = ctx.kernel_info()
    print("# shard %d x %d generated and uploaded in %.1f s; %s" % (cfg.n, cfg.d, t_up, info),
          file=sys.stderr, flush=True)

    warmup = 0
    t_warm = time.perf_counter()
    while warmup < a.warmup or (time.perf_counter() - t_warm) * 1e3 < settle_ms:
        ctx.loss_grad(theta)
        warmup += 1
    ctx.reset_timing()
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        g, loss, n = ctx.loss_grad(theta)   # synchronous: returns after the stream drained
    ctx.synchronize()
    elapsed = time.perf_counter() - t0
    _, kern_ms_sum, launches = ctx.timing()
    assert launches == a.steps and n == cfg.n
    kern_ms = kern_ms_sum / launches

    read_probe = ctx.probe_read_bandwidth(10)
    copy_probe = ctx.probe_copy_bandwidth(2 << 30, 5)   # read + written, runtime D2D copy
    bytes_step = cfg.algorithmic_bytes()
    achieved = bytes_step / (kern_ms * 1e-3) / 1e9
    whole = bytes_step / (elapsed / a.steps) / 1e9
    traffic, traffic_src = measured_traffic(cfg, info)
    out = {
        "metric": "lr_gradient_steps_per_sec",
        "value": a.steps / elapsed,
        "unit": "steps/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": warmup,
        "ms_per_step": 1e3 * elapsed / a.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {"workload": cfg.name, "n": cfg.n, "d": cfg.d,
                   "step": "plr_loss_grad: theta host->device, fused loss+gradient pass, "
                           "gsum+loss device->host",
                   "lambda": cfg.lam, "alpha": cfg.alpha, "beta": cfg.beta,
                   "kernel": kernel_code(info)},
        "kernel_info": info,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_source": traffic_src,
                     "kernel_ms": kern_ms, "algorithmic_bytes": bytes_step,
                     "whole_step_gbs": whole, "whole_step_frac": whole / HBM_PEAK_GBS,
                     # what a kernel that only reads the shard sustains, and the runtime's
                     # device-to-device copy (bytes read + written): probes, not bounds
                     "read_probe_gbs": read_probe,
                     "frac_of_read_probe": achieved / read_probe,
                     "copy_probe_gbs": copy_probe},
        "cpu_baseline": None,
        "loss_mean": loss / n,
    }
    if cfg.bias_first and not KEEP_BIAS_COLUMN:
        # the constant first column stays on the host: the kernel streams one column less
        # than the reference's row has; both byte counts, both fractions
        stored = bytes_step - 8 * cfg.n
        out["roofline"]["stored_bytes"] = stored
        out["roofline"]["frac_of_stored_bytes"] = stored / (kern_ms * 1e-3) / 1e9 / HBM_PEAK_GBS
    if with_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, Xs, ys, theta, *cpu_reps)
    ctx.close()
    return out


def run_parse(a, cfg):
    """Sample text -> resident shard (lr.cpp:76-93): plr_set_data_csv on the device against
    the host's threaded parser and the reference's std::stod per field on one core.  The
    text has the workload's width (k = d - 1 features + label, six decimals like the
    reference's sample data); ~2 GB of it are parsed in one call."""
    import tempfile

    import numpy as np

    from oracle import oracle
    from paracel_amd import Plr

    k = cfg.d - 1
    rng = np.random.default_rng(cfg.seed)
    block_rows = max(64, int(48e6 // (k * (len(getattr(a, "parse_format", "%.6f") % -0.123456789) + 1)
                                      + 2)))
    fmt = getattr(a, "parse_format", "%.6f")
    pool = np.array([fmt % v for v in rng.normal(size=200000) * cfg.spec.scale * 3])
    idx = rng.integers(0, pool.size, size=(block_rows, k))
    lab = rng.integers(0, 2, size=block_rows)
    t0 = time.time()
    block = "\n".join(",".join(pool[idx[i]]) + ",%d" % lab[i] for i in range(block_rows)) + "\n"
    block = block.encode()
    reps = max(1, int(2.0e9 // len(block)))
    print("# text block: %d rows x %d fields, %.1f MB, built in %.1f s; parsed %d times over "
          "(%.2f GB)" % (block_rows, k + 1, len(block) / 1e6, time.time() - t0, reps,
                         reps * len(block) / 1e9), file=sys.stderr, flush=True)
    ctx = Plr(0)
    ctx.set_data_csv(block)                          # warm-up: one block
    pieces = [block] * reps
    nbytes = reps * len(block)
    calls = []
    for _ in range(max(1, min(a.steps, 5))):
        t0 = time.perf_counter()
        n, d = ctx.set_data_csv(pieces)
        calls.append(time.perf_counter() - t0)
    assert (n, d) == (block_rows * reps, cfg.d)
    info = ctx.kernel_info()
    # the same with option "csv_overlap" off: the whole text transferred, then parsed; the
    # parsing kernel's own duration comes from this order (one launch over the whole text)
    ctx.set_option("csv_overlap", 0)
    serial = []
    for _ in range(3):
        t0 = time.perf_counter()
        ctx.set_data_csv(pieces)
        serial.append(time.perf_counter() - t0)
    kern_ms = ctx.timing()[0]
    ctx.set_option("csv_overlap", 1)
    ctx.set_data_csv(pieces)
    # the shard it left: spot-check against the oracle's parser on the first block
    Xo, yo = oracle.local_parser(block[:block.index(b"\n", 2000000) + 1].decode())
    X, y = ctx.get_data(0, Xo.shape[0])
    assert X.tobytes() == Xo.tobytes() and y.tobytes() == yo.tobytes()
    ctx.close()
    call = float(np.median(calls))
    # CPU: the reference's path (strtod per field, one core) on 20 MB; the host's own
    # threaded parser on one block through plr_shard_tool
    sample = block[:block.index(b"\n", min(len(block) - 2, 20000000)) + 1]
    t0 = time.perf_counter()
    oracle.local_parser(sample.decode())
    stod_s = time.perf_counter() - t0
    host = {}
    with tempfile.NamedTemporaryFile(suffix=".csv") as f:
        f.write(block)
        f.flush()
        for th in (1, cpu_threads()):
            r = subprocess.run([os.path.join(ROOT, "paracel_amd", "plr_shard_tool"), "time",
                                f.name, str(th), "0"], capture_output=True, text=True, check=True)
            nn, dd, t_split, t_parse = r.stdout.split()
            host[th] = (float(t_split), float(t_parse))
    fields = n * cfg.d
    # bytes the parsing kernel must move: the text once, 8 bytes per field written
    alg = nbytes + 8 * fields
    out = {
        "metric": "csv_parse_gb_per_sec", "value": nbytes / call / 1e9, "unit": "GB/s of text",
        "n_gpus": 1, "steps": len(calls), "warmup": 1, "ms_per_step": 1e3 * call,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8 -> f64",
        "data": "synthetic",
        "config": {"workload": cfg.name + " as text", "field_format": fmt, "rows": n,
                   "fields_per_row": cfg.d,
                   "text_bytes": nbytes, "step": "plr_set_data_csv: text host->device and, "
                   "stretch by stretch while it arrives, counted and parsed into the resident "
                   "shard (text in pageable host memory, so the call includes its PCIe "
                   "transfer)", "kernel": info,
                   "ms_per_call_transfer_then_parse": [round(1e3 * t, 2) for t in serial]},
        "roofline": {"bound": "hbm", "achieved": alg / (kern_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": alg / (kern_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": None, "kernel": "csv_parse_fields", "kernel_ms": kern_ms,
                     "algorithmic_bytes": alg,
                     "text_gbs_kernel_only": nbytes / (kern_ms * 1e-3) / 1e9},
        "cpu_baseline": {
            "value": len(block) / sum(host[cpu_threads()]) / 1e9, "unit": "GB/s of text",
            "cores": cpu_threads(), "kind": "port",
            "sample": "one %.0f MB block: line split %.2f s + parse %.2f s on %d threads "
                      "(shard_io.hpp's parser: std::stod's values, short decimals on an exact "
                      "fast path)" % (len(block) / 1e6, host[cpu_threads()][0],
                                      host[cpu_threads()][1], cpu_threads()),
            "value_1core": len(block) / sum(host[1]) / 1e9,
            "reference_stod_1core_gbs": len(sample) / stod_s / 1e9,
            "reference_stod_sample": "strtod per field as lr.cpp:76-93 does (oracle port), "
                                     "%.0f MB" % (len(sample) / 1e6)},
    }
    return out


def kernel_code(info):
    """'shard_pass<NCH=8,R=4,WCOL=1,WROW=4,ALLCH=1,TL=0> ...' -> 'shard_pass<8,4,1,4,1,0>' (+ what
    else distinguishes the variant: team shape, the constant column left on the host)."""
    import re

    m = re.match(r"(\w+)<([^>]*)>", info)
    code = info[:24] if not m else "%s<%s>" % (
        m.group(1), ",".join(v.split("=")[-1] for v in m.group(2).split(",")))
    t = re.search(r"(\d+) column blocks of (\d+-?) chunks", info)
    if t:
        code += " %sx%s" % (t.group(1), t.group(2))
    if "two sweeps" in info:
        code += " two-sweeps"
    if "not stored" in info:
        code += " col0-on-host"
    return code


# columns of the per_config / other_shapes rows
ROW_COLS = ["steps_per_s", "ms_per_step", "kernel_ms", "gb_per_s", "frac", "whole_step_frac",
            "read_probe_gb_per_s", "traffic_over_algorithmic", "cpu_steps_per_s_1core",
            "cpu_steps_per_s_16", "kernel"]


def compact_row(rec):
    """One bare-step record as a row of ROW_COLS."""
    r = rec["roofline"]
    c = rec["cpu_baseline"] or {}
    sig = lambda v, nd=4: None if v is None else float("%.*g" % (nd, v))  # noqa: E731
    return [sig(rec["value"]), sig(rec["ms_per_step"], 5), sig(r["kernel_ms"], 5),
            sig(r["achieved"]), sig(r["frac"]), sig(r["whole_step_frac"]),
            sig(r["read_probe_gbs"]),
            sig(r["traffic"] / r["algorithmic_bytes"], 5) if r["traffic"] else None,
            sig(c.get("value_1core"), 3), sig(c.get("value"), 3), rec["config"]["kernel"]]


def main():
    global KEEP_BIAS_COLUMN
    a = parse_args()
    KEEP_BIAS_COLUMN = a.keep_bias_column
    if a.gpus != 1:
        print("bench.py measures one GPU's shard: this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if a.ps_roundtrip:
        run_ps_roundtrip(a)
        return

    import numpy as np  # noqa: F401

    from paracel_amd.datagen import gen

    cfgs = gen.configs()
    name = a.workload or "c2_headline_1m_x_1000"
    if name not in cfgs:
        print("unknown workload %s; known: %s" % (name, ", ".join(cfgs)), file=sys.stderr)
        sys.exit(2)
    cfg = cfgs[name]
    if a.rows:
        cfg = cfg.scaled(a.rows)
    if a.e2e:
        rec = run_e2e(a, cfg, workers=a.workers)
        rec.pop("theta_cpu", None)
        print(json.dumps(rec), flush=True)
        return
    if a.train:
        run_train(a, cfg)
        return
    if a.parse:
        print(json.dumps(run_parse(a, cfg)), flush=True)
        return

    with_cpu = not a.no_cpu_baseline
    out = run_step(a, cfg, with_cpu, full_cpu_sample=(a.workload is None and not a.rows),
                   settle_ms=(a.settle_ms if a.workload is not None else 0.0))
    if a.workload is None:
        out.pop("kernel_info")  # (the long description: single-workload runs only)
    if a.workload is None and not a.headline_only and not a.rows:
        # Everything below rides in the same line, kept short: the harness keeps the tail of
        # what a run prints.  Rows of numbers under one list of column names.
        sig = lambda v, nd=4: None if v is None else float("%.*g" % (nd, v))  # noqa: E731
        out["row_cols"] = ROW_COLS
        # the other configurations, same steps / warmup, bounded CPU legs
        per = {}
        for other in PER_CONFIG:
            rec = run_step(a, cfgs[other], with_cpu, cpu_reps=(2, 6), settle_ms=a.settle_ms)
            per[other] = compact_row(rec)
        out["per_config"] = per
        # config 1 is an 80 MB shard (cache-resident): what its rounds cost end to end
        try:
            out["c1_latency_us"] = c1_latency(cfgs["c1_dense_100k_x_100"])
        except Exception as e:
            out["c1_latency_us"] = {"error": "%s: %s" % (type(e).__name__, e)}
        # config 5 as it is defined: 100 rounds through the parameter server -- by one worker,
        # and by 2 and 4 worker processes that share the GPU (n / W rows each)
        c5 = cfgs["c5_e2e_2m_x_512"]
        e2e = {"cols": ["workers", "iters_per_s", "ms_per_iter", "gpu_kernel_ms_per_iter",
                        "theta_rel_err_vs_cpu",
                        "worker0_ms:read,wait_for_gpu,pass,barrier,bupdate,barrier"],
               "rows": [], "rounds": 100}
        theta_cpu = None
        for W in (1, 2, 4):
            try:
                r = run_e2e(a, c5, rounds=100, workers=W, theta_cpu=theta_cpu)
                theta_cpu = r.pop("theta_cpu", theta_cpu)
                e2e["rows"].append([W, sig(r["value"]), sig(r["ms_per_step"]),
                                    sig(r["gpu_kernel_ms_per_iter"]),
                                    sig(r["theta_rel_err_vs_cpu"], 3),
                                    [round(v, 2) for v in r["worker0_phases_ms"] or []]])
                if W == 1:
                    e2e["final_loss"] = r["final_loss"]
                    e2e["cpu_iters_per_s"] = sig((r.get("cpu_baseline") or {}).get("value"))
                    e2e["cpu_cores"] = (r.get("cpu_baseline") or {}).get("cores")
            except Exception as e:
                e2e["rows"].append([W, "%s: %s" % (type(e).__name__, e)])
        out["c5_via_ps"] = e2e
        # the loader of the same configuration: its sample text parsed on the device
        try:
            pr = run_parse(a, c5)
            out["c5_text_to_shard"] = {
                "text_gb_per_s": sig(pr["value"]), "ms_per_call": sig(pr["ms_per_step"]),
                "text_bytes": pr["config"]["text_bytes"], "rows": pr["config"]["rows"],
                "parse_kernel_ms": sig(pr["roofline"]["kernel_ms"]),
                "parse_kernel_text_gb_per_s": sig(pr["roofline"]["text_gbs_kernel_only"]),
                "parse_kernel_frac_of_hbm": sig(pr["roofline"]["frac"]),
                "ms_per_call_transfer_then_parse": pr["config"]["ms_per_call_transfer_then_parse"],
                "cpu_text_gb_per_s_16": sig(pr["cpu_baseline"]["value"]),
                "cpu_text_gb_per_s_1core": sig(pr["cpu_baseline"]["value_1core"]),
                "reference_stod_1core_gb_per_s": sig(pr["cpu_baseline"]["reference_stod_1core_gbs"])}
        except Exception as e:
            out["c5_text_to_shard"] = {"error": "%s: %s" % (type(e).__name__, e)}
        extra = {}
        for other in OTHER_SHAPES:
            try:
                extra[other] = compact_row(run_step(a, cfgs[other], False, settle_ms=a.settle_ms))
            except Exception as e:  # the headline line must survive a shape that does not fit
                extra[other] = ["%s: %s" % (type(e).__name__, e)]
        out["other_shapes"] = extra
    print(json.dumps(out, separators=(",", ":")), flush=True)


def c1_latency(cfg):
    """Microseconds per call on the 100 000 x 100 shard, wall clock over 300 calls each:
    the bare step, the same with the timing events off, one round of plr_dgd_delta, and
    one device-resident round of plr_train_dgd (100 rounds per call)."""
    import numpy as np

    from paracel_amd import Plr

    with Plr(0) as ctx:
        X, y = cfg.rows(0, cfg.n)
        ctx.set_data(X, y)
        th = cfg.theta()

        def per_call(fn, reps=300):
            for _ in range(30):
                fn()
            t0 = time.perf_counter()
            for _ in range(reps):
                fn()
            return round((time.perf_counter() - t0) / reps * 1e6, 2)

        res = {"loss_grad": per_call(lambda: ctx.loss_grad(th))}
        ctx.set_timing(False)
        res["loss_grad_timing_off"] = per_call(lambda: ctx.loss_grad(th))
        res["dgd_delta_no_loss_timing_off"] = per_call(
            lambda: ctx.dgd_delta(th, cfg.alpha, cfg.beta, want_loss=False))
        z = np.zeros(cfg.d)
        ctx.train_dgd(z, cfg.alpha, cfg.beta, 100)
        t0 = time.perf_counter()
        for _ in range(10):
            ctx.train_dgd(z, cfg.alpha, cfg.beta, 100)
        res["train_dgd_per_round"] = round((time.perf_counter() - t0) / 1000 * 1e6, 2)
        ctx.set_timing(True)
    return res


if __name__ == "__main__":
    main()
