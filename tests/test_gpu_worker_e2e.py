"""End to end through the host parameter server: the C++ worker
(paracel_amd/worker, same call order as the reference's dgd_learning) reads
theta over ZeroMQ, computes delta on the GPU through the C ABI and pushes it
with paracel_bupdate into a server process whose reducer is the dlopen'ed
lr_theta_update plugin.  The final theta is compared with the CPU oracle's
training loop (tool/lr_serial.cpp:95-110 restated) on the same seeded data:
relative error <= 1e-8 after 100 iterations.
"""
import json
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "paracel_amd")


def rel(a, b):
    return np.linalg.norm(a - b) / np.linalg.norm(b)


@pytest.fixture()
def server_info():
    for f in ("plr_ps_server", "plr_lr_worker", "liblr_update.so"):
        assert os.path.exists(os.path.join(PKG, f)), "%s is not built" % f
    p = subprocess.Popen([os.path.join(PKG, "plr_ps_server")], stdout=subprocess.PIPE, text=True)
    info = p.stdout.readline().strip()
    yield info
    p.kill()
    p.wait()


def test_synthetic_100_rounds_match_oracle(server_info, oracle, gen, tmp_path):
    n, d, rounds = 20000, 512, 100
    cfg = gen.configs()["c5_e2e_2m_x_512"].scaled(n)
    alpha, beta = cfg.lr / n, cfg.lam / 2
    out = tmp_path / "theta.bin"
    cmd = [os.path.join(PKG, "plr_lr_worker"), "--server_info", server_info,
           "--synthetic", "%x,%d,%d,%.17g" % (cfg.seed, n, d, cfg.spec.scale),
           "--rounds", str(rounds), "--alpha", "%.17g" % alpha, "--beta", "%.17g" % beta,
           "--theta0", "zero", "--update_file", os.path.join(PKG, "liblr_update.so"),
           "--theta_out", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    rep = json.loads(r.stdout.strip().splitlines()[-1])
    print(rep)
    theta = np.fromfile(out)
    X, y = cfg.rows(0, n)
    theta_ref = oracle.train_dgd(X, y, np.zeros(d), alpha, beta, rounds)
    assert theta.shape == (d,)
    assert rel(theta, theta_ref) <= 1e-8
    assert abs(rep["final_loss"] - oracle.calc_loss(X, y, theta_ref)) <= 1e-10
    assert rep["rounds"] == rounds and rep["iters_per_sec"] > 0


def test_csv_driver_follows_the_reference_call_order(server_info, oracle, tmp_path):
    # training file "f1,...,fk,label" (lr.cpp:74-75), cfg keys of lr_driver.cpp:45-59
    rng = np.random.default_rng(3)
    n, k = 400, 6
    F = np.round(rng.normal(size=(n, k)), 4)
    lab = (rng.random(n) < 0.5).astype(int)
    train = tmp_path / "train.csv"
    with open(train, "w") as f:
        for i in range(n):
            f.write(",".join("%.4f" % v for v in F[i]) + ",%d\n" % lab[i])
    outdir = tmp_path / "out"
    cfgf = tmp_path / "cfg.json"
    cfgf.write_text(json.dumps({
        "training_input": str(train), "test_input": str(train), "predict_input": str(train),
        "output": str(outdir) + "/", "update_file": os.path.join(PKG, "liblr_update.so"),
        "update_func": "lr_theta_update", "method": "dgd", "rounds": 20,
        "alpha": 0.001, "beta": 0.01, "debug": True}, indent=2))
    r = subprocess.run([os.path.join(PKG, "plr_lr_worker"), "--server_info", server_info,
                        "--cfg_file", str(cfgf), "--theta0", "zero"],
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    X = np.hstack([np.ones((n, 1)), F])          # bias column first (lr.cpp:83)
    y = lab.astype(float)
    theta_ref = oracle.train_dgd(X, y, np.zeros(k + 1), 0.001, 0.01, 20)
    # lr_theta_<rank>: std::to_string (6 decimals) joined by '|' (lr.cpp:340, ps.hpp:1308)
    dumped = np.array([float(t) for t in (outdir / "lr_theta_0").read_text().strip().split("|")])
    np.testing.assert_allclose(dumped, theta_ref, atol=5.1e-7, rtol=0)
    loss_line = [ln for ln in r.stdout.splitlines() if ln.startswith("final loss:")][0]
    assert abs(float(loss_line.split(":")[1]) - oracle.calc_loss(X, y, theta_ref)) <= 1e-10
    assert "loss in test dataset is:" in r.stdout
    # pred_v_<rank>: "x0,x1,...,xk:h" per sample (lr.cpp:346, ps.hpp:1312-1319)
    plines = (outdir / "pred_v_0").read_text().splitlines()
    assert len(plines) == n
    pred = np.array([float(l.split(":")[1]) for l in plines])
    np.testing.assert_allclose(pred, oracle.predict(X, theta_ref), atol=5.1e-7, rtol=0)
    xs = np.array([[float(t) for t in l.split(":")[0].split(",")] for l in plines])
    np.testing.assert_allclose(xs, X, atol=5.1e-7, rtol=0)
    # debug: the loss after every sample of every round (lr.cpp:139-141, 341-343) -- n equal
    # entries per round, the mean loss at the theta read at the start of that round
    curve = np.array([float(t) for t in (outdir / "lr_loss_error_0").read_text().split()])
    assert curve.shape == (20 * n,)
    per_round = curve.reshape(20, n)
    assert np.all(per_round == per_round[:, :1])
    assert abs(per_round[0, 0] - np.log(2)) < 1e-6 and per_round[-1, 0] < per_round[0, 0]
    th = np.zeros(k + 1)
    for rd in range(20):
        assert abs(per_round[rd, 0] - oracle.calc_loss(X, y, th)) <= 5.1e-7
        th = th + oracle.dgd_delta(X, y, th, 0.001, 0.01)

    # the first run parsed the training text on the device and wrote the binary shard cache
    assert "parsed on the device: 400 x 7" in r.stdout and "lines got: 400" in r.stdout
    # second run: the text is not parsed again (binary shard cache), same result
    # (in the first run only test(), which re-reads the training file, found the cache)
    assert r.stdout.count("shard cache hit") == 1
    outdir2 = tmp_path / "out2"
    cfg2 = json.loads(cfgf.read_text())
    cfg2["output"] = str(outdir2) + "/"
    cfgf.write_text(json.dumps(cfg2))
    r2 = subprocess.run([os.path.join(PKG, "plr_lr_worker"), "--server_info", server_info,
                         "--cfg_file", str(cfgf), "--theta0", "zero"],
                        capture_output=True, text=True, timeout=110)
    assert r2.returncode == 0, r2.stderr
    assert r2.stdout.count("shard cache hit: 400 x 7") == 2
    assert (outdir2 / "lr_theta_0").read_text() == (outdir / "lr_theta_0").read_text()
    # third run, no cache and the host's parser: the same bytes in every output file
    os.remove(str(train) + ".plrshard.0of1")
    outdir3 = tmp_path / "out3"
    cfg2["output"] = str(outdir3) + "/"
    cfgf.write_text(json.dumps(cfg2))
    r3 = subprocess.run([os.path.join(PKG, "plr_lr_worker"), "--server_info", server_info,
                         "--cfg_file", str(cfgf), "--theta0", "zero"],
                        capture_output=True, text=True, timeout=110,
                        env=dict(os.environ, PLR_HOST_PARSE="1"))
    assert r3.returncode == 0, r3.stderr
    assert "parsed on the device" not in r3.stdout
    for name in ("lr_theta_0", "pred_v_0", "lr_loss_error_0"):
        assert (outdir3 / name).read_text() == (outdir / name).read_text()


def test_config_5_at_full_size_through_the_server(server_info, oracle, gen, tmp_path):
    # benchmark configuration 5 as it is defined: 2 000 000 x 512, 100 rounds of paracel_read ->
    # GPU delta -> paracel_bupdate; theta against the CPU oracle's 16-worker training
    cfg = gen.configs()["c5_e2e_2m_x_512"]
    n, d, rounds = cfg.n, cfg.d, 100
    out = tmp_path / "theta.bin"
    cmd = [os.path.join(PKG, "plr_lr_worker"), "--server_info", server_info,
           "--synthetic", "%x,%d,%d,%.17g" % (cfg.seed, n, d, cfg.spec.scale),
           "--rounds", str(rounds), "--alpha", "%.17g" % cfg.alpha, "--beta", "%.17g" % cfg.beta,
           "--theta0", "zero", "--update_file", os.path.join(PKG, "liblr_update.so"),
           "--theta_out", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    rep = json.loads(r.stdout.strip().splitlines()[-1])
    print(rep, flush=True)
    theta = np.fromfile(out)
    X = np.empty((n, d))
    y = np.empty(n)
    for lo in range(0, n, 262144):
        m = min(262144, n - lo)
        _, y[lo:lo + m] = cfg.rows(lo, m, out=X[lo:lo + m])
    theta_ref = oracle.train_dgd_workers(X, y, np.zeros(d), cfg.alpha, cfg.beta, rounds, 16)
    err = rel(theta, theta_ref)
    print("config 5 full size: theta rel err %.3e, %.1f iterations/s" %
          (err, rep["iters_per_sec"]), flush=True)
    assert err <= 1e-8
    assert abs(rep["final_loss"] - oracle.calc_loss(X, y, theta_ref)) <= 1e-10


def _write_csv(path, F, target, fmt="%.6f"):
    with open(path, "w") as f:
        for i in range(F.shape[0]):
            f.write(",".join(fmt % v for v in F[i]) + "," + target[i] + "\n")


@pytest.mark.parametrize("W", [2, 4])
def test_several_workers_share_the_gpu_and_the_server(server_info, oracle, tmp_path, W):
    # the reference's `mpirun -n W bin/lr`: W worker processes, each with its byte range of
    # one CSV (partition.hpp:57-86) as a shard of its own on the one GPU, one server adding
    # their deltas (update.cpp:26-32); paracel_sync is a real barrier, calc_loss a real
    # all-reduce (lr.cpp:143-145, 331-335)
    rng = np.random.default_rng(40 + W)
    n, k, rounds = 3001, 9, 20
    F = np.round(rng.normal(size=(n, k)), 5)
    lab = (rng.random(n) < 0.5).astype(int)
    train = tmp_path / "train.csv"
    _write_csv(train, F, [str(v) for v in lab], "%.5f")
    cfgf = tmp_path / "cfg.json"
    cfgf.write_text(json.dumps({
        "training_input": str(train), "test_input": "", "predict_input": "",
        "output": str(tmp_path / "out") + "/", "update_file": os.path.join(PKG, "liblr_update.so"),
        "update_func": "lr_theta_update", "method": "dgd", "rounds": rounds,
        "alpha": 0.1 / n, "beta": 0.005, "debug": False}))
    procs = []
    for r in range(W):
        cmd = [os.path.join(PKG, "plr_lr_worker"), "--server_info", server_info, "--cfg_file",
               str(cfgf), "--theta0", "zero", "--worker_id", str(r), "--worker_sz", str(W),
               "--theta_out", str(tmp_path / "theta.bin")]
        procs.append(subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                                      text=True))
    outs = []
    for p in procs:
        try:
            o, e = p.communicate(timeout=100)
        except subprocess.TimeoutExpired:
            for q in procs:
                q.kill()
            raise
        assert p.returncode == 0, e
        outs.append(o)
    X = np.hstack([np.ones((n, 1)), F])
    y = lab.astype(float)
    theta_ref = oracle.train_dgd_workers(X, y, np.zeros(k + 1), 0.1 / n, 0.005, rounds, W)
    theta = np.fromfile(tmp_path / "theta.bin")
    assert rel(theta, theta_ref) <= 1e-8
    # every worker reports the GLOBAL mean loss, and owns a different share of the lines
    want = oracle.calc_loss(X, y, theta_ref)
    got_lines = 0
    for o in outs:
        loss_line = [ln for ln in o.splitlines() if ln.startswith("final loss:")][0]
        assert abs(float(loss_line.split(":")[1]) - want) <= 1e-10
        got_lines += int([ln for ln in o.splitlines() if ln.startswith("lines got:")][0].split(":")[1])
        assert o.count("finished round:") == rounds
    assert got_lines == n


def test_two_workers_with_rows_wider_than_one_workgroup_holds(server_info, oracle, tmp_path):
    # 20 000 features + bias: past 19 456 stored columns a row is shared by several
    # workgroups, all of which must be resident at once.  Two processes on one GPU cannot
    # count on that, so the workers take turns at the device (a pass at a time), and a pass
    # that still finds compute units taken runs again in two sweeps
    # (lr.cpp:143-145, update.cpp:26-32, prun.py:169-172: mpirun -n W)
    W, n, k, rounds = 2, 600, 20000, 20
    rng = np.random.default_rng(2026)
    F = np.round(rng.normal(size=(n, k)) / np.sqrt(k), 6)
    lab = (rng.random(n) < 0.5).astype(int)
    train = tmp_path / "wide.csv"
    np.savetxt(train, np.hstack([F, lab[:, None]]), fmt=["%.6f"] * k + ["%d"], delimiter=",")
    cfgf = tmp_path / "cfg.json"
    cfgf.write_text(json.dumps({
        "training_input": str(train), "test_input": "", "predict_input": "",
        "output": str(tmp_path / "out") + "/", "update_file": os.path.join(PKG, "liblr_update.so"),
        "update_func": "lr_theta_update", "method": "dgd", "rounds": rounds,
        "alpha": 0.5 / n, "beta": 0.005, "debug": False}))
    procs = []
    for r in range(W):
        cmd = [os.path.join(PKG, "plr_lr_worker"), "--server_info", server_info, "--cfg_file",
               str(cfgf), "--theta0", "zero", "--worker_id", str(r), "--worker_sz", str(W),
               "--theta_out", str(tmp_path / "theta.bin")]
        procs.append(subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                                      text=True))
    outs = []
    for p in procs:
        try:
            o, e = p.communicate(timeout=100)
        except subprocess.TimeoutExpired:
            for q in procs:
                q.kill()
            raise
        assert p.returncode == 0, e
        outs.append(o)
    X = np.hstack([np.ones((n, 1)), F])
    y = lab.astype(float)
    theta_ref = oracle.train_dgd_workers(X, y, np.zeros(k + 1), 0.5 / n, 0.005, rounds, W)
    theta = np.fromfile(tmp_path / "theta.bin")
    assert theta.shape == (k + 1,) and rel(theta, theta_ref) <= 1e-8
    want = oracle.calc_loss(X, y, theta_ref)
    for o in outs:
        assert "team_pass" in o, o[-2000:]
        loss_line = [ln for ln in o.splitlines() if ln.startswith("final loss:")][0]
        assert abs(float(loss_line.split(":")[1]) - want) <= 1e-10
        assert o.count("finished round:") == rounds


def test_ridge_worker_end_to_end(server_info, oracle, tmp_path):
    # cfg keys and call order of ridge_driver.cpp:29-73; the batch trainer against the
    # oracle's batch form of ridge.hpp:79-84, loss / predictions against ridge.hpp:103-139
    for f in ("plr_ridge_worker",):
        assert os.path.exists(os.path.join(PKG, f)), "%s is not built" % f
    rng = np.random.default_rng(77)
    n, k, rounds = 1500, 80, 30
    F = np.round(rng.normal(size=(n, k)) / np.sqrt(k), 5)
    w = rng.normal(size=k)
    t = np.round(F @ w + 0.3 + 0.1 * rng.normal(size=n), 5)
    train = tmp_path / "train.csv"
    _write_csv(train, F, ["%.5f" % v for v in t], "%.5f")
    test = tmp_path / "test.csv"
    _write_csv(test, F[:200], ["%.5f" % v for v in t[:200]], "%.5f")
    outdir = tmp_path / "out"
    alpha, beta = 1.0 / n, 0.001
    cfgf = tmp_path / "cfg.json"
    cfgf.write_text(json.dumps({
        "training_input": str(train), "test_input": str(test), "predict_input": str(test),
        "output": str(outdir) + "/", "update_file": os.path.join(PKG, "liblr_update.so"),
        "update_func": "lr_theta_update", "rounds": rounds, "alpha": alpha, "beta": beta}))
    r = subprocess.run([os.path.join(PKG, "plr_ridge_worker"), "--server_info", server_info,
                        "--cfg_file", str(cfgf), "--theta0", "zero", "--theta_out",
                        str(tmp_path / "theta.bin")], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    X = np.hstack([np.ones((n, 1)), F])
    theta_ref = oracle.ridge_train_workers(X, t, np.zeros(k + 1), alpha, beta, rounds, 1)
    theta = np.fromfile(tmp_path / "theta.bin")
    assert rel(theta, theta_ref) <= 1e-8
    loss_line = [ln for ln in r.stdout.splitlines() if ln.startswith("final loss:")][0]
    want = oracle.ridge_loss_sum(X, t, theta_ref) / n
    assert abs(float(loss_line.split(":")[1]) - want) <= 1e-10 * want
    tl = [ln for ln in r.stdout.splitlines() if ln.startswith("loss in test dataset is:")][0]
    want_t = oracle.ridge_loss_sum(X[:200], t[:200], theta_ref) / 200
    assert abs(float(tl.split(":")[1]) - want_t) <= 2e-6 * want_t   # printed with 6 digits
    dumped = np.array([float(v) for v in (outdir / "ridge_theta_0").read_text().strip().split("|")])
    np.testing.assert_allclose(dumped, theta_ref, atol=5.1e-7, rtol=0)
    plines = (outdir / "pred_v_0").read_text().splitlines()
    assert len(plines) == 200
    pred = np.array([float(l.split(":")[1]) for l in plines])
    np.testing.assert_allclose(pred, oracle.predict_linear(X[:200], theta_ref), atol=5.1e-7, rtol=0)
