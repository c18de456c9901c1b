"""The HIP path against the committed golden vectors (exact-rational / 60-digit
expected values, tests/golden/make_golden.py)."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def golden_cases():
    with open(os.path.join(HERE, "golden", "lr_small.json")) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", golden_cases(), ids=lambda c: c["name"])
def test_hip_matches_golden(plr, case):
    X, y, th = np.array(case["X"]), np.array(case["y"]), np.array(case["theta"])
    plr.set_data(X, y)
    g, loss, n = plr.loss_grad(th)
    gs = np.array(case["gsum"])
    assert n == case["n"]
    assert np.max(np.abs(g - gs)) <= 1e-13 * max(1.0, np.max(np.abs(gs)))
    assert abs(loss - case["loss_sum"]) <= 1e-12 * abs(case["loss_sum"])
    loss_s, _ = plr.calc_loss(th, 1)
    assert abs(loss_s - case["loss_sum"]) <= 1e-13 * abs(case["loss_sum"])
    np.testing.assert_allclose(plr.predict(th), case["h"], rtol=0, atol=5e-16)
    delta, _ = plr.dgd_delta(th, case["alpha"], case["beta"])
    dl = np.array(case["delta"])
    assert np.max(np.abs(delta - dl)) <= 1e-13 * max(1e-3, np.max(np.abs(dl)))
    np.testing.assert_allclose(th + delta, case["theta_after_update"], rtol=0, atol=1e-13)


def test_plain_c_caller_on_a_golden_case(tmp_path):
    """plr_create -> plr_set_data -> plr_dgd_delta from a C99 program (no Python, no C++ on the
    caller's side) on the golden case with a bias column."""
    import subprocess

    tool = os.path.join(os.path.dirname(HERE), "paracel_amd", "plr_c_caller")
    assert os.path.exists(tool), "plr_c_caller is not built (__graft_entry__.build())"
    case = [c for c in golden_cases() if c["name"] == "n17_d5_bias"][0]
    inp = tmp_path / "in.txt"
    with open(inp, "w") as f:
        f.write("%d %d %.17g %.17g\n" % (case["n"], case["d"], case["alpha"], case["beta"]))
        for row in case["X"]:
            f.write(" ".join("%.17g" % v for v in row) + "\n")
        f.write(" ".join("%.17g" % v for v in case["y"]) + "\n")
        f.write(" ".join("%.17g" % v for v in case["theta"]) + "\n")
    r = subprocess.run([tool, str(inp)], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    delta = np.array([float(l.split("=")[1]) for l in lines if l.startswith("delta[")])
    loss = float([l for l in lines if l.startswith("loss_sum")][0].split("=")[1])
    dl = np.array(case["delta"])
    assert delta.shape == dl.shape
    assert np.max(np.abs(delta - dl)) <= 1e-13 * max(1e-3, np.max(np.abs(dl)))
    assert abs(loss - case["loss_sum"]) <= 1e-12 * abs(case["loss_sum"])
    assert lines[-1].startswith("plr ")
