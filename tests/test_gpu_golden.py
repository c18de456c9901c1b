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
