"""Pins the CPU oracle (oracle/lr_oracle.cpp) without the reference's help.

The reference has no test or fixture for its logistic-regression arithmetic,
so every oracle function is checked against what the mathematics fixes:
exact-rational / 60-digit golden values, closed forms, library routines and
invariants, chosen so that a dropped term, a flipped sign, a transposed
operand or a wrong index fails at least one of them.
"""
import json
import math
import os

import numpy as np
import pytest
from scipy.optimize import minimize
from scipy.special import expit

HERE = os.path.dirname(os.path.abspath(__file__))


def golden_cases():
    with open(os.path.join(HERE, "golden", "lr_small.json")) as f:
        return json.load(f)["cases"]


def rel(a, b):
    nb = np.linalg.norm(b)
    return np.linalg.norm(np.asarray(a) - np.asarray(b)) / (nb if nb > 0 else 1.0)


def rand_case(n, d, seed):
    rng = np.random.default_rng(seed)
    X = rng.normal(size=(n, d)) / np.sqrt(d)
    th = rng.normal(size=d)
    y = (rng.random(n) < expit(X @ th)).astype(float)
    return X, y, rng.normal(size=d)


@pytest.mark.parametrize("case", golden_cases(), ids=lambda c: c["name"])
def test_oracle_matches_golden(oracle, case):
    X, y, th = np.array(case["X"]), np.array(case["y"]), np.array(case["theta"])
    for i in range(case["n"]):
        assert abs(oracle.dot_product(X[i], th) - case["z"][i]) <= 1e-14 * max(1, abs(case["z"][i]))
        assert abs(oracle.lr_hypothesis(X[i], th) - case["h"][i]) <= 4e-16
    np.testing.assert_allclose(oracle.predict(X, th), case["h"], rtol=0, atol=4e-16)
    gs = np.array(case["gsum"])
    assert np.max(np.abs(oracle.gsum(X, y, th) - gs)) <= 1e-14 * max(1.0, np.max(np.abs(gs)))
    assert np.max(np.abs(oracle.gsum(X, y, th, hp=True) - gs)) <= 1e-15 * max(1.0, np.max(np.abs(gs)))
    assert abs(oracle.calc_loss_sum(X, y, th) - case["loss_sum"]) <= 1e-13 * abs(case["loss_sum"])
    mean = case["loss_sum"] / case["n"]
    assert abs(oracle.calc_loss(X, y, th) - mean) <= 1e-13 * max(1.0, mean)
    assert abs(oracle.calc_loss_sum_hp(X, y, th) - case["loss_sum"]) <= 1e-14 * abs(case["loss_sum"])
    assert abs(oracle.stable_loss_sum_hp(X, y, th) - case["loss_sum"]) <= 1e-14 * abs(case["loss_sum"])
    dl = np.array(case["delta"])
    got = oracle.dgd_delta(X, y, th, case["alpha"], case["beta"])
    assert np.max(np.abs(got - dl)) <= 1e-14 * max(1e-3, np.max(np.abs(dl)))
    got_hp = oracle.dgd_delta_hp(X, y, th, case["alpha"], case["beta"])
    assert np.max(np.abs(got_hp - dl)) <= 1e-15 * max(1e-3, np.max(np.abs(dl)))
    np.testing.assert_allclose(oracle.theta_update(th, got), case["theta_after_update"],
                               rtol=0, atol=1e-14)


def test_dot_product_is_strictly_sequential(oracle):
    # 1 + 2^-53 + 2^-53 ... left to right never leaves 1.0; any pairwise or
    # reversed order would (include/utils/ext_utility.hpp:171-174)
    a = np.array([1.0] + [2.0 ** -53] * 64)
    b = np.ones(65)
    assert oracle.dot_product(a, b) == 1.0
    assert oracle.dot_product(a[::-1].copy(), b) > 1.0
    assert oracle.dot_product(np.array([3.0, -2.0]), np.array([0.5, 4.0])) == -6.5


def test_hypothesis_closed_forms(oracle):
    one = np.ones(1)
    assert oracle.lr_hypothesis(np.zeros(1), one) == 0.5
    for z in (0.1, 1.0, 5.0, 20.0):
        hp, hm = oracle.lr_hypothesis(np.array([z]), one), oracle.lr_hypothesis(np.array([-z]), one)
        assert abs(hp + hm - 1.0) <= 3e-16                       # h(-z) = 1 - h(z)
        assert abs(hp - expit(z)) <= 3e-16
    # saturation points of the unclamped formula (lr.cpp:71)
    assert oracle.lr_hypothesis(np.array([37.0]), one) == 1.0     # exp(-z) < 2^-53
    assert oracle.lr_hypothesis(np.array([-800.0]), one) == 0.0   # exp overflows to inf
    assert 0.0 < oracle.lr_hypothesis(np.array([-700.0]), one) < 1e-300
    zs = np.linspace(-30, 30, 301)
    hs = np.array([oracle.lr_hypothesis(np.array([z]), one) for z in zs])
    assert np.all(np.diff(hs) >= 0)


def test_theta_zero_closed_forms(oracle):
    X, y, _ = rand_case(400, 13, 1)
    th = np.zeros(13)
    np.testing.assert_allclose(oracle.gsum(X, y, th), X.T @ (0.5 - y), rtol=1e-13, atol=1e-13)
    assert abs(oracle.calc_loss(X, y, th) - math.log(2.0)) <= 1e-14   # ln 2 whatever the labels
    alpha, beta = 0.01, 0.3
    # theta = 0 kills the L2 term: delta = alpha X^T (y - 1/2)
    np.testing.assert_allclose(oracle.dgd_delta(X, y, th, alpha, beta), alpha * (X.T @ (y - 0.5)),
                               rtol=1e-12, atol=1e-14)


def test_gsum_equals_numpy_gemv(oracle):
    X, y, th = rand_case(300, 40, 2)
    want = X.T @ (expit(X @ th) - y)
    assert rel(oracle.gsum(X, y, th), want) <= 1e-13
    assert rel(oracle.gsum(X, y, th, hp=True), want) <= 1e-13
    # a transposed operand or (y - h) sign would fail here
    assert rel(oracle.gsum(X, y, th), -want) > 1.0


def test_delta_formula_sign_scale_and_l2(oracle):
    X, y, th = rand_case(250, 9, 3)
    n = X.shape[0]
    alpha, beta = 0.003, 0.07
    g = X.T @ (expit(X @ th) - y)
    want = -alpha * g - 2 * alpha * beta * n * th      # L2 applied once per sample (lr.cpp:136)
    got = oracle.dgd_delta(X, y, th, alpha, beta)
    assert rel(got, want) <= 1e-12
    # X = 0: pure L2, exactly n additions of -coff2*theta
    got0 = oracle.dgd_delta(np.zeros_like(X), y, th, alpha, beta)
    np.testing.assert_allclose(got0, -2 * alpha * beta * n * th, rtol=1e-13)
    # linear in alpha at beta = 0
    a1 = oracle.dgd_delta(X, y, th, alpha, 0.0)
    a2 = oracle.dgd_delta(X, y, th, 2 * alpha, 0.0)
    np.testing.assert_allclose(a2, 2 * a1, rtol=1e-15, atol=0)   # doubling is exact
    # traversal order only moves rounding
    order = np.random.default_rng(0).permutation(n)
    assert rel(oracle.dgd_delta(X, y, th, alpha, beta, order=order), got) <= 1e-13
    assert rel(oracle.dgd_delta_hp(X, y, th, alpha, beta), got) <= 1e-13


def test_one_hot_rows(oracle):
    n, d = 200, 11
    rng = np.random.default_rng(4)
    cols = rng.integers(0, d, n)
    X = np.zeros((n, d))
    X[np.arange(n), cols] = 1.0
    y = (rng.random(n) < 0.5).astype(float)
    th = rng.normal(size=d)
    want = np.zeros(d)
    np.add.at(want, cols, expit(th[cols]) - y)
    np.testing.assert_allclose(oracle.gsum(X, y, th), want, rtol=1e-13, atol=1e-14)


def test_shard_additivity(oracle):
    X, y, th = rand_case(500, 20, 5)
    g = oracle.gsum(X, y, th)
    g1, g2 = oracle.gsum(X[:123], y[:123], th), oracle.gsum(X[123:], y[123:], th)
    assert rel(g1 + g2, g) <= 1e-14
    l = oracle.calc_loss_sum(X, y, th)
    assert abs(oracle.calc_loss_sum(X[:123], y[:123], th) + oracle.calc_loss_sum(X[123:], y[123:], th) - l) <= 1e-12 * l


def test_loss_closed_forms_and_symmetry(oracle):
    # n = 1, d = 1
    for z, lab in ((0.7, 1.0), (0.7, 0.0), (-2.5, 1.0), (3.0, 0.0)):
        got = oracle.calc_loss_sum(np.array([[z]]), np.array([lab]), np.ones(1))
        want = math.log1p(math.exp(-z)) if lab == 1.0 else math.log1p(math.exp(z))
        # -log(1-h) amplifies the rounding of h by 1/(1-h) (~21 at z=3)
        assert abs(got - want) <= 1e-14 * max(1, want)
    # l(z, 1) = l(-z, 0)
    X, y, th = rand_case(100, 6, 6)
    a = oracle.calc_loss_sum(X, np.ones(100), th)
    b = oracle.calc_loss_sum(-X, np.zeros(100), th)
    assert abs(a - b) <= 1e-13 * a
    # no L2 term in the loss (lr.cpp:322-330): scaling beta is not even an input;
    # any label other than exactly 1.0 is class 0
    y2 = y.copy()
    y2[y2 == 0.0] = 0.5
    assert oracle.calc_loss_sum(X, y2, th) == oracle.calc_loss_sum(X, y, th)
    # naive and stable forms agree for |z| <= 10
    Xs = np.linspace(-10, 10, 81).reshape(-1, 1)
    ys = (np.arange(81) % 2).astype(float)
    n1, s1 = oracle.calc_loss_sum(Xs, ys, np.ones(1)), oracle.stable_loss_sum_hp(Xs, ys, np.ones(1))
    assert abs(n1 - s1) <= 1e-12 * s1   # 1-h loses relative accuracy near h=1: 1e-12, not 1e-15
    # the naive formula overflows for a mislabelled saturated row, the stable one does not
    assert math.isinf(oracle.calc_loss_sum(np.array([[40.0]]), np.zeros(1), np.ones(1)))
    assert abs(oracle.stable_loss_sum_hp(np.array([[40.0]]), np.zeros(1), np.ones(1)) - 40.0) <= 1e-14


def test_ridge_pieces_against_numpy(oracle):
    # ridge.hpp:103-109,130-139: squared residuals and the linear prediction
    X, _, th = rand_case(300, 17, 11)
    y = np.random.default_rng(12).normal(size=300)
    z = X @ th
    np.testing.assert_allclose(oracle.predict_linear(X, th), z, rtol=1e-13, atol=1e-14)
    assert abs(oracle.ridge_loss_sum(X, y, th) - np.sum((z - y) ** 2)) <= 1e-12 * np.sum((z - y) ** 2)
    assert rel(oracle.lsq_gsum(X, y, th), X.T @ (z - y)) <= 1e-13
    # exact closed forms: theta = 0 -> loss = sum y^2, gsum = -X^T y; y = X theta -> 0
    assert abs(oracle.ridge_loss_sum(X, y, np.zeros(17)) - np.sum(y * y)) <= 1e-12 * np.sum(y * y)
    assert rel(oracle.lsq_gsum(X, y, np.zeros(17)), -(X.T @ y)) <= 1e-13
    assert oracle.ridge_loss_sum(X, oracle.predict_linear(X, th), th) == 0.0


def test_ridge_batch_delta_and_training(oracle):
    # the batch form of ridge.hpp:79-84: delta = alpha X^T(y - X theta) - 2 alpha beta n theta
    X, _, th = rand_case(400, 13, 21)
    y = np.random.default_rng(22).normal(size=400)
    n = 400
    alpha, beta = 3.0 / n, 0.02
    want = alpha * (X.T @ (y - X @ th)) - 2 * alpha * beta * n * th
    assert rel(oracle.ridge_delta(X, y, th, alpha, beta), want) <= 1e-13
    # X = 0: only the L2 term, n times; theta = 0: only the data term
    assert rel(oracle.ridge_delta(np.zeros((50, 13)), y[:50], th, alpha, beta),
               -2 * alpha * beta * 50 * th) <= 1e-14
    assert rel(oracle.ridge_delta(X, y, np.zeros(13), alpha, beta), alpha * (X.T @ y)) <= 1e-13
    # a dropped sign or a transposed operand fails this: delta vanishes exactly at the ridge
    # solution (X^T X + 2 beta n I) theta = X^T y, and training contracts towards it
    star = np.linalg.solve(X.T @ X + 2 * beta * n * np.eye(13), X.T @ y)
    assert np.linalg.norm(oracle.ridge_delta(X, y, star, alpha, beta)) <= 1e-13
    t = oracle.ridge_train_workers(X, y, np.zeros(13), alpha, beta, 400, 1)
    assert rel(t, star) <= 1e-9
    # shards add up: W workers give the single worker's theta to rounding
    for w in (2, 3, 7):
        assert rel(oracle.ridge_train_workers(X, y, np.zeros(13), alpha, beta, 25, w),
                   oracle.ridge_train_workers(X, y, np.zeros(13), alpha, beta, 25, 1)) <= 1e-13


def test_theta_update_is_elementwise_add(oracle):
    a, b = np.array([1.23, -4.0, 1e300]), np.array([3.21, 4.0, 1e300])
    np.testing.assert_array_equal(oracle.theta_update(a, b), a + b)   # test_proxy.cpp:45-54: 1.23+3.21


def test_training_reaches_the_regularised_optimum(oracle):
    # alpha = lr/n, beta = lam/2 makes the reference update plain gradient descent on
    # mean log-loss + (lam/2)|theta|^2; its fixed point satisfies (1/n)X^T(h-y) + lam theta = 0
    X, y, _ = rand_case(2000, 8, 7)
    X = X * np.sqrt(8)
    n, lam, lr = X.shape[0], 0.05, 1.0
    th = oracle.train_dgd(X, y, np.zeros(8), lr / n, lam / 2, 600)

    def f(t):
        z = X @ t
        return np.mean(np.logaddexp(0, z) - y * z) + 0.5 * lam * t @ t

    def g(t):
        return X.T @ (expit(X @ t) - y) / n + lam * t

    opt = minimize(f, np.zeros(8), jac=g, method="BFGS", options={"gtol": 1e-12})
    assert np.linalg.norm(g(th)) <= 1e-9
    assert rel(th, opt.x) <= 1e-7
    # one round equals delta followed by the server-side add (update.cpp:26-32)
    t1 = oracle.train_dgd(X, y, th, lr / n, lam / 2, 1)
    np.testing.assert_array_equal(t1, oracle.theta_update(th, oracle.dgd_delta(X, y, th, lr / n, lam / 2)))


def test_multi_worker_training_matches_single_worker(oracle):
    # P workers + server-side folding only regroups the sums (shard additivity)
    X, y, _ = rand_case(3000, 12, 9)
    n = X.shape[0]
    t1 = oracle.train_dgd(X, y, np.zeros(12), 0.5 / n, 0.01, 30)
    assert np.array_equal(t1, oracle.train_dgd_workers(X, y, np.zeros(12), 0.5 / n, 0.01, 30, 1))
    t4 = oracle.train_dgd_workers(X, y, np.zeros(12), 0.5 / n, 0.01, 30, 4)
    assert rel(t4, t1) <= 1e-13


def test_local_parser(oracle):
    # lr.cpp:76-93: "f1,...,fk,label" -> [1.0, f1..fk], label; empty fields are dropped
    X, y = oracle.local_parser("0.5,2,1\n-1e-3,4.25,0\n")
    np.testing.assert_array_equal(X, [[1.0, 0.5, 2.0], [1.0, -1e-3, 4.25]])
    np.testing.assert_array_equal(y, [1.0, 0.0])
    X, y = oracle.local_parser("3,,7,1")        # str_split skips the empty token
    np.testing.assert_array_equal(X, [[1.0, 3.0, 7.0]])
    with pytest.raises(ValueError):
        oracle.local_parser("1,2,1\n1,1\n")     # ragged
    with pytest.raises(ValueError):
        oracle.local_parser("1,abc,1\n")        # std::stod would throw
    X, y = oracle.local_parser("1|2|0", sep="|")
    np.testing.assert_array_equal(X, [[1.0, 1.0, 2.0]])


def test_baseline_timer_computes_the_same_delta(oracle):
    X, y, th = rand_case(1000, 30, 8)
    want = oracle.dgd_delta(X, y, th, 0.01, 0.02)
    sec, d1, ls, lv = oracle.baseline_time(X, y, th, 0.01, 0.02, threads=1, reps=1)
    np.testing.assert_array_equal(d1, want)           # same instruction stream, same bits
    assert lv == oracle.calc_loss_sum(X, y, th) and sec > 0 and ls > 0
    _, d4, _, lv4 = oracle.baseline_time(X, y, th, 0.01, 0.02, threads=4, reps=2)
    assert rel(d4, want) <= 1e-13 and abs(lv4 - lv) <= 1e-12 * lv
