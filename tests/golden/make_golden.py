#!/usr/bin/env python3
"""Writes tests/golden/lr_small.json: small logistic-regression cases with
expected values computed independently of both the oracle and the HIP path.

The reference ships no fixture for this path, so the expected values come from
the mathematics: dot products in exact rational arithmetic (fractions.Fraction
over the exact binary values of the doubles), exp/log in 60-digit decimal
arithmetic, one final rounding to double.  Inputs are drawn from Python's
Mersenne Twister with fixed seeds and rounded to a few bits so that they are
exactly representable and the file stays small.

Run from the repo root:  python tests/golden/make_golden.py
"""
import json
import os
import random
from decimal import Decimal, getcontext
from fractions import Fraction

getcontext().prec = 60


def dec(fr):
    return Decimal(fr.numerator) / Decimal(fr.denominator)


def case(name, n, d, seed, xs=1.0, ts=1.0, alpha=0.01, beta=0.05, special=None):
    rnd = random.Random(seed)
    q = 1 << 10
    X = [[round(rnd.uniform(-xs, xs) * q) / q for _ in range(d)] for _ in range(n)]
    theta = [round(rnd.uniform(-ts, ts) * q) / q for _ in range(d)]
    y = [float(rnd.random() < 0.5) for _ in range(n)]
    if special == "bias":
        for r in X:
            r[0] = 1.0
    if special == "zero_theta":
        theta = [0.0] * d
    if special == "odd_labels":
        y = [[0.0, 1.0, 0.5, -1.0, 2.0][i % 5] for i in range(n)]
    Xf = [[Fraction(v) for v in r] for r in X]
    tf = [Fraction(v) for v in theta]
    z = [sum(a * b for a, b in zip(r, tf)) for r in Xf]            # exact
    h = [Decimal(1) / (Decimal(1) + (-dec(zi)).exp()) for zi in z]  # 60 digits
    res = [hi - Decimal(yi) for hi, yi in zip(h, y)]
    gsum = [sum(res[i] * dec(Xf[i][j]) for i in range(n)) for j in range(d)]
    # lr.cpp:325-329: label == 1.0 exactly selects -log(h), anything else -log(1-h)
    loss = sum(-(hi.ln()) if yi == 1.0 else -((Decimal(1) - hi).ln()) for hi, yi in zip(h, y))
    A, B = Decimal(alpha), Decimal(beta)
    # lr.cpp:119,134-137: delta_j = sum_i (alpha (y_i - h_i) x_ij - 2 beta alpha theta_j)
    delta = [-A * gsum[j] - Decimal(2) * B * A * n * dec(tf[j]) for j in range(d)]
    return {
        "name": name, "n": n, "d": d, "alpha": alpha, "beta": beta,
        "X": X, "y": y, "theta": theta,
        "z": [float(dec(v)) for v in z],
        "h": [float(v) for v in h],
        "gsum": [float(v) for v in gsum],
        "loss_sum": float(loss),
        "delta": [float(v) for v in delta],
        "theta_after_update": [float(dec(tf[j]) + delta[j]) for j in range(d)],
    }


def main():
    cases = [
        case("n1_d1", 1, 1, 1),
        case("n3_d2", 3, 2, 2),
        case("n17_d5_bias", 17, 5, 3, special="bias"),
        case("n64_d17", 64, 17, 4, xs=2.0),
        case("n33_d16_zero_theta", 33, 16, 5, special="zero_theta"),
        case("n40_d7_odd_labels", 40, 7, 6, special="odd_labels"),
        case("n25_d9_large_z", 25, 9, 7, xs=4.0, ts=2.0),
        case("n50_d3_readme_knobs", 50, 3, 8, alpha=0.001, beta=0.01),
        # rows wider than 64 columns reach the other device kernels: one ragged chunk,
        # chunk + tail stage, two chunks + wide tail, eight chunks + tail
        case("n6_d70", 6, 70, 9, xs=0.5),
        case("n7_d130_tail", 7, 130, 10, xs=0.5),
        case("n4_d300_tail", 4, 300, 11, xs=0.25),
        case("n2_d1030_tail", 2, 1030, 12, xs=0.125),
    ]
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lr_small.json")
    with open(out, "w") as f:
        json.dump({"cases": cases}, f, separators=(",", ":"))
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
