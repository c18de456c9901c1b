"""The seeded shard generator: reproducible, split-invariant, right distributions."""
import numpy as np
from scipy.stats import norm


def test_counter_based_and_split_invariant(gen):
    spec = gen.GenSpec(1234, gen.NORMAL, 0, 1.0, 0.0, 1.0)
    whole = gen.gen_X(spec, 0, 1000, 37, threads=3)
    parts = np.vstack([gen.gen_X(spec, 0, 400, 37, threads=1), gen.gen_X(spec, 400, 600, 37, threads=8)])
    np.testing.assert_array_equal(whole, parts)
    np.testing.assert_array_equal(whole, gen.gen_X(spec, 0, 1000, 37))
    assert whole[5, 7] == gen.normal(1234, 1, 5, 7)
    other = gen.gen_X(gen.GenSpec(1235, gen.NORMAL, 0, 1.0, 0.0, 1.0), 0, 10, 37)
    assert not np.array_equal(other, whole[:10])


def _sm64_mix(z):
    M = (1 << 64) - 1
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
    return z ^ (z >> 31)


def _u01_py(seed, stream, i, j):
    M, G = (1 << 64) - 1, 0x9E3779B97F4A7C15
    rk = _sm64_mix((_sm64_mix((seed + stream * G) & M) + (i + 1) * G) & M)
    bits = _sm64_mix((rk + (j + 1) * G) & M)
    return ((bits >> 11) + 0.5) / 9007199254740992.0


def test_known_answers(gen):
    # pins the bit stream: splitmix64 finaliser keyed by (seed, stream, row), element j --
    # restated here in Python integers
    for key in ((1, 1, 2, 3), (0x5EED0002, 1, 999_999, 999), (7, 4, 0, 0), (2**63, 6, 12345, 77)):
        assert gen.u01(*key) == _u01_py(*key)
    assert gen.u01(1, 1, 2, 3) == 0.5211329322530509
    assert gen.normal(1, 1, 2, 3) == 0.05299720396923816


def test_inverse_cdf_matches_scipy(gen):
    us = np.array([gen.u01(9, 1, i, 0) for i in range(2000)])
    zs = np.array([gen.normal(9, 1, i, 0) for i in range(2000)])
    np.testing.assert_allclose(zs, norm.ppf(us), rtol=1e-13, atol=1e-15)
    assert us.min() > 0 and us.max() < 1


def test_distributions(gen):
    n, d = 4000, 64
    X = gen.gen_X(gen.GenSpec(7, gen.NORMAL, 0, 0.5, 0.0, 1.0), 0, n, d)
    assert abs(X.mean()) < 5e-3 and abs(X.std() - 0.5) < 5e-3
    U = gen.gen_X(gen.GenSpec(7, gen.UNIFORM, 0, 1.0, 0.0, 1.0), 0, n, d)
    assert U.min() >= -1 and U.max() <= 1 and abs(U.mean()) < 5e-3 and abs(U.std() - 1 / np.sqrt(3)) < 5e-3
    Z = gen.gen_X(gen.GenSpec(7, gen.NORMAL, 0, 1.0, 0.9, 1.0), 0, n, d)
    assert abs((Z == 0).mean() - 0.9) < 5e-3
    O = gen.gen_X(gen.GenSpec(7, gen.UNIFORM, 100, 1.0, 0.0, 100.0), 0, 20000, 4)
    big = (np.abs(O).max(axis=1) > 1.0).mean()
    assert 0.005 < big < 0.015


def test_labels_follow_the_model(gen):
    cfg = gen.configs()["c1_dense_100k_x_100"].scaled(20000)
    X, y = cfg.rows(0, cfg.n)
    assert set(np.unique(y)) <= {0.0, 1.0}
    p = 1 / (1 + np.exp(-(X @ cfg.theta_star())))
    # calibration: mean label matches mean probability
    assert abs(y.mean() - p.mean()) < 0.01
    hi = p > 0.9
    assert y[hi].mean() > 0.9


def test_configs_match_the_baseline_shapes(gen):
    c = gen.configs()
    assert (c["c1_dense_100k_x_100"].n, c["c1_dense_100k_x_100"].d) == (100_000, 100)
    assert (c["c2_headline_1m_x_1000"].n, c["c2_headline_1m_x_1000"].d) == (1_000_000, 1000)
    assert (c["c3_tall_10m_x_256"].n, c["c3_tall_10m_x_256"].d) == (10_000_000, 256)
    assert (c["c4_wide_200k_x_16384"].n, c["c4_wide_200k_x_16384"].d) == (200_000, 16384)
    assert c["c4b_wide_200k_x_16385"].d == 16385
    assert (c["c5_e2e_2m_x_512"].n, c["c5_e2e_2m_x_512"].d) == (2_000_000, 512)
    c1 = c["c1_dense_100k_x_100"]
    assert abs(c1.alpha - 1e-6) < 1e-20 and c1.beta == 0.005 and not c1.theta().any()
    assert c["c2_headline_1m_x_1000"].algorithmic_bytes() == 8_008_016_008
    ts = c["c4_wide_200k_x_16384"].theta_star()
    assert 0.03 < (ts != 0).mean() < 0.07
