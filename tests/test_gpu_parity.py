"""GPU parity: the HIP shard pass, called through the C ABI, against the CPU
oracle on identical seeded inputs.

Tolerances (fp64): relative L2 error <= 1e-10 per gradient / delta, <= 1e-8 on
theta after 100 iterations; loss sums relative <= 1e-10 where no row is
saturated (|z| moderate), stated per test otherwise.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GRAD_TOL = 1e-10
LOSS_TOL = 1e-10


def rel(a, b):
    nb = np.linalg.norm(b)
    return np.linalg.norm(a - b) / (nb if nb > 0 else 1.0)


def make(gen, n, d, seed=0xABCD, scale=None, theta_scale=1.0):
    spec = gen.GenSpec(seed, gen.NORMAL, 0, scale if scale else 1.0 / np.sqrt(d), 0.0, 1.0)
    X = gen.gen_X(spec, 0, n, d)
    ts = gen.gen_vec(seed, gen.STREAM_THETA_STAR, d, gen.NORMAL, theta_scale)
    y = gen.gen_labels(spec, 0, X, ts) if n else np.zeros(0)
    th = gen.gen_vec(seed, gen.STREAM_THETA, d, gen.NORMAL, theta_scale)
    return X, y, th


# every kernel variant (d <= 128, 256, 512, 1024, 2048, 4096, 8192, 16384,
# 19456), widths that are not multiples of the 128-column chunk or of 2, and
# row counts around the tile sizes
SHAPES = [
    (1, 1), (5, 2), (7, 3), (64, 17), (300, 64), (1000, 100), (257, 127), (1030, 128),
    (515, 129), (1000, 255), (4099, 256), (333, 257), (1001, 512), (2051, 1000),
    (700, 1024), (300, 1025), (260, 2047), (130, 4097), (70, 8193), (40, 16384),
    (37, 16385), (21, 19456),
    # several tiles per row group and a partial last tile, for every tile height
    (40003, 256), (20005, 512), (9001, 1000), (6149, 2047), (3077, 4097), (2053, 8193),
    (8195, 100), (515, 16384),
    # 8 waves side by side with 9..19 chunks each: every count has a variant of its own
    # (exact multiples of 1024 columns, and rows that leave the last wave short)
    (70, 9000), (33, 9216), (45, 10000), (40, 11000), (31, 11264), (40, 12288), (36, 13000),
    (29, 13312), (33, 14000), (30, 15000), (27, 15360), (30, 17000), (25, 18000), (23, 18432),
    (25, 19000),
    # 65..96 columns: a half-wave per row (pair_pass), 16 rows per tile
    (1, 65), (15, 66), (16, 67), (17, 72), (1000, 80), (4099, 95), (40003, 96), (300, 97),
]


@pytest.mark.parametrize("n,d", SHAPES)
def test_loss_grad_matches_oracle(plr, oracle, gen, n, d):
    print("case n=%d d=%d" % (n, d), flush=True)
    X, y, th = make(gen, n, d)
    plr.set_data(X, y)
    print(plr.kernel_info(), flush=True)
    g, loss, n_out = plr.loss_grad(th)
    assert n_out == n
    g_ref = oracle.gsum(X, y, th)
    assert rel(g, g_ref) <= GRAD_TOL
    # long-double arbiter agrees too
    assert rel(g, oracle.gsum(X, y, th, hp=True)) <= GRAD_TOL
    loss_ref = oracle.calc_loss_sum(X, y, th)
    assert abs(loss - loss_ref) <= LOSS_TOL * abs(loss_ref)


# rows that end a few columns past a 128-column chunk boundary (the file path's
# bias column makes 2^k + 1 the common width): (full chunks, leftover columns)
# for every tail-stage variant at its smallest and largest leftover, odd and
# even widths, with row counts that leave partial tiles and partial tail loads
TAIL_CASES = [(k, t) for k in (1, 2) for t in (1, 2, 7, 8, 9, 16, 17, 31, 32, 33, 63, 64)] + \
             [(k, t) for k in (3, 4) for t in (1, 15, 16, 17, 32)] + \
             [(k, t) for k in (6, 7, 9, 10, 11) for t in (1, 32)] + \
             [(8, t) for t in (1, 31, 32, 33, 64)] + \
             [(k, t) for k in (12, 13, 14, 15, 16) for t in (1, 64)] + \
             [(32, 1), (32, 32), (64, 1), (64, 17), (64, 64), (128, 1), (128, 100)]


@pytest.mark.parametrize("k,t", TAIL_CASES)
def test_rows_just_past_a_chunk_boundary(plr, oracle, gen, k, t):
    d = 128 * k + t
    for n in (1, 3, 77, 1543):
        print("case n=%d d=%d" % (n, d), flush=True)
        if d > 4096 and n > 100:
            n = 131
        X, y, th = make(gen, n, d, seed=0x7A11 + d)
        plr.set_data(X, y)
        if n == 1:
            print(plr.kernel_info(), flush=True)
            pitch = d + (d & 1) if d < 2048 else (d + 15) // 16 * 16
            assert "tail=%d " % (pitch - 128 * k) in plr.kernel_info()
        g, loss, n_out = plr.loss_grad(th)
        assert n_out == n
        assert rel(g, oracle.gsum(X, y, th)) <= GRAD_TOL
        loss_ref = oracle.calc_loss_sum(X, y, th)
        assert abs(loss - loss_ref) <= LOSS_TOL * abs(loss_ref)
        # the passes without a gradient take their own instances
        l2, _ = plr.calc_loss(th)
        assert abs(l2 - loss_ref) <= LOSS_TOL * abs(loss_ref)
        h = plr.predict(th)
        assert np.max(np.abs(h - oracle.predict(X, th))) <= 1e-14
    # the last column matters: a spike there must show in its gradient entry alone
    X2 = X.copy()
    X2[:, d - 1] += 1.0
    plr.set_data(X2, y)
    g2, _, _ = plr.loss_grad(np.zeros(d))
    assert rel(g2, X2.T @ (0.5 - y)) <= GRAD_TOL


@pytest.mark.parametrize("chunks", list(range(17, 33)))
def test_rows_of_17_to_32_chunks(plr, oracle, gen, chunks):
    # one exact kernel variant per chunk count; the widths that fill a
    # several-waves variant exactly (18, 21, 24, 28, 32 chunks) take that one
    for d in (128 * chunks, 128 * chunks - 1, 128 * (chunks - 1) + 17):
        for n in (1, 5, 517):
            print("case n=%d d=%d" % (n, d), flush=True)
            X, y, th = make(gen, n, d, seed=0xC0DE + d)
            plr.set_data(X, y)
            if n == 1:
                print(plr.kernel_info(), flush=True)
            g, loss, _ = plr.loss_grad(th)
            assert rel(g, oracle.gsum(X, y, th)) <= GRAD_TOL
            loss_ref = oracle.calc_loss_sum(X, y, th)
            assert abs(loss - loss_ref) <= LOSS_TOL * abs(loss_ref)
            l2, _ = plr.calc_loss(th)
            assert abs(l2 - loss_ref) <= LOSS_TOL * abs(loss_ref)
            assert np.max(np.abs(plr.predict(th) - oracle.predict(X, th))) <= 1e-14
    X2 = X.copy()
    X2[:, d - 1] += 1.0
    plr.set_data(X2, y)
    g2, _, _ = plr.loss_grad(np.zeros(d))
    assert rel(g2, X2.T @ (0.5 - y)) <= GRAD_TOL


@pytest.mark.parametrize("n,d", [(1000, 100), (2051, 1000), (333, 257), (70, 8193), (37, 16385),
                                 (1500, 70)])
def test_dgd_delta_matches_oracle(plr, oracle, gen, n, d):
    X, y, th = make(gen, n, d)
    plr.set_data(X, y)
    alpha, beta = 0.1 / n, 0.005
    delta, loss = plr.dgd_delta(th, alpha, beta)
    d_ref = oracle.dgd_delta(X, y, th, alpha, beta)
    assert rel(delta, d_ref) <= GRAD_TOL
    assert rel(delta, oracle.dgd_delta_hp(X, y, th, alpha, beta)) <= GRAD_TOL
    # a shuffled traversal (the reference shuffles with a time seed) only moves rounding
    order = np.random.default_rng(1).permutation(n)
    assert rel(delta, oracle.dgd_delta(X, y, th, alpha, beta, order=order)) <= GRAD_TOL
    assert abs(loss - oracle.calc_loss_sum(X, y, th)) <= LOSS_TOL * abs(loss)
    # the reference's own knobs (README: alpha=0.001, beta=0.01)
    delta2, _ = plr.dgd_delta(th, 0.001, 0.01, want_loss=False)
    assert rel(delta2, oracle.dgd_delta(X, y, th, 0.001, 0.01)) <= GRAD_TOL


@pytest.mark.parametrize("n,d", [(999, 100), (2051, 1000), (130, 4097), (999, 72)])
def test_calc_loss_and_predict(plr, oracle, gen, n, d):
    X, y, th = make(gen, n, d)
    plr.set_data(X, y)
    loss, n_out = plr.calc_loss(th)
    assert n_out == n
    ref = oracle.calc_loss_sum(X, y, th)
    assert abs(loss - ref) <= LOSS_TOL * abs(ref)
    h = plr.predict(th)
    h_ref = oracle.predict(X, th)
    assert np.max(np.abs(h - h_ref)) <= 1e-14
    # fused pass and loss-only pass agree with each other
    _, loss2, _ = plr.loss_grad(th)
    assert abs(loss2 - loss) <= 1e-12 * abs(loss)


@pytest.mark.parametrize("n,d", [(999, 100), (2051, 1000), (70, 8193), (999, 90)])
def test_linear_model_pieces(plr, oracle, gen, n, d):
    # the ridge worker's loss and prediction (alg/regression/ridge/ridge.hpp:103-109,130-139)
    # and the least-squares gradient, on the same streaming pass with the identity link
    X, _, th = make(gen, n, d)
    y = gen.gen_vec(99, gen.STREAM_THETA, n)
    plr.set_data(X, y)
    z = plr.predict_linear(th)
    np.testing.assert_allclose(z, oracle.predict_linear(X, th), rtol=0, atol=1e-13)
    loss, n_out = plr.calc_loss(th, 3)
    want = oracle.ridge_loss_sum(X, y, th)
    assert n_out == n and abs(loss - want) <= 1e-12 * want
    g, loss2, _ = plr.loss_grad(th, 3)
    assert rel(g, oracle.lsq_gsum(X, y, th)) <= GRAD_TOL
    assert rel(g, X.T @ (X @ th - y)) <= 1e-12
    assert abs(loss2 - want) <= 1e-12 * want


# one shape per kernel family: lane_pass, lane2_pass, pair_pass, one-chunk shard_pass, tail
# stage, one wave per row, several waves side by side, theta in LDS + tail, and the two
# wide-row paths (team_pass, two sweeps)
LINEAR_SHAPES = [(3000, 16, 0), (2500, 41, 0), (1500, 70, 0), (1000, 100, 0), (333, 257, 0),
                 (2051, 1000, 0), (130, 4097, 0), (37, 16385, 0), (300, 20001, 0),
                 (300, 20001, 1), (64, 65536, 0), (64, 65536, 1)]


@pytest.mark.parametrize("first_col_one", [0, 1])
@pytest.mark.parametrize("n,d,two_sweeps", LINEAR_SHAPES)
def test_linear_delta_matches_oracle(plr, oracle, gen, n, d, two_sweeps, first_col_one):
    # the identity link in every kernel family: the ridge worker's batch step
    # (alg/regression/ridge/ridge.hpp:79-84 summed at a fixed theta), its loss (:103-109)
    # and its prediction (:130-139), with the constant first column stored and not
    print("case n=%d d=%d two_sweeps=%d first_col_one=%d" % (n, d, two_sweeps, first_col_one),
          flush=True)
    X, _, th = make(gen, n, d, seed=0x1D + d)
    if first_col_one:
        X[:, 0] = 1.0
    y = X @ gen.gen_vec(7, gen.STREAM_THETA_STAR, d) + 0.3 * gen.gen_vec(99, gen.STREAM_THETA, n)
    plr.set_option("column_blocks_two_sweeps", two_sweeps)
    plr.set_option("first_column_is_one", first_col_one)
    plr.set_data(X, y)
    info = plr.kernel_info()
    print(info, flush=True)
    assert ("not stored" in info) == bool(first_col_one)
    if d > 19456:
        assert ("team_pass" in info) == (not two_sweeps)
    alpha, beta = 0.1 / n, 0.005
    delta, loss = plr.dgd_delta_linear(th, alpha, beta)
    assert rel(delta, oracle.ridge_delta(X, y, th, alpha, beta)) <= GRAD_TOL
    # the textbook form of the same step
    assert rel(delta, alpha * (X.T @ (y - X @ th)) - 2 * alpha * beta * n * th) <= 1e-11
    want = oracle.ridge_loss_sum(X, y, th)
    assert abs(loss - want) <= 1e-12 * want
    g, loss2, n_out = plr.loss_grad(th, 3)
    assert n_out == n and rel(g, oracle.lsq_gsum(X, y, th)) <= GRAD_TOL
    assert abs(loss2 - want) <= 1e-12 * want
    l3, _ = plr.calc_loss(th, 3)
    assert abs(l3 - want) <= 1e-12 * want
    np.testing.assert_allclose(plr.predict_linear(th), oracle.predict_linear(X, th), rtol=0,
                               atol=1e-12)
    # the reference's own knobs (ridge README: alpha=0.01, beta=0.01 scale) and repeatability
    d2, _ = plr.dgd_delta_linear(th, 0.01, 0.01)
    assert rel(d2, oracle.ridge_delta(X, y, th, 0.01, 0.01)) <= GRAD_TOL
    d3, _ = plr.dgd_delta_linear(th, 0.01, 0.01)
    np.testing.assert_array_equal(d2, d3)


@pytest.mark.parametrize("two_sweeps", [0, 1])
@pytest.mark.parametrize("n,d", [(19, 19457), (300, 33000), (1030, 20001), (64, 65536),
                                 (700, 32768), (515, 24577), (40, 131072), (12, 140000),
                                 (9, 262144), (5, 262200), (3, 524288), (3, 524300),
                                 (3, 20000), (2100, 20016)])
def test_rows_wider_than_the_fused_kernels(plr, oracle, gen, n, d, two_sweeps):
    # past 19456 columns the row is processed in column blocks: by teams of workgroups that
    # exchange partial dot products (X read once; up to 64 blocks of 8192 columns), or in two
    # sweeps over X
    print("case n=%d d=%d two_sweeps=%d" % (n, d, two_sweeps), flush=True)
    X, y, th = make(gen, n, d)
    plr.set_option("column_blocks_two_sweeps", two_sweeps)
    plr.set_data(X, y)
    assert ("team_pass" in plr.kernel_info()) == (not two_sweeps and d <= 524288)
    print(plr.kernel_info(), flush=True)
    g, loss, n_out = plr.loss_grad(th)
    assert n_out == n
    assert rel(g, oracle.gsum(X, y, th)) <= GRAD_TOL
    want = oracle.calc_loss_sum(X, y, th)
    assert abs(loss - want) <= LOSS_TOL * want
    g2, loss2, _ = plr.loss_grad(th)
    np.testing.assert_array_equal(g, g2)
    assert loss == loss2
    delta, _ = plr.dgd_delta(th, 0.1 / n, 0.005)
    assert rel(delta, oracle.dgd_delta(X, y, th, 0.1 / n, 0.005)) <= GRAD_TOL
    l3, _ = plr.calc_loss(th, 1)
    assert abs(l3 - want) <= LOSS_TOL * want
    assert np.max(np.abs(plr.predict(th) - oracle.predict(X, th))) <= 1e-14
    t5 = plr.train_dgd(np.zeros(d), 0.1 / n, 0.005, 5)
    assert rel(t5, oracle.train_dgd(X, y, np.zeros(d), 0.1 / n, 0.005, 5)) <= 1e-10
    # the identity link on the same shard: squared loss, least-squares gradient, x.theta
    wq = oracle.ridge_loss_sum(X, y, th)
    gq, lq, _ = plr.loss_grad(th, 3)
    assert rel(gq, oracle.lsq_gsum(X, y, th)) <= GRAD_TOL
    assert abs(lq - wq) <= 1e-12 * wq
    lq2, _ = plr.calc_loss(th, 3)
    assert abs(lq2 - wq) <= 1e-12 * wq
    np.testing.assert_allclose(plr.predict_linear(th), oracle.predict_linear(X, th), rtol=0,
                               atol=1e-12)


@pytest.mark.parametrize("n,d", [(300, 2), (1000, 3), (4099, 17), (2051, 65), (2000, 66), (999, 98),
                                 (3001, 129), (40003, 257), (2051, 1001), (1500, 1025),
                                 (700, 2049), (130, 4097), (70, 8193), (37, 16385), (90, 19458),
                                 (200, 33001)])
def test_constant_first_column_is_not_stored(plr, oracle, gen, n, d):
    # "first_column_is_one": the bias column the file path prepends (lr.cpp:83) stays on the
    # host; every result must be what the stored column gives (the oracle sees the full X)
    from paracel_amd import PlrError

    print("case n=%d d=%d" % (n, d), flush=True)
    X, _, th = make(gen, n, d, seed=0xB1A5 + d)
    X[:, 0] = 1.0
    spec = gen.GenSpec(77, gen.NORMAL, 0, 1.0, 0.0, 1.0)
    y = gen.gen_labels(spec, 0, X, gen.gen_vec(77, gen.STREAM_THETA_STAR, d, gen.NORMAL, 1.0))
    plr.set_option("first_column_is_one", 1)
    plr.set_data(X, y)
    info = plr.kernel_info()
    print(info, flush=True)
    assert "not stored" in info and plr.shape == (n, d)
    g, loss, n_out = plr.loss_grad(th)
    g_ref = oracle.gsum(X, y, th)
    assert n_out == n and g.shape == (d,)
    assert rel(g, g_ref) <= GRAD_TOL
    assert abs(g[0] - g_ref[0]) <= 1e-10 * max(abs(g_ref[0]), np.linalg.norm(g_ref) / d)
    want = oracle.calc_loss_sum(X, y, th)
    assert abs(loss - want) <= LOSS_TOL * want
    delta, _ = plr.dgd_delta(th, 0.1 / n, 0.005)
    assert rel(delta, oracle.dgd_delta(X, y, th, 0.1 / n, 0.005)) <= GRAD_TOL
    l1, _ = plr.calc_loss(th, 1)
    assert abs(l1 - want) <= LOSS_TOL * want
    assert np.max(np.abs(plr.predict(th) - oracle.predict(X, th))) <= 1e-14
    np.testing.assert_allclose(plr.predict_linear(th), X @ th, rtol=0, atol=1e-12)
    t5 = plr.train_dgd(np.zeros(d), 0.1 / n, 0.005, 5)
    assert rel(t5, oracle.train_dgd(X, y, np.zeros(d), 0.1 / n, 0.005, 5)) <= 1e-10
    # chunked upload of the same shard, same bits
    plr.alloc_data(n, d)
    h = n // 2
    plr.set_data_chunk(h, X[h:], y[h:])
    plr.set_data_chunk(0, X[:h], y[:h])
    g2, loss2, _ = plr.loss_grad(th)
    np.testing.assert_array_equal(g, g2)
    assert loss == loss2
    # a row that does not start with 1.0 is refused, by row number
    Xb = X.copy()
    Xb[n // 3, 0] = 1.0000001
    Xb[n - 1, 0] = 0.0      # a later one too (another upload thread may meet it first)
    with pytest.raises(PlrError) as e:
        plr.set_data(Xb, y)
    assert e.value.code == -1 and "row %d" % (n // 3) in str(e.value)
    # the refused shard does not stay resident, half uploaded
    assert plr.shape == (0, 0)
    with pytest.raises(PlrError) as e:
        plr.loss_grad(np.zeros(0))
    assert e.value.code == -4  # PLR_ERR_NODATA
    # switched off again: the column is stored, same results to rounding
    plr.set_option("first_column_is_one", 0)
    plr.set_data(X, y)
    assert "not stored" not in plr.kernel_info()
    g3, loss3, _ = plr.loss_grad(th)
    assert rel(g3, g) <= 1e-12 and abs(loss3 - loss) <= 1e-12 * loss


def test_wide_row_exchange_gives_up_instead_of_hanging(plr, oracle, gen):
    # a workgroup that never hears from its partners must not spin for ever: with the poll
    # limit at 0 every wait that does not find its partial at the first look gives up, the
    # kernel runs to its end and -- with the fallback switched off -- the call reports the
    # failure (a pass in which every first look happens to succeed is correct and also accepted)
    from paracel_amd import PlrError

    X, y, th = make(gen, 600, 20001)
    plr.set_data(X, y)
    assert "team_pass" in plr.kernel_info()
    g_ref = oracle.gsum(X, y, th)
    plr.set_option("team_fallback", 0)
    plr.set_option("team_spin_limit", 0)
    try:
        g, _, _ = plr.loss_grad(th)
        assert rel(g, g_ref) <= GRAD_TOL
        print("every first look succeeded", flush=True)
    except PlrError as e:
        assert e.code == -2 and "gave up waiting" in str(e)
    # several rounds enqueued back to back: a give-up in ANY of them must surface -- what may
    # never come back is success with a theta that later rounds built on a discarded pass
    alpha, beta = 0.1 / 600, 0.005
    t_ref = oracle.train_dgd(X, y, np.zeros(20001), alpha, beta, 8)
    try:
        t8 = plr.train_dgd(np.zeros(20001), alpha, beta, 8)
        assert rel(t8, t_ref) <= 1e-8
        print("every first look of 8 rounds succeeded", flush=True)
    except PlrError as e:
        assert e.code == -2 and "gave up waiting" in str(e)
    # the context is usable again once the limit is back
    plr.set_option("team_spin_limit", 1 << 22)
    g, _, _ = plr.loss_grad(th)
    assert rel(g, g_ref) <= GRAD_TOL
    with pytest.raises(PlrError):
        plr.set_option("no_such_option", 1)


def test_a_wide_row_pass_that_gives_up_runs_again_in_two_sweeps(plr, oracle, gen):
    # the default: a team pass whose workgroups are not all resident (other processes or
    # streams on the compute units) is run again in two sweeps, which need no residency; the
    # caller gets the shard's results either way, and after two such passes the shard stays on
    # two sweeps.  Forced here from the host with the poll limit at 0.
    X, y, th = make(gen, 600, 20001, seed=0xFA11)
    plr.set_data(X, y)
    assert "team_pass" in plr.kernel_info() and "gave up" not in plr.kernel_info()
    g_ref = oracle.gsum(X, y, th)
    l_ref = oracle.calc_loss_sum(X, y, th)
    alpha, beta = 0.1 / 600, 0.005
    t_ref = oracle.train_dgd(X, y, np.zeros(20001), alpha, beta, 8)
    plr.set_option("team_spin_limit", 0)
    for _ in range(3):
        g, loss, _ = plr.loss_grad(th)
        assert rel(g, g_ref) <= GRAD_TOL and abs(loss - l_ref) <= LOSS_TOL * l_ref
        t8 = plr.train_dgd(np.zeros(20001), alpha, beta, 8)
        assert rel(t8, t_ref) <= 1e-8
        h = plr.predict(th)
        assert np.max(np.abs(h - oracle.predict(X, th))) <= 1e-14
    print(plr.kernel_info(), flush=True)
    plr.set_option("team_spin_limit", 1 << 22)
    g, loss, _ = plr.loss_grad(th)
    assert rel(g, g_ref) <= GRAD_TOL and abs(loss - l_ref) <= LOSS_TOL * l_ref
    # a fresh shard starts on the team path again
    plr.set_data(X, y)
    assert "team_pass" in plr.kernel_info() and "gave up" not in plr.kernel_info()
    g, _, _ = plr.loss_grad(th)
    assert rel(g, g_ref) <= GRAD_TOL


NARROW = [(n, d) for d in (1, 2, 3, 4, 5, 8, 9, 16, 17, 31, 32, 33, 48, 63, 64)
          for n in (1, 65, 100003)] + [(63, 7), (64, 7), (127, 32), (128, 32), (255, 64), (256, 2),
                                       (257, 2), (511, 4), (513, 8), (1000000, 6)]


@pytest.mark.parametrize("n,d", NARROW)
def test_narrow_rows_lane_per_row(plr, oracle, gen, n, d):
    # d <= 64: the shard is stored in tiles of 64 rows, column pair by column pair, and a
    # lane owns a row
    print("case n=%d d=%d" % (n, d), flush=True)
    X, y, th = make(gen, n, d, scale=1.0 / np.sqrt(d), theta_scale=1.0)
    plr.set_data(X, y)
    g, loss, n_out = plr.loss_grad(th)
    assert n_out == n
    assert rel(g, oracle.gsum(X, y, th)) <= GRAD_TOL
    want = oracle.calc_loss_sum(X, y, th)
    assert abs(loss - want) <= LOSS_TOL * want
    g2, loss2, _ = plr.loss_grad(th)
    np.testing.assert_array_equal(g, g2)
    assert loss2 == loss
    if n <= 1000:
        delta, _ = plr.dgd_delta(th, 0.1 / n, 0.005)
        assert rel(delta, oracle.dgd_delta(X, y, th, 0.1 / n, 0.005)) <= GRAD_TOL
        np.testing.assert_allclose(plr.predict(th), oracle.predict(X, th), rtol=0, atol=1e-14)
        ls, _ = plr.calc_loss(th, 1)
        assert abs(ls - want) <= LOSS_TOL * want
        lq, _ = plr.calc_loss(th, 3)
        wq = oracle.ridge_loss_sum(X, y, th)
        assert abs(lq - wq) <= 1e-12 * wq
        np.testing.assert_allclose(plr.predict_linear(th), oracle.predict_linear(X, th), rtol=0,
                                   atol=1e-13)


def test_every_narrow_width_and_the_tiling_of_uploaded_rows(plr, oracle, gen):
    # every width of the row-tiled layout, rows sent in pieces that start and end inside a
    # tile, from host rows with a stride, and with the constant first column left on the host
    for d in range(1, 65):
        n = 64 * 9 + (d * 7) % 61
        print("case d=%d n=%d" % (d, n), flush=True)
        X, y, th = make(gen, n, d, scale=1.0 / np.sqrt(d), theta_scale=1.0)
        want_g, want_l = oracle.gsum(X, y, th), oracle.calc_loss_sum(X, y, th)
        plr.set_data(X, y)
        g, loss, _ = plr.loss_grad(th)
        assert rel(g, want_g) <= GRAD_TOL and abs(loss - want_l) <= LOSS_TOL * want_l
        # the same rows in three pieces, out of order, the host rows 3 doubles apart
        wide = np.zeros((n, d + 3))
        wide[:, :d] = X
        cuts = [0, 37 + d, 64 * 5 - 1, n]
        plr.alloc_data(n, d)
        for k in (2, 0, 1):
            lo, hi = cuts[k], cuts[k + 1]
            plr.set_data_chunk(lo, wide[lo:hi, :d], y[lo:hi])
        g2, loss2, _ = plr.loss_grad(th)
        np.testing.assert_array_equal(g2, g)
        assert loss2 == loss
        np.testing.assert_allclose(plr.predict(th), oracle.predict(X, th), rtol=0, atol=1e-14)
        if d >= 2:
            Xb = X.copy()
            Xb[:, 0] = 1.0
            plr.set_option("first_column_is_one", 1)
            try:
                plr.set_data(Xb, y)
                gb, lb, _ = plr.loss_grad(th)
            finally:
                plr.set_option("first_column_is_one", 0)
            wl = oracle.calc_loss_sum(Xb, y, th)
            assert rel(gb, oracle.gsum(Xb, y, th)) <= GRAD_TOL and abs(lb - wl) <= LOSS_TOL * wl


def test_theta_zero_closed_forms(plr, gen):
    # theta = 0 => h = 1/2 exactly: gsum = X^T (1/2 - y) (a plain GEMV), loss = n ln 2
    X, y, _ = make(gen, 3001, 300)
    plr.set_data(X, y)
    g, loss, n = plr.loss_grad(np.zeros(300))
    assert rel(g, X.T @ (0.5 - y)) <= 1e-13
    assert abs(loss - n * np.log(2.0)) <= 1e-12 * n
    for flags in (0, 1):
        l2, _ = plr.calc_loss(np.zeros(300), flags)
        assert abs(l2 - n * np.log(2.0)) <= 1e-12 * n


def test_x_zero_gives_pure_l2_delta(plr, gen):
    # X = 0 => delta = -2 alpha beta n theta exactly (up to one rounding)
    n, d = 777, 130
    X = np.zeros((n, d))
    y = (np.arange(n) % 2).astype(float)
    th = gen.gen_vec(3, gen.STREAM_THETA, d)
    plr.set_data(X, y)
    delta, _ = plr.dgd_delta(th, 1e-3, 0.25)
    np.testing.assert_allclose(delta, -2 * 1e-3 * 0.25 * n * th, rtol=4e-16, atol=0)


def test_one_hot_rows_count_columns(plr):
    # one-hot rows with theta = 0: gsum[j] = sum over rows hitting j of (1/2 - y)
    n, d = 1000, 200
    rng = np.random.default_rng(5)
    cols = rng.integers(0, d, n)
    X = np.zeros((n, d))
    X[np.arange(n), cols] = 1.0
    y = (rng.random(n) < 0.3).astype(float)
    plr.set_data(X, y)
    g, _, _ = plr.loss_grad(np.zeros(d))
    want = np.zeros(d)
    np.add.at(want, cols, 0.5 - y)
    np.testing.assert_array_equal(g, want)  # halves add exactly


def test_shard_additivity(plr, gen):
    # gsum(S1 u S2) = gsum(S1) + gsum(S2): the multi-worker invariant of update.cpp:26-32
    X, y, th = make(gen, 5000, 700)
    plr.set_data(X, y)
    g, loss, _ = plr.loss_grad(th)
    plr.set_data(X[:1777], y[:1777])
    g1, l1, _ = plr.loss_grad(th)
    plr.set_data(X[1777:], y[1777:])
    g2, l2, _ = plr.loss_grad(th)
    assert rel(g1 + g2, g) <= 1e-13
    assert abs(l1 + l2 - loss) <= 1e-13 * abs(loss)


def test_bitwise_reproducible(plr, gen):
    X, y, th = make(gen, 9000, 1000)
    plr.set_data(X, y)
    g1, l1, _ = plr.loss_grad(th)
    g2, l2, _ = plr.loss_grad(th)
    np.testing.assert_array_equal(g1, g2)
    assert l1 == l2


def test_chunked_upload_equals_whole(plr, gen):
    X, y, th = make(gen, 3000, 513)
    plr.set_data(X, y)
    g, loss, _ = plr.loss_grad(th)
    plr.alloc_data(3000, 513)
    for lo, hi in ((2000, 3000), (0, 700), (700, 2000)):
        plr.set_data_chunk(lo, X[lo:hi], y[lo:hi])
    g2, loss2, _ = plr.loss_grad(th)
    np.testing.assert_array_equal(g, g2)
    assert loss == loss2


def test_rows_never_uploaded_read_as_zero_rows(plr, oracle, gen):
    # plr_alloc_data reserves a zero-filled shard: a row range the caller never sends behaves
    # as rows of zeros with label 0 (h = 1/2 each), not as whatever the memory held before
    X, y, th = make(gen, 3000, 130)
    plr.set_data(np.full((3000, 130), 7.5), np.ones(3000))   # leave something behind
    plr.alloc_data(3000, 130)
    plr.set_data_chunk(0, X[:1000], y[:1000])
    plr.set_data_chunk(2000, X[2000:], y[2000:])
    Xz, yz = X.copy(), y.copy()
    Xz[1000:2000] = 0.0
    yz[1000:2000] = 0.0
    g, loss, _ = plr.loss_grad(th)
    assert rel(g, oracle.gsum(Xz, yz, th)) <= GRAD_TOL
    assert abs(loss - oracle.calc_loss_sum(Xz, yz, th)) <= LOSS_TOL * loss


def test_pitched_input(plr, oracle, gen):
    X, y, th = make(gen, 500, 333)
    wide = np.full((500, 400), np.nan)
    wide[:, :333] = X
    plr.set_data(wide[:, :333], y)  # ldx = 400 > d, NaNs outside must not be read
    g, _, _ = plr.loss_grad(th)
    assert rel(g, oracle.gsum(X, y, th)) <= GRAD_TOL


def test_host_pitch_equal_to_device_pitch_with_pad_column(plr, oracle, gen):
    # d odd -> device pitch d+1; a host buffer with the same pitch holds foreign values in
    # that extra column, which must not reach the device's zero pad column
    X, y, th = make(gen, 300, 333)
    wide = np.full((300, 334), np.nan)
    wide[:, :333] = X
    plr.set_data(wide[:, :333], y)
    g, loss, _ = plr.loss_grad(th)
    assert np.all(np.isfinite(g)) and np.isfinite(loss)
    assert rel(g, oracle.gsum(X, y, th)) <= GRAD_TOL


def test_saturated_rows_stable_vs_reference_loss(plr, oracle, gen):
    # rows scaled x100 saturate the sigmoid: the reference formula returns
    # +inf once exp(-z) < 2^-53 (lr.cpp:328 with h == 1.0); the stable form
    # stays finite and matches the long-double value
    n, d = 2000, 256
    spec = gen.GenSpec(77, gen.UNIFORM, 100, 1.0, 0.0, 100.0)
    X = gen.gen_X(spec, 0, n, d)
    ts = gen.gen_vec(77, gen.STREAM_THETA_STAR, d, gen.NORMAL, 0.1)
    y = gen.gen_labels(spec, 0, X, ts)
    th = 3.0 * ts
    # flip a label on a saturated row so the naive formula overflows
    z = X @ th
    i = int(np.argmax(z))
    assert z[i] > 40
    y[i] = 0.0
    plr.set_data(X, y)
    _, loss_ref_formula, _ = plr.loss_grad(th, 0)
    assert np.isinf(loss_ref_formula) and np.isinf(oracle.calc_loss_sum(X, y, th))
    g, loss_stable, _ = plr.loss_grad(th, 1)
    want = oracle.stable_loss_sum_hp(X, y, th)
    assert np.isfinite(loss_stable)
    assert abs(loss_stable - want) <= 1e-12 * abs(want)
    # the gradient is insensitive to saturation
    assert rel(g, oracle.gsum(X, y, th, hp=True)) <= GRAD_TOL


def test_stable_loss_equals_reference_loss_when_unsaturated(plr, gen):
    X, y, th = make(gen, 4000, 100)
    plr.set_data(X, y)
    a, _ = plr.calc_loss(th, 0)
    b, _ = plr.calc_loss(th, 1)
    assert abs(a - b) <= 1e-13 * abs(a)


def test_labels_other_than_one_are_class_zero(plr, oracle, gen):
    # lr.cpp:325 compares labels[i] == 1. exactly; anything else takes the -log(1-h) branch
    X, y, th = make(gen, 500, 60)
    y[::7] = 0.5
    y[::11] = -1.0
    plr.set_data(X, y)
    g, loss, _ = plr.loss_grad(th)
    assert abs(loss - oracle.calc_loss_sum(X, y, th)) <= LOSS_TOL * abs(loss)
    assert rel(g, oracle.gsum(X, y, th)) <= GRAD_TOL


@pytest.mark.parametrize("d", [300, 80, 40])
def test_non_finite_inputs_propagate_like_the_reference(plr, oracle, gen, d):
    # the reference does no input checking: a NaN or an infinity in a sample poisons
    # exactly the entries IEEE arithmetic says it should, on the device as on the host
    X, y, th = make(gen, 200, d)
    for kind, val in (("nan", np.nan), ("inf", np.inf), ("-inf", -np.inf)):
        Xb = X.copy()
        Xb[17, 5] = val
        plr.set_data(Xb, y)
        g, loss, _ = plr.loss_grad(th)
        g_ref = oracle.gsum(Xb, y, th)
        with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
            loss_ref = oracle.calc_loss_sum(Xb, y, th)
        np.testing.assert_array_equal(np.isnan(g), np.isnan(g_ref), err_msg=kind)
        np.testing.assert_array_equal(np.isinf(g), np.isinf(g_ref), err_msg=kind)
        ok = np.isfinite(g_ref)
        assert rel(g[ok], g_ref[ok]) <= GRAD_TOL
        assert (np.isnan(loss) and np.isnan(loss_ref)) or loss == loss_ref or \
            abs(loss - loss_ref) <= 1e-9 * abs(loss_ref)
    # a NaN label poisons every column its row touches
    yb = y.copy()
    yb[3] = np.nan
    plr.set_data(X, yb)
    g, _, _ = plr.loss_grad(th)
    np.testing.assert_array_equal(np.isnan(g), np.isnan(oracle.gsum(X, yb, th)))


def test_timing_switch(plr, gen):
    X, y, th = make(gen, 500, 130)
    plr.set_data(X, y)
    plr.reset_timing()
    g1, l1, _ = plr.loss_grad(th)
    assert plr.timing()[2] == 1 and plr.timing()[0] > 0
    plr.set_timing(False)
    g2, l2, _ = plr.loss_grad(th)
    d2, _ = plr.dgd_delta(th, 1e-3, 1e-2)
    assert plr.timing()[2] == 1               # nothing recorded while off
    np.testing.assert_array_equal(g1, g2)
    assert l1 == l2
    plr.set_timing(True)
    plr.loss_grad(th)
    assert plr.timing()[2] == 2


def test_results_watched_for_in_host_memory(plr, gen):
    # option "poll_results" (default on): the caller's thread takes the results as soon as the
    # finishing kernel has written them and their pass number to host memory.  Many calls in a
    # row with theta changing every time -- a stale result of the call before, or one taken
    # before all of it had arrived, would differ from the same call with the option off.
    X, y, th = make(gen, 3000, 300)          # 19 finishing blocks, each with a word of its own
    plr.set_data(X, y)
    thetas = [th * (1.0 + 0.01 * k) for k in range(200)]
    got = [plr.loss_grad(t) for t in thetas]
    got_delta = [plr.dgd_delta(t, 1e-3, 1e-2) for t in thetas]
    plr.set_option("poll_results", 0)
    try:
        for k, t in enumerate(thetas):
            g, loss, cnt = plr.loss_grad(t)
            assert np.array_equal(g, got[k][0]) and loss == got[k][1] and cnt == got[k][2], k
            dl, loss = plr.dgd_delta(t, 1e-3, 1e-2)
            assert np.array_equal(dl, got_delta[k][0]) and loss == got_delta[k][1], k
    finally:
        plr.set_option("poll_results", 1)


def test_bandwidth_probes(plr, gen):
    X, y, _ = make(gen, 4096, 512)
    plr.set_data(X, y)
    assert plr.probe_read_bandwidth(2) > 100.0       # GB/s; a 16 MB shard sits in cache
    assert plr.probe_copy_bandwidth(64 << 20, 2) > 100.0


def test_empty_shard(plr):
    plr.set_data(np.zeros((0, 10)), np.zeros(0))
    g, loss, n = plr.loss_grad(np.ones(10))
    assert n == 0 and loss == 0.0
    np.testing.assert_array_equal(g, np.zeros(10))
    delta, _ = plr.dgd_delta(np.ones(10), 0.1, 0.1)
    np.testing.assert_array_equal(np.abs(delta), np.zeros(10))
    assert plr.predict(np.ones(10)).size == 0


def test_errors(plr):
    from paracel_amd import PlrError

    with pytest.raises(PlrError) as e:
        plr.loss_grad(np.zeros(0))
    assert e.value.code == -4  # PLR_ERR_NODATA
    with pytest.raises(PlrError) as e:
        plr.alloc_data(10, 0)
    assert e.value.code == -1
    plr.set_data(np.ones((4, 3)), np.ones(4))
    with pytest.raises(ValueError):
        plr.loss_grad(np.zeros(5))
    with pytest.raises(PlrError) as e:
        plr.set_data_chunk(3, np.ones((2, 3)), np.ones(2))
    assert e.value.code == -1


def test_a_shard_that_does_not_fit_is_refused_cleanly(plr, oracle, gen):
    from paracel_amd import PlrError

    X, y, th = make(gen, 300, 257)
    plr.set_data(X, y)
    # 2^40 rows of 1000 doubles = 8 PB: the device allocation fails, nothing is computed
    with pytest.raises(PlrError) as e:
        plr.alloc_data(1 << 40, 1000)
    assert e.value.code == -3  # PLR_ERR_NOMEM
    assert "hipMalloc" in str(e.value)
    # the context holds no shard afterwards (the old one was dropped, the new one never existed)
    assert plr.shape == (0, 0)
    with pytest.raises(PlrError) as e:
        plr.loss_grad(np.zeros(0))
    assert e.value.code == -4
    # a row count whose byte size wraps around 64 bits is refused before any allocation
    # (it must not come back as a small allocation that the kernels then run past)
    for n_bad, d_bad in ((1 << 61, 1000), (1 << 62, 3), ((1 << 63) - 1, 70), (1 << 58, 40000)):
        with pytest.raises(PlrError) as e:
            plr.alloc_data(n_bad, d_bad)
        assert e.value.code == -1 and "64 bits" in str(e.value), (n_bad, d_bad, str(e.value))
        assert plr.shape == (0, 0)
    # and is usable again
    plr.set_data(X, y)
    g, _, _ = plr.loss_grad(th)
    assert rel(g, oracle.gsum(X, y, th)) <= GRAD_TOL


def test_config1_trajectory_100_iterations(plr, oracle, gen):
    # dense n=100000 d=100, theta0=0, lr=0.1, lam=0.01 => alpha=lr/n, beta=lam/2;
    # 100 full-batch rounds of read theta -> delta -> theta += delta
    # (lr.cpp:124-146 with update.cpp:26-32).  theta rel error <= 1e-8.
    cfg = gen.configs()["c1_dense_100k_x_100"]
    X, y = cfg.rows(0, cfg.n)
    plr.set_data(X, y)
    theta = np.zeros(cfg.d)
    worst = 0.0
    for it in range(100):
        delta, _ = plr.dgd_delta(theta, cfg.alpha, cfg.beta, want_loss=False)
        if it in (0, 50, 99):
            worst = max(worst, rel(delta, oracle.dgd_delta(X, y, theta, cfg.alpha, cfg.beta)))
        theta = theta + delta
    theta_ref = oracle.train_dgd(X, y, np.zeros(cfg.d), cfg.alpha, cfg.beta, 100)
    print("per-step delta rel-L2 worst %.3e, theta rel %.3e" % (worst, rel(theta, theta_ref)))
    assert worst <= GRAD_TOL
    assert rel(theta, theta_ref) <= 1e-8
    loss, n = plr.calc_loss(theta)
    assert abs(loss / n - oracle.calc_loss(X, y, theta_ref)) <= 1e-9


def test_device_resident_training_matches_oracle_and_per_round_path(plr, oracle, gen):
    # tool/lr_serial.cpp:95-110: rounds of delta + theta += delta, theta kept on the device
    cfg = gen.configs()["c1_dense_100k_x_100"].scaled(30000)
    X, y = cfg.rows(0, cfg.n)
    alpha, beta = cfg.lr / cfg.n, cfg.beta
    plr.set_data(X, y)
    theta, curve = plr.train_dgd(np.zeros(cfg.d), alpha, beta, 100, want_curve=True)
    theta_ref = oracle.train_dgd(X, y, np.zeros(cfg.d), alpha, beta, 100)
    assert rel(theta, theta_ref) <= 1e-8
    # the same rounds driven from the host, one plr_dgd_delta per round: identical bits
    th = np.zeros(cfg.d)
    losses = []
    for _ in range(100):
        delta, l = plr.dgd_delta(th, alpha, beta)
        losses.append(l)
        th = th + delta
    np.testing.assert_array_equal(theta, th)
    np.testing.assert_array_equal(curve, np.array(losses))
    assert abs(curve[0] - cfg.n * np.log(2.0)) <= 1e-12 * cfg.n and curve[-1] < curve[0]
    # zero rounds leave theta alone; no curve requested works too
    t0 = gen.gen_vec(5, gen.STREAM_THETA, cfg.d)
    np.testing.assert_array_equal(plr.train_dgd(t0, alpha, beta, 0), t0)
    np.testing.assert_array_equal(plr.train_dgd(np.zeros(cfg.d), alpha, beta, 100), theta)


@pytest.mark.parametrize("n,d", [(3000, 16), (2500, 81), (2000, 257), (1500, 1025), (500, 2500),
                                 (300, 4097), (200, 16385), (120, 20001)])
def test_device_resident_training_in_every_kernel_family(plr, oracle, gen, n, d):
    # packed rows, tail stage, one wave per row, several waves + tail, column blocks:
    # device-resident rounds give the bits of the host-driven loop, and the oracle's theta
    X, y, _ = make(gen, n, d, seed=0x7EA + d)
    alpha, beta = 0.1 / n, 0.005
    plr.set_data(X, y)
    print(plr.kernel_info(), flush=True)
    theta, curve = plr.train_dgd(np.zeros(d), alpha, beta, 6, want_curve=True)
    th = np.zeros(d)
    losses = []
    for _ in range(6):
        delta, l = plr.dgd_delta(th, alpha, beta)
        losses.append(l)
        th = th + delta
    np.testing.assert_array_equal(theta, th)
    np.testing.assert_array_equal(curve, np.array(losses))
    assert rel(theta, oracle.train_dgd(X, y, np.zeros(d), alpha, beta, 6)) <= 1e-8


def test_every_width_up_to_4400_against_numpy(plr):
    # variant selection has a case per chunk count, tail capacity and pitch rule: walk
    # every width (small shards, so this is about indexing, not bandwidth) against a
    # library-routine reference -- numpy GEMV + scipy expit / logaddexp in fp64
    from scipy.special import expit

    rng = np.random.default_rng(123)
    widths = list(range(1, 4400)) + list(range(4400, 20600, 97)) + [19455, 19456, 19457]
    for d in widths:
        n = 23 if d < 4400 else 11
        X = rng.normal(size=(n, d)) / np.sqrt(d)
        y = (rng.random(n) < 0.5) * 1.0
        th = rng.normal(size=d)
        plr.set_data(X, y)
        g, loss, n_out = plr.loss_grad(th, 1)
        z = X @ th
        g_ref = X.T @ (expit(z) - y)
        l_ref = np.sum(np.logaddexp(0.0, np.where(y == 1.0, -z, z)))
        ok = n_out == n and rel(g, g_ref) <= 1e-11 and abs(loss - l_ref) <= 1e-11 * l_ref
        assert ok, "d=%d: %s" % (d, plr.kernel_info())


@pytest.mark.parametrize("d", [3, 16, 64, 66, 95, 100, 130, 257, 1000, 1025, 2500, 4097, 16385,
                               20001])
def test_every_row_count_around_the_tile_sizes(plr, d):
    # partial tiles, partial tail loads, fewer rows than row groups: n = 0..139 in every family
    from scipy.special import expit

    rng = np.random.default_rng(d)
    Xall = rng.normal(size=(139, d)) / np.sqrt(d)
    yall = (rng.random(139) < 0.5) * 1.0
    th = rng.normal(size=d)
    for n in range(0, 140):
        X, y = Xall[:n], yall[:n]
        plr.set_data(X, y)
        g, loss, n_out = plr.loss_grad(th, 1)
        z = X @ th
        g_ref = X.T @ (expit(z) - y)
        l_ref = np.sum(np.logaddexp(0.0, np.where(y == 1.0, -z, z)))
        assert n_out == n
        assert np.linalg.norm(g - g_ref) <= 1e-11 * max(np.linalg.norm(g_ref), 1e-300), (n, d)
        assert abs(loss - l_ref) <= 1e-11 * max(l_ref, 1e-300), (n, d)
        h = plr.predict(th)
        assert h.shape == (n,) and (n == 0 or np.max(np.abs(h - expit(z))) <= 1e-14)


def _random_shapes(count, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        # widths spread over every kernel family, biased towards chunk / variant boundaries
        kind = rng.integers(0, 4)
        if kind == 0:
            d = int(rng.integers(1, 130))
        elif kind == 1:
            d = int(rng.choice([128, 256, 512, 1024, 2048, 4096, 8192]) + rng.integers(-3, 4))
        elif kind == 2:
            d = int(rng.integers(130, 9000))
        else:
            d = int(rng.integers(9000, 24000))
        n = int(rng.integers(1, max(2, min(3000, 3_000_000 // d))))
        out.append((n, d))
    return out


def test_random_shape_sweep(plr, oracle, gen):
    # 60 seeded shapes across all kernel families, gradient + loss against the oracle
    worst = 0.0
    for n, d in _random_shapes(60, 20240607):
        print("case n=%d d=%d" % (n, d), flush=True)
        X, y, th = make(gen, n, d, seed=n * 131 + d)
        plr.set_data(X, y)
        g, loss, n_out = plr.loss_grad(th)
        e = rel(g, oracle.gsum(X, y, th))
        worst = max(worst, e)
        assert n_out == n and e <= GRAD_TOL, (n, d, e, plr.kernel_info())
        want = oracle.calc_loss_sum(X, y, th)
        assert abs(loss - want) <= LOSS_TOL * want, (n, d, plr.kernel_info())
    print("worst gradient rel-L2 over the sweep: %.3e" % worst)
