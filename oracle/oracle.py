"""ctypes loader of the CPU oracle (liblr_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py -- never by the paracel_amd package.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "liblr_oracle.so")
_dp = C.POINTER(C.c_double)
_i64p = C.POINTER(C.c_int64)
_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_PATH):
            raise ImportError("%s is missing: run `make -C oracle`" % _PATH)
        L = C.CDLL(_PATH)
        shp = [_dp, C.c_int64, C.c_int64, C.c_int64]
        L.oracle_dot_product.restype = C.c_double
        L.oracle_dot_product.argtypes = [_dp, _dp, C.c_int64]
        L.oracle_lr_hypothesis.restype = C.c_double
        L.oracle_lr_hypothesis.argtypes = [_dp, _dp, C.c_int64]
        L.oracle_dgd_delta.restype = None
        L.oracle_dgd_delta.argtypes = shp + [_dp, _dp, C.c_double, C.c_double, _i64p, _dp]
        for f in ("oracle_calc_loss_sum", "oracle_calc_loss", "oracle_calc_loss_sum_hp",
                  "oracle_stable_loss_sum_hp", "oracle_ridge_loss_sum"):
            getattr(L, f).restype = C.c_double
            getattr(L, f).argtypes = shp + [_dp, _dp]
        L.oracle_theta_update.restype = None
        L.oracle_theta_update.argtypes = [_dp, _dp, C.c_int64, _dp]
        for f in ("oracle_predict", "oracle_predict_linear"):
            getattr(L, f).restype = None
            getattr(L, f).argtypes = shp + [_dp, _dp]
        for f in ("oracle_gsum", "oracle_gsum_hp", "oracle_lsq_gsum"):
            getattr(L, f).restype = None
            getattr(L, f).argtypes = shp + [_dp, _dp, _dp]
        L.oracle_train_dgd.restype = None
        L.oracle_train_dgd.argtypes = shp + [_dp, _dp, C.c_double, C.c_double, C.c_int]
        L.oracle_train_dgd_workers.restype = None
        L.oracle_train_dgd_workers.argtypes = shp + [_dp, _dp, C.c_double, C.c_double, C.c_int, C.c_int]
        L.oracle_ridge_delta.restype = None
        L.oracle_ridge_delta.argtypes = shp + [_dp, _dp, C.c_double, C.c_double, _dp]
        L.oracle_ridge_train_workers.restype = None
        L.oracle_ridge_train_workers.argtypes = shp + [_dp, _dp, C.c_double, C.c_double, C.c_int,
                                                       C.c_int]
        L.oracle_dgd_delta_hp.restype = None
        L.oracle_dgd_delta_hp.argtypes = shp + [_dp, _dp, C.c_double, C.c_double, _dp]
        L.oracle_local_parser.restype = C.c_int64
        L.oracle_local_parser.argtypes = [C.c_char_p, C.c_int64, C.c_char, _dp, _dp, C.c_int64]
        L.oracle_baseline_time.restype = C.c_double
        L.oracle_baseline_time.argtypes = shp + [_dp, _dp, C.c_double, C.c_double, C.c_int,
                                                 C.c_int, _dp, _dp, _dp]
        _lib = L
    return _lib


def _c(a):
    return np.ascontiguousarray(a, dtype=np.float64)


def _p(a):
    return a.ctypes.data_as(_dp)


def _shape(X):
    X = _c(X)
    if X.ndim != 2:
        raise ValueError("X must be 2-D")
    n, d = X.shape
    return X, n, d


def dot_product(a, b):
    a, b = _c(a), _c(b)
    return load().oracle_dot_product(_p(a), _p(b), a.size)


def lr_hypothesis(x, theta):
    x, theta = _c(x), _c(theta)
    return load().oracle_lr_hypothesis(_p(x), _p(theta), x.size)


def dgd_delta(X, y, theta, alpha, beta, order=None):
    X, n, d = _shape(X)
    y, theta = _c(y), _c(theta)
    out = np.empty(d)
    op = None
    if order is not None:
        order = np.ascontiguousarray(order, dtype=np.int64)
        op = order.ctypes.data_as(_i64p)
    load().oracle_dgd_delta(_p(X), n, d, d, _p(y), _p(theta), alpha, beta, op, _p(out))
    return out


def dgd_delta_hp(X, y, theta, alpha, beta):
    X, n, d = _shape(X)
    y, theta = _c(y), _c(theta)
    out = np.empty(d)
    load().oracle_dgd_delta_hp(_p(X), n, d, d, _p(y), _p(theta), alpha, beta, _p(out))
    return out


def _loss(fn, X, y, theta):
    X, n, d = _shape(X)
    y, theta = _c(y), _c(theta)
    return getattr(load(), fn)(_p(X), n, d, d, _p(y), _p(theta))


def calc_loss_sum(X, y, theta):
    return _loss("oracle_calc_loss_sum", X, y, theta)


def calc_loss(X, y, theta):
    return _loss("oracle_calc_loss", X, y, theta)


def calc_loss_sum_hp(X, y, theta):
    return _loss("oracle_calc_loss_sum_hp", X, y, theta)


def stable_loss_sum_hp(X, y, theta):
    return _loss("oracle_stable_loss_sum_hp", X, y, theta)


def ridge_loss_sum(X, y, theta):
    return _loss("oracle_ridge_loss_sum", X, y, theta)


def predict_linear(X, theta):
    X, n, d = _shape(X)
    theta = _c(theta)
    out = np.empty(n)
    load().oracle_predict_linear(_p(X), n, d, d, _p(theta), _p(out))
    return out


def lsq_gsum(X, y, theta):
    X, n, d = _shape(X)
    y, theta = _c(y), _c(theta)
    out = np.empty(d)
    load().oracle_lsq_gsum(_p(X), n, d, d, _p(y), _p(theta), _p(out))
    return out


def ridge_delta(X, y, theta, alpha, beta):
    X, n, d = _shape(X)
    y, theta = _c(y), _c(theta)
    out = np.empty(d)
    load().oracle_ridge_delta(_p(X), n, d, d, _p(y), _p(theta), alpha, beta, _p(out))
    return out


def ridge_train_workers(X, y, theta0, alpha, beta, rounds, workers=1):
    X, n, d = _shape(X)
    y = _c(y)
    theta = np.array(theta0, dtype=np.float64, copy=True)
    load().oracle_ridge_train_workers(_p(X), n, d, d, _p(y), _p(theta), alpha, beta, rounds,
                                      workers)
    return theta


def theta_update(a, b):
    a, b = _c(a), _c(b)
    out = np.empty_like(a)
    load().oracle_theta_update(_p(a), _p(b), a.size, _p(out))
    return out


def predict(X, theta):
    X, n, d = _shape(X)
    theta = _c(theta)
    out = np.empty(n)
    load().oracle_predict(_p(X), n, d, d, _p(theta), _p(out))
    return out


def gsum(X, y, theta, hp=False):
    X, n, d = _shape(X)
    y, theta = _c(y), _c(theta)
    out = np.empty(d)
    getattr(load(), "oracle_gsum_hp" if hp else "oracle_gsum")(_p(X), n, d, d, _p(y), _p(theta),
                                                               _p(out))
    return out


def train_dgd(X, y, theta0, alpha, beta, rounds):
    X, n, d = _shape(X)
    y = _c(y)
    theta = np.array(theta0, dtype=np.float64, copy=True)
    load().oracle_train_dgd(_p(X), n, d, d, _p(y), _p(theta), alpha, beta, rounds)
    return theta


def train_dgd_workers(X, y, theta0, alpha, beta, rounds, workers):
    X, n, d = _shape(X)
    y = _c(y)
    theta = np.array(theta0, dtype=np.float64, copy=True)
    load().oracle_train_dgd_workers(_p(X), n, d, d, _p(y), _p(theta), alpha, beta, rounds, workers)
    return theta


def local_parser(text, sep=",", k_expected=-1):
    lines = [ln for ln in text.split("\n") if ln != ""]
    nlines = len(lines)
    blob = "\n".join(lines).encode()
    width = max(len(ln.split(sep)) for ln in lines) + 1 if lines else 1
    X = np.zeros(nlines * width)
    y = np.zeros(nlines)
    D = load().oracle_local_parser(blob, nlines, sep.encode(), _p(X), _p(y), k_expected)
    if D < 0:
        raise ValueError("unparsable or ragged input")
    return X[: nlines * D].reshape(nlines, D).copy(), y


def baseline_time(X, y, theta, alpha, beta, threads=1, reps=1, with_loss=True):
    """seconds per traversal (lr.cpp:132-138) in the reference's own layout."""
    X, n, d = _shape(X)
    y, theta = _c(y), _c(theta)
    delta = np.empty(d)
    ls, lv = C.c_double(), C.c_double()
    sec = load().oracle_baseline_time(_p(X), n, d, d, _p(y), _p(theta), alpha, beta, threads, reps,
                                      _p(delta), C.byref(ls) if with_loss else None,
                                      C.byref(lv) if with_loss else None)
    return sec, delta, (ls.value if with_loss else None), (lv.value if with_loss else None)
