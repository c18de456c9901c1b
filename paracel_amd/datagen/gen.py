import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(os.path.dirname(_HERE), "libplr_gen.so")

NORMAL, UNIFORM = 0, 1
STREAM_THETA, STREAM_THETA_STAR = 5, 6


class GenSpec(C.Structure):
    _fields_ = [("seed", C.c_uint64), ("kind", C.c_int32), ("outlier_mod", C.c_int32),
                ("scale", C.c_double), ("zero_prob", C.c_double), ("outlier_scale", C.c_double)]


_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise ImportError("%s is missing: run __graft_entry__.build()" % _LIB)
        lib = C.CDLL(_LIB)
        dp = C.POINTER(C.c_double)
        lib.plr_gen_X.argtypes = [C.POINTER(GenSpec), C.c_int64, C.c_int64, C.c_int64, C.c_int64, dp, C.c_int]
        lib.plr_gen_X.restype = None
        lib.plr_gen_vec.argtypes = [C.c_uint64, C.c_uint64, C.c_int, C.c_double, C.c_double, C.c_int64, dp]
        lib.plr_gen_vec.restype = None
        lib.plr_gen_labels.argtypes = [C.POINTER(GenSpec), C.c_int64, C.c_int64, C.c_int64, C.c_int64, dp, dp, dp, C.c_int]
        lib.plr_gen_labels.restype = None
        lib.plr_gen_u01.argtypes = [C.c_uint64] * 4
        lib.plr_gen_u01.restype = C.c_double
        lib.plr_gen_normal.argtypes = [C.c_uint64] * 4
        lib.plr_gen_normal.restype = C.c_double
        _lib = lib
    return _lib


def _dp(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


def default_threads():
    return max(1, min(16, os.cpu_count() or 1))


def gen_X(spec, row0, nrows, d, threads=None, out=None):
    X = out if out is not None else np.empty((nrows, d), dtype=np.float64)
    assert X.flags.c_contiguous and X.shape == (nrows, d)
    _load().plr_gen_X(C.byref(spec), row0, nrows, d, d, _dp(X), threads or default_threads())
    return X


def gen_vec(seed, stream, n, kind=NORMAL, scale=1.0, nonzero_frac=1.0):
    out = np.empty(n, dtype=np.float64)
    _load().plr_gen_vec(seed, stream, kind, scale, nonzero_frac, n, _dp(out))
    return out


def gen_labels(spec, row0, X, theta_star, threads=None):
    n, d = X.shape
    y = np.empty(n, dtype=np.float64)
    ts = np.ascontiguousarray(theta_star, dtype=np.float64)
    _load().plr_gen_labels(C.byref(spec), row0, n, d, d, _dp(X), _dp(ts), _dp(y),
                           threads or default_threads())
    return y


def u01(seed, stream, i, j):
    return _load().plr_gen_u01(seed, stream, i, j)


def normal(seed, stream, i, j):
    return _load().plr_gen_normal(seed, stream, i, j)


class Config:
    """One benchmark configuration: shape, distributions, hyper-parameters.

    alpha/beta are the reference's knobs (lr.cpp:119,134): the un-normalised
    update applies the L2 term once per sample, so plain gradient descent with
    step lr on mean log-loss + (lam/2)|theta|^2 is alpha = lr/n, beta = lam/2.
    """

    def __init__(self, name, n, d, seed, kind, scale, lam, lr=0.1, zero_prob=0.0,
                 outlier_mod=0, outlier_scale=1.0, theta_scale=1.0, theta_nonzero=1.0,
                 theta0_zero=False, bias_first=False):
        self.name, self.n, self.d, self.seed = name, n, d, seed
        self.spec = GenSpec(seed, kind, outlier_mod, scale, zero_prob, outlier_scale)
        self.lam, self.lr = lam, lr
        self.theta_scale, self.theta_nonzero = theta_scale, theta_nonzero
        self.theta0_zero = theta0_zero
        # column 0 is the constant 1.0 the worker's parser prepends (lr.cpp:83)
        self.bias_first = bias_first

    @property
    def alpha(self):
        return self.lr / self.n

    @property
    def beta(self):
        return self.lam / 2.0

    def scaled(self, n):
        """Same distributions and seed on the first n rows (alpha keeps the full n)."""
        c = Config.__new__(Config)
        c.__dict__.update(self.__dict__)
        c.n = n
        return c

    def theta_star(self):
        return gen_vec(self.seed, STREAM_THETA_STAR, self.d, NORMAL, self.theta_scale,
                       self.theta_nonzero)

    def theta(self):
        """theta the timed gradient step is evaluated at."""
        if self.theta0_zero:
            return np.zeros(self.d)
        return self.theta_star()

    def rows(self, row0, nrows, threads=None, out=None):
        """Rows [row0, row0+nrows) of the shard and their labels.  `out` (a
        C-contiguous nrows x d array) is filled in place when given."""
        X = gen_X(self.spec, row0, nrows, self.d, threads, out=out)
        if self.bias_first:
            X[:, 0] = 1.0
        y = gen_labels(self.spec, row0, X, self.theta_star(), threads)
        return X, y

    def algorithmic_bytes(self):
        """X once + y + theta in + gradient out + loss."""
        return 8 * self.n * self.d + 8 * self.n + 16 * self.d + 8


def configs():
    d2 = 1000
    return {
        # dense, CPU-runnable: X~N(0,1), theta*~N(0,1), theta0=0, lam=0.01, lr=0.1
        "c1_dense_100k_x_100": Config("c1_dense_100k_x_100", 100_000, 100, 0x5EED0001, NORMAL, 1.0,
                                      lam=0.01, theta0_zero=True),
        # headline: X~N(0,1/d), theta~N(0,1), y~Bernoulli(sigmoid(X theta))
        "c2_headline_1m_x_1000": Config("c2_headline_1m_x_1000", 1_000_000, d2, 0x5EED0002, NORMAL,
                                        1.0 / np.sqrt(d2), lam=0.01),
        # tall-skinny: U[-1,1], 1% of rows x100, theta*~N(0, sigma=0.1)
        "c3_tall_10m_x_256": Config("c3_tall_10m_x_256", 10_000_000, 256, 0x5EED0003, UNIFORM, 1.0,
                                    lam=0.001, outlier_mod=100, outlier_scale=100.0,
                                    theta_scale=0.1),
        # wide: 90% exact zeros, theta* nonzero on 5% of coordinates
        "c4_wide_200k_x_16384": Config("c4_wide_200k_x_16384", 200_000, 16384, 0x5EED0004, NORMAL,
                                       1.0, lam=0.1, zero_prob=0.9, theta_nonzero=0.05),
        "c4b_wide_200k_x_16385": Config("c4b_wide_200k_x_16385", 200_000, 16385, 0x5EED0004, NORMAL,
                                        1.0, lam=0.1, zero_prob=0.9, theta_nonzero=0.05),
        # config 3 as the file path sees it: 256 features + the bias column (lr.cpp:83) -- a row
        # that ends two columns past a chunk boundary (tail-stage kernel variant)
        "x_bias_10m_x_257": Config("x_bias_10m_x_257", 10_000_000, 257, 0x5EED0008, UNIFORM, 1.0,
                                   lam=0.001, outlier_mod=100, outlier_scale=100.0,
                                   theta_scale=0.1, bias_first=True),
        # 2048 features + the bias column
        "x_bias_1m_x_2049": Config("x_bias_1m_x_2049", 1_000_000, 2049, 0x5EED000C, NORMAL,
                                   1.0 / np.sqrt(2049), lam=0.01, bias_first=True),
        # rows of 65..96 columns at HBM-resident size: the half-wave-per-row kernel
        "x_short_30m_x_66": Config("x_short_30m_x_66", 30_000_000, 66, 0x5EED0009, NORMAL,
                                   1.0 / np.sqrt(66), lam=0.01),
        "x_short_30m_x_72": Config("x_short_30m_x_72", 30_000_000, 72, 0x5EED000A, NORMAL,
                                   1.0 / np.sqrt(72), lam=0.01),
        # config 1's shape (the reference tutorial's 100 features) at HBM-resident size
        "x_c1shape_20m_x_100": Config("x_c1shape_20m_x_100", 20_000_000, 100, 0x5EED000B, NORMAL,
                                      1.0, lam=0.01, theta0_zero=True),
        # narrow rows: the row-tiled layout, a lane per row
        "x_narrow_30m_x_16": Config("x_narrow_30m_x_16", 30_000_000, 16, 0x5EED0007, NORMAL, 0.25,
                                    lam=0.01),
        # ... at the narrowest width: one exp (and, with the loss, one log) per 16 bytes
        "x_narrow_100m_x_2": Config("x_narrow_100m_x_2", 100_000_000, 2, 0x5EED0010, NORMAL,
                                    1.0 / np.sqrt(2), lam=0.01),
        # ... at a width that is neither a power of two nor even
        "x_narrow_10m_x_41": Config("x_narrow_10m_x_41", 10_000_000, 41, 0x5EED000D, NORMAL,
                                    1.0 / np.sqrt(41), lam=0.01),
        # eight waves side by side, theta in LDS, the last wave one chunk short (71 chunks = 7 x 9 + 8)
        "x_wide_250k_x_9000": Config("x_wide_250k_x_9000", 250_000, 9000, 0x5EED0011, NORMAL,
                                     1.0 / np.sqrt(9000), lam=0.01),
        # wider than the widest one-workgroup kernel: column blocks, a team of workgroups per row
        "x_verywide_100k_x_32768": Config("x_verywide_100k_x_32768", 100_000, 32768, 0x5EED0006,
                                          NORMAL, 1.0, lam=0.1, zero_prob=0.9, theta_nonzero=0.05),
        # ... on dense data, at widths that do not fill the workgroups of a team evenly
        "x_wide_75k_x_20000": Config("x_wide_75k_x_20000", 75_000, 20000, 0x5EED000E, NORMAL,
                                     1.0 / np.sqrt(20000), lam=0.01),
        "x_wide_30k_x_50000": Config("x_wide_30k_x_50000", 30_000, 50000, 0x5EED000F, NORMAL,
                                     1.0 / np.sqrt(50000), lam=0.01),
        # end-to-end through the host parameter server
        "c5_e2e_2m_x_512": Config("c5_e2e_2m_x_512", 2_000_000, 512, 0x5EED0005, NORMAL,
                                  1.0 / np.sqrt(512), lam=0.01, theta0_zero=True),
    }
