"""ctypes binding of the C ABI in ``include/plr.h``.

Thin by design: every method is one ``plr_*`` call on host numpy buffers.  The
binding is what the parity tests and ``bench.py`` drive; the C++ worker in
``paracel_amd/worker`` calls the same entry points directly.
"""
import ctypes as C
import os

import numpy as np

PLR_LOSS_REFERENCE = 0
PLR_LOSS_STABLE = 1
PLR_LOSS_NONE = 2
PLR_LOSS_SQUARED = 3

_HERE = os.path.dirname(os.path.abspath(__file__))

# every symbol include/plr.h declares: (name, restype, argtypes)
_dp = C.POINTER(C.c_double)
_i64p = C.POINTER(C.c_int64)
_ctx = C.c_void_p
SYMBOLS = [
    ("plr_create", C.c_int, [C.POINTER(_ctx), C.c_int]),
    ("plr_destroy", None, [_ctx]),
    ("plr_set_data", C.c_int, [_ctx, _dp, C.c_int64, C.c_int64, C.c_int64, _dp]),
    ("plr_alloc_data", C.c_int, [_ctx, C.c_int64, C.c_int64]),
    ("plr_set_data_chunk", C.c_int, [_ctx, C.c_int64, C.c_int64, _dp, C.c_int64, _dp]),
    ("plr_set_data_csv", C.c_int, [_ctx, C.POINTER(C.c_char_p), _i64p, C.c_int, C.c_char, _i64p,
                                   _i64p]),
    ("plr_get_data", C.c_int, [_ctx, C.c_int64, C.c_int64, _dp, C.c_int64, _dp]),
    ("plr_loss_grad", C.c_int, [_ctx, _dp, _dp, _dp, _i64p, C.c_uint]),
    ("plr_dgd_delta", C.c_int, [_ctx, _dp, C.c_double, C.c_double, _dp, _dp]),
    ("plr_dgd_delta_linear", C.c_int, [_ctx, _dp, C.c_double, C.c_double, _dp, _dp]),
    ("plr_train_dgd", C.c_int, [_ctx, _dp, C.c_double, C.c_double, C.c_int, _dp]),
    ("plr_calc_loss", C.c_int, [_ctx, _dp, _dp, _i64p, C.c_uint]),
    ("plr_predict", C.c_int, [_ctx, _dp, _dp]),
    ("plr_predict_linear", C.c_int, [_ctx, _dp, _dp]),
    ("plr_loss_grad_noalloc", C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                        C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_uint]),
    ("plr_synchronize", C.c_int, [_ctx]),
    ("plr_set_timing", C.c_int, [_ctx, C.c_int]),
    ("plr_set_option", C.c_int, [_ctx, C.c_char_p, C.c_int64]),
    ("plr_probe_copy_bandwidth", C.c_int, [_ctx, C.c_int64, C.c_int, C.POINTER(C.c_double)]),
    ("plr_get_shape", C.c_int, [_ctx, _i64p, _i64p]),
    ("plr_get_timing", C.c_int, [_ctx, _dp, _dp, _i64p]),
    ("plr_reset_timing", C.c_int, [_ctx]),
    ("plr_probe_read_bandwidth", C.c_int, [_ctx, C.c_int, _dp]),
    ("plr_kernel_info", C.c_char_p, [_ctx]),
    ("plr_last_error", C.c_char_p, [_ctx]),
    ("plr_version", C.c_char_p, []),
]


class PlrError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("plr error %d: %s" % (code, msg))
        self.code = code


def lib_path():
    return os.path.join(_HERE, "libplr.so")


_lib = None


def load_library():
    """Load libplr.so and type every entry point; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError(
            "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(hipcc --offload-arch=gfx950); there is no CPU fallback" % path)
    lib = C.CDLL(path)
    for name, res, args in SYMBOLS:
        fn = getattr(lib, name)  # AttributeError if the ABI lost a symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _vec(a, n=None, name="array"):
    a = np.ascontiguousarray(a, dtype=np.float64)
    if n is not None and a.size != n:
        raise ValueError("%s has %d entries, expected %d" % (name, a.size, n))
    return a


def _p(a):
    return a.ctypes.data_as(_dp) if a is not None else None


def loss_grad_noalloc(dX, dy, n, d, ldx, dtheta, dout, flags=PLR_LOSS_REFERENCE, device=0,
                      stream=None):
    """plr_loss_grad_noalloc on raw DEVICE addresses (ints); enqueues on `stream`
    (a hipStream_t as an int, None = the default stream) and returns at once."""
    lib = load_library()
    rc = lib.plr_loss_grad_noalloc(int(device), C.c_void_p(stream), C.c_void_p(dX),
                                   C.c_void_p(dy), n, d, ldx, C.c_void_p(dtheta),
                                   C.c_void_p(dout), flags)
    if rc != 0:
        raise PlrError(rc, lib.plr_last_error(None).decode())


class Plr:
    """One shard context (``plr_ctx``) on one GPU."""

    def __init__(self, device=0):
        self._lib = load_library()
        h = _ctx()
        rc = self._lib.plr_create(C.byref(h), int(device))
        if rc != 0:
            raise PlrError(rc, self._lib.plr_last_error(None).decode())
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._lib.plr_destroy(self._h)
            self._h = None

    __del__ = close

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _check(self, rc):
        if rc != 0:
            raise PlrError(rc, self._lib.plr_last_error(self._h).decode())

    # -- shard ------------------------------------------------------------
    def set_data(self, X, y):
        X = np.asarray(X, dtype=np.float64)
        if X.ndim != 2:
            raise ValueError("X must be 2-D")
        if X.shape[0] and X.strides[1] != 8:
            X = np.ascontiguousarray(X)
        n, d = X.shape
        ldx = X.strides[0] // 8 if n > 1 else d
        if ldx < d:
            X = np.ascontiguousarray(X)
            ldx = d
        y = _vec(y, n, "y")
        self._shape = None
        self._check(self._lib.plr_set_data(self._h, _p(X), n, d, ldx, _p(y)))

    def alloc_data(self, n, d):
        self._shape = None
        self._check(self._lib.plr_alloc_data(self._h, n, d))

    def set_data_chunk(self, row0, X, y):
        X = np.asarray(X, dtype=np.float64)
        if X.ndim != 2:
            raise ValueError("X must be 2-D")
        if X.shape[0] and X.strides[1] != 8:
            X = np.ascontiguousarray(X)
        m, d = X.shape
        ldx = X.strides[0] // 8 if m > 1 else d
        if ldx < d:
            X = np.ascontiguousarray(X)
            ldx = d
        y = _vec(y, m, "y")
        self._check(self._lib.plr_set_data_chunk(self._h, row0, m, _p(X), ldx, _p(y)))

    def set_data_csv(self, texts, sep=","):
        """Sample text (bytes, or a list of pieces) -> resident shard, parsed on the device;
        returns (n, d) with d counting the constant first column."""
        if isinstance(texts, (bytes, bytearray, memoryview)):
            texts = [texts]
        texts = [bytes(t) for t in texts]
        arr = (C.c_char_p * len(texts))(*texts)
        lens = (C.c_int64 * len(texts))(*[len(t) for t in texts])
        n, d = C.c_int64(), C.c_int64()
        self._shape = None
        self._check(self._lib.plr_set_data_csv(self._h, arr, lens, len(texts),
                                               sep.encode()[0:1], C.byref(n), C.byref(d)))
        return n.value, d.value

    def get_data(self, row0=0, nrows=None):
        """Rows of the resident shard as (X, y) in the form set_data takes."""
        n, d = self.shape
        if nrows is None:
            nrows = n - row0
        X = np.empty((nrows, d))
        y = np.empty(nrows)
        self._check(self._lib.plr_get_data(self._h, row0, nrows, _p(X), d, _p(y)))
        return X, y

    @property
    def shape(self):
        # asked of the library once per resident shard (the per-step calls use it)
        if getattr(self, "_shape", None) is None:
            n, d = C.c_int64(), C.c_int64()
            self._check(self._lib.plr_get_shape(self._h, C.byref(n), C.byref(d)))
            if n.value == 0 and d.value == 0:
                return 0, 0
            self._shape = (n.value, d.value)
        return self._shape

    # -- compute ----------------------------------------------------------
    def loss_grad(self, theta, flags=PLR_LOSS_REFERENCE):
        """(gsum[d], loss_sum, n) = one fused pass over the resident shard."""
        d = self.shape[1]
        theta = _vec(theta, d, "theta")
        g = np.empty(d, dtype=np.float64)
        loss, n = C.c_double(), C.c_int64()
        self._check(self._lib.plr_loss_grad(self._h, _p(theta), _p(g), C.byref(loss),
                                            C.byref(n), flags))
        return g, loss.value, n.value

    def dgd_delta(self, theta, alpha, beta, want_loss=True):
        d = self.shape[1]
        theta = _vec(theta, d, "theta")
        delta = np.empty(d, dtype=np.float64)
        loss = C.c_double()
        self._check(self._lib.plr_dgd_delta(self._h, _p(theta), alpha, beta, _p(delta),
                                            C.byref(loss) if want_loss else None))
        return delta, (loss.value if want_loss else None)

    def dgd_delta_linear(self, theta, alpha, beta):
        """(delta, squared-loss sum) of the linear model's full-batch round."""
        d = self.shape[1]
        theta = _vec(theta, d, "theta")
        delta = np.empty(d, dtype=np.float64)
        loss = C.c_double()
        self._check(self._lib.plr_dgd_delta_linear(self._h, _p(theta), alpha, beta, _p(delta),
                                                   C.byref(loss)))
        return delta, loss.value

    def train_dgd(self, theta0, alpha, beta, rounds, want_curve=False):
        """theta after `rounds` device-resident rounds (and the per-round loss sums)."""
        d = self.shape[1]
        theta = np.array(_vec(theta0, d, "theta"), copy=True)
        curve = np.empty(rounds, dtype=np.float64) if want_curve else None
        self._check(self._lib.plr_train_dgd(self._h, _p(theta), alpha, beta, rounds, _p(curve)))
        return (theta, curve) if want_curve else theta

    def calc_loss(self, theta, flags=PLR_LOSS_REFERENCE):
        d = self.shape[1]
        theta = _vec(theta, d, "theta")
        loss, n = C.c_double(), C.c_int64()
        self._check(self._lib.plr_calc_loss(self._h, _p(theta), C.byref(loss), C.byref(n), flags))
        return loss.value, n.value

    def predict(self, theta):
        n, d = self.shape
        theta = _vec(theta, d, "theta")
        h = np.empty(n, dtype=np.float64)
        self._check(self._lib.plr_predict(self._h, _p(theta), _p(h)))
        return h

    def predict_linear(self, theta):
        n, d = self.shape
        theta = _vec(theta, d, "theta")
        z = np.empty(n, dtype=np.float64)
        self._check(self._lib.plr_predict_linear(self._h, _p(theta), _p(z)))
        return z

    def synchronize(self):
        self._check(self._lib.plr_synchronize(self._h))

    # -- timing / info ----------------------------------------------------
    def timing(self):
        last, total, cnt = C.c_double(), C.c_double(), C.c_int64()
        self._check(self._lib.plr_get_timing(self._h, C.byref(last), C.byref(total), C.byref(cnt)))
        return last.value, total.value, cnt.value

    def reset_timing(self):
        self._check(self._lib.plr_reset_timing(self._h))

    def set_timing(self, enabled):
        """Timing events on (default) or off (saves 6-8 us per call)."""
        self._check(self._lib.plr_set_timing(self._h, 1 if enabled else 0))

    def set_option(self, key, value):
        """plr_set_option: "column_blocks_two_sweeps", "team_spin_limit"."""
        self._check(self._lib.plr_set_option(self._h, key.encode(), int(value)))

    def probe_copy_bandwidth(self, nbytes=1 << 30, reps=5):
        """GB/s (read + written) of the runtime's device-to-device copy of nbytes."""
        gbs = C.c_double()
        self._check(self._lib.plr_probe_copy_bandwidth(self._h, nbytes, reps, C.byref(gbs)))
        return gbs.value

    def probe_read_bandwidth(self, reps=10):
        """GB/s a pure streaming read of the resident shard sustains."""
        gbs = C.c_double()
        self._check(self._lib.plr_probe_read_bandwidth(self._h, reps, C.byref(gbs)))
        return gbs.value

    def kernel_info(self):
        return self._lib.plr_kernel_info(self._h).decode()
