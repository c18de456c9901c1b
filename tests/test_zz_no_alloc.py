"""plr_loss_grad_noalloc (the entry point that allocates nothing: static device
scratch, device pointers in and out) against plr_loss_grad on the same shard,
through the C ABI: two calls in a row, the second with a smaller input, then
the refusals.  The device buffers the caller passes come from the HIP runtime
itself (hipMalloc / hipMemcpy through ctypes), as a C caller's would."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL = 1e-12  # both entry points run the same kernels; the bar of the parity tests is 1e-10


class DevBuf:
    """A device allocation filled from (and read back into) a numpy array."""

    _hip = None

    @classmethod
    def hip(cls):
        if cls._hip is None:
            h = C.CDLL("libamdhip64.so.7")  # the runtime libplr.so is linked against
            h.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
            h.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
            h.hipFree.argtypes = [C.c_void_p]
            cls._hip = h
        return cls._hip

    def __init__(self, host):
        host = np.ascontiguousarray(host, dtype=np.float64)
        self.shape = host.shape
        self.nbytes = max(host.nbytes, 8)
        p = C.c_void_p()
        assert self.hip().hipMalloc(C.byref(p), self.nbytes) == 0
        self.ptr = p.value
        if host.nbytes:
            assert self.hip().hipMemcpy(self.ptr, host.ctypes.data, host.nbytes, 1) == 0

    def numpy(self):
        out = np.empty(self.shape)
        assert self.hip().hipDeviceSynchronize() == 0
        if out.nbytes:
            assert self.hip().hipMemcpy(out.ctypes.data, self.ptr, out.nbytes, 2) == 0
        return out

    def free(self):
        if self.ptr:
            self.hip().hipFree(self.ptr)
            self.ptr = None


def _device_inputs(X, y, theta, ldx):
    n, d = X.shape
    Xp = np.zeros((n, ldx))
    Xp[:, :d] = X
    # dout poisoned, so that anything the call leaves unwritten shows
    return DevBuf(Xp), DevBuf(y), DevBuf(theta), DevBuf(np.full(d + 1, np.nan))


def _one(capi, plr, gen, n, d, ldx, seed, flags=0):
    spec = gen.GenSpec(seed, gen.NORMAL, 0, 1.0 / np.sqrt(d), 0.0, 1.0)
    X = gen.gen_X(spec, 0, n, d)
    y = gen.gen_labels(spec, 0, X, gen.gen_vec(seed, gen.STREAM_THETA_STAR, d, gen.NORMAL, 1.0))
    theta = gen.gen_vec(seed, gen.STREAM_THETA, d, gen.NORMAL, 1.0)
    plr.set_data(X, y)
    g_ref, loss_ref, n_ref = plr.loss_grad(theta, flags)
    dX, dy, dth, dout = _device_inputs(X, y, theta, ldx)
    capi.loss_grad_noalloc(dX.ptr, dy.ptr, n, d, ldx, dth.ptr, dout.ptr, flags)
    out = dout.numpy()  # synchronises the device first
    for b in (dX, dy, dth, dout):
        b.free()
    assert n_ref == n
    assert np.all(np.isfinite(out)), "the call left part of dout unwritten"
    eg = np.linalg.norm(out[:d] - g_ref) / np.linalg.norm(g_ref)
    el = abs(out[d] - loss_ref) / abs(loss_ref)
    print("noalloc n=%d d=%d ldx=%d: grad rel %.2e loss rel %.2e bitwise=%s" %
          (n, d, ldx, eg, el, np.array_equal(out[:d], g_ref) and out[d] == loss_ref), flush=True)
    assert eg <= REL and el <= REL, (eg, el)


def test_noalloc_matches_loss_grad_on_two_calls_the_second_smaller(plr, gen):
    from paracel_amd import capi

    # big first, then smaller in rows AND columns: whatever the first call left in the
    # static array (theta beyond the new width, partials of more workgroups) must not leak
    _one(capi, plr, gen, 40000, 1000, 1024, 11)
    _one(capi, plr, gen, 777, 100, 128, 12)
    # and up again, other formulas, a pitch with spare chunks
    _one(capi, plr, gen, 5000, 257, 384, 13, flags=1)
    _one(capi, plr, gen, 3000, 513, 2048, 14, flags=3)


def test_noalloc_empty_shard_and_refusals(plr, gen):
    from paracel_amd import PlrError, capi

    d, ldx = 100, 128
    dth, dout = DevBuf(np.zeros(d)), DevBuf(np.full(d + 1, np.nan))
    capi.loss_grad_noalloc(None, None, 0, d, ldx, dth.ptr, dout.ptr)
    assert np.array_equal(dout.numpy(), np.zeros(d + 1))

    dX, dy = DevBuf(np.zeros((4, 4096))), DevBuf(np.zeros(4))
    dth, dout = DevBuf(np.zeros(4096)), DevBuf(np.zeros(4097))
    for args, what in [((4, 3000, 4096), "limit"),      # beyond the static array
                       ((4, 100, 100), "multiple of 128"),  # pitch not whole chunks
                       ((4, 200, 128), "multiple of 128"),  # ldx < d
                       ((-1, 100, 128), "n >= 0")]:
        with pytest.raises(PlrError) as e:
            capi.loss_grad_noalloc(dX.ptr, dy.ptr, args[0], args[1], args[2], dth.ptr, dout.ptr)
        assert e.value.code == -1 and what in str(e.value), str(e.value)
    with pytest.raises(PlrError):
        capi.loss_grad_noalloc(dX.ptr, dy.ptr, 4, 100, 128, None, dout.ptr)
