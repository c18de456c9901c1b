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


def _free_bytes(hip):
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_noalloc_leaves_device_memory_as_it_found_it(plr, gen):
    # what the name promises: once the first call on the device has looked up the static
    # array, calls neither take nor return device memory, whatever their size
    from paracel_amd import PlrError, capi

    hip = DevBuf.hip()
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    rng = np.random.default_rng(3)
    n, d, ldx = 5000, 300, 384
    X = rng.normal(size=(n, d)) / np.sqrt(d)
    y = (rng.random(n) < 0.5) * 1.0
    dX, dy, dth, dout = _device_inputs(X, y, rng.normal(size=d), ldx)
    capi.loss_grad_noalloc(dX.ptr, dy.ptr, n, d, ldx, dth.ptr, dout.ptr)   # first call: set-up
    assert hip.hipDeviceSynchronize() == 0
    before = _free_bytes(hip)
    for rows, cols, pitch, flags in ((n, d, ldx, 0), (n // 3, 200, ldx, 1), (17, d, ldx, 3),
                                     (0, d, ldx, 0), (n, d, ldx, 2)):
        capi.loss_grad_noalloc(dX.ptr, dy.ptr, rows, cols, pitch, dth.ptr, dout.ptr, flags)
    assert hip.hipDeviceSynchronize() == 0
    assert _free_bytes(hip) == before
    # the pass loads X 16 bytes per lane: a pointer that is not 16-byte aligned is refused
    with pytest.raises(PlrError) as e:
        capi.loss_grad_noalloc(dX.ptr + 8, dy.ptr, n - 1, d, ldx, dth.ptr, dout.ptr)
    assert e.value.code == -1 and "16-byte aligned" in str(e.value)
    for b in (dX, dy, dth, dout):
        b.free()


def test_noalloc_under_stream_capture(plr, gen):
    # the caller it is for: a stream under capture.  The first call per device and pitch (the
    # look-ups) is made before the capture begins; the captured call then only enqueues
    # kernels.  The graph is replayed several times, with eager work and synchronisations in
    # between, and every replay must give the eager call's bits.
    from paracel_amd import capi

    hip = DevBuf.hip()
    for f, args in (("hipStreamCreate", [C.POINTER(C.c_void_p)]),
                    ("hipStreamBeginCapture", [C.c_void_p, C.c_int]),
                    ("hipStreamEndCapture", [C.c_void_p, C.POINTER(C.c_void_p)]),
                    ("hipGraphInstantiate", [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p,
                                             C.c_char_p, C.c_size_t]),
                    ("hipGraphLaunch", [C.c_void_p, C.c_void_p]),
                    ("hipStreamSynchronize", [C.c_void_p]),
                    ("hipGraphExecDestroy", [C.c_void_p]), ("hipGraphDestroy", [C.c_void_p]),
                    ("hipStreamDestroy", [C.c_void_p])):
        getattr(hip, f).argtypes = args
    rng = np.random.default_rng(8)
    n, d, ldx = 9000, 500, 512
    X = rng.normal(size=(n, d)) / np.sqrt(d)
    y = (rng.random(n) < 0.5) * 1.0
    theta = rng.normal(size=d)
    dX, dy, dth, dout = _device_inputs(X, y, theta, ldx)
    stream = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(stream)) == 0
    # eager, on the same stream: the reference bits, and the set-up of this device and pitch
    capi.loss_grad_noalloc(dX.ptr, dy.ptr, n, d, ldx, dth.ptr, dout.ptr, stream=stream.value)
    assert hip.hipStreamSynchronize(stream) == 0
    want = dout.numpy()
    assert np.all(np.isfinite(want))
    graph, gexec = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 0) == 0          # hipStreamCaptureModeGlobal
    try:
        capi.loss_grad_noalloc(dX.ptr, dy.ptr, n, d, ldx, dth.ptr, dout.ptr, stream=stream.value)
    finally:
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
    poison = np.full(d + 1, np.nan)
    for replay in range(4):
        assert hip.hipMemcpy(dout.ptr, poison.ctypes.data, poison.nbytes, 1) == 0
        assert hip.hipGraphLaunch(gexec, stream) == 0
        assert hip.hipStreamSynchronize(stream) == 0
        got = dout.numpy()
        assert np.array_equal(got, want), "replay %d differs from the eager call" % replay
        # the program's own eager work between replays: another shape through the same array
        capi.loss_grad_noalloc(dX.ptr, dy.ptr, 333, 100, ldx, dth.ptr, dout.ptr,
                               stream=stream.value)
        assert hip.hipStreamSynchronize(stream) == 0
    assert hip.hipGraphExecDestroy(gexec) == 0 and hip.hipGraphDestroy(graph) == 0
    assert hip.hipStreamDestroy(stream) == 0
    for b in (dX, dy, dth, dout):
        b.free()
