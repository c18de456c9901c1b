"""The parameter-server shim and codec on the wire, driven from Python with the
real msgpack implementation and libzmq's C API (ctypes): requests are built the
way the reference's client builds them (include/client.hpp:523-539,
include/packer.hpp:43-51) and the replies are decoded with python-msgpack, so a
deviation of the C++ codec from the msgpack format shows up here.

Reference tests this mirrors: test/test_packer.cpp:128-147 (vector<double>
round trip), test/test_proxy.cpp:45-54 (update_proxy on packed values),
test/test_paste.cpp (field join/split).
"""
import ctypes as C
import os
import struct
import subprocess

import msgpack
import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "paracel_amd")
SEP = b"_PARACEL_"
ZMQ_REQ = 3


def _need_host_binaries():
    if not all(os.path.exists(os.path.join(PKG, f)) for f in
               ("plr_ps_server", "liblr_update.so")):
        subprocess.run(["make", "-C", os.path.join(PKG, "worker"), os.path.join("..", "plr_ps_server"),
                        os.path.join("..", "liblr_update.so")], check=True)


def field(obj):
    """packer::pack: 8-byte native size_t + msgpack bytes"""
    body = msgpack.packb(obj, use_bin_type=False)
    return struct.pack("=Q", len(body)) + body


def unfield(b):
    (n,) = struct.unpack("=Q", b[:8])
    assert len(b) == 8 + n
    return msgpack.unpackb(b[8:], raw=False)


class Zmq:
    def __init__(self):
        self.lib = C.CDLL("/opt/conda/lib/libzmq.so.5")
        self.lib.zmq_ctx_new.restype = C.c_void_p
        self.lib.zmq_socket.restype = C.c_void_p
        self.lib.zmq_socket.argtypes = [C.c_void_p, C.c_int]
        self.lib.zmq_connect.argtypes = [C.c_void_p, C.c_char_p]
        self.lib.zmq_send.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.c_int]
        self.lib.zmq_recv.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.c_int]
        self.lib.zmq_close.argtypes = [C.c_void_p]
        self.lib.zmq_setsockopt.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t]
        self.ctx = self.lib.zmq_ctx_new()
        self.socks = {}

    def req(self, host, port, payload):
        key = (host, port)
        if key not in self.socks:
            s = self.lib.zmq_socket(self.ctx, ZMQ_REQ)
            tmo = C.c_int(5000)
            self.lib.zmq_setsockopt(s, 27, C.byref(tmo), 4)  # ZMQ_RCVTIMEO
            zero = C.c_int(0)
            self.lib.zmq_setsockopt(s, 17, C.byref(zero), 4)  # ZMQ_LINGER
            assert self.lib.zmq_connect(s, ("tcp://%s:%s" % (host, port)).encode()) == 0
            self.socks[key] = s
        s = self.socks[key]
        assert self.lib.zmq_send(s, payload, len(payload), 0) == len(payload)
        buf = C.create_string_buffer(1 << 20)
        n = self.lib.zmq_recv(s, buf, len(buf), 0)
        assert n >= 0, "no reply from the server"
        return buf.raw[:n]

    def close(self):
        for s in self.socks.values():
            self.lib.zmq_close(s)


@pytest.fixture()
def server():
    _need_host_binaries()
    p = subprocess.Popen([os.path.join(PKG, "plr_ps_server")], stdout=subprocess.PIPE, text=True)
    info = p.stdout.readline().strip()
    host, ports = info.split(":")
    z = Zmq()
    yield z, host, ports.split(","), info
    z.close()
    p.kill()
    p.wait()


def test_server_info_format(server):
    _, host, ports, info = server
    assert host == "127.0.0.1" and len(ports) == 5 and all(p.isdigit() for p in ports)


def test_push_pull_bupdate_roundtrip(server):
    z, host, ports, _ = server
    theta = [1.23, -4.5, 1e-300, 3.0, 2.0 ** 60]
    # push on port[1]: the server stores the packed field verbatim and answers packed true
    r = z.req(host, ports[1], SEP.join([field("push"), field("theta"), field(theta)]))
    assert unfield(r) is True
    # pull on port[0]: the stored bytes come back unchanged
    r = z.req(host, ports[0], SEP.join([field("pull"), field("theta")]))
    assert r == field(theta) and unfield(r) == theta
    # contains
    assert unfield(z.req(host, ports[0], SEP.join([field("contains"), field("theta")]))) is True
    assert unfield(z.req(host, ports[0], SEP.join([field("contains"), field("nope")]))) is False
    # a missing key is answered with the raw bytes "nokey" (server.hpp:237-247)
    assert z.req(host, ports[0], SEP.join([field("pull"), field("missing")])) == b"nokey"
    # register the reducer plugin on port[3], then bupdate on the same port
    so = os.path.join(PKG, "liblr_update.so")
    r = z.req(host, ports[3], SEP.join([field("register_bupdate"), field(so), field("lr_theta_update")]))
    assert unfield(r) is True
    delta = [3.21, 0.5, 1e-300, -3.0, 1.0]
    r = z.req(host, ports[3], SEP.join([field("bupdate"), field("theta"), field(delta)]))
    want = [a + b for a, b in zip(theta, delta)]       # update.cpp:26-32; 1.23+3.21 as test_proxy.cpp
    assert unfield(r) == want                           # the reply is the new value
    assert unfield(z.req(host, ports[0], SEP.join([field("pull"), field("theta")]))) == want
    # first bupdate of a missing key = set (server.hpp:88-100)
    r = z.req(host, ports[3], SEP.join([field("bupdate"), field("fresh"), field(delta)]))
    assert unfield(r) == delta
    # integer table on the fifth port (client.hpp:456-467)
    assert unfield(z.req(host, ports[4], SEP.join([field("push_int"), field("worker_sz"), field(4)]))) is True
    assert unfield(z.req(host, ports[4], SEP.join([field("pull_int"), field("worker_sz")]))) == 4


def test_vector_lengths_cross_every_array_header(server):
    # fixarray (<=15), array16 (<=65535), array32
    z, host, ports, _ = server
    rng = np.random.default_rng(0)
    so = os.path.join(PKG, "liblr_update.so")
    z.req(host, ports[3], SEP.join([field("register_bupdate"), field(so), field("lr_theta_update")]))
    for n in (0, 1, 15, 16, 513, 65535, 65536):
        a, b = rng.normal(size=n).tolist(), rng.normal(size=n).tolist()
        key = "v%d" % n
        assert unfield(z.req(host, ports[1], SEP.join([field("push"), field(key), field(a)]))) is True
        r = z.req(host, ports[3], SEP.join([field("bupdate"), field(key), field(b)]))
        got = unfield(r)
        assert got == [x + y for x, y in zip(a, b)]
        # the C++ encoder emits the same bytes python-msgpack does
        assert r == field(got)


def test_integers_arrive_as_doubles(server):
    # msgpack-c converts integer objects to double on request; a vector packed as ints must add up
    z, host, ports, _ = server
    so = os.path.join(PKG, "liblr_update.so")
    z.req(host, ports[3], SEP.join([field("register_bupdate"), field(so), field("lr_theta_update")]))
    z.req(host, ports[1], SEP.join([field("push"), field("ints"), field([1, -2, 300, 70000, -70000])]))
    r = z.req(host, ports[3], SEP.join([field("bupdate"), field("ints"), field([0.5] * 5)]))
    assert unfield(r) == [1.5, -1.5, 300.5, 70000.5, -69999.5]
