import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _ensure_cpu_libs():
    """The CPU-side helpers (oracle, generator) are cheap to build on demand;
    the HIP library is never built from a test."""
    import subprocess

    if not os.path.exists(os.path.join(ROOT, "oracle", "liblr_oracle.so")):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True)
    if not os.path.exists(os.path.join(ROOT, "paracel_amd", "libplr_gen.so")):
        from paracel_amd import build

        build.build_libplr_gen()


_ensure_cpu_libs()


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o

    o.load()
    return o


@pytest.fixture(scope="session")
def gen():
    from paracel_amd.datagen import gen as g

    return g


@pytest.fixture()
def plr():
    """A fresh shard context on GPU 0 (fails loudly if libplr.so is absent)."""
    from paracel_amd import Plr

    ctx = Plr(0)
    yield ctx
    ctx.close()
