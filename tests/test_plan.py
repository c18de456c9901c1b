"""The width -> kernel-variant choice (paracel_amd/csrc/plr_plan.hpp), checked
on the host for every width: pitch rules, chunk coverage, tail capacities,
LDS budget, and that no variant of the table is dead."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "paracel_amd", "plr_plan_check")


@pytest.fixture(scope="module", autouse=True)
def _tool():
    if not os.path.exists(TOOL):
        subprocess.run(["g++", "-O2", "-std=c++17", "-o", TOOL,
                        os.path.join(ROOT, "paracel_amd", "csrc", "plr_plan_check.cpp")], check=True)


def plan(d, n=None):
    args = [TOOL, str(d)] + ([str(n)] if n is not None else [])
    out = subprocess.run(args, capture_output=True, text=True, check=True).stdout
    return dict(kv.split("=") for kv in out.split()[0:] if "=" in kv)


def test_every_width_satisfies_the_kernels_assumptions():
    r = subprocess.run([TOOL], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout
    assert r.stdout.strip().startswith("ok: 600000 widths")


def test_the_benchmark_shapes_take_the_intended_variants():
    p = plan(100, 100000)   # config 1 (80 MB): one chunk, 16 rows per tile
    assert (p["path"], p["NCH"], p["R"], p["WCOL"], p["tail"]) == ("fused", "1", "16", "1", "0")
    p = plan(100, 20000000)  # its shape at 16 GB, and when the rows are not known: 32 rows per tile
    assert (p["path"], p["NCH"], p["R"], p["WCOL"], p["tail"]) == ("fused", "1", "32", "1", "0")
    assert plan(100)["R"] == "32" and plan(128, 1000000)["R"] == "16" and plan(128, 1500000)["R"] == "32"
    assert plan(1000, 1000)["R"] == plan(1000, 1000000)["R"] == "4"   # one entry: no choice
    p = plan(1000)       # config 2: one wave, 8 chunks
    assert (p["NCH"], p["R"], p["WCOL"], p["allch"], p["pitch"]) == ("8", "4", "1", "1", "1000")
    p = plan(256)        # config 3
    assert (p["NCH"], p["R"], p["WCOL"]) == ("2", "32", "1")
    p = plan(16384)      # config 4: 8 waves x 16 chunks, theta in LDS
    assert (p["NCH"], p["WCOL"], p["THL"], p["allch"]) == ("16", "8", "1", "1")
    p = plan(16385)      # ... plus the bias column: same variant with a tail stage
    assert (p["NCH"], p["WCOL"], p["TL"], p["tail"], p["pitch"]) == ("16", "8", "1", "16", "16400")
    p = plan(512)        # config 5
    assert (p["NCH"], p["R"], p["WCOL"]) == ("4", "16", "1")
    p = plan(257)        # 256 features + bias: two chunks and a two-column tail
    assert (p["NCH"], p["TL"], p["tail"], p["pitch"]) == ("2", "1", "2", "258")
    assert plan(16)["path"] == "lane" and plan(64)["np"] == "32"
    assert plan(41)["np"] == "21" and plan(41)["pitch"] == "42"   # no padding beyond an even width
    assert plan(65)["path"] == "pair"
    assert plan(19456)["path"] == "fused" and plan(19457)["path"] == "blocked"
