"""The host-side shard producer (paracel_amd/worker/shard_io.hpp) through its
command-line tool: the reference's byte-range line partition
(include/load/partition.hpp:57-86,121-139; the reference's own
test/test_partition.cpp checks line continuity for np = 1..99), the CSV parser
(lr.cpp:76-93) against the oracle's restatement, and the binary shard cache."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "paracel_amd", "plr_shard_tool")


@pytest.fixture(scope="module", autouse=True)
def _tool():
    if not os.path.exists(TOOL):
        subprocess.run(["make", "-C", os.path.join(ROOT, "paracel_amd", "worker"),
                        os.path.join("..", "plr_shard_tool")], check=True)


def run(*args):
    return subprocess.run([TOOL] + [str(a) for a in args], capture_output=True, text=True)


def make_csv(path, n, k, seed, ragged_len=True):
    rng = np.random.default_rng(seed)
    lines = []
    for i in range(n):
        kk = k
        vals = rng.normal(size=kk)
        # fields of varying printed width so that byte ranges cut lines at every position
        fmt = ["%.1f", "%.6f", "%.12g", "%e"][i % 4] if ragged_len else "%.6f"
        lines.append(",".join(fmt % v for v in vals) + ",%d" % (i % 2))
    path.write_text("\n".join(lines) + "\n")
    return lines


@pytest.mark.parametrize("np_", [1, 2, 3, 4, 7, 16, 33, 99])
def test_partition_covers_every_line_once(tmp_path, np_):
    f = tmp_path / "a.csv"
    lines = make_csv(f, 250, 5, 1)
    got = []
    for r in range(np_):
        out = run("lines", f, r, np_)
        assert out.returncode == 0, out.stderr
        got.extend(out.stdout.splitlines())
    assert got == lines                      # no line lost, duplicated or split; order kept


def test_partition_when_a_boundary_hits_a_newline(tmp_path):
    # 4 lines of 9 bytes + newline = 40 bytes; np=4 puts every boundary right after a newline
    f = tmp_path / "b.csv"
    lines = ["1.0,2.0,%d" % (i % 2) for i in range(4)]
    f.write_text("\n".join(lines) + "\n")
    for r in range(4):
        assert run("lines", f, r, 4).stdout.splitlines() == [lines[r]]
    # and np=8: every second range owns nothing
    owned = [run("lines", f, r, 8).stdout.splitlines() for r in range(8)]
    assert sum(owned, []) == lines


@pytest.mark.parametrize("np_", [1, 2, 3, 5, 8])
def test_directory_and_glob_inputs_are_one_byte_stream(tmp_path, np_):
    # files laid end to end in glob order, then the same byte-range rule
    # (include/load/partition.hpp:57-86,141-175)
    d = tmp_path / "parts"
    d.mkdir()
    (d / "sub").mkdir()
    all_lines = []
    for name, n, seed in (("a.csv", 40, 1), ("b.csv", 7, 2), ("sub/c.csv", 25, 3)):
        all_lines.append(make_csv(d / name, n, 4, seed))
    flat = sum(all_lines, [])
    for spec, want in ((d, flat), (str(d) + "/*.csv", all_lines[0] + all_lines[1])):
        got = []
        for r in range(np_):
            out = run("lines", spec, r, np_)
            assert out.returncode == 0, out.stderr
            got.extend(out.stdout.splitlines())
        assert got == want
    assert run("lines", str(d) + "/*.nothing", 0, 1).returncode == 1


def _owners_by_definition(blobs, np_):
    """Brute force of the rule itself: lay the files end to end, cut the stream into np
    ranges of floor(total/np) bytes (the last takes the rest), and give every non-blank
    line to the range its FIRST byte falls in.  Lines never span two files."""
    total = sum(len(b) for b in blobs)
    part = total // np_
    owned = [[] for _ in range(np_)]
    base = 0
    for b in blobs:
        pos = 0
        while pos < len(b):
            nl = b.find(b"\n", pos)
            stop = len(b) if nl < 0 else nl
            if stop > pos:
                start = base + pos
                r = np_ - 1 if part == 0 else min(start // part, np_ - 1)
                owned[r].append(b[pos:stop].decode())
            pos = stop + 1
        base += len(b)
    return owned


@pytest.mark.parametrize("case", ["one_file", "three_files", "no_final_newline", "tiny_lines"])
def test_ownership_rule_by_brute_force_for_np_1_to_99(tmp_path, case):
    # the reference's own test (test/test_partition.cpp) checks line continuity for
    # np = 1..99 on one file; here the definition is evaluated directly, byte by byte,
    # also over several files, files that lack the final newline and one-byte lines
    rng = np.random.default_rng(len(case))
    d = tmp_path / "in"
    d.mkdir()

    def text(n, maxlen):
        return "".join("".join(rng.choice(list("0123456789.,-e"), size=rng.integers(1, maxlen)))
                       + "\n" for _ in range(n))

    if case == "one_file":
        files = {"a.csv": text(300, 40)}
    elif case == "three_files":
        files = {"a.csv": text(120, 30), "b.csv": text(5, 200), "c.csv": text(211, 12)}
    elif case == "no_final_newline":
        files = {"a.csv": text(50, 25)[:-1], "b.csv": text(70, 25)[:-1], "c.csv": text(3, 9)}
    else:
        files = {"a.csv": text(150, 2), "b.csv": "7\n" * 90}
    for name, t in files.items():
        (d / name).write_text(t)
    blobs = [files[k].encode() for k in sorted(files)]   # glob order = sorted names
    out = run("owners", d, 1, 99)
    assert out.returncode == 0, out.stderr
    got = {}
    for ln in out.stdout.splitlines():
        a, b, line = ln.split(" ", 2)
        got.setdefault(int(a), {}).setdefault(int(b), []).append(line)
    for np_ in range(1, 100):
        want = _owners_by_definition(blobs, np_)
        for r in range(np_):
            assert got.get(np_, {}).get(r, []) == want[r], (case, np_, r)


def test_blank_lines_are_dropped(tmp_path):
    f = tmp_path / "e.csv"
    f.write_text("1,2,1\n\n3,4,0\n\n\n5,6,1\n")
    for np_ in (1, 2, 5):
        got = sum((run("lines", f, r, np_).stdout.splitlines() for r in range(np_)), [])
        assert got == ["1,2,1", "3,4,0", "5,6,1"]


def test_parser_matches_oracle_and_cache_roundtrip(tmp_path, oracle):
    f = tmp_path / "c.csv"
    lines = make_csv(f, 300, 7, 2)
    out = run("parse", f, 0, 1)
    assert out.returncode == 0, out.stderr
    assert out.stdout.split() == ["300", "8"]            # bias column added: D = k + 1
    raw = np.fromfile(str(f) + ".plrshard.0of1", dtype=np.uint8)
    hdr = raw[:48]
    assert bytes(hdr[:8]) == b"PLRSHARD"
    n, d = np.frombuffer(hdr[16:32].tobytes(), dtype=np.int64)
    body = np.frombuffer(raw[48:].tobytes(), dtype=np.float64)
    X, y = body[: n * d].reshape(n, d), body[n * d:]
    Xo, yo = oracle.local_parser(f.read_text())
    np.testing.assert_array_equal(X, Xo)                 # bit-exact: same strtod
    np.testing.assert_array_equal(y, yo)
    assert np.all(X[:, 0] == 1.0)
    assert run("info", f, 0, 1).stdout.split() == ["300", "8"]
    # the mapped read and the slab-by-slab writer (the GPU workers' routes) keep every byte
    for slab in (64, 1000, 1 << 26):
        out = run("recache", f, 0, 1, slab)
        assert out.returncode == 0 and out.stdout.split() == ["rewritten", "300", "8"], out.stderr
        assert np.array_equal(np.fromfile(str(f) + ".plrshard.0of1", dtype=np.uint8), raw)
    # touching the source invalidates the cache
    os.utime(f, ns=(1, 1))
    assert run("recache", f, 0, 1, 4096).returncode == 1
    assert run("info", f, 0, 1).returncode == 1
    # per-rank shards concatenate to the whole
    parts = []
    for r in range(3):
        assert run("parse", f, r, 3).returncode == 0
        rr = np.fromfile(str(f) + ".plrshard.%dof3" % r, dtype=np.uint8)
        nn, dd = np.frombuffer(rr[16:32].tobytes(), dtype=np.int64)
        parts.append(np.frombuffer(rr[48:48 + 8 * nn * dd].tobytes(), dtype=np.float64).reshape(nn, dd))
    np.testing.assert_array_equal(np.vstack(parts), Xo)


def test_cache_written_in_slabs_while_the_next_is_fetched(tmp_path):
    # a few slabs and one: the writer thread and the fetch alternate between two buffers
    f = tmp_path / "big.csv"
    make_csv(f, 40000, 7, 5, ragged_len=False)
    assert run("parse", f, 0, 1).stdout.split() == ["40000", "8"]
    raw = np.fromfile(str(f) + ".plrshard.0of1", dtype=np.uint8)
    assert raw.size == 48 + 40000 * 9 * 8
    for slab in (1 << 18, 1 << 20, 1 << 26):
        out = run("recache", f, 0, 1, slab)
        assert out.returncode == 0, out.stderr
        assert np.array_equal(np.fromfile(str(f) + ".plrshard.0of1", dtype=np.uint8), raw)


def test_parser_errors(tmp_path):
    f = tmp_path / "d.csv"
    f.write_text("1,2,1\n1,1\n")
    assert run("parse", f, 0, 1).returncode == 1        # ragged
    f.write_text("1,abc,1\n")
    assert run("parse", f, 0, 1).returncode == 1        # std::stod throws
    f.write_text("3,,7,1\n")                            # empty field dropped (str_split)
    assert run("parse", f, 0, 1).stdout.split() == ["1", "3"]
    assert run("parse", tmp_path / "missing.csv", 0, 1).returncode == 1


def test_field_parser_equals_stod_bit_for_bit():
    # the short-decimal fast path against std::stod itself on random spellings:
    # digit counts around 15, exponents around +-22, zeros, signs, hex floats,
    # inf/nan, blanks, garbage -- values and exceptions must agree
    for seed in (1, 0xBEEF):
        out = run("selftest", 1500000, seed, 0)
        assert out.returncode == 0, out.stdout + out.stderr
        assert out.stdout.startswith("ok 1500000 fields")


def test_parser_against_python_float(tmp_path):
    # python's float() is correctly rounded, like strtod: fields written with few
    # digits (fast path) and with 17 (library path) in one file
    rng = np.random.default_rng(11)
    vals = rng.normal(size=(200, 6)) * 10.0 ** rng.integers(-30, 30, size=(200, 6))
    lines = []
    for i, row in enumerate(vals):
        fmt = ["%.3f", "%.17g", "%.14e", "%r"][i % 4]
        lines.append(",".join((fmt % v) if fmt != "%r" else repr(float(v)) for v in row) + ",1")
    f = tmp_path / "p.csv"
    f.write_text("\n".join(lines) + "\n")
    assert run("parse", f, 0, 1).returncode == 0
    raw = np.fromfile(str(f) + ".plrshard.0of1", dtype=np.uint8)
    X = np.frombuffer(raw[48:48 + 8 * 200 * 7].tobytes(), dtype=np.float64).reshape(200, 7)
    want = np.array([[float(t) for t in l.split(",")[:-1]] for l in lines])
    assert X[:, 1:].tobytes() == want.tobytes()
