"""plr_set_data_csv: the reference's local_parser (lr.cpp:76-93) on the device.

The shard it leaves resident must be, bit for bit, what the oracle's restatement of
local_parser (strtod per field, str_split's empty-field rule, the leading 1.0) builds
from the same text -- whichever route a field's conversion took, the device's exact
one-rounding path or std::stod on the host.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def plr():
    from paracel_amd import Plr

    with Plr(0) as c:
        yield c


@pytest.fixture(scope="module")
def oracle():
    from oracle import oracle as o

    return o


def spell(rng, v, kind):
    """One spelling of the number v (kind picks the route it will take)."""
    if kind == 0:
        return "%.6f" % v                       # short decimal: device
    if kind == 1:
        return "%.14e" % v                      # 15 significant digits + exponent: device
    if kind == 2:
        return repr(float(v))                   # shortest round-trip, up to 17 digits: mostly host
    if kind == 3:
        return "%d" % int(v * 1000)             # integer
    if kind == 4:
        return "%.17g" % v                      # 17 digits: host
    if kind == 5:
        return ("%.3f" % v).lstrip("0") if 0 <= v < 1 else "%.3f" % v   # ".123"
    if kind == 6:
        return "%.2fE%+d" % (v, int(rng.integers(-25, 26)))             # exponent near +-22
    if kind == 7:
        return "%d." % int(v * 10)              # "12."
    return "%.9g" % v


def make_text(rng, n, k, kinds, sep=",", eol="\n", blank_every=0):
    vals = rng.normal(size=(n, k)) * 10.0 ** rng.integers(-3, 4, size=(n, k))
    lines = []
    for i in range(n):
        f = [spell(rng, vals[i, j], kinds[(i * k + j) % len(kinds)]) for j in range(k)]
        f.append(str(int(rng.integers(0, 2))))
        lines.append(sep.join(f))
        if blank_every and i % blank_every == 0:
            lines.append("")
    return eol.join(lines) + eol


def check_equal(plr, oracle, text, pieces=None, sep=","):
    Xo, yo = oracle.local_parser(text, sep=sep)
    data = text.encode()
    n, d = plr.set_data_csv(pieces if pieces is not None else data, sep=sep)
    assert (n, d) == Xo.shape
    assert "not stored" in plr.kernel_info()
    assert any(("a %s per %s" % k) in plr.kernel_info()
               for k in (("lane", "field"), ("lane", "row"), ("wave", "row")))
    X, y = plr.get_data()
    assert X.tobytes() == Xo.tobytes()
    assert y.tobytes() == yo.tobytes()
    return Xo, yo


@pytest.mark.parametrize("n,k", [(1, 1), (3, 2), (70, 5), (1000, 16), (129, 31), (257, 63),
                                 (500, 64), (300, 65), (200, 100), (150, 257), (64, 1000),
                                 (9, 5000), (5, 20000)])
def test_device_parser_builds_the_oracles_shard(plr, oracle, n, k):
    rng = np.random.default_rng(1000 * n + k)
    print("case n=%d k=%d" % (n, k), flush=True)
    text = make_text(rng, n, k, kinds=[0, 1, 3, 5, 6, 7, 8])
    Xo, yo = check_equal(plr, oracle, text)
    # ... and the passes over it are those of the same rows sent with plr_set_data
    th = rng.normal(size=k + 1)
    g, loss, cnt = plr.loss_grad(th)
    plr.set_option("first_column_is_one", 1)
    try:
        plr.set_data(Xo, yo)
        g2, loss2, _ = plr.loss_grad(th)
    finally:
        plr.set_option("first_column_is_one", 0)
    assert cnt == n
    np.testing.assert_array_equal(g, g2)
    assert loss == loss2


def test_fields_the_host_converts_and_odd_lines(plr, oracle):
    rng = np.random.default_rng(5)
    # 17-digit spellings, shortest round-trip reprs, blank lines, CR LF line ends
    text = make_text(rng, 400, 9, kinds=[2, 4, 0, 1], blank_every=7)
    check_equal(plr, oracle, text)
    text = make_text(rng, 300, 70, kinds=[4, 2])
    check_equal(plr, oracle, text)
    crlf = make_text(rng, 50, 6, kinds=[0, 3], eol="\r\n")
    check_equal(plr, oracle, crlf)
    # the carriage return ends a line's last number as it does for std::stod: no field of a
    # CR LF text is left to the host for that reason
    assert int(plr.kernel_info().split("), ")[-1].split(" ")[0]) == 0
    # inf, nan, hex floats, blanks, a plus sign, trailing characters, very long digit strings,
    # empty fields (dropped), another separator
    odd = ("inf,-inf,0x1p3, 2.5,+3,4.5abc,1\n"
           "1e22,1e23,123456789012345,1234567890123456,-0,-0.0,0\n"
           "0.000000000000000000000000000000000001,1%s,1e-5,00000000000000000000012.5,7,8,1\n"
           % ("0" * 40))
    Xo, _ = check_equal(plr, oracle, odd)
    assert np.isinf(Xo[0, 1]) and Xo[0, 3] == 8.0 and np.signbit(Xo[1, 5])
    # blanks and tabs in front of a number, and a blank behind it with whatever follows, are
    # what std::stod skips and ignores: converted on the device like the bare number
    spaced = "".join("%.3f, %.2f,\t%d ,%.1f  x, -%.4f,1\n" % (v[0], v[1], int(v[2]), v[3], abs(v[4]))
                     for v in rng.normal(size=(300, 5)) * 7)
    check_equal(plr, oracle, spaced)
    assert host_converted(plr) == 0
    check_equal(plr, oracle, "1e 5,2,1\n3 e2, 4 5,0\n")      # "1e 5" is 1, and the host's
    assert host_converted(plr) == 1
    check_equal(plr, oracle, "1,,2,,,3,1\n4,5,,6,0\n")
    check_equal(plr, oracle, "1;2;1\n3;4;0\n", sep=";")
    # a blank or a tab as the separator: white space of the other kind still belongs to a field
    check_equal(plr, oracle, "1.5\t2.5\t1\n 3\t4 \t0\n\t5\t\t6\t1\n", sep="\t")
    check_equal(plr, oracle, "1.5 2.5 1\n\t3 4\t 0\n", sep=" ")
    nan_line = "nan,1,1\n"
    n, d = plr.set_data_csv(nan_line.encode())
    X, y = plr.get_data()
    assert (n, d) == (1, 3) and np.isnan(X[0, 1]) and X[0, 2] == 1.0 and y[0] == 1.0


def host_converted(plr):
    return int(plr.kernel_info().split("), ")[-1].split(" ")[0])


def test_long_mantissas_are_converted_on_the_device_and_still_exact(plr, oracle):
    # 16..19 significant digits (what "%.17g", repr() and "%.18e" write): scaled in
    # double-double arithmetic on the device, left to the host only next to a rounding tie
    rng = np.random.default_rng(77)
    n, k = 4000, 24
    vals = rng.normal(size=(n, k)) * 10.0 ** rng.integers(-12, 13, size=(n, k))
    fmts = ["%.17g", "%.18e", "%.16g", "%.17e", "%r", "%.19g"]
    lines = []
    for i in range(n):
        f = []
        for j in range(k):
            fmt = fmts[(i + j) % len(fmts)]
            f.append(repr(float(vals[i, j])) if fmt == "%r" else fmt % vals[i, j])
        lines.append(",".join(f) + ",1")
    check_equal(plr, oracle, "\n".join(lines) + "\n")
    assert host_converted(plr) <= n * k // 200      # "%.19g" digits beyond 2^64 and the like
    # integers and decimals of 16..19 random digits, scaled by 10^-44..10^44
    lines = []
    for i in range(3000):
        f = []
        for j in range(12):
            nd = int(rng.integers(16, 20))
            m = "".join(str(int(t)) for t in rng.integers(0, 10, size=nd))
            m = str(int(rng.integers(1, 10))) + m[1:]
            cut = int(rng.integers(0, nd + 1))
            body = (m[:cut] + "." + m[cut:]) if j % 3 else m
            if j % 4 == 1:
                body += "e%+d" % int(rng.integers(-30, 31))
            f.append(("-" if (i + j) % 5 == 0 else "") + body)
        lines.append(",".join(f) + ",0")
    check_equal(plr, oracle, "\n".join(lines) + "\n")
    # a larger sample over 80 decades: 600 000 fields of 17 digits
    n, k = 3000, 200
    vals = rng.normal(size=(n, k)) * 10.0 ** rng.integers(-38, 24, size=(n, k))
    text = "\n".join(",".join("%.17g" % v for v in row) + ",1" for row in vals) + "\n"
    check_equal(plr, oracle, text)
    print("600000 fields of 17 digits: %d converted on the host" % host_converted(plr), flush=True)
    # exact ties and their neighbours: 2^53 + 1 is halfway between two doubles
    ties = ["9007199254740993", "9007199254740992", "9007199254740994", "9007199254740995",
            "9007199254740993.0000", "9.007199254740993e15", "4503599627370497.5",
            "0.50000000000000005551", "1.0000000000000001110", "2.00000000000000022204",
            "1152921504606846977", "18446744073709551615", "9999999999999999999",
            "0.9999999999999999444", "1.00000000000000011102230246251565"]
    check_equal(plr, oracle, "\n".join(t + ",1,1" for t in ties) + "\n")


def test_pieces_of_text_and_rows_across_windows(plr, oracle):
    rng = np.random.default_rng(9)
    text = make_text(rng, 333, 12, kinds=[0, 1, 8])
    data = text.encode()
    # pieces cut at line ends, the last without its newline; an empty piece in between
    cut1 = data.index(b"\n", len(data) // 3) + 1
    cut2 = data.index(b"\n", 2 * len(data) // 3) + 1
    pieces = [data[:cut1], b"", data[cut1:cut2], data[cut2:-1]]
    check_equal(plr, oracle, text, pieces=pieces)
    # rows of every length around the 64-byte window, fields of 1..14 digits: field starts
    # and ends fall on every lane, many fields run on into the next window
    lines = []
    for _ in range(700):
        f = [str(int(rng.integers(0, 10 ** int(rng.integers(1, 15))))) for _ in range(12)]
        lines.append(",".join(f + [str(int(rng.integers(0, 2)))]))
    check_equal(plr, oracle, "\n".join(lines) + "\n")


@pytest.fixture()
def overlap(plr):
    plr.set_option("csv_overlap", 1)     # the default, whatever a test before left
    yield plr
    plr.set_option("csv_overlap", 1)


def test_text_parsed_while_it_arrives(overlap, oracle):
    # option "csv_overlap" (on by default): from 256 MiB on the text is parsed stretch by stretch while the rest
    # is still on its way from the host (the shard reserved for an estimated row count); same
    # shard, bit for bit, as with the whole text transferred first
    plr = overlap
    rng = np.random.default_rng(11)
    block = make_text(rng, 2000, 512, kinds=[0]).encode()
    reps = (300 << 20) // len(block) + 1
    pieces = [block] * (reps - 1) + [block[:-1]]        # the last line without its newline
    print("text: %d x %.1f MB" % (reps, len(block) / 1e6), flush=True)
    n, d = plr.set_data_csv(pieces)
    assert (n, d) == (2000 * reps, 513)
    info = plr.kernel_info()
    print(info, flush=True)
    assert "while it arrived" in info
    X, y = plr.get_data()
    Xo, yo = oracle.local_parser(block.decode())
    assert X[:2000].tobytes() == Xo.tobytes() and y[:2000].tobytes() == yo.tobytes()
    Xr = X.reshape(reps, 2000, 513)
    assert all(Xr[i].tobytes() == Xo.tobytes() for i in range(reps))
    assert y.reshape(reps, 2000).tobytes() == np.tile(yo, reps).tobytes()
    th = rng.normal(size=513)
    g, loss, cnt = plr.loss_grad(th)
    # the other order: transfer, then parse
    plr.set_option("csv_overlap", 0)
    try:
        assert plr.set_data_csv(pieces) == (n, d)
        assert "while it arrived" not in plr.kernel_info()
        X2, y2 = plr.get_data()
        g2, loss2, _ = plr.loss_grad(th)
    finally:
        plr.set_option("csv_overlap", 1)
    assert X2.tobytes() == X.tobytes() and y2.tobytes() == y.tobytes()
    np.testing.assert_array_equal(g, g2)
    assert cnt == n and loss == loss2
    # a ragged line deep in the text is still named by its number
    from paracel_amd import PlrError

    bad = block.replace(b",", b";", 1)                   # one line with a field less
    with pytest.raises(PlrError) as e:
        plr.set_data_csv([block] * 40 + [bad] + [block] * (reps - 41))
    assert e.value.code == -1 and "ragged sample line %d" % (40 * 2000) in str(e.value)
    assert plr.shape == (0, 0)


def test_more_rows_than_the_sampled_lines_suggest(overlap):
    # (with "csv_overlap") the row count is estimated from the lengths of lines sampled at regular
    # distances; text whose short lines mostly hide between the samples has half as many rows
    # again as reserved, and the call must notice
    # and start over (transfer, count, parse) instead of writing past the shard
    long_line, short_line = b"0.12345678901234,1\n", b".5,0\n"
    plr = overlap
    pattern = long_line * 40000 + short_line * 60000
    pieces = [pattern] * 256
    assert sum(len(p) for p in pieces) >= 256 << 20
    n, d = plr.set_data_csv(pieces)
    assert (n, d) == (256 * 100000, 2)
    assert "while it arrived" not in plr.kernel_info()
    X, y = plr.get_data()
    want_x = np.tile(np.r_[np.full(40000, 0.12345678901234), np.full(60000, 0.5)], 256)
    want_y = np.tile(np.r_[np.ones(40000), np.zeros(60000)], 256)
    assert np.array_equal(X[:, 0], np.ones(n)) and np.array_equal(X[:, 1], want_x)
    assert np.array_equal(y, want_y)


def test_errors_are_the_reference_parsers(plr):
    from paracel_amd import PlrError

    with pytest.raises(PlrError) as e:
        plr.set_data_csv(b"1,2,1\n3,4,5,0\n6,7,1\n")
    assert e.value.code == -1 and "ragged sample line 1" in str(e.value)
    with pytest.raises(PlrError) as e:
        plr.set_data_csv(b"1,2,1\n3,abc,0\n")
    assert e.value.code == -1 and "sample line 1" in str(e.value)
    with pytest.raises(PlrError) as e:
        plr.set_data_csv(b"1,1e999,1\n")        # std::stod: out of range
    assert e.value.code == -1
    with pytest.raises(PlrError) as e:
        plr.set_data_csv(b"1\n0\n")             # a label and no feature
    assert e.value.code == -5
    # no sample line: an empty shard, no error
    assert plr.set_data_csv(b"\n\n") == (0, 0)
    assert plr.set_data_csv([]) == (0, 0)
    # the context is usable afterwards
    assert plr.set_data_csv(b"1,2,1\n") == (1, 3)
    X, y = plr.get_data()
    assert X.tolist() == [[1.0, 1.0, 2.0]] and y.tolist() == [1.0]


def test_get_data_returns_what_set_data_took(plr):
    rng = np.random.default_rng(3)
    # (the last shape: a row longer than one 4 MiB block of the upload lanes, cut by columns)
    for n, d in [(100, 7), (130, 64), (77, 66), (50, 300), (10, 20001), (3, 530001)]:
        X = rng.normal(size=(n, d))
        y = rng.integers(0, 2, size=n).astype(float)
        plr.set_data(X, y)
        X2, y2 = plr.get_data()
        assert X2.tobytes() == X.tobytes() and y2.tobytes() == y.tobytes()
        X3, y3 = plr.get_data(n // 3, n // 2)
        assert X3.tobytes() == X[n // 3:n // 3 + n // 2].tobytes()
        assert y3.tobytes() == y[n // 3:n // 3 + n // 2].tobytes()


def _random_field(rng):
    k = rng.integers(0, 12)
    v = rng.normal() * 10.0 ** rng.integers(-6, 7)
    if k == 0:
        return "%.6f" % v
    if k == 1:
        return "%.14e" % v
    if k == 2:
        return repr(float(v))
    if k == 3:
        return "%d" % int(v)
    if k == 4:
        return "%.17g" % v
    if k == 5:
        return "%.*f" % (int(rng.integers(0, 12)), v)
    if k == 6:
        return "%.2fE%+d" % (v % 10, int(rng.integers(-30, 31)))
    if k == 7:
        return "%d." % int(v)
    if k == 8:
        return "0" * int(rng.integers(1, 25)) + "%.3f" % abs(v)
    if k == 9:
        return "%.9g" % v
    if k == 10:
        return "-0" if rng.random() < 0.5 else ".5"
    if rng.random() < 0.3:
        # blanks and tabs as std::stod treats them: skipped in front, the end of the number
        # behind it (whatever follows), an error when nothing else is there
        if rng.random() < 0.002:
            return str(rng.choice(["- 5", " . 5", "  "]))       # no number: the text is refused
        return str(rng.choice([" %.3f" % v, "\t%.4f " % v, "%.2f  " % v, "  %d\t" % int(v),
                               "%.3f abc" % v, "%.1f 7" % v, "1e 5", "%.2e\tx" % v, " -.5",
                               "5. ", " 1"]))
    return "%.1f" % v + "0" * int(rng.integers(0, 30))   # tails that pass 32 characters


def _random_text(rng):
    k = int(rng.choice([1, 2, 3, 5, 8, 15, 16, 17, 31, 40, 63, 64, 65, 100, 257, 600, 3000]))
    target = int(rng.choice([300, 4000, 4096, 8192, 20000, 70000, 300000]))   # bytes
    eol = "\r\n" if rng.random() < 0.15 else "\n"
    lines, size = [], 0
    while size < target:
        f = [_random_field(rng) for _ in range(k)] + [str(int(rng.integers(0, 2)))]
        if rng.random() < 0.05:
            f.insert(int(rng.integers(0, len(f))), "")      # an empty field: dropped
        lines.append(",".join(f))
        size += len(lines[-1]) + 1
        if rng.random() < 0.03:
            lines.append("")                                # a blank line ("\r" with CR LF)
    text = eol.join(lines)
    if rng.random() < 0.7:
        text += eol
    if rng.random() < 0.2:
        text = eol * int(rng.integers(1, 4)) + text
    return text


def test_random_texts_against_the_oracle(plr, oracle):
    # widths from 2 to 3001 fields, texts from a fraction of a 4 KiB block to 70 blocks, every
    # spelling class mixed within a line, empty fields, blank lines, CR LF -- where the oracle's
    # parser refuses a text (a line that is only "\r"), the device must refuse it too
    from paracel_amd import PlrError

    refused = 0
    for seed in range(250):
        rng = np.random.default_rng(seed)
        text = _random_text(rng)
        try:
            Xo, yo = oracle.local_parser(text)
        except ValueError:
            with pytest.raises(PlrError):
                plr.set_data_csv(text.encode())
            refused += 1
            continue
        n, d = plr.set_data_csv(text.encode())
        X, y = plr.get_data()
        assert (n, d) == Xo.shape, seed
        assert X.tobytes() == Xo.tobytes() and y.tobytes() == yo.tobytes(), seed
    assert refused < 90
