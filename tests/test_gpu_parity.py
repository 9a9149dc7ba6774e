"""GPU parity: the HIP path, called through the C ABI, against the reference's known-answer
vectors and against the host oracle on seeded inputs.  Bit-exact (integer work)."""
import numpy as np
import pytest

from tests import golden_cases as gc
from tests.golden_cases import strings
from cudf_amd.arrow_host import HostStringsColumn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nv():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from cudf_amd import nvtext
    from cudf_amd import _capi
    _capi.load()  # fails loudly if the HIP library is missing
    return nvtext


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


def dev(nv, host):
    return nv.DeviceStringsColumn.from_host(host)


def assert_same(got, exp, what=""):
    assert got.size == exp.size, what
    assert got.null_count == exp.null_count, what
    assert got.child.dtype == exp.child.dtype, what
    assert np.array_equal(got.validity(), exp.validity()), what
    assert got.offsets.size == exp.offsets.size, what
    assert np.array_equal(got.offsets, exp.offsets), what
    if not np.array_equal(got.child, exp.child):
        bad = np.flatnonzero(got.child != exp.child)
        raise AssertionError(f"{what}: {bad.size} child values differ, first at {bad[:5]}: "
                             f"got {got.child[bad[:5]]} expected {exp.child[bad[:5]]}")


# ----------------------------------------------------------------------------- minhash golden
@pytest.mark.parametrize("case", gc.minhash_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_minhash_golden(nv, case, dtype):
    col = dev(nv, strings(case["rows"], dtype))
    if "expected32" in case:
        got = nv.minhash(col, case["seed"], np.array(case["a"], np.uint32), np.array(case["b"], np.uint32), case["width"]).to_host()
        assert gc.expected_list_equal(got.to_pylist(), case["expected32"])
    if "expected64" in case:
        got = nv.minhash64(col, case["seed"], np.array(case["a"], np.uint64), np.array(case["b"], np.uint64), case["width"]).to_host()
        assert gc.expected_list_equal(got.to_pylist(), case["expected64"])


def random_rows(rng, n, max_len, utf8=False, p_null=0.05, p_empty=0.05):
    ascii_alpha = list("abcdefghijklmnopqrstuvwxyz      .,")
    wide = list("éüñßçøå") + list("漢字仮名日本語中文") + ["😀", "𝄞"]
    rows = []
    for _ in range(n):
        u = rng.random()
        if u < p_null:
            rows.append(None)
            continue
        if u < p_null + p_empty:
            rows.append("")
            continue
        ln = int(rng.integers(1, max_len))
        if utf8:
            pool = ascii_alpha + wide
            rows.append("".join(rng.choice(pool, ln)))
        else:
            rows.append("".join(rng.choice(ascii_alpha, ln)))
    return rows


@pytest.mark.parametrize("utf8", [False, True], ids=["ascii", "utf8"])
@pytest.mark.parametrize("P,width", [(1, 3), (3, 4), (4, 2), (5, 6), (16, 9), (26, 12), (32, 24), (33, 7), (64, 5), (100, 2), (128, 8),
                                     (129, 4), (192, 3), (256, 5), (260, 12), (320, 24), (321, 5), (700, 6)])
def test_minhash_random_vs_oracle(nv, orc, utf8, P, width):
    rng = np.random.default_rng(1000 + P + width + int(utf8))
    rows = random_rows(rng, 300, 700, utf8=utf8)
    rows += ["a", "ab", "é", "abcde" * 1000, "x" * 255, "y" * 256, "z" * 257, "w" * 1023, "v" * 1025]
    host = strings(rows)
    col = dev(nv, host)
    a32 = rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32)
    b32 = rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32)
    assert_same(nv.minhash(col, 42, a32, b32, width).to_host(), orc.minhash(host, 42, a32, b32, width, nthreads=8), "minhash")
    a64 = rng.integers(1, 2**64, P, dtype=np.uint64)
    b64 = rng.integers(0, 2**64, P, dtype=np.uint64)
    assert_same(nv.minhash64(col, 7, a64, b64, width).to_host(), orc.minhash64(host, 7, a64, b64, width, nthreads=8), "minhash64")


def test_minhash_long_rows_cross_workgroups(nv, orc):
    """Rows longer than one workgroup span (16 KiB) take the multi-workgroup + atomic-min route."""
    rng = np.random.default_rng(5)
    words = ["".join(rng.choice(list("abcdefghij"), int(rng.integers(1, 9)))) for _ in range(500)]

    def doc(nbytes):
        out, ln = [], 0
        while ln < nbytes:
            w = words[int(rng.integers(0, len(words)))]
            out.append(w)
            ln += len(w) + 1
        return " ".join(out)[:nbytes]

    rows = [doc(16384), doc(16385), doc(40000), None, "", doc(300000), doc(100), doc(16383), doc(70000) + "é漢" * 3000]
    host = strings(rows, np.int64)
    col = dev(nv, host)
    a32 = rng.integers(1, 2**32, 128, dtype=np.uint64).astype(np.uint32)
    b32 = rng.integers(0, 2**32, 128, dtype=np.uint64).astype(np.uint32)
    assert_same(nv.minhash(col, 9, a32, b32, 5).to_host(), orc.minhash(host, 9, a32, b32, 5, nthreads=8), "minhash long")
    a64 = rng.integers(1, 2**64, 128, dtype=np.uint64)
    b64 = rng.integers(0, 2**64, 128, dtype=np.uint64)
    assert_same(nv.minhash64(col, 7, a64, b64, 5).to_host(), orc.minhash64(host, 7, a64, b64, 5, nthreads=8), "minhash64 long")


@pytest.mark.parametrize("P", [65, 68, 72, 80, 96, 129, 150, 200, 224, 260, 273, 288])
def test_minhash_parameters_beyond_the_last_full_set_of_64(nv, orc, P):
    """65 to 288 parameters of which at most 32 lie beyond the last full set of 64: those share the lanes of a wavefront in
    sets (4, 8, 16 or 32 lanes to a set) beside the full sets.  Short rows (a wavefront each), rows shared by a workgroup
    and rows of several spans (the extra workgroups, merged with atomic minima), empty and null rows."""
    rng = np.random.default_rng(3000 + P)
    rows = random_rows(rng, 40, 900, utf8=True) + ["a", "", None, "abcdefg " * 700, "".join(rng.choice(list("abcdefghijk "), 50000)),
                                                   "é漢x " * 9000, "q" * 16384, "r" * 16385, "ab"]
    host = strings(rows, np.int64)
    col = dev(nv, host)
    a32 = rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32)
    b32 = rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32)
    assert_same(nv.minhash(col, 11, a32, b32, 4).to_host(), orc.minhash(host, 11, a32, b32, 4, nthreads=8), f"minhash P={P}")
    a64 = rng.integers(1, 2**64, P, dtype=np.uint64)
    b64 = rng.integers(0, 2**64, P, dtype=np.uint64)
    assert_same(nv.minhash64(col, 12, a64, b64, 6).to_host(), orc.minhash64(host, 12, a64, b64, 6, nthreads=8), f"minhash64 P={P}")


@pytest.mark.parametrize("rows", [140_000, 300_000, 600_000, 1_100_000])
def test_minhash_many_rows_several_short_rows_to_a_wavefront(nv, orc, rows):
    """From 131,072 rows on a wavefront takes 2, 4, 8 and, from 1,048,576 rows on, 16 short rows of its workgroup's group
    instead of one.  Mostly rows of a few bytes, nulls and empty rows among them, rows of the group's last places, rows
    just below and above the lengths that a wavefront does alone (1024 bytes, 4096 with several rows to a wavefront), and
    rows of several workgroup spans."""
    from cudf_amd.arrow_host import HostStringsColumn, pack_validity
    rng = np.random.default_rng(rows)
    lengths = rng.integers(0, 24, rows)
    lengths[rng.integers(0, rows, rows // 200)] = rng.integers(1000, 1050, rows // 200)   # either side of 1024 bytes
    lengths[rng.integers(0, rows, 60)] = rng.integers(4080, 4112, 60)                      # and of 4096 (the limit with several rows to a wavefront)
    lengths[rng.integers(0, rows, 40)] = rng.integers(5000, 70000, 40)                     # shared by a workgroup; extra workgroups
    lengths[-1] = 1500
    lengths[-2] = 3
    offsets = np.zeros(rows + 1, np.int64)
    np.cumsum(lengths, out=offsets[1:])
    chars = rng.integers(97, 105, int(offsets[-1]), dtype=np.uint8)
    chars[rng.random(chars.size) < 0.2] = 32
    valid = rng.random(rows) > 0.05
    host = HostStringsColumn(chars, offsets.astype(np.int32), pack_validity(valid), rows, 0, int((~valid).sum()))
    col = dev(nv, host)
    for P in (3, 70):
        a32 = rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32)
        b32 = rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32)
        assert_same(nv.minhash(col, 5, a32, b32, 4).to_host(), orc.minhash(host, 5, a32, b32, 4, nthreads=8), f"minhash rows={rows} P={P}")
    a64 = rng.integers(1, 2**64, 5, dtype=np.uint64)
    b64 = rng.integers(0, 2**64, 5, dtype=np.uint64)
    assert_same(nv.minhash64(col, 6, a64, b64, 7).to_host(), orc.minhash64(host, 6, a64, b64, 7, nthreads=8), f"minhash64 rows={rows}")
    # a slice whose first row is not the first of a group
    lo, hi = 3, rows - 5
    hs = host.slice(lo, hi)
    assert_same(nv.minhash(col.slice(lo, hi, hs.null_count), 5, a32, b32, 4).to_host(), orc.minhash(hs, 5, a32, b32, 4, nthreads=8), f"sliced rows={rows}")


def test_minhash_few_parameters_share_the_lanes_of_a_wavefront(nv, orc):
    """With at most 32 parameters the lanes work in sets that each fold a part of the hashes; long rows (every wavefront
    of a workgroup, the extra workgroups) and rows of fewer windows than sets must still give the minimum over all."""
    rng = np.random.default_rng(26)
    rows = random_rows(rng, 60, 3000) + ["k" * 40000, "".join(rng.choice(list("abcdefg "), 70000)), "ab", "abc", "abcd", "abcdefgh", "", None]
    host = strings(rows)
    col = dev(nv, host)
    for P in (1, 2, 7, 8, 26, 31, 32):
        a32 = rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32)
        b32 = rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32)
        assert_same(nv.minhash(col, 0, a32, b32, 12).to_host(), orc.minhash(host, 0, a32, b32, 12, nthreads=8), f"minhash P={P}")
        a64 = rng.integers(1, 2**64, P, dtype=np.uint64)
        b64 = rng.integers(0, 2**64, P, dtype=np.uint64)
        assert_same(nv.minhash64(col, 0, a64, b64, 24).to_host(), orc.minhash64(host, 0, a64, b64, 24, nthreads=8), f"minhash64 P={P}")


def test_minhash_more_rows_than_a_grid_has_workgroups(nv, orc):
    """More rows than a launch has workgroups along x (2^15 groups of them, 64 rows each at this size): the rest lie along z."""
    rows = (1 << 22) + 12345
    rng = np.random.default_rng(17)
    lengths = rng.integers(0, 6, rows)
    offsets = np.zeros(rows + 1, np.int32)
    np.cumsum(lengths, out=offsets[1:])
    chars = rng.integers(97, 123, int(offsets[-1]), dtype=np.uint8)
    valid = rng.random(rows) > 0.01
    from cudf_amd.arrow_host import HostStringsColumn, pack_validity
    host = HostStringsColumn(chars, offsets, pack_validity(valid), rows, 0, int((~valid).sum()))
    col = dev(nv, host)
    a = np.array([3, 5], np.uint32)
    b = np.array([1, 2], np.uint32)
    assert_same(nv.minhash(col, 1, a, b, 3).to_host(), orc.minhash(host, 1, a, b, 3, nthreads=8), "many rows")
    a64, b64 = a.astype(np.uint64), b.astype(np.uint64)
    assert_same(nv.minhash64(col, 1, a64, b64, 3).to_host(), orc.minhash64(host, 1, a64, b64, 3, nthreads=8), "many rows 64")


def test_minhash_very_wide_window(nv, orc):
    """width*4 bytes beyond the staged halo: bytes are read straight from global memory."""
    rng = np.random.default_rng(6)
    rows = random_rows(rng, 40, 900, utf8=True) + ["q" * 50, "ab" * 300]
    host = strings(rows)
    col = dev(nv, host)
    a = rng.integers(1, 2**32, 5, dtype=np.uint64).astype(np.uint32)
    assert_same(nv.minhash(col, 1, a, a, 40).to_host(), orc.minhash(host, 1, a, a, 40), "wide window")
    a64 = rng.integers(1, 2**64, 5, dtype=np.uint64)
    assert_same(nv.minhash64(col, 1, a64, a64, 100).to_host(), orc.minhash64(host, 1, a64, a64, 100), "wide window 64")


def test_windows_over_runs_of_continuation_bytes(nv, orc):
    """Bytes that continue no character count for nothing in the walk to `width` characters
    (cpp/include/cudf/strings/string_view.cuh:67-80), so a run of them stretches a window past the 4 * width bytes that
    well-formed text needs: the same rows at several places of the 256-position tiles, for minhash and jaccard_index."""
    rng = np.random.default_rng(66)
    rows = []
    for shift in (0, 1, 100, 200, 250, 255, 256, 257, 300):
        head = bytes(rng.integers(97, 123, shift, dtype=np.uint8))
        for run in (4, 17, 60, 129, 300, 700):
            rows.append(head + b"ab" + b"\x80" * run + b"cdefgh" + b"\xbf" * (run // 2) + b"ij klmnop")
            rows.append(head + "é".encode() + b"\x9a" * run)          # the run ends the row: only the first window may be short
            rows.append(head + b"\xe6\xbc" + b"\xa2" * run + b"xyz")
    host = HostStringsColumn.from_pylist(rows)
    col = dev(nv, host)
    a = rng.integers(1, 2**32, 9, dtype=np.uint64).astype(np.uint32)
    b = rng.integers(0, 2**32, 9, dtype=np.uint64).astype(np.uint32)
    for width in (2, 5, 12, 40):
        assert_same(nv.minhash(col, 3, a, b, width).to_host(), orc.minhash(host, 3, a, b, width, nthreads=4), f"minhash width {width}")
        a64, b64 = a.astype(np.uint64) << np.uint64(7), b.astype(np.uint64)
        assert_same(nv.minhash64(col, 3, a64, b64, width).to_host(), orc.minhash64(host, 3, a64, b64, width, nthreads=4), f"minhash64 width {width}")
        n = len(rows) - 1
        got = nv.jaccard_index(col.slice(0, n, 0), col.slice(1, n + 1, 0), width).to_host()
        exp = orc.jaccard_index(host.slice(0, n), host.slice(1, n + 1), width, nthreads=4)
        assert got.equals(exp), f"jaccard_index width {width}"


def test_minhash64_reduction_edge(nv, orc):
    """Parameters that drive (h*a+b) mod 2^64 onto p, p+1.. and 2^64-1 exercise the final subtraction."""
    p = 2**61 - 1
    host = strings(["hello world", "abc", "x" * 600])
    col = dev(nv, host)
    a = np.array([0, 0, 0, 0, 0, 1, 2**63], np.uint64)
    b = np.array([p, p + 1, p + 7, 2**64 - 1, p - 1, 0, 2**64 - 1], np.uint64)
    assert_same(nv.minhash64(col, 0, a, b, 4).to_host(), orc.minhash64(host, 0, a, b, 4), "mod edge")


def test_minhash_sliced_and_nulls(nv, orc):
    rng = np.random.default_rng(8)
    rows = random_rows(rng, 200, 300, p_null=0.2, p_empty=0.1)
    host = strings(rows)
    a = rng.integers(1, 2**32, 64, dtype=np.uint64).astype(np.uint32)
    for lo, hi in [(0, 200), (3, 150), (33, 97), (64, 128), (199, 200)]:
        hs = host.slice(lo, hi)
        ds = dev(nv, host).slice(lo, hi, hs.null_count)
        assert_same(nv.minhash(ds, 3, a, a, 4).to_host(), orc.minhash(hs, 3, a, a, 4), f"slice {lo}:{hi}")


def test_minhash_errors_and_empty(nv):
    col = dev(nv, strings(["this string intentionally left blank"]))
    e32, e64 = np.zeros(0, np.uint32), np.zeros(0, np.uint64)
    with pytest.raises(ValueError):
        nv.minhash(col, 0, e32, e32, 0)
    with pytest.raises(ValueError):
        nv.minhash64(col, 0, e64, e64, 0)
    with pytest.raises(ValueError):
        nv.minhash(col, 0, e32, e32, 4)
    with pytest.raises(ValueError):
        nv.minhash64(col, 0, e64, e64, 4)
    with pytest.raises(ValueError):
        nv.minhash(col, 0, np.ones(3, np.uint32), np.ones(2, np.uint32), 4)
    big = dev(nv, strings([""] * 50000))
    with pytest.raises(OverflowError):
        nv.minhash(big, 0, np.zeros(50000, np.uint32), np.zeros(50000, np.uint32), 4)
    with pytest.raises(OverflowError):
        nv.minhash64(big, 0, np.zeros(50000, np.uint64), np.zeros(50000, np.uint64), 4)
    empty = dev(nv, strings([]))
    got = nv.minhash(empty, 0, np.ones(3, np.uint32), np.ones(3, np.uint32), 4).to_host()
    assert got.size == 0 and got.child.size == 0
    got = nv.minhash64(empty, 0, np.ones(3, np.uint64), np.ones(3, np.uint64), 4).to_host()
    assert got.size == 0 and got.child.size == 0


# ----------------------------------------------------------------------------- minhash_ngrams
def ldev(nv, host):
    return nv.DeviceListStringsColumn.from_host(host)


@pytest.mark.parametrize("case", gc.minhash_ngrams_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_minhash_ngrams_golden(nv, case, dtype):
    host = gc.list_strings(case["rows"], dtype)
    d = ldev(nv, host)
    if "slice" in case:
        lo, hi = case["slice"]
        d = d.slice(lo, hi, 0)
    a32, b32 = np.array(case["a"], np.uint32), np.array(case["b"], np.uint32)
    assert nv.minhash_ngrams(d, case["ngrams"], case["seed"], a32, b32).to_host().to_pylist() == case["expected32"]
    got = nv.minhash64_ngrams(d, case["ngrams"], case["seed"], a32.astype(np.uint64), b32.astype(np.uint64)).to_host()
    assert got.to_pylist() == case["expected64"] and got.child.dtype == np.uint64


@pytest.mark.parametrize("P,ngrams", [(3, 2), (64, 5), (100, 3), (260, 10)])
def test_minhash_ngrams_random_vs_oracle(nv, orc, P, ngrams):
    rng = np.random.default_rng(1000 + P)
    letters = list("abcdefghijé漢 ")
    rows = []
    for _ in range(700):
        u = rng.random()
        if u < 0.05:
            rows.append(None)
            continue
        n = 0 if u < 0.1 else int(rng.integers(1, 40)) if u < 0.9 else int(rng.integers(200, 600))
        row = []
        for _ in range(n):
            t = rng.random()
            row.append(None if t < 0.04 else "" if t < 0.08 else "".join(rng.choice(letters, int(rng.integers(1, 14)))))
        rows.append(row)
    for dtype in (np.int32, np.int64):
        host = gc.list_strings(rows, dtype)
        d = ldev(nv, host)
        a = rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32)
        b = rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32)
        assert_same(nv.minhash_ngrams(d, ngrams, 7, a, b).to_host(), orc.minhash_ngrams(host, ngrams, 7, a, b, nthreads=4), f"ngrams u32 P={P}")
        a64 = rng.integers(1, 2**64, P, dtype=np.uint64)
        b64 = rng.integers(0, 2**64, P, dtype=np.uint64)
        assert_same(nv.minhash64_ngrams(d, ngrams, 99, a64, b64).to_host(), orc.minhash64_ngrams(host, ngrams, 99, a64, b64, nthreads=4),
                    f"ngrams u64 P={P}")
        for lo, hi in [(3, 650), (100, 101)]:
            hs = host.slice(lo, hi)
            assert_same(nv.minhash_ngrams(d.slice(lo, hi, hs.null_count), ngrams, 7, a, b).to_host(),
                        orc.minhash_ngrams(hs, ngrams, 7, a, b), f"ngrams slice {lo}:{hi}")


@pytest.mark.parametrize("rows", [150_000, 1_100_000])
def test_minhash_ngrams_many_rows_several_short_rows_to_a_wavefront(nv, orc, rows):
    """From 131,072 rows on a wavefront takes several short rows of its workgroup's group (16 from 1,048,576 rows on) and
    does a row of up to 2048 positions alone.  Mostly rows of a few elements, empty and null rows and null elements among
    them, rows either side of 2048 positions, a row of many more."""
    from cudf_amd.arrow_host import HostListStringsColumn, HostStringsColumn, pack_validity
    rng = np.random.default_rng(rows + 1)
    sizes = rng.integers(0, 7, rows)
    sizes[rng.integers(0, rows, 30)] = rng.integers(2040, 2060, 30)
    sizes[rng.integers(0, rows, 200)] = rng.integers(60, 400, 200)
    sizes[rows // 2] = 9000
    sizes[-1] = 70
    offsets = np.zeros(rows + 1, np.int32)
    np.cumsum(sizes, out=offsets[1:])
    count = int(offsets[-1])
    lengths = rng.integers(0, 6, count)
    eoff = np.zeros(count + 1, np.int32)
    np.cumsum(lengths, out=eoff[1:])
    chars = rng.integers(97, 103, int(eoff[-1]), dtype=np.uint8)
    evalid = rng.random(count) > 0.03
    elements = HostStringsColumn(chars, eoff, pack_validity(evalid), count, 0, int((~evalid).sum()))
    valid = rng.random(rows) > 0.05
    host = HostListStringsColumn(offsets, elements, pack_validity(valid), rows, 0, int((~valid).sum()))
    d = ldev(nv, host)
    a = rng.integers(1, 2**32, 5, dtype=np.uint64).astype(np.uint32)
    b = rng.integers(0, 2**32, 5, dtype=np.uint64).astype(np.uint32)
    assert_same(nv.minhash_ngrams(d, 3, 7, a, b).to_host(), orc.minhash_ngrams(host, 3, 7, a, b, nthreads=8), f"ngrams u32 rows={rows}")
    a64 = rng.integers(1, 2**64, 70, dtype=np.uint64)
    b64 = rng.integers(0, 2**64, 70, dtype=np.uint64)
    assert_same(nv.minhash64_ngrams(d, 2, 9, a64, b64).to_host(), orc.minhash64_ngrams(host, 2, 9, a64, b64, nthreads=8), f"ngrams u64 rows={rows}")
    lo, hi = 5, rows - 3
    hs = host.slice(lo, hi)
    assert_same(nv.minhash_ngrams(d.slice(lo, hi, hs.null_count), 3, 7, a, b).to_host(), orc.minhash_ngrams(hs, 3, 7, a, b, nthreads=8), f"sliced rows={rows}")


def test_minhash_ngrams_wide_row_and_errors(nv, orc):
    rng = np.random.default_rng(5)
    words = ["".join(rng.choice(list("abcdef"), int(rng.integers(1, 9)))) for _ in range(300_000)]
    host = gc.list_strings([words, words[:3], words[:70_000]])
    a = np.arange(1, 6, dtype=np.uint32)
    assert_same(nv.minhash_ngrams(ldev(nv, host), 5, 0, a, a).to_host(), orc.minhash_ngrams(host, 5, 0, a, a, nthreads=8), "wide rows")
    d = ldev(nv, gc.list_strings([["a", "b"]]))
    with pytest.raises(ValueError):
        nv.minhash_ngrams(d, 1, 0, a, a)
    with pytest.raises(ValueError):
        nv.minhash_ngrams(d, 2, 0, a[:0], a[:0])
    with pytest.raises(ValueError):
        nv.minhash64_ngrams(d, 2, 0, np.zeros(3, np.uint64), np.zeros(2, np.uint64))
    empty = nv.minhash_ngrams(ldev(nv, gc.list_strings([])), 4, 0, a, a).to_host()
    assert empty.size == 0 and empty.child.size == 0


# ----------------------------------------------------------------------------- jaccard_index
def assert_same_fixed(got, exp, what=""):
    assert got.size == exp.size and got.null_count == exp.null_count, what
    assert (got.mask is None) == (exp.mask is None), what
    v = exp.validity()
    assert np.array_equal(got.validity(), v), what
    a, b = got.values.view(np.uint32)[v], exp.values.view(np.uint32)[v]
    if not np.array_equal(a, b):
        bad = np.flatnonzero(a != b)
        raise AssertionError(f"{what}: {bad.size} values differ, first at {bad[:5]}: got {got.values[v][bad[:5]]} expected {exp.values[v][bad[:5]]}")


@pytest.mark.parametrize("case", gc.jaccard_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_jaccard_golden(nv, orc, case, dtype):
    h1, h2 = strings(case["input1"], dtype), strings(case["input2"], dtype)
    got = nv.jaccard_index(dev(nv, h1), dev(nv, h2), case["width"]).to_host()
    assert_same_fixed(got, orc.jaccard_index(h1, h2, case["width"]), case["name"])
    exp = np.array(case["expected"], np.float32)
    valid = np.array(case.get("expected_valid", [True] * len(exp)))
    assert np.allclose(got.values[valid], exp[valid], atol=case.get("tolerance", 0), rtol=0)


@pytest.mark.parametrize("width", [2, 5, 40])
def test_jaccard_random_vs_oracle(nv, orc, width):
    rng = np.random.default_rng(400 + width)
    alphabet = list("abcdefgé漢 ")
    r1, r2 = [], []
    for _ in range(1200):
        common = "".join(rng.choice(alphabet, int(rng.integers(0, 300))))
        u = rng.random()
        r1.append(None if u < 0.04 else "" if u < 0.08 else "".join(rng.choice(alphabet, int(rng.integers(0, 40)))) + common)
        u = rng.random()
        r2.append(None if u < 0.04 else "" if u < 0.08 else common + "".join(rng.choice(alphabet, int(rng.integers(0, 80)))))
    # pairs beyond the 4096 bytes of the LDS set, and one far beyond
    for n1, n2 in [(3000, 3000), (9000, 100), (100, 20000), (300_000, 250_000)]:
        base = "".join(rng.choice(alphabet[:6], 64))
        r1.append((base * (n1 // 64 + 1))[:n1])
        r2.append("".join(rng.choice(alphabet[:6], n2 // 2)) + (base * (n2 // 128 + 1))[: n2 // 2])
    for dtype in (np.int32, np.int64):
        h1, h2 = strings(r1, dtype), strings(r2, dtype)
        d1, d2 = dev(nv, h1), dev(nv, h2)
        assert_same_fixed(nv.jaccard_index(d1, d2, width).to_host(), orc.jaccard_index(h1, h2, width, nthreads=8), f"jaccard width={width}")
        lo, hi = 7, 1150
        s1, s2 = h1.slice(lo, hi), h2.slice(lo + 3, hi + 3)
        assert_same_fixed(nv.jaccard_index(d1.slice(lo, hi, s1.null_count), d2.slice(lo + 3, hi + 3, s2.null_count), width).to_host(),
                          orc.jaccard_index(s1, s2, width, nthreads=4), "jaccard sliced")
    # no nulls: no mask; same column twice: all ones (or 0 for empty rows)
    clean = strings([x or "" for x in r1[:300]])
    same = nv.jaccard_index(dev(nv, clean), dev(nv, clean), width).to_host()
    assert same.mask is None and same.null_count == 0
    lens = np.diff(clean.offsets)
    assert np.array_equal(same.values, np.where(lens > 0, np.float32(1), np.float32(0)))


def test_jaccard_errors_and_empty(nv):
    three, two = dev(nv, strings(["1", "2", "3"])), dev(nv, strings(["1", "2"]))
    with pytest.raises(ValueError):
        nv.jaccard_index(three, three, 1)
    with pytest.raises(ValueError):
        nv.jaccard_index(three, two, 5)
    empty = nv.jaccard_index(dev(nv, strings([])), dev(nv, strings([])), 5).to_host()
    assert empty.size == 0 and empty.values.size == 0


# ----------------------------------------------------------------------------- wordpiece
@pytest.mark.parametrize("case", gc.wordpiece_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_wordpiece_golden(nv, case, dtype):
    vocab = nv.WordPieceVocabulary(dev(nv, strings(case["vocab"])))
    host = strings(case["rows"], dtype)
    col = dev(nv, host)
    if "slice" in case:
        lo, hi = case["slice"]
        col = col.slice(lo, hi, host.slice(lo, hi).null_count)
    for run in case["runs"]:
        got = nv.wordpiece_tokenize(col, vocab, run["max_words"]).to_host()
        assert gc.expected_list_equal(got.to_pylist(), run["expected"]), (case["name"], run["max_words"])
        assert got.child.dtype == np.int32


def test_wordpiece_bert_sentences(nv):
    d = gc.bert_case()
    vocab = nv.WordPieceVocabulary(dev(nv, strings(d["vocab"])))
    assert vocab.unk_id == 100
    col = dev(nv, strings(d["rows"]))
    for mw, exp in d["expected"].items():
        got = nv.wordpiece_tokenize(col, vocab, int(mw)).to_host()
        assert gc.expected_list_equal(got.to_pylist(), exp), mw


def test_wordpiece_errors_and_empty(nv):
    with pytest.raises(ValueError):
        nv.WordPieceVocabulary(dev(nv, strings([])))
    with pytest.raises(ValueError):
        nv.WordPieceVocabulary(dev(nv, strings([None, None, None])))
    v = nv.WordPieceVocabulary(dev(nv, strings(["x"])))
    assert v.unk_id == -1
    with pytest.raises(ValueError):
        nv.wordpiece_tokenize(dev(nv, strings(["  "])), v, -1)
    v2 = nv.WordPieceVocabulary(dev(nv, strings([""])))
    for mw in (0, 10):
        got = nv.wordpiece_tokenize(dev(nv, strings([])), v2, mw).to_host()
        assert got.size == 0 and got.offsets.size == 0


def make_vocab(rng, n, letters, with_unk=True):
    vocab = (["[PAD]", "[UNK]"] if with_unk else ["[PAD]"]) + list(letters) + ["##" + c for c in letters]
    seen = set(vocab)
    while len(vocab) < n:
        ln = int(rng.integers(2, 14))
        s = "".join(rng.choice(list(letters), ln))
        if rng.random() < 0.4:
            s = "##" + s
        if s not in seen:
            seen.add(s)
            vocab.append(s)
    return vocab


@pytest.fixture(params=["column", "2", "8"], ids=["ranges_by_column_size", "ranges_of_2_tiles", "ranges_of_8_tiles"])
def range_tiles(request):
    """The tokenizer gives a wavefront ranges of 1 to 8 tiles, the fewer the smaller the column; the columns of these
    tests are all small, so the tests that take this fixture run a second time with the size that a column of a
    gigabyte gets (set through the library's test knob, nvtext_amd_profile_set_range_tiles)."""
    from cudf_amd import _capi
    _capi.set_range_tiles(0 if request.param == "column" else int(request.param))
    yield request.param
    _capi.set_range_tiles(0)


@pytest.mark.parametrize("max_words", [0, 7, 1000])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_wordpiece_random_vs_oracle(nv, orc, max_words, dtype, range_tiles):
    rng = np.random.default_rng(77 + max_words)
    letters = "abcdefghijkl"
    vocab = make_vocab(rng, 3000, letters)
    stems = [v for v in vocab[2:] if not v.startswith("##")]
    rows = []
    for _ in range(1500):
        u = rng.random()
        if u < 0.03:
            rows.append(None)
            continue
        if u < 0.06:
            rows.append("")
            continue
        nw = int(rng.integers(1, 120))
        ws = []
        for _ in range(nw):
            t = rng.random()
            if t < 0.7:
                ws.append(stems[int(rng.integers(0, len(stems)))])
            elif t < 0.97:
                ws.append("".join(rng.choice(list(letters + "xyz"), int(rng.integers(1, 20)))))
            else:
                ws.append("".join(rng.choice(list(letters), int(rng.integers(150, 260)))))
        sep = " " if max_words else ("  " if rng.random() < 0.1 else " ")
        s = sep.join(ws)
        if rng.random() < 0.2:
            s = " " + s
        if rng.random() < 0.2:
            s = s + " "  # a single trailing space is well defined in both paths
        rows.append(s)
    rows += ["a", " ", "a b", "ab", "  a", "a" * 199, "a" * 200, "a" * 600 + " b"]
    host = strings(rows, dtype)
    hv = strings(vocab)
    got = nv.wordpiece_tokenize(dev(nv, host), nv.WordPieceVocabulary(dev(nv, hv)), max_words).to_host()
    exp = orc.wordpiece_tokenize(host, orc.Vocabulary(hv), max_words, nthreads=8)
    assert_same(got, exp, f"wordpiece mw={max_words}")
    assert exp.child.size > (5000 if max_words == 7 else 50000)


def _tile_kernel_launches(nv, fn):
    """Runs fn() with the library's kernel timing on; returns its result and the number of tile-pass launches."""
    from cudf_amd import _capi
    import torch
    _capi.profile_enable(True)
    _capi.profile_read()
    try:
        out = fn()
        torch.cuda.synchronize()
        names = [n for n, _ in _capi.profile_read()]
    finally:
        _capi.profile_enable(False)
    return out, sum(1 for n in names if n == "wordpiece_word_kernel")


@pytest.fixture(params=[False, True], ids=["sized_by_default", "sized_by_sample"])
def sizing_sample(request):
    """wordpiece_tokenize sizes its first attempt from a sample of the column; without the sample (the library's test
    knob) a column that needs more than the default sizes reaches the second attempt."""
    from cudf_amd import _capi
    _capi.set_sizing_sample(request.param)
    yield request.param
    _capi.set_sizing_sample(True)


@pytest.mark.parametrize("max_words", [0, 5, 100000])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
@pytest.mark.parametrize("shape", ["few rows", "many rows"])
def test_wordpiece_more_tokens_than_the_first_attempt_has_room_for(nv, orc, shape, dtype, max_words, range_tiles, sizing_sample):
    """Text whose ranges give more than three tokens per eight bytes (here two-letter words that are not in the
    vocabulary and fall apart into letters: two tokens per three bytes) does not fit the arena of an attempt with
    the default sizes: the call has to notice, run the tile pass again with room for a token per byte, and give the
    same result as the oracle (greedy rule: cpp/src/text/wordpiece_tokenize.cu:349-407).  A million such words, in
    a few long rows and in many short ones; the launches are read off the library's kernel timing: two without the
    sample of the column that sizes the first attempt, one with it."""
    rng = np.random.default_rng(5)
    letters = "abcdefgh"
    vocab = ["[UNK]"] + list(letters) + ["##" + c for c in letters] + ["abcdefgh"]
    words = ["".join(rng.choice(list(letters), 2)) for _ in range(4096)]
    per_row = 125000 if shape == "few rows" else 7
    nrows = 8 if shape == "few rows" else 150000
    rows = [" ".join(words[int(j) % 4096] for j in rng.integers(0, 4096, per_row)) for _ in range(nrows)]
    rows[1] = None
    rows[2] = ""
    host = strings(rows, dtype)
    hv = strings(vocab)
    dcol, dvoc = dev(nv, host), nv.WordPieceVocabulary(dev(nv, hv))
    got, launches = _tile_kernel_launches(nv, lambda: nv.wordpiece_tokenize(dcol, dvoc, max_words))
    exp = orc.wordpiece_tokenize(host, orc.Vocabulary(hv), max_words, nthreads=8)
    assert_same(got.to_host(), exp, f"{shape}, max_words={max_words}")
    if max_words != 5 or shape == "many rows":
        # (five words of a long row are too few tokens to fill anything; the sample looks at the text, not at the limit)
        assert launches == (1 if sizing_sample else 2), launches
        assert exp.child.size > 1_000_000
    # ordinary text right afterwards: one launch, nothing left over from the call before
    plain = strings(["abcdefgh " * 2000] * 50, dtype)
    got, launches = _tile_kernel_launches(nv, lambda: nv.wordpiece_tokenize(dev(nv, plain), dvoc, max_words))
    if sizing_sample:
        assert launches == 1   # (without the sample a word that the table keeps outside its home bucket is queued every time)
    assert_same(got.to_host(), orc.wordpiece_tokenize(plain, orc.Vocabulary(hv), max_words, nthreads=8), "plain text afterwards")


def test_wordpiece_rows_of_one_byte_and_tiles_of_more_words_than_a_unit(nv, orc, range_tiles):
    """Every byte a row of its own (row starts separate words as spaces do: cpp/src/text/wordpiece_tokenize.cu:515-523), so a
    tile of 2048 bytes holds 2048 words, four times what is looked up at a time, and a token per byte; then the
    same bytes as words of one letter between spaces (1024 words per tile).  With a word limit a one-byte row has
    room for no word at all (limit = bytes / 2, :780)."""
    rng = np.random.default_rng(6)
    letters = "abcdefgh"
    vocab = ["[UNK]"] + list(letters) + ["##" + c for c in letters]
    hv = strings(vocab)
    dvoc, ovoc = nv.WordPieceVocabulary(dev(nv, hv)), orc.Vocabulary(hv)
    n = 300_000
    chars = rng.choice(list(letters + "xy"), n)
    for dtype in (np.int32, np.int64):
        one_byte_rows = strings(list(chars), dtype)
        spaced = strings([" ".join(chars[i:i + 5000]) for i in range(0, n, 5000)] + ["x", " ", ""], dtype)
        for host in (one_byte_rows, spaced):
            for max_words in (0, 3):
                got = nv.wordpiece_tokenize(dev(nv, host), dvoc, max_words).to_host()
                assert_same(got, orc.wordpiece_tokenize(host, ovoc, max_words, nthreads=8), f"max_words={max_words}")
    assert orc.wordpiece_tokenize(one_byte_rows, ovoc, 0, nthreads=8).child.size == n


def test_wordpiece_utf8_vs_oracle(nv, orc, range_tiles):
    rng = np.random.default_rng(99)
    base = list("abcdeé漢字ñ語😀")
    vocab = ["[unk]"] + base + ["##" + c for c in base[:8]]
    seen = set(vocab)
    while len(vocab) < 1500:
        s = "".join(rng.choice(base, int(rng.integers(2, 6))))
        if rng.random() < 0.4:
            s = "##" + s
        if s not in seen:
            seen.add(s)
            vocab.append(s)
    rows = [" ".join("".join(rng.choice(base + ["z"], int(rng.integers(1, 9)))) for _ in range(int(rng.integers(1, 60))))
            for _ in range(800)]
    host = strings(rows, np.int64)
    hv = strings(vocab)
    for mw in (0, 16):
        got = nv.wordpiece_tokenize(dev(nv, host), nv.WordPieceVocabulary(dev(nv, hv)), mw).to_host()
        assert_same(got, orc.wordpiece_tokenize(host, orc.Vocabulary(hv), mw, nthreads=4), f"utf8 mw={mw}")


def test_wordpiece_sliced_nulls_vs_oracle(nv, orc, range_tiles):
    rng = np.random.default_rng(123)
    vocab = make_vocab(rng, 500, "abcdef")
    rows = []
    for _ in range(400):
        if rng.random() < 0.25:
            rows.append(None)
        else:
            rows.append(" ".join("".join(rng.choice(list("abcdefg"), int(rng.integers(1, 8)))) for _ in range(int(rng.integers(0, 30)))))
    host = strings(rows)
    hv = strings(vocab)
    dv = nv.WordPieceVocabulary(dev(nv, hv))
    ov = orc.Vocabulary(hv)
    for lo, hi in [(0, 400), (5, 390), (33, 65), (100, 101)]:
        hs = host.slice(lo, hi)
        ds = dev(nv, host).slice(lo, hi, hs.null_count)
        for mw in (0, 5):
            assert_same(nv.wordpiece_tokenize(ds, dv, mw).to_host(), orc.wordpiece_tokenize(hs, ov, mw), f"slice {lo}:{hi} mw={mw}")


def test_wordpiece_row_longer_than_chunks(nv, orc, range_tiles):
    """One row spanning many 256-byte chunks, with words straddling chunk boundaries."""
    rng = np.random.default_rng(321)
    vocab = make_vocab(rng, 2000, "abcdefgh")
    words = ["".join(rng.choice(list("abcdefghz"), int(rng.integers(1, 30)))) for _ in range(20000)]
    rows = [" ".join(words), " ".join(words[:7000]), "x", " ".join(words[100:5000])]
    host = strings(rows)
    hv = strings(vocab)
    for mw in (0, 3000):
        got = nv.wordpiece_tokenize(dev(nv, host), nv.WordPieceVocabulary(dev(nv, hv)), mw).to_host()
        assert_same(got, orc.wordpiece_tokenize(host, orc.Vocabulary(hv), mw, nthreads=4), f"long row mw={mw}")


def test_wordpiece_long_keys_and_many_pieces(nv, orc):
    """Keys of 1..60 bytes that share their first bytes (so the per-prefix length filter has several bits,
    including the one for 34 bytes and more), multi-byte characters at byte 2 and 3 of keys and words,
    and words that split into more than eight pieces."""
    rng = np.random.default_rng(2024)
    base = list("abcé漢😀")
    vocab = ["[UNK]"] + base + ["##" + c for c in base]
    seen = set(vocab)
    heads = ["ab", "aé", "a漢", "é漢", "漢a", "😀", "abc", "b"]
    while len(vocab) < 1200:
        n = int(rng.choice([1, 2, 3, 4, 6, 9, 15, 31, 32, 33, 34, 35, 40, 60]))
        s = heads[int(rng.integers(0, len(heads)))]
        while len(s.encode()) < n:
            s += base[int(rng.integers(0, len(base)))]
        if rng.random() < 0.5:
            s = "##" + s
        if s not in seen and len(s.encode()) < 199:
            seen.add(s)
            vocab.append(s)
    keys = [v[2:] if v.startswith("##") else v for v in vocab[1:]]
    rows = []
    for _ in range(600):
        ws = []
        for _ in range(int(rng.integers(1, 25))):
            t = rng.random()
            if t < 0.5:  # several keys glued together: pieces of every length class
                ws.append("".join(keys[int(rng.integers(0, len(keys)))] for _ in range(int(rng.integers(1, 5)))))
            elif t < 0.8:  # single letters: one piece per character, often more than eight
                ws.append("".join(rng.choice(base, int(rng.integers(1, 30)))))
            else:  # a key cut short or followed by a letter outside the vocabulary
                k = keys[int(rng.integers(0, len(keys)))]
                ws.append(k[: max(1, len(k) - int(rng.integers(0, 3)))] + ("z" if rng.random() < 0.5 else ""))
        rows.append(" ".join(w for w in ws if w))
    host = strings(rows, np.int32)
    hv = strings(vocab)
    for mw in (0, 10):
        got = nv.wordpiece_tokenize(dev(nv, host), nv.WordPieceVocabulary(dev(nv, hv)), mw).to_host()
        exp = orc.wordpiece_tokenize(host, orc.Vocabulary(hv), mw, nthreads=4)
        assert_same(got, exp, f"long keys mw={mw}")
    assert exp.child.size > 5000


@pytest.mark.parametrize("letters", [5, 7, 8, 12])
def test_wordpiece_every_word_splits_into_as_many_pieces_as_it_has_letters(nv, orc, letters, range_tiles):
    """A vocabulary of single letters only, so that a word of k letters is k tokens: rounds of the library's last pass
    in which every word brings five tokens (its usual way of writing them), seven (more tokens in a round than it puts in
    order before writing: each word's are then written by themselves), eight and twelve (more than a word's record
    keeps: tokenized again into place)."""
    rng = np.random.default_rng(100 + letters)
    alphabet = list("abcdefgh")
    vocab = ["[UNK]"] + alphabet + ["##" + c for c in alphabet]
    rows = []
    for _ in range(400):
        n = int(rng.integers(0, 60))
        rows.append(" ".join("".join(rng.choice(alphabet, letters)) for _ in range(n)))
    rows[7] = ""
    host = strings(rows, np.int32)
    hv = strings(vocab)
    for mw in (0, 11):
        got = nv.wordpiece_tokenize(dev(nv, host), nv.WordPieceVocabulary(dev(nv, hv)), mw).to_host()
        exp = orc.wordpiece_tokenize(host, orc.Vocabulary(hv), mw, nthreads=4)
        assert_same(got, exp, f"{letters} letters mw={mw}")
    assert exp.child.size > 400 * 5 * letters


def test_wordpiece_pieces_of_letters_and_of_their_neighbours(nv, orc):
    """Later pieces of a word ("##" keys) over an alphabet of lower-case letters and the bytes next to them in ASCII
    ('`' before 'a', '{' after 'z', capitals, digits): the library serves the pieces that begin with two or three
    lower-case letters from small tables of their own and the others from the general ones, and both have to say the
    same as the oracle; keys of every length from 1 to 20 bytes, so that the lengths that the three-letter table names
    one by one (3 to 9) and those that share its last bit are met, and fourth bytes that share a bit of its fourth-byte
    mask ('z' and 'b', 'a' and 'A' and '9') with and without a key of their own."""
    rng = np.random.default_rng(77)
    letters = list("azmb")
    others = list("`{AZ09")
    alphabet = letters * 3 + others
    vocab = ["[UNK]"]
    seen = set(vocab)
    for c in letters + others[:3]:
        for v in (c, "##" + c):
            seen.add(v)
            vocab.append(v)
    while len(vocab) < 2500:
        n = int(rng.choice([2, 2, 3, 3, 3, 4, 5, 6, 8, 9, 12, 15, 16, 17, 18, 19, 20]))
        k = "".join(rng.choice(alphabet if rng.random() < 0.6 else letters, n))
        v = "##" + k if rng.random() < 0.7 else k
        if v not in seen:
            seen.add(v)
            vocab.append(v)
    keys = [v[2:] if v.startswith("##") else v for v in vocab[1:]]
    rows = []
    for _ in range(3000):
        ws = []
        for _ in range(int(rng.integers(1, 20))):
            t = rng.random()
            if t < 0.6:  # keys glued together, cut to the 16 bytes and fewer that the short-word path takes, or longer
                w = "".join(keys[int(rng.integers(0, len(keys)))] for _ in range(int(rng.integers(1, 4))))
                ws.append(w[: int(rng.integers(1, 17))] if rng.random() < 0.7 else w)
            else:
                ws.append("".join(rng.choice(alphabet, int(rng.integers(1, 17)))))
        rows.append(" ".join(ws))
    host = strings(rows, np.int32)
    hv = strings(vocab)
    for mw in (0, 7):
        got = nv.wordpiece_tokenize(dev(nv, host), nv.WordPieceVocabulary(dev(nv, hv)), mw).to_host()
        exp = orc.wordpiece_tokenize(host, orc.Vocabulary(hv), mw, nthreads=4)
        assert_same(got, exp, f"letters and neighbours mw={mw}")
    assert exp.child.size > 30000
    # the test means to meet known and unknown words alike
    unk = int((exp.child == 0).sum())
    assert 0 < unk < exp.child.size


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_wordpiece_very_long_rows_are_cut_at_spaces(nv, orc, dtype, range_tiles):
    """Rows of hundreds of kilobytes (which the library tokenizes in pieces cut at spaces when there is no word limit)
    among short ones: with words of every length at the places where the cuts fall, a row that is one long word, a
    row that is mostly spaces, null rows, and the same column sliced."""
    rng = np.random.default_rng(77)
    letters = list("abcdefghij")
    vocab = ["[UNK]"] + letters + ["##" + c for c in letters] + ["ab", "abc", "##cd", "hello", "##llo"]
    def text(nbytes, max_word):
        words, total = [], 0
        while total < nbytes:
            w = "".join(rng.choice(letters, int(rng.integers(1, max_word + 1))))
            words.append(w)
            total += len(w) + 1
        return " ".join(words)
    rows = ["hello ab", text(70_000, 6), None, "", text(300_000, 40), "abc", "z" * 150_000, " " * 90_000 + "ab" + " " * 90_000,
            text(1_100_000, 12), text(32_768, 3)[:32_768], text(32_769, 3)[:32_769], None, "ab cd"]
    host = strings(rows, dtype)
    dv = nv.WordPieceVocabulary(dev(nv, strings(vocab)))
    ov = orc.Vocabulary(strings(vocab))
    for view in (host, host.slice(1, 10)):
        got = nv.wordpiece_tokenize(dev(nv, view), dv, 0).to_host()
        assert_same(got, orc.wordpiece_tokenize(view, ov, 0, nthreads=8), "very long rows")
    # with a word limit the rows are not cut (and end after the limit)
    got = nv.wordpiece_tokenize(dev(nv, host), dv, 50).to_host()
    assert_same(got, orc.wordpiece_tokenize(host, ov, 50, nthreads=8), "very long rows, word limit")


@pytest.mark.parametrize("max_words", [0, 4])
def test_wordpiece_long_runs_of_rows_without_bytes(nv, orc, max_words, range_tiles):
    """Hundreds of thousands of empty and null rows in a row, before, between and after rows with text: the rows are
    shared out by work, and rows without bytes must neither be lost nor all fall to one group of lanes."""
    vocab = strings(["[UNK]", "hello", "world", "##s", "a", "b"])
    rows = [""] * 300_000 + ["hello worlds a b zzz"] * 500 + [None] * 200_000 + ["a"] + [""] * 100_000 + ["b hello"] * 3 + [None] * 7
    host = strings(rows, np.int32)
    got = nv.wordpiece_tokenize(dev(nv, host), nv.WordPieceVocabulary(dev(nv, vocab)), max_words).to_host()
    assert_same(got, orc.wordpiece_tokenize(host, orc.Vocabulary(vocab), max_words, nthreads=4), f"max_words={max_words}")
    assert got.offsets[300_000] == 0 and got.offsets[-1] == got.child.size > 0


@pytest.mark.parametrize("which", ["bert 30k", "multilingual 250k"])
def test_wordpiece_every_vocabulary_entry_is_its_own_token(nv, orc, which):
    """Each entry of a generated vocabulary, as a word in the middle of a row and as the only word of a row: its
    token is its own index (the first one, if the entry occurs twice).  This reaches every key wherever the table
    put it -- in its home bucket, carried past one full bucket or past several -- and every key length."""
    from cudf_amd import datagen
    vocab = (datagen.make_vocab(datagen.VOCAB_BERT, 30522, seed=1001) if which == "bert 30k"
             else datagen.make_vocab(datagen.VOCAB_MULTILINGUAL, 250000, seed=1005))
    entries = vocab.to_pylist()
    first = {}
    for i, e in enumerate(entries):
        first.setdefault(e, i)
    words = [(e, first[e]) for e in entries if e and not e.startswith(b"##") and b" " not in e and len(e) < 199]
    assert len(words) > 0.5 * len(entries)
    dv = nv.WordPieceVocabulary(dev(nv, vocab))
    # alone in their rows
    alone = HostStringsColumn.from_pylist([w for w, _ in words])
    got = nv.wordpiece_tokenize(dev(nv, alone), dv, 0).to_host()
    assert np.array_equal(got.offsets, np.arange(len(words) + 1, dtype=np.int32))
    assert np.array_equal(got.child, np.array([i for _, i in words], np.int32))
    # sixteen to a row, and against the oracle
    rows = [b" ".join(w for w, _ in words[k: k + 16]) for k in range(0, len(words), 16)]
    packed = HostStringsColumn.from_pylist(rows)
    got = nv.wordpiece_tokenize(dev(nv, packed), dv, 0).to_host()
    assert np.array_equal(got.child, np.array([i for _, i in words], np.int32))
    assert_same(got, orc.wordpiece_tokenize(packed, orc.Vocabulary(vocab), 0, nthreads=8), which)


def test_cpp_api_program():
    """The C++ mirror of the nvtext API (cudf_amd/include) run on the reference's gtest cases."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "nvtext_api_test")
    assert os.path.exists(exe), "build it with __graft_entry__.build() or make -C tests/cpp"
    p = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "ALL PASSED" in p.stdout


# ----------------------------------------------------------------------------- the caller's stream
def test_every_operation_on_streams_of_the_caller(nv, orc):
    """Everything so far ran on the default stream.  Here the inputs are uploaded and the operations issued on two
    streams the caller made (which do not synchronise with the default stream), calls alternating between them; a
    kernel or copy that the library put on another stream than the one it was given would race with the upload or
    with the result's download."""
    import torch
    from cudf_amd import datagen
    from oracle import normalize_py
    w = datagen.config5(0.02)  # 160k UTF-8 rows, int64 offsets, 250k-entry vocabulary
    host, p = w.rows, w.params
    a32, b32 = datagen.make_params(32, 32, 1)
    a64, b64 = datagen.make_params(32, 64, 2)
    lists = datagen.words_as_lists(datagen.config3(0.005).rows)
    h1, h2 = host.slice(0, host.size - 1), host.slice(1, host.size)
    ov = orc.Vocabulary(w.vocab)
    expected = {
        "tokens": orc.wordpiece_tokenize(host, ov, p["max_words_per_row"], nthreads=8),
        "minhash": orc.minhash(host, 3, a32, b32, 5, nthreads=8),
        "minhash64": orc.minhash64(host, 4, a64, b64, 7, nthreads=8),
        "ngrams": orc.minhash_ngrams(lists, 3, 5, a32, b32, nthreads=8),
        "normalized": normalize_py.normalize_characters_native(host, True, [b"[CLS]"], nthreads=8),
        "jaccard": orc.jaccard_index(h1, h2, 5, nthreads=8),
    }
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [{}, {}]
    for turn in range(2):
        for k, s in enumerate(streams):
            with torch.cuda.stream(s):
                if turn == 0:
                    d = dev(nv, host)
                    got[k]["d"] = d
                    got[k]["vocab"] = nv.WordPieceVocabulary(dev(nv, w.vocab))
                    got[k]["normalizer"] = nv.CharacterNormalizer(True, dev(nv, strings(["[CLS]"])))
                    got[k]["minhash"] = nv.minhash(d, 3, a32, b32, 5)
                    got[k]["minhash64"] = nv.minhash64(d, 4, a64, b64, 7)
                    got[k]["ngrams"] = nv.minhash_ngrams(nv.DeviceListStringsColumn.from_host(lists), 3, 5, a32, b32)
                else:
                    d = got[k]["d"]
                    got[k]["tokens"] = nv.wordpiece_tokenize(d, got[k]["vocab"], p["max_words_per_row"])
                    got[k]["normalized"] = nv.normalize_characters(d, got[k]["normalizer"])
                    got[k]["jaccard"] = nv.jaccard_index(d.slice(0, host.size - 1, 0), d.slice(1, host.size, 0), 5)
    for k, s in enumerate(streams):
        with torch.cuda.stream(s):
            for name in ("tokens", "minhash", "minhash64", "ngrams"):
                assert_same(got[k][name].to_host(), expected[name], f"{name} on stream {k}")
            n = got[k]["normalized"].to_host()
            assert np.array_equal(n.offsets, expected["normalized"].offsets) and np.array_equal(n.chars, expected["normalized"].chars), f"normalized on stream {k}"
            j = got[k]["jaccard"].to_host()
            assert np.array_equal(j.values.view(np.uint32), expected["jaccard"].values.view(np.uint32)), f"jaccard on stream {k}"
    torch.cuda.synchronize()


# ----------------------------------------------------------------------------- a failing allocator
def test_allocation_failures_are_reported_and_leak_nothing(nv, orc):
    """The caller's allocator refuses the n-th request of a call and every later one, for every n until the call
    succeeds.  Each failed call reports NVTEXT_AMD_ALLOC_FAILED (MemoryError in this binding) and has given back what
    it had been given; the call that succeeds has the oracle's result."""
    from oracle import normalize_py
    from cudf_amd import datagen
    rng = np.random.default_rng(3)
    vocab = strings(["[UNK]", "hello", "world", "##s", "a", "b", "##b", "ab"])
    words = ["hello", "worlds", "a", "abb", "zzz", "b"]
    rows = [None if i % 7 == 3 else " ".join(rng.choice(words, int(rng.integers(0, 30)))) for i in range(2000)]
    rows[11] = " ".join(rng.choice(words, 12_000))   # beyond 32 KiB: cut into pieces when there is no word limit
    rows[12] = rows[11][:30_000]                      # a pair for jaccard_index' set in global memory
    host = strings(rows, np.int64)
    d = dev(nv, host)
    dv, ov = nv.WordPieceVocabulary(dev(nv, vocab)), orc.Vocabulary(vocab)
    a32, b32 = datagen.make_params(20, 32, 1)
    a64, b64 = datagen.make_params(20, 64, 2)
    lists = gc.list_strings([None if i % 5 == 2 else [str(w) for w in rng.choice(words, int(rng.integers(0, 9)))] for i in range(300)])
    dl = nv.DeviceListStringsColumn.from_host(lists)
    h1, h2 = host.slice(0, host.size - 1), host.slice(1, host.size)
    d1, d2 = d.slice(0, host.size - 1, h1.null_count), d.slice(1, host.size, h2.null_count)
    normalizer = nv.CharacterNormalizer(True, None)

    def lists_equal(got, exp, what):
        assert_same(got.to_host(), exp, what)

    def strings_equal(got, exp, what):
        g = got.to_host()
        assert np.array_equal(g.offsets, exp.offsets) and np.array_equal(g.chars, exp.chars), what
        assert np.array_equal(g.validity(), exp.validity()), what

    def floats_equal(got, exp, what):
        g, v = got.to_host(), exp.validity()
        assert g.null_count == exp.null_count and np.array_equal(g.validity(), v), what
        assert np.array_equal(g.values.view(np.uint32)[v], exp.values.view(np.uint32)[v]), what

    calls = [
        ("tokenize", lambda: nv.wordpiece_tokenize(d, dv, 0), lambda: orc.wordpiece_tokenize(host, ov, 0, nthreads=4), lists_equal),
        ("tokenize, word limit", lambda: nv.wordpiece_tokenize(d, dv, 5), lambda: orc.wordpiece_tokenize(host, ov, 5, nthreads=4), lists_equal),
        ("minhash", lambda: nv.minhash(d, 1, a32, b32, 4), lambda: orc.minhash(host, 1, a32, b32, 4, nthreads=4), lists_equal),
        ("minhash64", lambda: nv.minhash64(d, 1, a64, b64, 4), lambda: orc.minhash64(host, 1, a64, b64, 4, nthreads=4), lists_equal),
        ("minhash_ngrams", lambda: nv.minhash_ngrams(dl, 2, 1, a32, b32), lambda: orc.minhash_ngrams(lists, 2, 1, a32, b32), lists_equal),
        ("minhash64_ngrams", lambda: nv.minhash64_ngrams(dl, 2, 1, a64, b64), lambda: orc.minhash64_ngrams(lists, 2, 1, a64, b64), lists_equal),
        ("normalize", lambda: nv.normalize_characters(d, normalizer),
         lambda: normalize_py.normalize_characters_native(host, True, [], nthreads=4), strings_equal),
        ("jaccard", lambda: nv.jaccard_index(d1, d2, 5), lambda: orc.jaccard_index(h1, h2, 5, nthreads=4), floats_equal),
    ]
    mr = nv._mr()
    held = len(mr.live)
    try:
        for name, call, expect, same in calls:
            refused = 0
            for n in range(40):
                mr.fail_after = n
                try:
                    got = call()
                except MemoryError:
                    refused += 1
                    assert len(mr.live) == held, f"{name}: buffers kept after the failure of request {n}"
                    continue
                finally:
                    mr.fail_after = None
                assert len(mr.live) == held, f"{name}: buffers kept after success"
                same(got, expect(), name)
                break
            else:
                raise AssertionError(f"{name} still fails with 40 requests granted")
            assert refused >= 2, f"{name}: only {refused} requests seen"
    finally:
        mr.fail_after = None


# ----------------------------------------------------------------------------- several host threads
def test_host_threads_share_a_vocabulary_and_a_normalizer(nv, orc):
    """Four host threads, each with a stream of its own, call the operations at the same time on the same input
    columns, vocabulary and normalizer (which are immutable once made); every result is the oracle's."""
    import torch
    from concurrent.futures import ThreadPoolExecutor
    from cudf_amd import datagen
    from oracle import normalize_py
    w = datagen.config5(0.01)
    host, p = w.rows, w.params
    a32, b32 = datagen.make_params(16, 32, 1)
    a64, b64 = datagen.make_params(16, 64, 2)
    h1, h2 = host.slice(0, host.size - 1), host.slice(1, host.size)
    ov = orc.Vocabulary(w.vocab)
    exp_tokens = orc.wordpiece_tokenize(host, ov, p["max_words_per_row"], nthreads=8)
    exp_mh = orc.minhash(host, 3, a32, b32, 5, nthreads=8)
    exp_mh64 = orc.minhash64(host, 4, a64, b64, 7, nthreads=8)
    exp_norm = normalize_py.normalize_characters_native(host, True, [], nthreads=8)
    exp_j = orc.jaccard_index(h1, h2, 5, nthreads=8)
    d = dev(nv, host)
    dv = nv.WordPieceVocabulary(dev(nv, w.vocab))
    normalizer = nv.CharacterNormalizer(True, None)
    d1, d2 = d.slice(0, host.size - 1, 0), d.slice(1, host.size, 0)
    torch.cuda.synchronize()

    def worker(k):
        out = []
        with torch.cuda.stream(torch.cuda.Stream()):
            for turn in range(3):
                order = [(turn + k + i) % 5 for i in range(5)]
                for what in order:
                    if what == 0:
                        out.append(("tokens", nv.wordpiece_tokenize(d, dv, p["max_words_per_row"]).to_host()))
                    elif what == 1:
                        out.append(("minhash", nv.minhash(d, 3, a32, b32, 5).to_host()))
                    elif what == 2:
                        out.append(("minhash64", nv.minhash64(d, 4, a64, b64, 7).to_host()))
                    elif what == 3:
                        out.append(("normalized", nv.normalize_characters(d, normalizer).to_host()))
                    else:
                        out.append(("jaccard", nv.jaccard_index(d1, d2, 5).to_host()))
        return out

    with ThreadPoolExecutor(4) as pool:
        results = list(pool.map(worker, range(4)))
    for k, out in enumerate(results):
        assert len(out) == 15
        for name, got in out:
            what = f"{name} from thread {k}"
            if name == "tokens":
                assert_same(got, exp_tokens, what)
            elif name == "minhash":
                assert_same(got, exp_mh, what)
            elif name == "minhash64":
                assert_same(got, exp_mh64, what)
            elif name == "normalized":
                assert np.array_equal(got.offsets, exp_norm.offsets) and np.array_equal(got.chars, exp_norm.chars), what
            else:
                assert np.array_equal(got.values.view(np.uint32), exp_j.values.view(np.uint32)), what
