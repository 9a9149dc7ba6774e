"""The five benchmark workloads (cudf_amd.datagen.config1..5) as parity cases.

Host part (no GPU): the generator is deterministic and produces the stated shapes, and the oracle runs
configuration 1 end to end.  GPU part: every configuration at its full size through the C ABI, compared
bit for bit with the oracle where the oracle finishes in seconds (all of C1, C2 and C5's tokenization,
row samples of the minhash workloads, the longest rows of C4) and through size-independent properties on
the whole output: a slice of the input gives the matching slice of the output, a subset of the (a, b)
parameters gives the matching columns, null rows have no slots, offsets are the expected arithmetic
progression.
"""
import zlib

import numpy as np
import pytest

from cudf_amd import datagen
from cudf_amd.arrow_host import HostStringsColumn


def _crc(col):
    return zlib.crc32(np.ascontiguousarray(col.offsets).tobytes(), zlib.crc32(np.ascontiguousarray(col.chars).tobytes()))


# ----------------------------------------------------------------------------- host
def test_generator_is_deterministic_and_shaped():
    a = datagen.config2(0.002)
    b = datagen.config2(0.002)
    assert _crc(a.rows) == _crc(b.rows) and _crc(a.vocab) == _crc(b.vocab)
    assert a.rows.size == 8000 and a.rows.offsets.dtype == np.int32 and a.vocab.size == 30522
    mean = a.rows.chars_bytes / a.rows.size
    assert 200 < mean < 320
    c5 = datagen.config5(0.0005)
    assert c5.rows.offsets.dtype == np.int64 and c5.vocab.size == 250000
    assert (np.frombuffer(np.ascontiguousarray(c5.rows.chars), np.uint8) >= 0x80).mean() > 0.05  # multi-byte text
    c4 = datagen.config4(0.02)
    assert 0.05 < c4.rows.null_count / c4.rows.size < 0.15
    lens = np.diff(c4.rows.offsets.astype(np.int64))
    assert lens.max() <= (1 << 20)


def test_config1_on_the_oracle():
    from oracle import pyoracle as orc
    w = datagen.config1()
    p = w.params
    assert w.rows.size == 10000 and w.rows.null_count > 0
    tok = orc.wordpiece_tokenize(w.rows, orc.Vocabulary(w.vocab), p["max_words_per_row"], nthreads=4)
    valid = w.rows.validity()
    lens = np.diff(w.rows.offsets.astype(np.int64))
    counts = np.diff(tok.offsets.astype(np.int64))
    # single spaces, no leading or trailing ones: words = spaces + 1, and every word gives at least one token
    chars = np.frombuffer(np.ascontiguousarray(w.rows.chars), np.uint8)
    spaces = np.add.reduceat((chars == 0x20).astype(np.int64), np.minimum(w.rows.offsets[:-1].astype(np.int64), chars.size - 1))
    words = np.where(lens > 0, spaces + 1, 0)
    assert np.all(counts >= words) and np.all(counts[lens == 0] == 0)
    assert tok.null_count == w.rows.null_count
    a, b = datagen.make_params(p["P"], 32, p["param_seed"])
    mh = orc.minhash(w.rows, p["seed"], a, b, p["width"], nthreads=4)
    assert mh.child.size == int(valid.sum()) * p["P"]
    assert np.array_equal(np.diff(mh.offsets), np.where(valid, p["P"], 0))


# ----------------------------------------------------------------------------- GPU
@pytest.fixture(scope="module")
def nv():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from cudf_amd import nvtext
    from cudf_amd import _capi
    _capi.load()
    return nvtext


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


def _same(got, exp, what):
    assert got.size == exp.size and got.null_count == exp.null_count, what
    assert np.array_equal(got.validity(), exp.validity()), what
    assert np.array_equal(got.offsets, exp.offsets), what
    assert got.child.dtype == exp.child.dtype and np.array_equal(got.child, exp.child), what


def _params(nv, p):
    import torch
    a, b = datagen.make_params(p["P"], p["hash_bits"], p["param_seed"])
    signed = np.int32 if p["hash_bits"] == 32 else np.int64
    return a, b, torch.from_numpy(a.view(signed)).cuda(), torch.from_numpy(b.view(signed)).cuda()


def _child(out):
    """The child of a device list column as a typed tensor."""
    import torch
    t = {4: torch.int32, 8: torch.int64}[out.child_dtype.itemsize]
    return out.child.view(t)[: out.child_size]


def _minhash_properties(nv, fn, ofn, w, dcol, da, db, a, b, sample_rows, what):
    """Checks on a full-size minhash result `fn(dcol, ...)`; returns the device result."""
    import torch
    p = w.params
    P = p["P"]
    host = w.rows
    full = fn(dcol, p["seed"], da, db, p["width"])
    valid = host.validity()
    assert full.size == host.size and full.null_count == host.null_count
    assert full.child_size == int(valid.sum()) * P
    offs = full.offsets.view(torch.int32)[: host.size + 1].cpu().numpy()
    assert np.array_equal(np.diff(offs), np.where(valid, P, 0)), what + ": offsets"
    child = _child(full)
    # exact on row ranges the oracle finishes in seconds
    for lo, hi in sample_rows:
        hs = host.slice(lo, hi)
        exp = ofn(hs, p["seed"], a, b, p["width"], nthreads=16)
        got = fn(dcol.slice(lo, hi, hs.null_count), p["seed"], da, db, p["width"])
        _same(got.to_host(), exp, f"{what}: rows {lo}:{hi} against the oracle")
        # the slice's output is the matching part of the whole output
        assert torch.equal(_child(got), child[int(offs[lo]): int(offs[hi])]), f"{what}: slice {lo}:{hi} of the whole"
    # a subset of the parameters gives the matching columns (only meaningful without null rows in between,
    # so compare through the valid rows' view)
    k = P // 2 + 3
    part = fn(dcol, p["seed"], da[5:5 + k].contiguous(), db[5:5 + k].contiguous(), p["width"])
    nvalid = int(valid.sum())
    assert torch.equal(_child(part).view(nvalid, k), child.view(nvalid, P)[:, 5:5 + k]), what + ": parameter subset"
    return full


gpu = pytest.mark.gpu


@gpu
def test_config1_end_to_end(nv, orc):
    w = datagen.config1()
    p = w.params
    d = nv.DeviceStringsColumn.from_host(w.rows)
    got = nv.wordpiece_tokenize(d, nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(w.vocab)), p["max_words_per_row"]).to_host()
    _same(got, orc.wordpiece_tokenize(w.rows, orc.Vocabulary(w.vocab), p["max_words_per_row"], nthreads=8), "C1 tokenize")
    a, b, da, db = _params(nv, p)
    _same(nv.minhash(d, p["seed"], da, db, p["width"]).to_host(), orc.minhash(w.rows, p["seed"], a, b, p["width"], nthreads=8), "C1 minhash")


@gpu
def test_config2_tokenize_full_size(nv, orc):
    w = datagen.config2()
    assert w.rows.size == 4_000_000
    mw = w.params["max_words_per_row"]
    d = nv.DeviceStringsColumn.from_host(w.rows)
    got = nv.wordpiece_tokenize(d, nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(w.vocab)), mw).to_host()
    exp = orc.wordpiece_tokenize(w.rows, orc.Vocabulary(w.vocab), mw, nthreads=16)
    _same(got, exp, "C2 tokenize, all 4M rows")
    assert exp.child.size > 150_000_000


@gpu
def test_config3_minhash_full_size(nv, orc):
    w = datagen.config3()
    assert w.rows.size == 2_000_000 and w.rows.offsets.dtype == np.int64
    a, b, da, db = _params(nv, w.params)
    d = nv.DeviceStringsColumn.from_host(w.rows)
    _minhash_properties(nv, nv.minhash, orc.minhash, w, d, da, db, a, b, [(0, 8000), (1_234_567, 1_240_000), (1_999_000, 2_000_000)], "C3")


@gpu
def test_config4_minhash64_full_size(nv, orc):
    w = datagen.config4()
    assert w.rows.size == 100_000 and w.rows.null_count > 5000
    lens = np.diff(w.rows.offsets.astype(np.int64))
    assert lens.max() >= 256 * 1024, "the workload must hold rows past 256 KiB"
    a, b, da, db = _params(nv, w.params)
    d = nv.DeviceStringsColumn.from_host(w.rows)
    longest = [int(i) for i in np.argsort(lens)[-4:]]
    ranges = [(0, 600), (50_000, 50_400)] + [(i, i + 1) for i in longest]
    _minhash_properties(nv, nv.minhash64, orc.minhash64, w, d, da, db, a, b, ranges, "C4")


def _utf8_pipeline(nv, orc, w, token_ranges, normalize_ranges, minhash_ranges, what):
    """tokenize, normalize_characters and minhash64 of the whole column `w.rows`; exact against the oracle on the given
    row ranges, each also run as a slice of the column and compared with the matching part of the whole result."""
    import torch
    p = w.params
    d = nv.DeviceStringsColumn.from_host(w.rows)
    dv = nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(w.vocab))
    ov = orc.Vocabulary(w.vocab)
    full = nv.wordpiece_tokenize(d, dv, p["max_words_per_row"])
    offs = full.offsets.view(torch.int32)[: w.rows.size + 1].cpu().numpy()
    assert np.all(np.diff(offs) >= 0) and int(offs[-1]) == full.child_size
    child = _child(full)
    # exact against the oracle on row ranges, each also as a slice of the whole
    for lo, hi in token_ranges:
        hs = w.rows.slice(lo, hi)
        exp = orc.wordpiece_tokenize(hs, ov, p["max_words_per_row"], nthreads=16)
        got = nv.wordpiece_tokenize(d.slice(lo, hi, hs.null_count), dv, p["max_words_per_row"])
        _same(got.to_host(), exp, f"{what} tokenize rows {lo}:{hi}")
        assert torch.equal(_child(got), child[int(offs[lo]): int(offs[hi])]), f"{what} tokenize: slice {lo}:{hi} of the whole"
        assert np.array_equal(exp.offsets.astype(np.int64) + int(offs[lo]), offs[lo: hi + 1].astype(np.int64))
    del full, child
    torch.cuda.empty_cache()
    # normalize_characters of the whole column (the output passes 2 GiB: int64 offsets), exact against the oracle on
    # row ranges, each also as a slice of the whole
    from oracle import normalize_py
    tokens = ["[CLS]", "[SEP]", "[PAD]", "[MASK]", "[UNK]"]
    normalizer = nv.CharacterNormalizer(True, nv.DeviceStringsColumn.from_host(HostStringsColumn.from_pylist(tokens)))
    whole = nv.normalize_characters(d, normalizer)
    assert whole.offsets.dtype == torch.int64 and whole.size == w.rows.size
    woff = whole.offsets.cpu().numpy()
    assert woff[0] == 0 and np.all(np.diff(woff) >= 0) and int(woff[-1]) == whole.chars.numel() > 0x7FFFFFFF
    for lo, hi in normalize_ranges:
        hs = w.rows.slice(lo, hi)
        exp = normalize_py.normalize_characters_native(hs, True, [t.encode() for t in tokens], nthreads=16)
        got = nv.normalize_characters(d.slice(lo, hi, hs.null_count), normalizer)
        gh = got.to_host()
        assert np.array_equal(gh.offsets, exp.offsets) and np.array_equal(gh.chars, exp.chars), f"{what} normalize rows {lo}:{hi}"
        assert torch.equal(got.chars, whole.chars[int(woff[lo]): int(woff[hi])]), f"{what} normalize: slice {lo}:{hi} of the whole"
        assert np.array_equal(exp.offsets.astype(np.int64) + int(woff[lo]), woff[lo: hi + 1])
    del whole
    torch.cuda.empty_cache()
    a, b, da, db = _params(nv, p)
    _minhash_properties(nv, nv.minhash64, orc.minhash64, w, d, da, db, a, b, minhash_ranges, what + " minhash64")
    return d


@gpu
def test_config5_utf8_pipeline_full_size(nv, orc):
    w = datagen.config5()
    assert w.rows.size == 8_000_000 and w.rows.offsets.dtype == np.int64
    _utf8_pipeline(nv, orc, w, [(0, 1_000_000), (3_999_999, 4_600_001), (7_400_000, 8_000_000)],
                   [(0, 400_000), (3_999_999, 4_300_001), (7_700_000, 8_000_000)], [(0, 20_000), (6_000_000, 6_010_000)], "C5")


@gpu
def test_utf8_pipeline_on_more_than_4_gib_of_chars(nv, orc):
    """The same pipeline on a column a third larger than C5: its chars pass 2^32 bytes (byte offsets that need more than
    32 bits) and its words pass 2^31 slots of the tokenizer's word table.  The row ranges checked against the oracle
    straddle that place and lie beyond it."""
    w = datagen.config5(1.3)
    rows, off = w.rows.size, w.rows.offsets
    assert off.dtype == np.int64 and int(off[-1]) > (1 << 32) + (1 << 29)
    at = int(np.searchsorted(off, 1 << 32))  # the first row that begins at or beyond 4 GiB
    assert 200_000 < at < rows - 600_000
    d = _utf8_pipeline(nv, orc, w, [(at - 200_000, at + 200_000), (rows - 500_000, rows)],
                       [(at - 100_000, at + 100_000), (rows - 300_000, rows)], [(at - 5_000, at + 5_000), (rows - 10_000, rows)],
                       "C5 x1.3")
    # minhash (uint32) and jaccard_index of rows r / r + 1 across the same place and at the end
    a, b = datagen.make_params(32, 32, 7)
    for lo, hi in [(at - 20_000, at + 20_000), (rows - 20_001, rows - 1)]:
        h1, h2 = w.rows.slice(lo, hi), w.rows.slice(lo + 1, hi + 1)
        d1, d2 = d.slice(lo, hi, 0), d.slice(lo + 1, hi + 1, 0)
        _same(nv.minhash(d1, 3, a, b, 6).to_host(), orc.minhash(h1, 3, a, b, 6, nthreads=16), f"C5 x1.3 minhash rows {lo}:{hi}")
        got, exp = nv.jaccard_index(d1, d2, 5).to_host(), orc.jaccard_index(h1, h2, 5, nthreads=16)
        assert got.size == exp.size and got.null_count == exp.null_count == 0
        assert np.array_equal(got.values.view(np.uint32), exp.values.view(np.uint32)), f"C5 x1.3 jaccard rows {lo}:{hi}"


@gpu
@pytest.mark.parametrize("rows", [4096, 40])
def test_tokenize_reports_more_tokens_than_a_list_column_holds(nv, rows):
    """2^31 one-letter words and a few more: the child would pass INT32_MAX entries, which the reference reports as
    std::overflow_error (cpp/include/cudf/detail/sizes_to_offsets_iterator.cuh:331-335).  With 4096 rows each is a
    megabyte, with 40 each is a hundred megabytes; either way the rows are tokenized in pieces, so the error
    comes from the call over the pieces.  The library must give everything back and go on working afterwards."""
    import torch
    per_row = (1 << 31) // rows + 1                      # words per row
    chars = np.tile(np.frombuffer(b"a ", np.uint8), per_row * rows)
    offsets = np.arange(rows + 1, dtype=np.int64) * (2 * per_row)
    host = HostStringsColumn(chars, offsets, None, rows, 0, 0)
    dv = nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(HostStringsColumn.from_pylist(["[UNK]", "a", "b"])))
    d = nv.DeviceStringsColumn.from_host(host)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    with pytest.raises(OverflowError, match="exceeds the column size limit"):
        nv.wordpiece_tokenize(d, dv, 0)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    # one row less stays below the limit: the same call succeeds and every word is the token of "a"
    fewer = nv.wordpiece_tokenize(d.slice(0, rows - 1, 0), dv, 0)
    assert fewer.child_size == per_row * (rows - 1)
    child = _child(fewer)
    assert int(child.min()) == 1 and int(child.max()) == 1
    offs = fewer.offsets.view(torch.int32)[:rows].cpu().numpy()
    assert np.array_equal(offs.astype(np.int64), np.arange(rows, dtype=np.int64) * per_row)


@gpu
def test_rows_of_gigabytes(nv, orc):
    """A row of 2.1 GB (2047 copies of a megabyte of text: near the 2^31 - 1 bytes a row may have) and one of 0.3 GB
    among short rows.  What the oracle says of one copy fixes the result: the tokens and the normalized bytes of
    the row are those of the copy, repeated (a copy ends with a space), and its windows are those of the copy
    continued by its own first width - 1 bytes."""
    import torch
    from oracle import normalize_py
    w = datagen.config2(0.004)
    text = w.rows.chars
    def block(at):
        b = text[at: at + (1 << 20)].copy()
        b[-1] = 0x20
        assert b[0] != 0x20
        return b
    A, B = block(0), block(1 << 21)
    kA, kB, width = 2047, 300, 5
    small = [np.frombuffer(b"hello ab", np.uint8), np.frombuffer(b"ab", np.uint8)]
    parts = [small[0], np.tile(A, kA), np.tile(B, kB), small[1]]
    sizes = [len(parts[0]), len(parts[1]), 0, len(parts[2]), len(parts[3])]          # row 2 is null
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    host = HostStringsColumn(np.concatenate(parts), offsets, np.array([0b11011], np.uint32), 5, 0, 1)
    assert int(offsets[2] - offsets[1]) == kA << 20 > (1 << 31) - (1 << 21)
    d = nv.DeviceStringsColumn.from_host(host)
    def one(chars):
        return HostStringsColumn(np.ascontiguousarray(chars), np.array([0, len(chars)], np.int64), None, 1, 0, 0)
    copies = [(one(small[0]), 1), (one(A), kA), None, (one(B), kB), (one(small[1]), 1)]
    wrapped = [one(small[0]), one(np.concatenate([A, A[:width - 1]])), None, one(np.concatenate([B, B[:width - 1]])), one(small[1])]

    # wordpiece_tokenize: without a word limit (the long rows are tokenized in pieces), and with one
    dv = nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(w.vocab))
    ov = orc.Vocabulary(w.vocab)
    for max_words in (0, 1000):
        exp = [np.zeros(0, np.int32) if c is None else
               (np.tile(orc.wordpiece_tokenize(c[0], ov, 0, nthreads=1).child, c[1]) if max_words == 0
                else orc.wordpiece_tokenize(c[0], ov, max_words, nthreads=1).child) for c in copies]
        got = nv.wordpiece_tokenize(d, dv, max_words)
        assert got.size == 5 and got.null_count == 1
        offs = got.offsets.view(torch.int32)[:6].cpu().numpy()
        assert np.array_equal(offs, np.concatenate([[0], np.cumsum([len(e) for e in exp])])), f"max_words={max_words}"
        child = _child(got)
        for r in range(5):
            assert torch.equal(child[int(offs[r]): int(offs[r + 1])].cpu(), torch.from_numpy(exp[r])), f"tokens of row {r}, max_words={max_words}"
        del got, child
    torch.cuda.empty_cache()

    # minhash, minhash64
    for fn, ofn, bits in ((nv.minhash, orc.minhash, 32), (nv.minhash64, orc.minhash64, 64)):
        a, b = datagen.make_params(8, bits, 5)
        got = fn(d, 9, a, b, width).to_host()
        assert np.array_equal(got.offsets, [0, 8, 16, 16, 24, 32]) and got.null_count == 1
        for r, c in enumerate(wrapped):
            if c is not None:
                at = int(got.offsets[r])
                assert np.array_equal(got.child[at: at + 8], ofn(c, 9, a, b, width, nthreads=1).child), f"minhash{bits} of row {r}"

    # normalize_characters
    norm = nv.normalize_characters(d, nv.CharacterNormalizer(True, None))
    noff = norm.offsets.cpu().numpy()
    for r, c in enumerate(copies):
        lo, hi = int(noff[r]), int(noff[r + 1])
        if c is None:
            assert lo == hi
            continue
        e = torch.from_numpy(normalize_py.normalize_characters_native(c[0], True, [], nthreads=1).chars)
        assert hi - lo == len(e) * c[1], f"normalized size of row {r}"
        assert bool((norm.chars[lo:hi].view(c[1], len(e)).cpu() == e).all()), f"normalized bytes of row {r}"
    del norm
    torch.cuda.empty_cache()

    # jaccard_index: 300 copies of B against 300 copies of A share what the two copies (continued) share; a pair of
    # more than 2^32 / 3 bytes together is refused
    other = HostStringsColumn(np.concatenate([small[0], np.tile(A, kB), small[0]]),
                              np.array([0, 8, 8 + (kB << 20), 16 + (kB << 20)], np.int64), None, 3, 0, 0)
    d2 = nv.DeviceStringsColumn.from_host(other)
    got = nv.jaccard_index(d.slice(2, 5, 1), d2, width).to_host()
    assert got.size == 3 and got.null_count == 1 and list(got.validity()) == [False, True, True]
    exp = orc.jaccard_index(wrapped[3], wrapped[1], width, nthreads=1)
    assert got.values.view(np.uint32)[1] == exp.values.view(np.uint32)[0]
    assert got.values[2] == orc.jaccard_index(one(small[1]), one(small[0]), width, nthreads=1).values[0]
    with pytest.raises(OverflowError, match="row pair is too long"):
        nv.jaccard_index(d.slice(1, 2, 0), d.slice(1, 2, 0), width)


@gpu
def test_minhash_ngrams_on_a_child_of_more_than_4_gib(nv, orc):
    """LIST<STRING> rows whose strings child holds 4.7 GB (int64 child offsets): the rows whose elements lie across
    byte 2^32 of the child, and the last ones, against the oracle; each range also as a slice of the whole."""
    import torch
    from cudf_amd.arrow_host import HostListStringsColumn
    rng = np.random.default_rng(5)
    chars = np.tile(rng.integers(97, 123, 1 << 26, dtype=np.uint8), 70)
    each, per_row = 47, 37                       # bytes per element, elements per row
    elements = len(chars) // each
    rows = elements // per_row
    child = HostStringsColumn(chars, np.arange(elements + 1, dtype=np.int64) * each, None, elements, 0, 0)
    host = HostListStringsColumn(np.arange(rows + 1, dtype=np.int32) * per_row, child, None, rows, 0, 0)
    assert int(child.offsets[rows * per_row]) > (1 << 32) + (1 << 28)
    d = nv.DeviceListStringsColumn.from_host(host)
    at = (1 << 32) // (each * per_row)           # the row that holds byte 2^32
    for fn, ofn, bits in ((nv.minhash_ngrams, orc.minhash_ngrams, 32), (nv.minhash64_ngrams, orc.minhash64_ngrams, 64)):
        a, b = datagen.make_params(16, bits, 3)
        whole = fn(d, 4, 11, a, b)
        assert whole.size == rows and whole.child_size == rows * 16
        child_all = _child(whole).view(rows, 16)
        for lo, hi in [(at - 3000, at + 3000), (rows - 6000, rows)]:
            exp = ofn(host.slice(lo, hi), 4, 11, a, b, nthreads=16)
            got = fn(d.slice(lo, hi, 0), 4, 11, a, b)
            _same(got.to_host(), exp, f"ngrams{bits} rows {lo}:{hi}")
            assert torch.equal(_child(got).view(hi - lo, 16), child_all[lo:hi]), f"ngrams{bits}: slice {lo}:{hi} of the whole"
        del whole, child_all
