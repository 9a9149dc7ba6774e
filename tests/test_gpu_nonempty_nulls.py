"""GPU parity on null rows that keep their bytes.  libcudf input may hold such rows (cpp/include/cudf/copying.hpp:946-962);
wordpiece_tokenize with max_words_per_row == 0 never reads the validity and tokenizes them
(cpp/src/text/wordpiece_tokenize.cu:503-568), with a word limit it gives them no words (:778); minhash drops their
slots (cpp/src/text/minhash.cu:605-630); jaccard_index treats them as rows without hashes.  The columns are built by
hand: mask bit 0 and off[i + 1] > off[i].  Every operation against the host oracle, int32 and int64 offsets, sliced."""
import numpy as np
import pytest

from cudf_amd.arrow_host import HostListStringsColumn, HostStringsColumn, pack_validity

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


def column_with_nulls_that_keep_bytes(rng, rows, dtype, long_rows=False):
    """Text rows, every fifth or so null without losing its bytes; some nulls and some valid rows are empty."""
    letters = list("abcdefg")
    texts, valid = [], []
    for i in range(rows):
        u = rng.random()
        words = 0 if u < 0.1 else int(rng.integers(1, 30))
        if long_rows and i % 97 == 5:
            words = 6000  # a row of several tiles, null or not
        texts.append(" ".join("".join(rng.choice(letters, int(rng.integers(1, 9)))) for _ in range(words)))
        valid.append(rng.random() > 0.2)
    valid[0] = False
    texts[0] = "abc de abc"
    valid[-1] = False
    texts[-1] = "f gab c"
    base = HostStringsColumn.from_pylist(texts, offsets_dtype=dtype)
    valid = np.asarray(valid)
    return HostStringsColumn(base.chars, base.offsets, pack_validity(valid), rows, 0, int((~valid).sum())), valid


def small_vocab():
    return ["[UNK]", "abc", "de", "f", "gab", "c", "a", "b", "##c", "##a", "##b", "##d", "##e", "ab", "##g", "g", "##f", "e", "d"]


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_wordpiece_tokenize_null_rows_with_bytes(nv, orc, dtype):
    rng = np.random.default_rng(11)
    host, valid = column_with_nulls_that_keep_bytes(rng, 3000, dtype, long_rows=True)
    hv = HostStringsColumn.from_pylist(small_vocab())
    dcol = nv.DeviceStringsColumn.from_host(host)
    dv = nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(hv))
    ov = orc.Vocabulary(hv)
    lens = np.diff(host.offsets.astype(np.int64))
    for max_words in (0, 3, 100000):
        exp = orc.wordpiece_tokenize(host, ov, max_words, nthreads=4)
        got = nv.wordpiece_tokenize(dcol, dv, max_words).to_host()
        assert got.equals(exp), f"max_words={max_words}"
        counts = np.diff(got.offsets)
        kept = (~valid) & (lens > 0)
        assert got.null_count == int((~valid).sum())
        if max_words == 0:
            assert (counts[kept] > 0).all()   # tokens appear, the row stays null
        else:
            assert (counts[~valid] == 0).all()
        for lo, hi in ((0, 1), (1, 2999), (5, 6), (700, 2204), (2999, 3000)):
            hs = host.slice(lo, hi)
            ds = dcol.slice(lo, hi, hs.null_count)
            assert nv.wordpiece_tokenize(ds, dv, max_words).to_host().equals(orc.wordpiece_tokenize(hs, ov, max_words)), f"slice {lo}:{hi} max_words={max_words}"


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_minhash_and_jaccard_null_rows_with_bytes(nv, orc, dtype):
    rng = np.random.default_rng(12)
    host, valid = column_with_nulls_that_keep_bytes(rng, 2000, dtype, long_rows=True)
    other, _ = column_with_nulls_that_keep_bytes(rng, 2000, dtype)
    dcol, dother = nv.DeviceStringsColumn.from_host(host), nv.DeviceStringsColumn.from_host(other)
    P = 7
    a = rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32)
    b = rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32)
    a64 = rng.integers(1, 2**64, P, dtype=np.uint64)
    b64 = rng.integers(0, 2**64, P, dtype=np.uint64)
    for lo, hi in ((0, 2000), (0, 1), (3, 1990), (1999, 2000)):
        hs, ho = host.slice(lo, hi), other.slice(lo, hi)
        ds, do = dcol.slice(lo, hi, hs.null_count), dother.slice(lo, hi, ho.null_count)
        got = nv.minhash(ds, 3, a, b, 4).to_host()
        assert got.equals(orc.minhash(hs, 3, a, b, 4, nthreads=4)), f"minhash {lo}:{hi}"
        assert got.child.size == (hi - lo - hs.null_count) * P   # a null row has no slots, bytes or not
        assert nv.minhash64(ds, 9, a64, b64, 5).to_host().equals(orc.minhash64(hs, 9, a64, b64, 5, nthreads=4)), f"minhash64 {lo}:{hi}"
        assert nv.jaccard_index(ds, do, 3).to_host().equals(orc.jaccard_index(hs, ho, 3, nthreads=4)), f"jaccard_index {lo}:{hi}"


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_minhash_ngrams_null_rows_and_null_elements_with_bytes(nv, orc, dtype):
    rng = np.random.default_rng(13)
    # the elements: a strings column whose null elements keep their bytes; the rows: lists of them, the null rows keep their elements
    elements, _ = column_with_nulls_that_keep_bytes(rng, 6000, dtype)
    sizes = rng.integers(0, 12, 900)
    sizes[::50] = 0
    offsets = np.zeros(sizes.size + 1, np.int32)
    np.cumsum(sizes, out=offsets[1:])
    assert offsets[-1] <= elements.size
    row_valid = rng.random(sizes.size) > 0.15
    row_valid[0] = False
    lists = HostListStringsColumn(offsets, elements, pack_validity(row_valid), sizes.size, 0, int((~row_valid).sum()))
    assert ((~row_valid) & (sizes > 0)).any()
    dl = nv.DeviceListStringsColumn.from_host(lists)
    P = 5
    a = rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32)
    b = rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32)
    a64 = rng.integers(1, 2**64, P, dtype=np.uint64)
    b64 = rng.integers(0, 2**64, P, dtype=np.uint64)
    for lo, hi in ((0, sizes.size), (1, 890), (0, 1)):
        hs = lists.slice(lo, hi)
        ds = dl.slice(lo, hi, hs.null_count)
        assert nv.minhash_ngrams(ds, 2, 5, a, b).to_host().equals(orc.minhash_ngrams(hs, 2, 5, a, b, nthreads=4)), f"minhash_ngrams {lo}:{hi}"
        assert nv.minhash64_ngrams(ds, 3, 6, a64, b64).to_host().equals(orc.minhash64_ngrams(hs, 3, 6, a64, b64, nthreads=4)), f"minhash64_ngrams {lo}:{hi}"


def test_wordpiece_retry_on_a_column_of_many_more_ranges_than_wavefronts(nv, orc):
    """Forty megabytes of two-letter words that are not in the vocabulary, cut into ranges of one tile: twenty thousand
    ranges for some six thousand resident wavefronts, and several times the queue entries that the first attempt has.
    Which ranges a wavefront gets, and so how many entries it reserves in chunks, differs between the attempts; the
    second attempt must have room whatever the assignment (greedy rule: cpp/src/text/wordpiece_tokenize.cu:349-407)."""
    from cudf_amd import _capi
    rng = np.random.default_rng(14)
    words = 13_000_000
    chars = np.full(3 * words, 32, np.uint8)
    chars[0::3] = rng.integers(97, 105, words, dtype=np.uint8)
    chars[1::3] = rng.integers(97, 105, words, dtype=np.uint8)
    per_row = 100
    rows = words // per_row
    offsets = (np.arange(rows + 1, dtype=np.int64) * (3 * per_row)).astype(np.int32)
    host = HostStringsColumn(chars, offsets, None, rows, 0, 0)
    letters = "abcdefgh"
    hv = HostStringsColumn.from_pylist(["[UNK]"] + list(letters) + ["##" + c for c in letters] + ["abcdefgh"])
    dcol = nv.DeviceStringsColumn.from_host(host)
    dv = nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(hv))
    exp = orc.wordpiece_tokenize(host, orc.Vocabulary(hv), 0, nthreads=8)
    assert exp.child.size == 2 * words
    _capi.set_range_tiles(1)
    _capi.set_sizing_sample(False)   # (the sample of the column would size the first attempt right: no second one)
    try:
        for attempt in range(3):
            _capi.profile_enable(True)
            _capi.profile_read()
            got = nv.wordpiece_tokenize(dcol, dv, 0)
            launches = sum(1 for name, _ in _capi.profile_read() if name == "wordpiece_word_kernel")
            _capi.profile_enable(False)
            assert launches == 2, launches
            assert got.to_host().equals(exp), f"call {attempt}"
        _capi.set_sizing_sample(True)
        _capi.profile_enable(True)
        _capi.profile_read()
        got = nv.wordpiece_tokenize(dcol, dv, 0)
        launches = sum(1 for name, _ in _capi.profile_read() if name == "wordpiece_word_kernel")
        assert launches == 1, launches
        assert got.to_host().equals(exp), "sized by the sample"
    finally:
        _capi.profile_enable(False)
        _capi.set_range_tiles(0)
        _capi.set_sizing_sample(True)
