"""Pins the host oracle to every known-answer vector the reference holds for this path,
to published MurmurHash3 values, to an independent library (HF `tokenizers` WordPiece)
and to closed forms a plausible mistake would break.  CPU only."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from oracle.pyoracle import OracleError
from tests import golden_cases as gc
from tests.golden_cases import strings


# ----------------------------------------------------------------------------- hashes
def test_murmur32_public_vectors():
    for v in gc.murmur32_vectors():
        assert orc.murmur3_x86_32(bytes.fromhex(v["hex"]), v["seed"]) == v["hash"], v


def test_murmur64_reference_vectors():
    v = gc.murmur64_vectors()
    for s, e0, e7 in zip(v["strings"], v["seed0"], v["seed7"]):
        b = s.encode("utf-8")
        assert orc.murmur3_x64_128(b, 0)[0] == e0, s
        assert orc.murmur3_x64_128(b, 7)[0] == e7, s


def test_murmur64_tail_lengths_change_hash():
    # every tail length 0..31 goes through a different switch arm; all distinct
    seen = {orc.murmur3_x64_128(b"q" * n, 7) for n in range(32)}
    assert len(seen) == 32


# ----------------------------------------------------------------------------- minhash
@pytest.mark.parametrize("case", gc.minhash_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_minhash_golden(case, dtype):
    col = strings(case["rows"], dtype)
    if "expected32" in case:
        got = orc.minhash(col, case["seed"], case["a"], case["b"], case["width"], nthreads=2)
        assert gc.expected_list_equal(got.to_pylist(), case["expected32"])
        assert got.child.dtype == np.uint32 and got.offsets.dtype == np.int32
    if "expected64" in case:
        got = orc.minhash64(col, case["seed"], case["a"], case["b"], case["width"], nthreads=2)
        assert gc.expected_list_equal(got.to_pylist(), case["expected64"])
        assert got.child.dtype == np.uint64


def test_minhash_single_window_closed_form():
    # a row shorter than width contributes exactly one hash: out[j] = max(h,1)*a_j + b_j
    a = np.array([10, 0xFFFFFFFF, 3], np.uint32)
    b = np.array([10, 7, 0xFFFFFFF0], np.uint32)
    for s in ["d", "ab", "xyz", "é"]:
        h = max(orc.murmur3_x86_32(s.encode(), 0), 1)
        got = orc.minhash(strings([s]), 0, a, b, 4).to_pylist()[0]
        assert got == [(h * int(x) + int(y)) % 2**32 for x, y in zip(a, b)]
        h64 = max(orc.murmur3_x64_128(s.encode(), 7)[0], 1)
        a64 = np.array([2, 2**63 + 5], np.uint64)
        b64 = np.array([5, 2**64 - 1], np.uint64)
        got = orc.minhash64(strings([s]), 7, a64, b64, 4).to_pylist()[0]
        assert got == [((h64 * int(x) + int(y)) % 2**64) % (2**61 - 1) for x, y in zip(a64, b64)]


def test_minhash_invariants():
    rng = np.random.default_rng(3)
    a = rng.integers(1, 2**32, 17, dtype=np.uint64).astype(np.uint32)
    b = rng.integers(0, 2**32, 17, dtype=np.uint64).astype(np.uint32)
    # a run of one repeated character has one distinct window -> equals the single-window row
    one = orc.minhash(strings(["zzzzz"]), 42, a, b, 5).to_pylist()[0]
    many = orc.minhash(strings(["z" * 300]), 42, a, b, 5).to_pylist()[0]
    assert one == many
    # appending a copy of the text that re-creates only existing windows does not change the result
    base = orc.minhash(strings(["abcabc"]), 42, a, b, 3).to_pylist()[0]
    more = orc.minhash(strings(["abcabcabcabc"]), 42, a, b, 3).to_pylist()[0]
    assert base == more
    # the minimum over a union of window sets is the element-wise minimum
    x = orc.minhash(strings(["hello world"]), 1, a, b, 4).to_pylist()[0]
    y = orc.minhash(strings(["world hello"]), 1, a, b, 4).to_pylist()[0]
    xy = orc.minhash(strings(["hello world hello"]), 1, a, b, 4).to_pylist()[0]
    assert xy == [min(p, q) for p, q in zip(x, y)]


def test_minhash_utf8_windows_are_characters():
    # width counts characters: "ééé" (6 bytes) with width 3 is ONE window = whole row
    a = np.array([1], np.uint32)
    b = np.array([0], np.uint32)
    h = max(orc.murmur3_x86_32("ééé".encode(), 0), 1)
    assert orc.minhash(strings(["ééé"]), 0, a, b, 3).to_pylist()[0] == [h]
    # "éaé" + "b": width 3 -> windows "éaé", "aéb"; continuation bytes never start a window
    hs = [max(orc.murmur3_x86_32(w.encode(), 0), 1) for w in ["éaé", "aéb"]]
    assert orc.minhash(strings(["éaéb"]), 0, a, b, 3).to_pylist()[0] == [min(hs)]


def test_minhash_nulls_empty_sliced():
    rows = ["abcdef", None, "", "xyzuvw", None, "k"]
    a = np.array([3, 5], np.uint32)
    col = strings(rows)
    got = orc.minhash(col, 0, a, a, 4)
    assert got.null_count == 2 and got.size == 6
    assert got.offsets.tolist() == [0, 2, 2, 4, 6, 6, 8]
    pl = got.to_pylist()
    assert pl[1] is None and pl[4] is None and pl[2] == [0, 0]
    sl = col.slice(2, 5)
    got_s = orc.minhash(sl, 0, a, a, 4)
    assert got_s.to_pylist() == pl[2:5]
    assert got_s.offsets.tolist() == [0, 2, 4, 4]


def test_minhash_errors_and_empty():
    col = strings(["this string intentionally left blank"])
    e = np.zeros(0, np.uint32)
    with pytest.raises(OracleError) as ei:
        orc.minhash(col, 0, e, e, 0)
    assert ei.value.code == orc.INVALID_ARGUMENT
    with pytest.raises(OracleError):
        orc.minhash(col, 0, e, e, 4)
    with pytest.raises(OracleError):
        orc.minhash(col, 0, np.ones(2, np.uint32), np.ones(2, np.uint32), 1)
    big = strings([""] * 50000)
    z = np.zeros(50000, np.uint32)
    with pytest.raises(OracleError) as ei:
        orc.minhash(big, 0, z, z, 4)
    assert ei.value.code == orc.OVERFLOW_ERROR
    empty = strings([])
    got = orc.minhash(empty, 0, np.ones(3, np.uint32), np.ones(3, np.uint32), 4)
    assert got.size == 0 and got.child.size == 0


# ----------------------------------------------------------------------------- wordpiece
def check_jaccard_case(got, case):
    exp = np.array(case["expected"], np.float32)
    valid = np.array(case.get("expected_valid", [True] * len(exp)))
    assert got.size == len(exp) and np.array_equal(got.validity(), valid)
    assert got.null_count == int((~valid).sum()) and (got.mask is not None) == ("expected_valid" in case)
    if "tolerance" in case:  # values printed with six digits
        assert np.allclose(got.values[valid], exp[valid], atol=case["tolerance"], rtol=0)
    else:  # float32 literals: bit-exact
        assert np.array_equal(got.values[valid].view(np.uint32), exp[valid].view(np.uint32))


@pytest.mark.parametrize("case", gc.jaccard_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_jaccard_golden(case, dtype):
    got = orc.jaccard_index(strings(case["input1"], dtype), strings(case["input2"], dtype), case["width"])
    check_jaccard_case(got, case)
    check_jaccard_case(orc.jaccard_index(strings(case["input2"], dtype), strings(case["input1"], dtype), case["width"]), case)


def brute_force_jaccard(s1, s2, width):
    """The definition on the substrings themselves (no hashing), as the reference's Python test builds it from
    character_ngrams (test_text_methods.py:971-1010); rows shorter than width contribute the whole row."""
    def grams(t):
        if len(t) == 0:
            return set()
        return {t} if len(t) < width else {t[i:i + width] for i in range(len(t) - width + 1)}
    a, b = grams(s1), grams(s2)
    u = len(a | b)
    return np.float32(len(a & b)) / np.float32(u) if u else np.float32(0)


def test_jaccard_matches_the_set_definition():
    rng = np.random.default_rng(31)
    alphabet = list("abcdé漢 ")
    rows1, rows2 = [], []
    for _ in range(400):
        common = "".join(rng.choice(alphabet, int(rng.integers(0, 60))))
        rows1.append("".join(rng.choice(alphabet, int(rng.integers(0, 12)))) + common)
        rows2.append("".join(rng.choice(alphabet, int(rng.integers(0, 25)))) + common)
    for width in (2, 5, 9):
        got = orc.jaccard_index(strings(rows1), strings(rows2), width, nthreads=2)
        exp = np.array([brute_force_jaccard(x, y, width) for x, y in zip(rows1, rows2)], np.float32)
        assert np.array_equal(got.values.view(np.uint32), exp.view(np.uint32)), width
    with pytest.raises(OracleError):
        orc.jaccard_index(strings(["1", "2", "3"]), strings(["1", "2", "3"]), 1)
    with pytest.raises(OracleError):
        orc.jaccard_index(strings(["1", "2", "3"]), strings(["1", "2"]), 5)
    assert orc.jaccard_index(strings([]), strings([]), 5).size == 0


@pytest.mark.parametrize("case", gc.minhash_ngrams_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_minhash_ngrams_golden(case, dtype):
    col = gc.list_strings(case["rows"], dtype)
    if "slice" in case:
        col = col.slice(*case["slice"])
    a32, b32 = np.array(case["a"], np.uint32), np.array(case["b"], np.uint32)
    assert orc.minhash_ngrams(col, case["ngrams"], case["seed"], a32, b32).to_pylist() == case["expected32"]
    got = orc.minhash64_ngrams(col, case["ngrams"], case["seed"], a32.astype(np.uint64), b32.astype(np.uint64))
    assert got.to_pylist() == case["expected64"]
    assert got.child.dtype == np.uint64 and got.null_count == 0


def test_minhash_ngrams_rules():
    """What the vectors do not spell out: a run is ngrams + 1 elements unless the row is shorter (then only the
    run from element 0 exists); null elements start no run; null rows have no slots; empty rows are zeros; a row
    whose every run is skipped keeps the all-ones start value."""
    a, b = np.array([3, 5], np.uint32), np.array([7, 11], np.uint32)
    words = ["aa", "b", "cc", "ddd", "e", "ff", "g"]
    col = gc.list_strings([words, None, [], words[:3], [None, "x", "y", "z"]])
    got = orc.minhash_ngrams(col, 2, 9, a, b)
    assert got.null_count == 1 and list(np.diff(got.offsets)) == [2, 0, 2, 2, 2]
    rows = got.to_pylist()
    # row 0: runs of three elements starting at 0..4 (the run starting at 5 would be clamped and is dropped)
    hs = [max(orc.murmur3_x86_32("".join(words[i:i + 3]).encode(), 9), 1) for i in range(5)]
    assert rows[0] == [min((h * int(x) + int(y)) & 0xFFFFFFFF for h in hs) for x, y in zip(a, b)]
    assert rows[1] is None and rows[2] == [0, 0]
    # row 3: positions 0 and 1; the run from 0 is whole, the run from 1 is clamped and dropped
    h = max(orc.murmur3_x86_32(b"aabcc", 9), 1)
    assert rows[3] == [(h * int(x) + int(y)) & 0xFFFFFFFF for x, y in zip(a, b)]
    # row 4: positions 0..2: element 0 is null, the run from 1 spans elements 1..3, the run from 2 is clamped
    h = max(orc.murmur3_x86_32(b"xyz", 9), 1)
    assert rows[4] == [(h * int(x) + int(y)) & 0xFFFFFFFF for x, y in zip(a, b)]
    only_null = gc.list_strings([[None, None]])
    assert orc.minhash_ngrams(only_null, 2, 0, a, b).to_pylist() == [[0xFFFFFFFF, 0xFFFFFFFF]]
    with pytest.raises(OracleError):
        orc.minhash_ngrams(col, 1, 0, a, b)
    with pytest.raises(OracleError):
        orc.minhash_ngrams(col, 2, 0, a[:0], b[:0])
    with pytest.raises(OracleError):
        orc.minhash64_ngrams(col, 2, 0, np.zeros(3, np.uint64), np.zeros(2, np.uint64))
    assert orc.minhash_ngrams(gc.list_strings([]), 4, 0, a, b).size == 0


@pytest.mark.parametrize("case", gc.wordpiece_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_wordpiece_golden(case, dtype):
    vocab = orc.Vocabulary(strings(case["vocab"]))
    col = strings(case["rows"], dtype)
    if "slice" in case:
        col = col.slice(*case["slice"])
    for run in case["runs"]:
        got = orc.wordpiece_tokenize(col, vocab, run["max_words"], nthreads=2)
        assert gc.expected_list_equal(got.to_pylist(), run["expected"]), (case["name"], run["max_words"])
        assert got.child.dtype == np.int32


def test_wordpiece_bert_sentences():
    d = gc.bert_case()
    vocab = orc.Vocabulary(strings(d["vocab"]))
    assert vocab.unk_id == 100
    col = strings(d["rows"])
    for mw, exp in d["expected"].items():
        got = orc.wordpiece_tokenize(col, vocab, int(mw))
        assert gc.expected_list_equal(got.to_pylist(), exp), mw


def test_wordpiece_errors_and_empty():
    with pytest.raises(OracleError):
        orc.Vocabulary(strings([]))
    with pytest.raises(OracleError):
        orc.Vocabulary(strings([None, None, None]))
    v = orc.Vocabulary(strings(["x"]))
    with pytest.raises(OracleError):
        orc.wordpiece_tokenize(strings(["  "]), v, -1)
    v2 = orc.Vocabulary(strings([""]))
    for mw in (0, 10):
        got = orc.wordpiece_tokenize(strings([]), v2, mw)
        assert got.size == 0 and got.offsets.size == 0


def test_wordpiece_long_word_and_cap_rules():
    v = orc.Vocabulary(strings(["[UNK]", "a", "##a", "b"]))
    # 199 bytes tokenizes piece by piece, 200 bytes is a single unknown token
    got = orc.wordpiece_tokenize(strings(["a" * 199, "a" * 200, "a" * 250 + " b"]), v, 0).to_pylist()
    assert got[0] == [1] + [2] * 198 and got[1] == [0] and got[2] == [0, 3]
    # cap = min(max_words, size_bytes // 2): "a b a" has 5 bytes -> 2 words, a 1-byte row -> none
    got = orc.wordpiece_tokenize(strings(["a b a", "a", "a b"]), v, 100).to_pylist()
    assert got == [[1, 3], [], [1]]
    # a null row with max_words > 0 has no tokens and stays null
    got = orc.wordpiece_tokenize(strings(["a b", None, "b"]), v, 3)
    assert got.to_pylist() == [[1], None, []] and got.null_count == 1


def test_wordpiece_matches_hf_tokenizers():
    """Independent implementation of the same greedy longest-match-first rule."""
    tokenizers = pytest.importorskip("tokenizers")
    from tokenizers.models import WordPiece
    rng = np.random.default_rng(11)
    letters = "abcdefgh"
    vocab = ["[PAD]", "[UNK]"] + list(letters) + ["##" + c for c in letters[:5]]
    seen = set(vocab)
    while len(vocab) < 400:
        n = int(rng.integers(2, 6))
        s = "".join(rng.choice(list(letters), n))
        if rng.random() < 0.4:
            s = "##" + s
        if s not in seen:
            seen.add(s)
            vocab.append(s)
    model = WordPiece({t: i for i, t in enumerate(vocab)}, unk_token="[UNK]", max_input_chars_per_word=100)
    words = ["".join(rng.choice(list(letters), int(rng.integers(1, 12)))) for _ in range(3000)]
    rows = [" ".join(words[i:i + 30]) for i in range(0, 3000, 30)]
    v = orc.Vocabulary(strings(vocab))
    got = orc.wordpiece_tokenize(strings(rows), v, 0).to_pylist()
    multi = 0
    for row, g in zip(rows, got):
        exp = []
        for w in row.split(" "):
            ids = [t.id for t in model.tokenize(w)]
            multi += len(ids) > 1
            exp.extend(ids)
        assert g == exp
    assert multi > 100  # the comparison exercised real sub-word splits


def test_wordpiece_concatenation_and_cap_equivalence():
    d = gc.bert_case()
    v = orc.Vocabulary(strings(d["vocab"]))
    rows = d["rows"]
    full = orc.wordpiece_tokenize(strings(rows), v, 0).to_pylist()
    # tokens of a row = concatenation of the tokens of its words
    for row, toks in zip(rows, full):
        words = [w for w in row.split(" ") if w]
        per_word = orc.wordpiece_tokenize(strings(words), v, 0).to_pylist()
        assert sum(per_word, []) == toks
    # a cap above the word count (and below size/2) changes nothing
    capped = orc.wordpiece_tokenize(strings(rows), v, 150).to_pylist()
    assert capped == full


def test_copy_bitmask_shift():
    col = strings(["a", None, "b", None, None, "c"] * 20)
    sl = col.slice(7, 101)
    m = orc.copy_bitmask(sl)
    from cudf_amd.arrow_host import unpack_validity
    assert np.array_equal(unpack_validity(m, sl.size), col.validity()[7:101])


# ----------------------------------------------------------------------------- null rows that keep their bytes
def test_null_rows_that_keep_bytes_reduce_to_covered_cases():
    """Non-empty nulls are legal libcudf input (cpp/include/cudf/copying.hpp:946-962) and no reference vector holds one.
    What the code says of them reduces each operation to a case the vectors do cover: without a word limit the tokenizer
    never reads the validity (cpp/src/text/wordpiece_tokenize.cu:503-568), so the tokens are those of the same buffers
    without a mask; with a limit a null row has no words (:778), as if it were empty; minhash drops the slots of null
    rows (cpp/src/text/minhash.cu:626-628), as if the rows had been emptied first."""
    from cudf_amd.arrow_host import HostStringsColumn, pack_validity
    texts = ["abc de abc", "de f", "", "gab c abc", "f", "c c c c"]
    valid = np.array([False, True, True, False, False, True])
    for dtype in (np.int32, np.int64):
        base = strings(texts, dtype)
        kept = HostStringsColumn(base.chars, base.offsets, pack_validity(valid), len(texts), 0, int((~valid).sum()))
        emptied = strings([t if v else None for t, v in zip(texts, valid)], dtype)
        vocab = orc.Vocabulary(strings(["[UNK]", "abc", "de", "f", "gab", "c"]))
        all_tokens = orc.wordpiece_tokenize(base, vocab, 0)
        got = orc.wordpiece_tokenize(kept, vocab, 0)
        assert np.array_equal(got.child, all_tokens.child) and np.array_equal(got.offsets, all_tokens.offsets)
        assert got.null_count == 3 and np.array_equal(got.validity(), valid)
        assert got.to_pylist()[1] == [2, 3] and got.child.tolist()[:3] == [1, 2, 1]   # the null row 0 has its three tokens
        for max_words in (1, 2, 50):
            assert orc.wordpiece_tokenize(kept, vocab, max_words).equals(orc.wordpiece_tokenize(emptied, vocab, max_words))
        a = np.array([3, 11, 7], np.uint32)
        b = np.array([1, 2, 5], np.uint32)
        assert orc.minhash(kept, 0, a, b, 4).equals(orc.minhash(emptied, 0, a, b, 4))
        assert orc.minhash64(kept, 7, a.astype(np.uint64), b.astype(np.uint64), 4).equals(
            orc.minhash64(emptied, 7, a.astype(np.uint64), b.astype(np.uint64), 4))
        other = strings(["abc de", "de f", "x", "gab c", "f f", "c c"], dtype)
        j1, j2 = orc.jaccard_index(kept, other, 2), orc.jaccard_index(emptied, other, 2)
        assert j1.equals(j2)
