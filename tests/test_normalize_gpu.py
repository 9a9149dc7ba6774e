"""GPU parity of normalize_characters: the HIP path through the C ABI against the reference's known answers and
against the host oracle on seeded inputs.  Bit-exact (byte work)."""
import numpy as np
import pytest

from cudf_amd.arrow_host import HostStringsColumn, pack_validity
from tests import golden_cases as gc
from tests.golden_cases import strings

pytestmark = pytest.mark.gpu

TILE = 1024  # input bytes per workgroup in the library: cases below put interesting bytes around its multiples


@pytest.fixture(scope="module")
def nv():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from cudf_amd import _capi, nvtext
    _capi.load()  # fails loudly if the HIP library is missing
    return nvtext


@pytest.fixture(scope="module")
def onorm():
    from oracle import normalize_py
    return normalize_py


def run(nv, host, do_lower, tokens=()):
    special = nv.DeviceStringsColumn.from_host(strings(list(tokens))) if tokens else None
    normalizer = nv.CharacterNormalizer(do_lower, special)
    return nv.normalize_characters(nv.DeviceStringsColumn.from_host(host), normalizer).to_host()


def assert_same(got, exp, what=""):
    assert got.size == exp.size and got.null_count == exp.null_count, what
    assert got.offsets.dtype == np.int32, what
    assert np.array_equal(got.validity(), exp.validity()), what
    if not np.array_equal(got.offsets, exp.offsets):
        bad = np.flatnonzero(got.offsets != exp.offsets)
        raise AssertionError(f"{what}: offsets differ first at row {bad[0]}: got {got.offsets[bad[:4]]} expected {exp.offsets[bad[:4]]}")
    if not np.array_equal(got.chars, exp.chars):
        m = min(got.chars.size, exp.chars.size)
        bad = np.flatnonzero(got.chars[:m] != exp.chars[:m])
        at = int(bad[0]) if bad.size else m
        raise AssertionError(f"{what}: chars differ at byte {at} of {got.chars.size}/{exp.chars.size}: "
                             f"got {got.chars[max(0, at - 8): at + 8].tobytes()!r} expected {exp.chars[max(0, at - 8): at + 8].tobytes()!r}")


def check(nv, onorm, host, do_lower, tokens=(), what=""):
    got = run(nv, host, do_lower, tokens)
    exp = onorm.normalize_characters(host, do_lower, [t.encode("utf-8") if isinstance(t, str) else t for t in tokens])
    assert_same(got, exp, what)
    return got


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
@pytest.mark.parametrize("case", gc.normalize_cases(), ids=lambda c: c["name"])
def test_normalize_golden(nv, onorm, case, dtype):
    host = strings(case["rows"], dtype)
    if "slice" in case:
        lo, n = case["slice"]
        host = host.slice(lo, lo + n)
    normalizer_tokens = case["special_tokens"]
    for _ in range(2):  # the reference's tests call twice with one normalizer; here a fresh one each time is as good
        got = run(nv, host, case["do_lower_case"], normalizer_tokens)
        assert got.to_pylist() == [None if r is None else r.encode("utf-8") for r in case["expected"]]
    check(nv, onorm, host, case["do_lower_case"], normalizer_tokens, case["name"])


def test_normalizer_is_reusable(nv):
    case = next(c for c in gc.normalize_cases() if c["name"] == "SpecialTokens lower")
    normalizer = nv.CharacterNormalizer(True, nv.DeviceStringsColumn.from_host(strings(case["special_tokens"])))
    col = nv.DeviceStringsColumn.from_host(strings(case["rows"]))
    first = nv.normalize_characters(col, normalizer).to_host().to_pylist()
    again = nv.normalize_characters(col, normalizer).to_host().to_pylist()
    assert first == again == [r.encode("utf-8") for r in case["expected"]]


PALETTE = (list("abcdefghijklmnopqrstuvwxyzABCDEFGHIJKLMNOPQRSTUVWXYZ0123456789") * 3 + list("  \t\n\r.,;:!?^$[](){}`~-_'\"") * 2
           + list("éèâîôÉÈÂĂĆĖÑÜüñßçøåİıŉǅΐΣς") + ["é", "́", "̧", " ", " ", "​", "­", "�", "\x00", "\x7f"]
           + list("漢字仮名丏丟乾乿中文") + list("한글각힣") + list("ﬃﬁǰẖ£€„“”«»") + ["😀", "𝄞", "\U00020000", "\U000e0001", "\U0010ffff"]
           + ["[PAD]", "[CLS]", "[SEP]", "[pad]", "[MASK]", "[UNK]", "[", "]", "[a]", "[é]"])


def random_rows(rng, n, max_items, p_null=0.05, p_empty=0.05):
    rows = []
    for _ in range(n):
        u = rng.random()
        if u < p_null:
            rows.append(None)
        elif u < p_null + p_empty:
            rows.append("")
        else:
            rows.append("".join(PALETTE[i] for i in rng.integers(0, len(PALETTE), rng.integers(1, max_items + 1))))
    return rows


@pytest.mark.parametrize("do_lower", [True, False])
@pytest.mark.parametrize("seed,dtype", [(1, np.int32), (2, np.int64)])
def test_normalize_random_utf8(nv, onorm, seed, dtype, do_lower):
    rng = np.random.default_rng(seed)
    host = strings(random_rows(rng, 2000, 60), dtype)
    tokens = ["[PAD]", "[CLS]", "[SEP]", "[MASK]", "[UNK]"]
    check(nv, onorm, host, do_lower, tokens, "with special tokens")
    check(nv, onorm, host, do_lower, (), "without special tokens")
    lo, hi = 37, 1251
    check(nv, onorm, host.slice(lo, hi), do_lower, tokens, "sliced")


@pytest.mark.parametrize("do_lower", [True, False])
def test_normalize_tokens_and_characters_across_tile_boundaries(nv, onorm, do_lower):
    tokens = ["[PAD]", "[SEP]", "[ABCD]"]
    for shift in range(0, 14):
        rows = ["a" * (TILE - 9 + shift) + "[PAD]" + "b" * (TILE - 7) + "[abcd]" + "c" * (TILE - 3) + "[SEP]",
                "丏é😀ﬃ한" * 3, "[PAD]"]
        check(nv, onorm, strings(rows), do_lower, tokens, f"shift {shift}")
    for shift in range(0, 6):
        rows = ["x" * (TILE - 4 + shift) + "😀丏éĂ한ﬃ" + "y" * (TILE - 20) + "ﬃ😀"]
        check(nv, onorm, strings(rows), do_lower, (), f"wide shift {shift}")
    # a token split between rows is still one token of the flat byte sequence
    check(nv, onorm, strings(["ab[PA", "D]cd", "[", "SEP", "]"]), do_lower, tokens, "token over rows")


@pytest.mark.parametrize("do_lower", [True, False])
def test_normalize_malformed_utf8(nv, onorm, do_lower):
    rng = np.random.default_rng(7)
    rows = [bytes(rng.integers(0, 256, rng.integers(0, 40), dtype=np.uint8)) for _ in range(200)]
    rows += [b"abc\xe4", b"\xf0\x9f", b"\xc3", b"\xf8\x80\x80\x80z", b"\xf4\x90\x80\x80", b"\xed\xa0\x80", b"\x80\x80a"]
    check(nv, onorm, strings(rows), do_lower, ["[PAD]"], "random bytes")
    # more than four output bytes per input byte (a first byte that swallows ASCII into a Hangul syllable, which then
    # decomposes, and the swallowed bytes count once more on their own): the tile's output no longer fits the LDS
    # staging and is written byte by byte
    rows = [b"\xea\x30\x21" * 2000, b"ab" + b"\xea\x30\x21" * 700 + b"cd", b"plain"]
    got = check(nv, onorm, strings(rows), do_lower, (), "expansion beyond the staging buffer")
    if do_lower:
        assert got.chars.size > 4 * sum(len(r) for r in rows[:2])
    # over-long encodings of '[' decode to it and open a special token like the plain byte does
    for opener in (b"\xc1\x9b", b"\xe0\x81\x9b", b"\xf0\x80\x81\x9b", b"\xc1\x1b"):
        for shift in range(0, 9):
            rows = [b"a" * (TILE - 6 + shift) + opener + b"PAD]" + b"b" * 40, opener + b"PAD]"]
            check(nv, onorm, strings(rows), do_lower, ["[PAD]"], f"over-long bracket {opener!r} shift {shift}")


def test_normalize_nulls_keep_their_bytes_and_empty_shapes(nv, onorm):
    # a null row whose offsets still span bytes: the flat pass normalizes them like any others
    base = strings(["Ab.", "Cd!", "", "Ef"])
    mask = pack_validity([True, False, True, True])
    host = HostStringsColumn(base.chars, base.offsets, mask, 4, 0, 1)
    got = check(nv, onorm, host, True)
    assert got.offsets.tolist() == [0, 5, 10, 10, 12] and got.null_count == 1
    # every row empty: offsets of zeros, no chars; with a mask it is copied
    got = run(nv, strings(["", None, ""]), True)
    assert got.offsets.tolist() == [0, 0, 0, 0] and got.chars.size == 0 and got.to_pylist() == [b"", None, b""]
    # empty column
    got = run(nv, strings([]), False)
    assert got.size == 0 and got.offsets.size == 0 and got.chars.size == 0
    # thousands of empty rows that all start at one byte position, before, between and after the text
    rows = [""] * 3000 + ["Ab, c"] + [""] * 2500 + ["D!"] + [""] * 1000
    got = check(nv, onorm, strings(rows), True)
    assert got.offsets[3000] == 0 and got.offsets[3001] == 7 and got.offsets[-1] == 7 + 4
    # sliced view whose first offset is not 0, int64 offsets
    host = strings(["skip me", "Keep, THIS", "and\tthis"], np.int64).slice(1, 3)
    assert check(nv, onorm, host, True).to_pylist() == [b"keep ,  this", b"and this"]


def test_special_tokens_rules(nv, onorm):
    with pytest.raises(ValueError):
        nv.CharacterNormalizer(True, nv.DeviceStringsColumn.from_host(strings(["[PAD]", None])))
    rows = ["[PAD]", "[PADS]", "[LONGER]", "x[pad]y", "[PAD", "[P-D]", "[[PAD]", "[ﬃ]", "[K]"]
    # sorted, then lower-cased, then searched by halving: with "[PADS]" present "[pad]" is not found (as in the reference)
    check(nv, onorm, strings(rows), True, ["[PAD]", "[PADS]", "[LONGER]"], "out of order after lower-casing")
    check(nv, onorm, strings(rows), False, ["[PAD]", "[PADS]", "[LONGER]"], "keep case")
    check(nv, onorm, strings(rows), True, ["[PAD]", "[[PAD]", "[FFI]", "[K]"], "nested and non-ASCII tokens")
    many = [f"[T{i:03d}]" for i in range(200)]
    rng = np.random.default_rng(3)
    text = ["".join(many[i] if rng.random() < 0.7 else f"[t{i}x]" for i in rng.integers(0, 200, 8)) for _ in range(64)]
    check(nv, onorm, strings(text), True, many, "200 tokens")
    check(nv, onorm, strings(text), False, many, "200 tokens, keep case")


@pytest.mark.parametrize("do_lower", [True, False])
def test_normalize_ascii_at_scale(nv, onorm, do_lower):
    # 64 MiB of ASCII in 1M rows against the table-driven numpy restatement, which is first checked against the
    # character-by-character oracle on a prefix
    rng = np.random.default_rng(11)
    alphabet = np.frombuffer(b"abcdefghijklmnopqrstuvwxyz     ABCDEFGHIJ.,;!?[]()\t\n\x00\x1f\x7f0123456789", np.uint8)
    n = 64 << 20
    chars = alphabet[rng.integers(0, alphabet.size, n)]
    cuts = np.sort(rng.integers(0, n + 1, (1 << 20) - 1))
    offsets = np.concatenate([[0], cuts, [n]]).astype(np.int64)
    host = HostStringsColumn(chars, offsets, None, 1 << 20, 0, 0)
    small = host.slice(5, 400)
    assert_same(onorm.normalize_ascii(small, do_lower), onorm.normalize_characters(small, do_lower), "numpy restatement")
    assert_same(run(nv, host, do_lower), onorm.normalize_ascii(host, do_lower), "64 MiB")


@pytest.mark.parametrize("total", [0x7FFFFFFF - 1, 0x7FFFFFFF, (1 << 31) + 4097])
def test_normalize_large_strings_offsets(nv, total):
    # lower-case letters and single spaces come back unchanged, so the result must equal the input; its offsets are
    # int32 below INT32_MAX bytes of chars and int64 from there on.  Built and compared on the device.
    import torch
    phrase = torch.tensor(list(b"the quick brown fox jumps over the lazy dog "), dtype=torch.uint8, device="cuda")
    chars = phrase.repeat(total // phrase.numel() + 1)[:total].contiguous()
    row = 65521
    offsets = torch.arange(0, total, row, dtype=torch.int64, device="cuda")
    offsets = torch.cat([offsets, torch.tensor([total], dtype=torch.int64, device="cuda")])
    col = nv.DeviceStringsColumn(chars, offsets, None, offsets.numel() - 1, 0, 0)
    out = nv.normalize_characters(col, nv.CharacterNormalizer(True))
    torch.cuda.synchronize()
    assert out.size == col.size and out.null_count == 0
    assert out.offsets.dtype == (torch.int64 if total >= 0x7FFFFFFF else torch.int32)
    assert out.chars.numel() == total and torch.equal(out.chars, chars)
    assert torch.equal(out.offsets.to(torch.int64), offsets)


def test_normalize_feeds_the_tokenizer(nv, onorm):
    # the BERT pipeline on the device: the STRING result of normalize_characters goes straight into wordpiece_tokenize
    from oracle import pyoracle as orc
    d = gc.bert_case()
    vocab = strings(d["vocab"])
    words = [v.decode("utf-8") for v in d["vocab"] if v.isalpha() and len(v) > 2][:500]
    rng = np.random.default_rng(21)
    styles = [str.upper, str.title, lambda s: s, lambda s: s + ",", lambda s: "(" + s + ")", lambda s: s.replace("e", "é"),
              lambda s: s + "\t", lambda s: "[CLS]" + s, lambda s: s + "丏", lambda s: s + "!?"]
    rows = [None if rng.random() < 0.05 else
            " ".join(styles[int(rng.integers(0, len(styles)))](words[int(rng.integers(0, len(words)))]) for _ in range(int(rng.integers(0, 40))))
            for _ in range(3000)]
    host = strings(rows)
    normalizer = nv.CharacterNormalizer(True, nv.DeviceStringsColumn.from_host(strings(["[CLS]"])))
    normalized = nv.normalize_characters(nv.DeviceStringsColumn.from_host(host), normalizer)
    got = nv.wordpiece_tokenize(normalized, nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(vocab)), 0).to_host()
    exp = orc.wordpiece_tokenize(onorm.normalize_characters(host, True, [b"[CLS]"]), orc.Vocabulary(vocab), 0)
    assert got.equals(exp)
    assert got.child.size > 3 * 3000
