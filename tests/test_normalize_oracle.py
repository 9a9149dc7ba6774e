"""The normalize_characters oracle against the reference's known answers, and the per-code-point rules (the
oracle's and the library's table generator's) against digests of the reference's tables."""
import importlib.util
import os

import numpy as np
import pytest

from oracle import normalize_py as onorm
from tests import golden_cases as gc
from tests.golden.digest_codepoint_metadata import LIMIT, canonical, digests

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_generator():
    spec = importlib.util.spec_from_file_location(
        "gen_codepoint_tables", os.path.join(ROOT, "cudf_amd", "csrc", "gen_codepoint_tables.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def case_column(case, dtype=np.int32):
    col = gc.strings(case["rows"], dtype)
    if "slice" in case:
        lo, n = case["slice"]
        col = col.slice(lo, lo + n)
    return col


def expected_bytes(case):
    return [None if r is None else r.encode("utf-8") for r in case["expected"]]


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
@pytest.mark.parametrize("case", gc.normalize_cases(), ids=lambda c: c["name"])
def test_normalize_golden(case, dtype):
    tokens = [t.encode("utf-8") for t in case["special_tokens"]]
    got = onorm.normalize_characters(case_column(case, dtype), case["do_lower_case"], tokens)
    assert got.to_pylist() == expected_bytes(case)
    assert got.offsets.dtype == np.int32


def mismatched_blocks(entries):
    want = gc.codepoint_behaviour_digests()
    got = digests(entries)
    assert len(got) == len(want["digests"])
    return [hex(i * want["block"]) for i, (g, w) in enumerate(zip(got, want["digests"])) if g != w]


def test_oracle_rules_match_reference_tables():
    def entries():
        for cp in range(LIMIT):
            kind, low = onorm.classify(cp)
            new = 0x20 if kind == onorm.REPLACE else (0 if low == [cp] or not low else low[0])
            multi = int(len(low) > 1)
            aux = ((low[1] << 32) | (low[2] if len(low) > 2 else 0)) if multi else 0
            yield canonical(kind, multi, new, aux)
    assert mismatched_blocks(entries()) == []


def test_generated_tables_match_reference_tables():
    gen = load_generator()

    def entries():
        for cp in range(LIMIT):
            v, a = gen.entry(cp)
            yield canonical((v >> 24) & 7, (v >> 23) & 1, v & 0x1FFFFF, a)
    assert mismatched_blocks(entries()) == []


def committed_tables():
    """The three arrays of cudf_amd/csrc/codepoint_tables.inc, the data the library is compiled from."""
    import re
    text = open(os.path.join(ROOT, "cudf_amd", "csrc", "codepoint_tables.inc")).read()

    def rows(name):
        body = re.search(name + r"\[\]\[\d\] = \{(.*?)\};", text, re.S).group(1)
        return [tuple(int(x.rstrip("UL"), 0) for x in r.split(",")) for r in re.findall(r"\{([^{}]*)\}", body)]
    return rows("kCodepointRuns"), rows("kCodepointSecond"), rows("kLowerCase")


def test_committed_tables_match_reference_tables():
    gen = load_generator()
    runs, second, _ = committed_tables()
    first = [gen.DEFAULT] * LIMIT
    for cp, count, value in runs:
        first[cp: cp + count] = [value] * count
    aux = dict(second)
    for cp in range(0xAC00, 0xD7A4):  # the library fills the Hangul syllables the same way
        first[cp], aux[cp] = gen.hangul(cp)
    entries = (canonical((v >> 24) & 7, (v >> 23) & 1, v & 0x1FFFFF, aux.get(cp, 0)) for cp, v in enumerate(first))
    assert mismatched_blocks(entries) == []


def test_committed_tables_are_what_the_generator_writes():
    import unicodedata
    if unicodedata.unidata_version != "13.0.0":
        pytest.skip("the tables were generated with the Unicode 13.0.0 database")
    gen = load_generator()
    runs, second, lower = committed_tables()
    want_runs, want_second = gen.tables()
    assert runs == want_runs and second == want_second and lower == gen.lower_map()


def test_lower_case_table_matches_ascii_and_latin1():
    _, _, lower = committed_tables()
    table = {row[0]: row[1:] for row in lower}
    for c in range(ord("A"), ord("Z") + 1):
        assert table[c] == (c + 32, 0, 0)
    assert table[0xC9] == (0xE9, 0, 0) and table[0x130] == (0x69, 0x307, 0) and table[0x212A] == (0x6B, 0, 0)
    assert all(cp <= 0xFFFF for cp in table) and ord("a") not in table


def test_special_tokens_sorted_then_lowered():
    # "[B]" sorts before "[a]" but lower-cases to "[b]": the halving search then misses "[a]" in a list of two
    # only when it looks at the wrong half; with these two it still finds both
    assert onorm.sorted_special_tokens([b"[a]", b"[B]"], True) == [b"[b]", b"[a]"]
    assert onorm._binary_search([b"[b]", b"[a]"], b"[a]") is False
    assert onorm._binary_search([b"[b]", b"[a]"], b"[b]") is False
    assert onorm._binary_search([b"[a]", b"[b]"], b"[b]") is True


def test_decode_follows_the_lead_byte():
    # a lead byte decides the length alone: continuation bytes are not checked, bytes past the end read as 0
    assert onorm._decode("é".encode(), 0) == 0xE9
    assert onorm._decode("丏".encode(), 0) == 0x4E0F
    assert onorm._decode("😀".encode(), 0) == 0x1F600
    assert onorm._decode(b"\xc3", 0) == (0x03 << 6)
    assert onorm._decode(b"\xe4\xb8", 0) == ((0x4 << 12) | (0x38 << 6))


def test_special_token_rules():
    # a token is recognised only when '[' ... ']' spans at most 6 input characters and matches exactly
    rows = ["[PAD]", "[PADS]", "[LONGER]", "x[pad]y", "[PAD", "[P-D]"]
    col = gc.strings(rows)
    got = onorm.normalize_characters(col, True, [b"[PAD]", b"[LONGER]", b"[XPADS]"]).to_pylist()
    assert got == [b" [PAD] ", b" [ pads ] ", b" [ longer ] ", b"x [PAD] y", b" [ pad", b" [ p - d ] "]
    got = onorm.normalize_characters(col, False, [b"[PAD]", b"[PADS]"]).to_pylist()
    assert got == [b" [PAD] ", b" [PADS] ", b" [ LONGER ] ", b"x [ pad ] y", b" [ PAD", b" [ P - D ] "]


def test_special_tokens_lowered_after_sorting_can_be_missed():
    # "[PADS]" sorts before "[PAD]" ('S' < ']'), "[pads]" after "[pad]" (']' < 's'): the reference sorts, then
    # lower-cases, then searches by halving, so with both tokens "[pad]" is no longer found
    col = gc.strings(["[PAD]", "[PADS]"])
    got = onorm.normalize_characters(col, True, [b"[PAD]", b"[PADS]", b"[LONGER]"]).to_pylist()
    assert got == [b" [ pad ] ", b" [PADS] "]


# Unicode blocks whose characters and properties have not changed for many Unicode versions: an implementation with
# older or newer character tables than the reference's (Unicode 11) must still agree there
STABLE_BLOCKS = [(1, 0x0780), (0x1E00, 0x1F00), (0x2000, 0x2070), (0x3000, 0x3100), (0x4E00, 0x9FA6), (0xAC00, 0xD7A4),
                 (0xFB00, 0xFB50), (0xFF00, 0xFFF0)]


def test_rules_match_hf_bert_normalizer_and_pre_tokenizer():
    """An independent implementation of the same BERT clean-up (tokenizers' BertNormalizer + BertPreTokenizer, written in
    Rust with its own character tables): the words it finds in "x<c>y" must be the words of the oracle's output, for every
    assigned character c of the stable blocks, lower-casing and not."""
    import unicodedata
    tokenizers = pytest.importorskip("tokenizers")
    from tokenizers import normalizers, pre_tokenizers
    pre = pre_tokenizers.BertPreTokenizer()
    checked = 0
    for lower in (True, False):
        norm = normalizers.BertNormalizer(clean_text=True, handle_chinese_chars=True, strip_accents=None if lower else False, lowercase=lower)
        for lo, hi in STABLE_BLOCKS:
            cps = [cp for cp in range(lo, hi) if unicodedata.category(chr(cp)) not in ("Cn", "Co")]
            rows = ["x" + chr(cp) + "y" for cp in cps]
            got = onorm.normalize_characters(gc.strings(rows), lower).to_pylist()
            for cp, text, g in zip(cps, rows, got):
                want = [w for w, _ in pre.pre_tokenize_str(norm.normalize_str(text))]
                assert [w for w in g.decode("utf-8").split(" ") if w] == want, (hex(cp), lower)
                checked += 1
    assert checked > 60000


def test_normalize_then_tokenize_matches_hf_bert_pipeline():
    """normalize_characters followed by wordpiece_tokenize is BERT's tokenizer: ids equal tokenizers' Bert pipeline."""
    tokenizers = pytest.importorskip("tokenizers")
    from tokenizers import Tokenizer, normalizers, pre_tokenizers
    from tokenizers.models import WordPiece
    from oracle import pyoracle as orc
    d = gc.bert_case()
    vocab = [v.decode("utf-8") for v in d["vocab"]]
    ids = {}
    for i, t in enumerate(vocab):
        ids.setdefault(t, i)
    tok = Tokenizer(WordPiece(ids, unk_token="[UNK]", max_input_chars_per_word=100))
    tok.normalizer = normalizers.BertNormalizer(clean_text=True, handle_chinese_chars=True, strip_accents=None, lowercase=True)
    tok.pre_tokenizer = pre_tokenizers.BertPreTokenizer()
    rng = np.random.default_rng(5)
    stems = [t for t in vocab if t.isalpha() and t.isascii() and len(t) > 2][:600]
    decorate = [str.upper, str.title, lambda s: s, lambda s: s + ",", lambda s: "(" + s + ")", lambda s: s.replace("e", "é").replace("a", "Â"),
                lambda s: s + "\t", lambda s: s + "ing", lambda s: "un" + s, lambda s: s + "丏", lambda s: s + "­", lambda s: s + "!?"]
    rows = [" ".join(decorate[int(rng.integers(0, len(decorate)))](stems[int(rng.integers(0, len(stems)))]) for _ in range(int(rng.integers(1, 25))))
            for _ in range(400)]
    normalized = onorm.normalize_characters(gc.strings(rows), True)
    got = orc.wordpiece_tokenize(normalized, orc.Vocabulary(gc.strings(d["vocab"])), 0).to_pylist()
    split = 0
    for row, g in zip(rows, got):
        want = tok.encode(row, add_special_tokens=False).ids
        assert g == want, row
        split += len(want) > len(row.split(" "))
    assert split > 200  # punctuation and sub-word splits were exercised


# ---- the C++ restatement (oracle/nvtext_oracle.cpp), which checks the large inputs

def test_rule_tables_hold_classify_of_every_code_point():
    kind, lower = onorm.rule_tables()
    lower = lower.reshape(-1, 3)
    for cp in range(0x110000):
        k, low = onorm.classify(cp)
        assert kind[cp] == k and [int(x) for x in lower[cp] if x] == [x for x in low if x], hex(cp)


@pytest.mark.parametrize("nthreads", [1, 4])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
@pytest.mark.parametrize("case", gc.normalize_cases(), ids=lambda c: c["name"])
def test_native_normalize_golden(case, dtype, nthreads):
    tokens = [t.encode("utf-8") for t in case["special_tokens"]]
    got = onorm.normalize_characters_native(case_column(case, dtype), case["do_lower_case"], tokens, nthreads)
    assert got.to_pylist() == expected_bytes(case)


def random_text_rows(rng, n, max_items):
    palette = (list("abcdefghijklmnopqrstuvwxyzABCDEFGHIJKLMNOPQRSTUVWXYZ0123456789") * 3 + list("  \t\n\r.,;:!?^$[](){}`~-_'\"") * 2
               + list("éèâîôÉÈÂĂĆĖÑÜüñßçøåİıŉǅΐΣς") + ["é", "́", "̧", " ", " ", "​", "­", "�", "\x00", "\x7f"]
               + list("漢字仮名丏丟乾乿中文한글각힣ﬃﬁǰẖ£€„“”«»") + ["😀", "𝄞", "\U00020000", "\U000e0001", "\U0010ffff"]
               + ["[PAD]", "[CLS]", "[SEP]", "[pad]", "[MASK]", "[UNK]", "[", "]", "[a]", "[é]"])
    rows = []
    for _ in range(n):
        u = rng.random()
        rows.append(None if u < 0.05 else "" if u < 0.1 else
                    "".join(palette[i] for i in rng.integers(0, len(palette), rng.integers(1, max_items + 1))))
    return rows


@pytest.mark.parametrize("do_lower", [True, False])
@pytest.mark.parametrize("seed,dtype", [(11, np.int32), (12, np.int64)])
def test_native_normalize_matches_the_python_loops(seed, dtype, do_lower):
    rng = np.random.default_rng(seed)
    col = gc.strings(random_text_rows(rng, 600, 60), dtype)
    tokens = [b"[PAD]", b"[CLS]", b"[SEP]", b"[MASK]", b"[UNK]"]
    for toks in (tokens, []):
        for view in (col, col.slice(23, 411)):
            exp = onorm.normalize_characters(view, do_lower, toks)
            for nthreads in (1, 3, 8):  # parts of 4096 bytes and more: the column has about 40 KB
                got = onorm.normalize_characters_native(view, do_lower, toks, nthreads)
                assert np.array_equal(got.chars, exp.chars) and np.array_equal(got.offsets, exp.offsets), (len(toks), nthreads)
                assert got.offsets.dtype == exp.offsets.dtype and got.null_count == exp.null_count


def test_native_normalize_malformed_bytes():
    rng = np.random.default_rng(5)
    data = rng.integers(0, 256, 30000, dtype=np.uint8)
    data[rng.random(data.size) < 0.3] = 0x5B  # plenty of '['
    data[rng.random(data.size) < 0.1] = 0x5D
    cuts = np.sort(rng.integers(0, data.size + 1, 299))
    offsets = np.concatenate([[0], cuts, [data.size]]).astype(np.int32)
    from cudf_amd.arrow_host import HostStringsColumn
    col = HostStringsColumn(data, offsets, None, 300, 0, 0)
    for do_lower in (True, False):
        exp = onorm.normalize_characters(col, do_lower, [b"[]", b"[a]"])
        for nthreads in (1, 5):
            got = onorm.normalize_characters_native(col, do_lower, [b"[]", b"[a]"], nthreads)
            assert np.array_equal(got.chars, exp.chars) and np.array_equal(got.offsets, exp.offsets)


def test_native_normalize_special_token_across_its_blocks():
    # the C++ restatement works through the chars 32 KiB at a time: a token that lies across such a boundary
    from cudf_amd.arrow_host import HostStringsColumn
    for shift in range(0, 7):
        text = b"a" * (32768 - shift) + b"[pad]" + b"b" * 100 + "É".encode() + b"[SEP]"
        col = HostStringsColumn(np.frombuffer(text, np.uint8).copy(), np.array([0, 5, len(text)], np.int32), None, 2, 0, 0)
        exp = onorm.normalize_characters(col, True, [b"[PAD]", b"[SEP]"])
        got = onorm.normalize_characters_native(col, True, [b"[PAD]", b"[SEP]"], 1)
        assert np.array_equal(got.chars, exp.chars) and np.array_equal(got.offsets, exp.offsets), shift
        assert bytes(got.chars).count(b"[PAD]") == 1 and bytes(got.chars).count(b"[SEP]") == 1
