"""Every operation against the host oracle on randomly shaped inputs: alphabets of 2 to 26 letters with or without
multi-byte characters, vocabularies of 5 to 40000 entries with keys of up to 40 bytes, 1 to 20000 rows with nulls,
empty rows, words of up to 260 bytes, double spaces, now and then a row of hundreds of kilobytes, int32 and int64
offsets, sliced views.  Bit-exact."""
import numpy as np
import pytest

from cudf_amd.arrow_host import HostStringsColumn

pytestmark = pytest.mark.gpu

LETTERS = list("abcdefghijklmnopqrstuvwxyz")
EXTRA = list("éüñ漢字😀")


@pytest.fixture(scope="module")
def nv():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from cudf_amd import _capi, nvtext
    _capi.load()  # fails loudly if the HIP library is missing
    return nvtext


def make_case(seed):
    rng = np.random.default_rng(seed)
    utf8 = rng.random() < 0.4
    alpha = LETTERS[: int(rng.integers(2, 27))] + (EXTRA if utf8 else [])
    wanted = int(rng.choice([5, 50, 500, 5000, 40000]))
    vocab = ["[UNK]"] if rng.random() < 0.9 else ["x0"]
    seen = set(vocab)
    longest = int(rng.choice([3, 6, 12, 24, 40]))
    tries = 0
    while len(vocab) < wanted and tries < 20 * wanted:
        tries += 1
        s = "".join(rng.choice(alpha, int(rng.integers(1, longest + 1))))
        if rng.random() < 0.4:
            s = "##" + s
        if s not in seen:
            seen.add(s)
            vocab.append(s)
    stems = [v for v in vocab if not v.startswith("##") and v != "[UNK]"] or ["a"]
    n = int(rng.choice([1, 3, 70, 1000, 20000]))
    p_null = float(rng.choice([0, 0.1]))
    long_at = int(rng.integers(0, n)) if rng.random() < 0.3 else -1
    rows = []
    for i in range(n):
        u = rng.random()
        if u < p_null:
            rows.append(None)
            continue
        if u < p_null + 0.05:
            rows.append("")
            continue
        words = []
        for _ in range(int(rng.integers(1, 60)) if i != long_at else int(rng.integers(8000, 40000))):
            t = rng.random()
            if t < 0.6:
                words.append(stems[int(rng.integers(0, len(stems)))])
            elif t < 0.9:
                words.append("".join(rng.choice(alpha, int(rng.integers(1, 20)))))
            else:
                words.append("".join(rng.choice(alpha, int(rng.integers(20, 260)))))
        rows.append((" " if rng.random() < 0.8 else "  ").join(words))
    host = HostStringsColumn.from_pylist(rows)
    if rng.random() < 0.3:
        host = HostStringsColumn(host.chars, host.offsets.astype(np.int64), host.mask, host.size, host.offset, host.null_count)
    if n > 4 and rng.random() < 0.4:
        lo = int(rng.integers(0, n // 2))
        host = host.slice(lo, int(rng.integers(lo + 1, n + 1)))
    return rng, host, HostStringsColumn.from_pylist(vocab)


@pytest.mark.parametrize("seed", range(1000, 1016))
def test_every_operation_on_a_random_column(nv, seed):
    from oracle import normalize_py
    from oracle import pyoracle as orc
    rng, host, vocab = make_case(seed)
    d = nv.DeviceStringsColumn.from_host(host)
    dv = nv.WordPieceVocabulary(nv.DeviceStringsColumn.from_host(vocab))
    ov = orc.Vocabulary(vocab)
    for max_words in (0, int(rng.choice([1, 5, 100]))):
        assert nv.wordpiece_tokenize(d, dv, max_words).to_host().equals(orc.wordpiece_tokenize(host, ov, max_words, nthreads=8)), max_words
    P, width = int(rng.choice([1, 7, 64, 256])), int(rng.choice([2, 4, 5, 9, 20]))
    a = rng.integers(1, 2**32, P, dtype=np.uint64).astype(np.uint32)
    b = rng.integers(0, 2**32, P, dtype=np.uint64).astype(np.uint32)
    assert nv.minhash(d, 7, a, b, width).to_host().equals(orc.minhash(host, 7, a, b, width, nthreads=8))
    a64, b64 = rng.integers(1, 2**63, P, dtype=np.uint64), rng.integers(0, 2**63, P, dtype=np.uint64)
    assert nv.minhash64(d, 11, a64, b64, width).to_host().equals(orc.minhash64(host, 11, a64, b64, width, nthreads=8))
    lower = bool(rng.random() < 0.5)
    tokens = [b"[CLS]", b"[SEP]"] if rng.random() < 0.5 else []
    special = nv.DeviceStringsColumn.from_host(HostStringsColumn.from_pylist([t.decode() for t in tokens])) if tokens else None
    got = nv.normalize_characters(d, nv.CharacterNormalizer(lower, special)).to_host()
    exp = normalize_py.normalize_characters_native(host, lower, tokens, nthreads=8)
    assert np.array_equal(got.chars, exp.chars) and np.array_equal(got.offsets, exp.offsets)
    if host.size >= 2:
        h1, h2 = host.slice(0, host.size - 1), host.slice(1, host.size)
        got = nv.jaccard_index(nv.DeviceStringsColumn.from_host(h1), nv.DeviceStringsColumn.from_host(h2), width).to_host()
        exp = orc.jaccard_index(h1, h2, width, nthreads=8)
        valid = exp.validity()
        assert got.size == exp.size and got.null_count == exp.null_count and np.array_equal(got.validity(), valid)
        assert np.array_equal(got.values.view(np.uint32)[valid], exp.values.view(np.uint32)[valid])
