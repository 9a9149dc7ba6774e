"""Loaders for the committed known-answer fixtures (tests/golden/*.json)."""
from __future__ import annotations

import json
import os
from typing import List, Optional

import numpy as np

from cudf_amd.arrow_host import HostListStringsColumn, HostStringsColumn

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _row(r):
    if isinstance(r, dict):
        s, n = r["repeat"]
        return s * n
    return r


def minhash_cases():
    d = json.load(open(os.path.join(GOLDEN, "minhash_vectors.json"), encoding="utf-8"))
    out = []
    for c in d["cases"]:
        c = dict(c)
        c["rows"] = [_row(r) for r in c["rows"]]
        out.append(c)
    return out


def minhash_ngrams_cases():
    """Each case: rows (list of lists of strings), optional slice, ngrams, seed, a, b, expected32, expected64."""
    d = json.load(open(os.path.join(GOLDEN, "minhash_ngrams_vectors.json"), encoding="utf-8"))
    out = []
    for c in d["cases"]:
        c = dict(c)
        if "repeat_rows" in c:
            c["rows"] = [[s] * n for s, n in c.pop("repeat_rows")]
        out.append(c)
    return out


def list_strings(rows, child_offsets_dtype=np.int32) -> HostListStringsColumn:
    return HostListStringsColumn.from_pylist(rows, child_offsets_dtype)


def jaccard_cases():
    return json.load(open(os.path.join(GOLDEN, "jaccard_vectors.json"), encoding="utf-8"))["cases"]


def normalize_cases():
    """Each case: rows (None = null row), optional slice [offset, size], do_lower_case, special_tokens, expected."""
    return json.load(open(os.path.join(GOLDEN, "normalize_vectors.json"), encoding="utf-8"))["cases"]


def codepoint_behaviour_digests():
    return json.load(open(os.path.join(GOLDEN, "codepoint_behaviour_digests.json"), encoding="utf-8"))


def murmur64_vectors():
    return json.load(open(os.path.join(GOLDEN, "minhash_vectors.json"), encoding="utf-8"))["murmurhash3_x64_128_word0"]


def murmur32_vectors():
    return json.load(open(os.path.join(GOLDEN, "minhash_vectors.json"), encoding="utf-8"))["murmurhash3_x86_32_public"]["vectors"]


def wordpiece_cases():
    return json.load(open(os.path.join(GOLDEN, "wordpiece_vectors.json"), encoding="utf-8"))["cases"]


def bert_case():
    d = json.load(open(os.path.join(GOLDEN, "wordpiece_bert_sentences.json"), encoding="utf-8"))
    with open(os.path.join(GOLDEN, d["vocab_file"]), "rb") as f:
        # cudf.read_text(delimiter="\n", strip_delimiters=True): one entry per line
        vocab = f.read().split(b"\n")
    if vocab and vocab[-1] == b"":
        vocab.pop()
    d["vocab"] = vocab
    return d


def expected_list_equal(got_pylist: List[Optional[List[int]]], expected) -> bool:
    if len(got_pylist) != len(expected):
        return False
    for g, e in zip(got_pylist, expected):
        if e is None or g is None:
            if not (e is None and g is None):
                return False
        elif [int(x) for x in g] != [int(x) for x in e]:
            return False
    return True


def strings(rows, dtype=np.int32, **kw) -> HostStringsColumn:
    return HostStringsColumn.from_pylist(rows, offsets_dtype=dtype, **kw)
