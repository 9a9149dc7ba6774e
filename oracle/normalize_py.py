"""Host restatement of nvtext::normalize_characters -- TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows cpp/src/text/normalize.cu: 331-388 (per-character replacement), 270-316 (special tokens),
491-561 (flat pass over the chars of the column, row sizes, nulls).  Pure Python over the Unicode database of
the running interpreter, so it is for small inputs.  The per-code-point rules are written out here on their
own (they are what the reference keeps in cpp/src/text/detail/codepoint_metadata.ah); tests compare them with
the tables the library is built from, code point by code point.

Pinned by: cpp/tests/text/normalize_tests.cpp:91-228 (WithNormalizer, SpecialTokens, NormalizeSlicedColumn) and
python/pylibcudf/tests/test_nvtext_normalize.py, transcribed into tests/golden/normalize_vectors.json.
"""
from __future__ import annotations

import unicodedata
from typing import List, Optional, Sequence

import numpy as np

# Code points added by Unicode 12.0 - 13.0 whose properties would matter: the reference's tables predate them.
_NEWER = frozenset([
    0x0B55, 0x0C77, 0x0D81, 0x0EBA, 0x1ABF, 0x1AC0, 0x2E4F, 0x2E52, 0xA7BA, 0xA7BC, 0xA7BE, 0xA7C2, 0xA7C4, 0xA7C5, 0xA7C6,
    0xA7C7, 0xA7C9, 0xA7F5, 0xA82C, 0xA9BD, 0x10EAB, 0x10EAC, 0x10EAD, 0x111CF, 0x1145A, 0x11938, 0x1193B, 0x1193C, 0x1193E,
    0x11943, 0x11944, 0x11945, 0x11946, 0x119D4, 0x119D5, 0x119D6, 0x119D7, 0x119DA, 0x119DB, 0x119E0, 0x119E2, 0x11FFF,
    0x13430, 0x13431, 0x13432, 0x13433, 0x13434, 0x13435, 0x13436, 0x13437, 0x13438, 0x16F4F, 0x16FE2, 0x16FE4,
    0x1E130, 0x1E131, 0x1E132, 0x1E133, 0x1E134, 0x1E135, 0x1E136, 0x1E2EC, 0x1E2ED, 0x1E2EE, 0x1E2EF])

PAD, PAD_IF_LOWER, REMOVE, REMOVE_IF_LOWER, REPLACE, PLAIN = range(6)


def _punct(cp: int) -> bool:
    if (33 <= cp <= 47) or (58 <= cp <= 64) or (91 <= cp <= 96) or (123 <= cp <= 126) or cp == 0x166D:
        return True
    return unicodedata.category(chr(cp)).startswith("P")


def _cjk(cp: int) -> bool:
    return any(lo <= cp <= hi for lo, hi in ((0x4E00, 0x9FFF), (0x3400, 0x4DBF), (0x20000, 0x2A6DF), (0x2A700, 0x2B73F),
                                              (0x2B740, 0x2B81F), (0x2B820, 0x2CEAF), (0xF900, 0xFAFF), (0x2F800, 0x2FA1F)))


def classify(cp: int):
    """(category, replacement code points when lower-casing) of one code point."""
    if cp >= 0x110000 or cp in _NEWER or 0xD800 <= cp <= 0xDFFF:
        return PLAIN, [cp]
    ch = chr(cp)
    cat = unicodedata.category(ch)
    if ch in "\t\n\r" or cat in ("Zs", "Zl", "Zp"):
        return REPLACE, [0x20]
    if cat in ("Cc", "Cf") or cp == 0 or cp == 0xFFFD:
        return REMOVE, []
    if cat == "Mn":
        return REMOVE_IF_LOWER, [cp]
    low = [ord(c) for c in unicodedata.normalize("NFD", ch.lower()) if unicodedata.category(c) != "Mn"] or [cp]
    kind = PLAIN
    if low != [cp] and _punct(low[0]):
        kind = PAD_IF_LOWER
    if _punct(cp) or _cjk(cp):
        kind = PAD
    return kind, low


def _decode(data: bytes, i: int) -> int:
    """The code point of the character whose first byte is data[i], read the way the reference does
    (cpp/include/cudf/strings/detail/utf8.hpp:68-97 and 118-140): the lead byte alone says how many bytes are packed,
    and the packed value's magnitude picks the decoding.  Bytes past the buffer read as 0."""
    b0 = data[i]
    n = 1 + (b0 >= 0xC0) + (b0 >= 0xE0) + (b0 >= 0xF0)
    packed = 0
    for k in range(n):
        packed = (packed << 8) | (data[i + k] if i + k < len(data) else 0)
    if packed < 0x80:
        return packed
    if packed < 0xE000:
        return ((packed & 0x1F00) >> 2) | (packed & 0x3F)
    if packed < 0xF00000:
        return ((packed & 0x0F0000) >> 4) | ((packed & 0x3F00) >> 2) | (packed & 0x3F)
    if packed <= 0xF8000000:
        return ((packed & 0x07000000) >> 6) | ((packed & 0x3F0000) >> 4) | ((packed & 0x3F00) >> 2) | (packed & 0x3F)
    return 0


def _utf8(cp: int) -> bytes:
    """cudf::strings::detail::codepoint_to_utf8 (utf8.hpp:170-197): plain arithmetic, surrogates included."""
    if cp < 0x80:
        return bytes([cp])
    if cp < 0x800:
        return bytes([0xC0 | (cp >> 6), 0x80 | (cp & 0x3F)])
    if cp < 0x10000:
        return bytes([0xE0 | (cp >> 12), 0x80 | ((cp >> 6) & 0x3F), 0x80 | (cp & 0x3F)])
    return bytes([0xF0 | ((cp >> 18) & 0x07), 0x80 | ((cp >> 12) & 0x3F), 0x80 | ((cp >> 6) & 0x3F), 0x80 | (cp & 0x3F)])


def _lower_bmp(token: bytes) -> bytes:
    """cudf::strings::to_lower of one string: per character, code points above U+FFFF unchanged
    (cpp/src/strings/case.cu:142-148)."""
    text = token.decode("utf-8", "surrogateescape")
    return "".join(c.lower() if ord(c) <= 0xFFFF and not 0xD800 <= ord(c) <= 0xDFFF else c for c in text).encode("utf-8", "surrogateescape")


def sorted_special_tokens(special_tokens: Sequence[bytes], do_lower_case: bool) -> List[bytes]:
    """normalize.cu:230-235: sorted by bytes first, lower-cased afterwards (which can leave them out of order)."""
    tokens = sorted(special_tokens)
    return [_lower_bmp(t) for t in tokens] if do_lower_case else tokens


def _binary_search(tokens: List[bytes], value: bytes) -> bool:
    """thrust::binary_search (normalize.cu:299): lower_bound by halving, then "not value < *it"; written out
    because the tokens need not be in order."""
    first, count = 0, len(tokens)
    while count > 0:
        half = count >> 1
        if tokens[first + half] < value:
            first += half + 1
            count -= half + 1
        else:
            count = half
    return first < len(tokens) and not value < tokens[first]


def normalize_flat(data: bytes, do_lower_case: bool, special_tokens: Sequence[bytes] = ()) -> List[List[bytes]]:
    """Per input byte, the three output slots (each the UTF-8 bytes of one character, b"" = nothing), after the
    special-token pass.  normalize.cu:331-388 then 270-316."""
    n = len(data)
    slots: List[List[bytes]] = [[b"", b"", b""] for _ in range(n)]
    for i in range(n):
        if (data[i] & 0xC0) == 0x80:
            continue
        cp = _decode(data, i)
        kind, low = classify(cp)
        if kind == REMOVE or (do_lower_case and kind == REMOVE_IF_LOWER):
            continue
        if kind == REPLACE:
            out = [0x20]
        elif do_lower_case:
            out = list(low)
        else:
            out = [cp]
        if (kind == PAD or (do_lower_case and kind == PAD_IF_LOWER)) and len(out) == 1:
            out = [0x20, out[0], 0x20]
        for k, c in enumerate(out):
            slots[i][k] = _utf8(c) if c else b""
    tokens = sorted_special_tokens(special_tokens, do_lower_case)
    if tokens:
        flat = lambda i, k: slots[i][k]
        for i in range(n):
            if slots[i][1] != b"[":
                continue
            span = min(6, n - i)
            # the slots after the one holding '[': `span` positions' worth (normalize.cu:286), which ends with
            # slot 0 of position i + span when there is one
            seq = [(i, 1), (i, 2)] + [(j, k) for j in range(i + 1, i + span) for k in range(3)]
            if i + span < n:
                seq.append((i + span, 0))
            close = next((p for p, (j, k) in enumerate(seq) if flat(j, k) == b"]"), None)
            if close is None:
                continue
            # one byte per character, its first (normalize.cu:289-294 narrows each slot to a char)
            cand = bytes(flat(j, k)[0] for j, k in seq[: close + 1] if flat(j, k) and flat(j, k) != b" ")
            if not _binary_search(tokens, cand):
                continue
            j, k = seq[1]
            slots[j][k] = b""                       # the space after '['
            j, k = seq[close - 1]
            slots[j][k] = b""                       # the space before ']'
            if do_lower_case:
                for j, k in seq[2: close - 2]:
                    v = slots[j][k]
                    if len(v) == 1 and ord("a") <= v[0] <= ord("z"):
                        slots[j][k] = bytes([v[0] - 32])
    return slots


def _offsets_dtype(total: int):
    """int64 offsets from the large-strings threshold on (cpp/include/cudf/strings/detail/strings_children.cuh:164-175,
    cpp/src/strings/utilities.cu:150-157: INT32_MAX unless the environment lowers it)."""
    return np.int64 if int(total) >= 0x7FFFFFFF else np.int32


def normalize_characters(col, do_lower_case: bool, special_tokens: Sequence[bytes] = ()):
    """col: cudf_amd.arrow_host.HostStringsColumn.  Returns a HostStringsColumn."""
    from cudf_amd.arrow_host import HostStringsColumn
    from oracle.pyoracle import copy_bitmask
    if col.size == 0:
        return HostStringsColumn(np.zeros(0, np.uint8), np.zeros(0, np.int32), None, 0, 0, 0)
    off = np.asarray(col.offsets).astype(np.int64)
    first, last = int(off[col.offset]), int(off[col.offset + col.size])
    data = bytes(np.ascontiguousarray(col.chars[first:last]))
    slots = normalize_flat(data, do_lower_case, special_tokens)
    pieces = [b"".join(s) for s in slots]
    sizes = np.array([len(p) for p in pieces], dtype=np.int64)
    prefix = np.concatenate([[0], np.cumsum(sizes)])
    out_off = prefix[off[col.offset: col.offset + col.size + 1] - first].astype(_offsets_dtype(prefix[-1]))
    chars = np.frombuffer(b"".join(pieces), dtype=np.uint8).copy()
    return HostStringsColumn(chars, out_off, copy_bitmask(col), col.size, 0, col.null_count)


_RULES = None


def rule_tables():
    """classify() of every code point as two arrays for oracle/nvtext_oracle.cpp: kind[cp] and lower[3 * cp + k]
    (the characters cp becomes when lower-casing, 0 = none).  Unassigned code points are all alike, so only the
    assigned ones go through classify()."""
    global _RULES
    if _RULES is None:
        kind = np.full(0x110000, PLAIN, np.uint8)
        lower = np.zeros((0x110000, 3), np.uint32)
        lower[:, 0] = np.arange(0x110000, dtype=np.uint32)
        plain_unassigned = classify(0x0378) == (PLAIN, [0x0378])  # an unassigned code point
        assert plain_unassigned
        for cp in range(0x110000):
            if unicodedata.category(chr(cp)) == "Cn" and not _cjk(cp):
                continue
            k, low = classify(cp)
            kind[cp] = k
            lower[cp, :] = 0
            lower[cp, :len(low)] = low
        _RULES = (kind, np.ascontiguousarray(lower.reshape(-1)))
    return _RULES


def normalize_characters_native(col, do_lower_case: bool, special_tokens: Sequence[bytes] = (), nthreads: int = 1):
    """normalize_characters through the C++ restatement in oracle/nvtext_oracle.cpp (same rules, from rule_tables()):
    for inputs too large for the loops above.  Tests hold the two against each other."""
    import ctypes as C
    from cudf_amd.arrow_host import HostStringsColumn
    from oracle import pyoracle
    if col.size == 0:
        return HostStringsColumn(np.zeros(0, np.uint8), np.zeros(0, np.int32), None, 0, 0, 0)
    kind, lower = rule_tables()
    tokens = sorted_special_tokens(special_tokens, do_lower_case)
    tok_chars = np.frombuffer(b"".join(tokens) or b"\0", dtype=np.uint8).copy()
    tok_off = np.concatenate([[0], np.cumsum([len(t) for t in tokens])]).astype(np.int32)
    keep, cargs = pyoracle._col_args(col)
    out_off = np.zeros(col.size + 1, np.int64)
    out_chars, out_bytes = C.c_void_p(), C.c_int64(0)
    rc = pyoracle.lib().oracle_normalize_characters(*cargs, pyoracle._p(kind), pyoracle._p(lower), int(bool(do_lower_case)),
                                                     pyoracle._p(tok_chars), pyoracle._p(tok_off), len(tokens), int(nthreads),
                                                     pyoracle._p(out_off), C.byref(out_chars), C.byref(out_bytes))
    if rc != pyoracle.OK:
        raise pyoracle.OracleError(rc)
    n = out_bytes.value
    chars = np.ctypeslib.as_array(C.cast(out_chars, C.POINTER(C.c_uint8)), shape=(max(n, 1),))[:n].copy()
    pyoracle.lib().oracle_free(out_chars)
    return HostStringsColumn(chars, out_off.astype(_offsets_dtype(n)), pyoracle.copy_bitmask(col), col.size, 0, col.null_count)


def normalize_ascii(col, do_lower_case: bool):
    """normalize_characters for a column whose bytes are all below 0x80, no special tokens: the same rules through a
    256-entry table and numpy, for inputs too large for the loops above.  Tests check it against
    normalize_characters on small inputs before relying on it."""
    from cudf_amd.arrow_host import HostStringsColumn
    from oracle.pyoracle import copy_bitmask
    table = np.zeros((128, 3), np.uint8)
    for cp in range(128):
        slots = normalize_flat(bytes([cp]), do_lower_case)[0]
        table[cp] = [s[0] if s else 0 for s in slots]
    off = np.asarray(col.offsets).astype(np.int64)
    first, last = int(off[col.offset]), int(off[col.offset + col.size])
    data = np.ascontiguousarray(col.chars[first:last])
    assert data.size == 0 or int(data.max()) < 0x80
    slots = table[data]                                   # (n, 3)
    keep = slots != 0
    prefix = np.concatenate([[0], np.cumsum(keep.sum(axis=1, dtype=np.int64))])
    out_off = prefix[off[col.offset: col.offset + col.size + 1] - first].astype(_offsets_dtype(prefix[-1]))
    return HostStringsColumn(slots[keep], out_off, copy_bitmask(col), col.size, 0, col.null_count)
