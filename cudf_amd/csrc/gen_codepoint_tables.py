#!/usr/bin/env python3
"""Generates codepoint_tables.inc: the per-code-point data of nvtext::normalize_characters.

The reference ships these tables as generated data (cpp/src/text/detail/codepoint_metadata.ah, read by
cpp/src/text/normalize.cu:131-186); they encode the BERT basic-tokenizer rules.  This script derives the
same information from the Unicode character database of the Python that runs it:

  entry(cp) = category << 24 | multi << 23 | replacement
    category 0  pad with spaces                (punctuation, CJK ideographs)
             1  pad with spaces when lower-casing (the lower-cased, accent-stripped form is punctuation)
             2  remove                          (control and format characters, U+0000, U+FFFD)
             3  remove when lower-casing        (nonspacing marks: the accents)
             4  replace always                  (whitespace -> U+0020)
             5  none of these
    replacement = first code point of lower(cp) decomposed (NFD) with the nonspacing marks dropped, 0 if
                  that is cp itself; multi = the result has two or three code points, the others are in the
                  second table as (second << 32 | third).

Only entries that differ from the default (category 5, no replacement) are written, as runs
(first code point, count, value) of equal values; the library expands them into dense arrays when a
normalizer is created.  The precomposed Hangul syllables are left out: their entries follow from arithmetic.  A third table holds the lower-case mapping of the Basic Multilingual Plane
(cpp/src/strings/case.cu:142-148 converts no code point above U+FFFF), which the library applies to the
special tokens of a lower-casing normalizer (cpp/src/text/normalize.cu:232-235).

The reference's tables were generated from Unicode 11.  Code points that Unicode 12.0 - 13.0 added with
properties that matter here are listed in ASSIGNED_AFTER_UNICODE_11 and keep the default entry, so that
the behaviour is the same for every code point (checked against the reference's tables when this was
written: no other entry differs in category, replacement or second-table value).
"""
import sys
import unicodedata

DEFAULT = 5 << 24

ASSIGNED_AFTER_UNICODE_11 = frozenset([
    0x0B55, 0x0C77, 0x0D81, 0x0EBA, 0x1ABF, 0x1AC0, 0x2E4F, 0x2E52,
    0xA7BA, 0xA7BC, 0xA7BE, 0xA7C2, 0xA7C4, 0xA7C5, 0xA7C6, 0xA7C7, 0xA7C9, 0xA7F5, 0xA82C, 0xA9BD,
    0x10EAB, 0x10EAC, 0x10EAD, 0x111CF, 0x1145A, 0x11938, 0x1193B, 0x1193C, 0x1193E, 0x11943, 0x11944, 0x11945, 0x11946,
    0x119D4, 0x119D5, 0x119D6, 0x119D7, 0x119DA, 0x119DB, 0x119E0, 0x119E2, 0x11FFF,
    0x13430, 0x13431, 0x13432, 0x13433, 0x13434, 0x13435, 0x13436, 0x13437, 0x13438,
    0x16F4F, 0x16FE2, 0x16FE4, 0x1E130, 0x1E131, 0x1E132, 0x1E133, 0x1E134, 0x1E135, 0x1E136,
    0x1E2EC, 0x1E2ED, 0x1E2EE, 0x1E2EF,
])
# U+166D CANADIAN SYLLABICS CHI SIGN was punctuation (Po) until Unicode 12 made it a symbol (So).
PUNCTUATION_IN_UNICODE_11 = frozenset([0x166D])


def is_cjk(cp):
    """The ranges of BERT's _is_chinese_char."""
    return ((0x4E00 <= cp <= 0x9FFF) or (0x3400 <= cp <= 0x4DBF) or (0x20000 <= cp <= 0x2A6DF) or (0x2A700 <= cp <= 0x2B73F)
            or (0x2B740 <= cp <= 0x2B81F) or (0x2B820 <= cp <= 0x2CEAF) or (0xF900 <= cp <= 0xFAFF) or (0x2F800 <= cp <= 0x2FA1F))


def is_punctuation(cp):
    """BERT's _is_punctuation: the ASCII symbol ranges and every P* category."""
    if (33 <= cp <= 47) or (58 <= cp <= 64) or (91 <= cp <= 96) or (123 <= cp <= 126) or cp in PUNCTUATION_IN_UNICODE_11:
        return True
    return unicodedata.category(chr(cp)).startswith("P")


def entry(cp):
    """(first-table value, second-table value) of a code point."""
    if cp in ASSIGNED_AFTER_UNICODE_11:
        return DEFAULT, 0
    if 0xD800 <= cp <= 0xDFFF:
        return DEFAULT, 0
    ch = chr(cp)
    cat = unicodedata.category(ch)
    if ch in "\t\n\r" or cat in ("Zs", "Zl", "Zp"):
        return (4 << 24) | 0x20, 0
    if cat in ("Cc", "Cf") or cp == 0 or cp == 0xFFFD:
        return 2 << 24, 0
    if cat == "Mn":
        return (3 << 24) | 0x20, 0
    rest = [ord(c) for c in unicodedata.normalize("NFD", ch.lower()) if unicodedata.category(c) != "Mn"]
    new, multi, second = 0, 0, 0
    if rest and rest != [cp]:
        new = rest[0]
        if len(rest) > 1:
            multi = 1
            second = (rest[1] << 32) | (rest[2] if len(rest) > 2 else 0)
            assert len(rest) <= 3, hex(cp)
    token_cat = 5
    if new and is_punctuation(new):
        token_cat = 1
    if is_punctuation(cp) or is_cjk(cp):
        token_cat = 0
    return (token_cat << 24) | (multi << 23) | new, second


def hangul(cp):
    """entry() of a precomposed Hangul syllable from its arithmetic decomposition (The Unicode Standard, 3.12):
    the library computes these 11172 entries instead of reading them from the tables."""
    s = cp - 0xAC00
    lead, vowel, trail = 0x1100 + s // 588, 0x1161 + (s % 588) // 28, s % 28
    return (5 << 24) | (1 << 23) | lead, (vowel << 32) | (0x11A7 + trail if trail else 0)


def tables():
    """(runs of the first table, entries of the second table), Hangul syllables left out."""
    runs, second = [], []
    for cp in range(0x110000):
        v, a = entry(cp)
        if 0xAC00 <= cp <= 0xD7A3:
            assert (v, a) == hangul(cp), hex(cp)
            continue
        if v != DEFAULT:
            if runs and runs[-1][2] == v and runs[-1][0] + runs[-1][1] == cp:
                runs[-1][1] += 1
            else:
                runs.append([cp, 1, v])
        if a:
            second.append((cp, a))
    return [tuple(r) for r in runs], second


def lower_map():
    """(code point, up to three code points of its lower-case form) for the BMP characters that have one."""
    out = []
    for cp in range(0x10000):
        if 0xD800 <= cp <= 0xDFFF:
            continue
        low = [ord(c) for c in chr(cp).lower()]
        if low != [cp]:
            assert len(low) <= 3, hex(cp)
            out.append((cp, low[0], low[1] if len(low) > 1 else 0, low[2] if len(low) > 2 else 0))
    return out


def main(path):
    first, second = tables()
    with open(path, "w") as f:
        f.write("// Generated by gen_codepoint_tables.py from Unicode %s; do not edit.\n" % unicodedata.unidata_version)
        f.write("// (first code point, count, entry) for every run of the first table that differs from the default 0x%08X\n" % DEFAULT)
        f.write("static const uint32_t kCodepointRuns[][3] = {\n")
        for i in range(0, len(first), 5):
            f.write("".join("{0x%X,%d,0x%X}," % p for p in first[i:i + 5]) + "\n")
        f.write("};\n// (code point, second << 32 | third) for every multi-code-point replacement\n")
        f.write("static const uint64_t kCodepointSecond[][2] = {\n")
        for i in range(0, len(second), 4):
            f.write("".join("{0x%X,0x%XULL}," % p for p in second[i:i + 4]) + "\n")
        f.write("};\n// (code point, lower-case form: up to three code points) for the BMP\n")
        f.write("static const uint32_t kLowerCase[][4] = {\n")
        lower = lower_map()
        for i in range(0, len(lower), 5):
            f.write("".join("{0x%X,0x%X,0x%X,0x%X}," % p for p in lower[i:i + 5]) + "\n")
        f.write("};\n")
    print("%s: %d runs, %d multi-code-point replacements, %d lower-case mappings (Unicode %s)"
          % (path, len(first), len(second), len(lower), unicodedata.unidata_version))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "codepoint_tables.inc")
