#!/usr/bin/env python3
"""Writes codepoint_behaviour_digests.json from the reference's generated tables.

The reference keeps what normalize_characters does with each code point in numeric tables
(cpp/src/text/detail/codepoint_metadata.ah, read by cpp/src/text/normalize.cu:131-186).  This script reads
those numbers, reduces every code point to what the normalizer's output depends on

    (category, multi, replacement, second << 32 | third)      -- replacement and the rest zeroed where the
                                                                  category removes the character

and stores one 64-bit digest per block of 4096 code points.  Tests rebuild the same digests from the rules
the oracle and the library's table generator are written from, so a wrong rule for any code point shows.

Run where the reference tree is present:  python tests/golden/digest_codepoint_metadata.py /root/reference
"""
import hashlib
import json
import os
import re
import struct
import sys

BLOCK = 4096
LIMIT = 0x110000
DEFAULT = 5 << 24


def canonical(cat, multi, new, aux):
    if cat in (2, 3):          # removed (always, or when lower-casing; kept as it is otherwise)
        return cat, 0, 0, 0
    return cat, multi, new, aux if multi else 0


def digests(entries):
    """entries: iterable over all code points of canonical tuples."""
    out, h = [], hashlib.sha256()
    for cp, e in enumerate(entries):
        h.update(struct.pack("<BBIQ", *e))
        if (cp + 1) % BLOCK == 0:
            out.append(h.hexdigest()[:16])
            h = hashlib.sha256()
    return out


def reference_entries(root):
    src = open(os.path.join(root, "cpp/src/text/detail/codepoint_metadata.ah")).read()

    def numbers(name):
        m = re.search(name + r"\[\]\s*=\s*\{(.*?)\};", src, re.S)
        return [int(x) for x in re.findall(r"\d+", m.group(1))]

    meta, tail = numbers("codepoint_metadata"), numbers("cp_metadata_917505_917999")
    aux = {0: numbers("aux_codepoint_data"), 44032: numbers("aux_cp_data_44032_55203"),
           70475: numbers("aux_cp_data_70475_71099"), 119134: numbers("aux_cp_data_119134_119232")}
    for cp in range(LIMIT):
        v = meta[cp] if cp < len(meta) else tail[cp - 917505] if 917505 <= cp <= 917999 else DEFAULT
        a = 0
        for lo, vals in aux.items():
            if lo <= cp < lo + len(vals):
                a = vals[cp - lo]
        yield canonical((v >> 24) & 7, (v >> 23) & 1, v & 0x1FFFFF, a)


if __name__ == "__main__":
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    here = os.path.dirname(os.path.abspath(__file__))
    doc = {"about": "sha256[:16] per block of 4096 code points over struct.pack('<BBIQ', category, multi, replacement, "
                    "second<<32|third) of the reference's normalizer tables; made by digest_codepoint_metadata.py",
           "block": BLOCK, "digests": digests(reference_entries(root))}
    json.dump(doc, open(os.path.join(here, "codepoint_behaviour_digests.json"), "w"), indent=0)
    print(len(doc["digests"]), "blocks")
