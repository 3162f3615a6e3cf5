"""Writes unicode_ranges.hpp beside this file: the code point ranges of the general categories L* (letters) and
N* (numbers) that the pre-tokeniser patterns of byte-pair vocabularies name as \\p{L} and \\p{N}, taken from the
Unicode database of the running Python (`unicodedata.unidata_version` goes into the header).

    python retrograd_amd/csrc/unicode_ranges.py
"""
from __future__ import annotations

import sys
import unicodedata
from pathlib import Path


def ranges(first_letter: str) -> list:
    out, start = [], None
    for cp in range(sys.maxunicode + 1):
        inside = unicodedata.category(chr(cp)).startswith(first_letter)
        if inside and start is None:
            start = cp
        elif not inside and start is not None:
            out.append((start, cp - 1))
            start = None
    if start is not None:
        out.append((start, sys.maxunicode))
    return out


def table(name: str, rs: list) -> str:
    rows = []
    for at in range(0, len(rs), 6):
        rows.append("    " + " ".join("{0x%04X, 0x%04X}," % r for r in rs[at:at + 6]))
    return "static const CodeRange %s[%d] = {\n%s\n};\n" % (name, len(rs), "\n".join(rows))


def main() -> None:
    text = (
        "// Code point ranges of the Unicode general categories L* and N* (Unicode %s).\n"
        "// Written by unicode_ranges.py beside this file; edit that, not this.\n"
        "#pragma once\n\n#include <cstdint>\n\nnamespace retro {\n\n"
        "struct CodeRange { uint32_t lo, hi; };\n\n%s\n%s\n}  // namespace retro\n"
    ) % (unicodedata.unidata_version, table("kUnicodeLetters", ranges("L")), table("kUnicodeNumbers", ranges("N")))
    Path(__file__).with_name("unicode_ranges.hpp").write_text(text)


if __name__ == "__main__":
    main()
