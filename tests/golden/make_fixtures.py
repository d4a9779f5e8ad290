#!/usr/bin/env python3
"""Extract the reference's known-answer tables into one JSON fixture file.

The reference keeps its hand-computed test vectors as C array initialisers in
``c/tests/test_*_buffers.h`` (one namespace per header; entries such as
``kF``, ``kG``, ``kH``, ``kNF``, ``kS`` ...; values written as ``a./b.``
rationals).  Both its C++ test mains (``c/tests/test_mcorrlcorr.cc:33-71``) and
its Python tests (``tests/test_mconv.py:25-65``) read those tables.  This
script reads the same headers *as text* and writes the numbers to
``tests/golden/reference_fixtures.json`` so that the vectors travel with this
repository while the headers do not.

Run from anywhere:  python tests/golden/make_fixtures.py [/path/to/reference]
Only data is copied: array names, integer parameters and float values.
"""
import json
import os
import re
import sys
from fractions import Fraction

HEADERS = [
    "mconv1d", "mcorr1d", "lconv1d", "lcorr1d", "mconvlconv", "mcorrlcorr",
    "snd2col", "col2snd", "lin2col", "col2lin", "spec2col", "col2spec",
]

_DECL = re.compile(r"const\s+(int|double)\s+(k[A-Za-z]+)\s*((?:\[[^\]]*\])*)\s*=")


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def _number(tok):
    tok = tok.strip()
    if "/" in tok:
        a, b = tok.split("/")
        return float(Fraction(a.strip().rstrip(".")) / Fraction(b.strip().rstrip(".")))
    return float(tok)


def _parse_braces(text, pos):
    """Parse a (possibly nested) brace initialiser starting at text[pos] == '{'."""
    assert text[pos] == "{"
    out, tok, pos = [], "", pos + 1
    while True:
        ch = text[pos]
        if ch == "{":
            sub, pos = _parse_braces(text, pos)
            out.append(sub)
            continue
        if ch in ",}":
            if tok.strip():
                out.append(_number(tok))
            tok = ""
            if ch == "}":
                return out, pos + 1
        else:
            tok += ch
        pos += 1


def parse_header(path):
    text = _strip_comments(open(path).read())
    entries = {}
    for m in _DECL.finditer(text):
        ctype, name, dims = m.groups()
        rest = text[m.end():].lstrip()
        if rest.startswith("{"):
            val, _ = _parse_braces(text, text.index("{", m.end()))
        else:
            val = _number(rest[: rest.index(";")])
        if ctype == "int":
            val = [int(v) for v in val] if isinstance(val, list) else int(val)
        entries[name] = val
    return entries


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    out = {}
    for name in HEADERS:
        path = os.path.join(ref, "c", "tests", "test_%s_buffers.h" % name)
        ent = parse_header(path)
        n = ent.pop("kNumTests")
        for key, val in ent.items():
            assert len(val) == n, (name, key, len(val), n)
        out[name] = {"num_tests": n, **ent}
        print("%-11s %2d cases, entries %s" % (name, n, sorted(ent)))
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_fixtures.json")
    with open(dst, "w") as fp:
        json.dump(out, fp, separators=(",", ":"))
        fp.write("\n")
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
