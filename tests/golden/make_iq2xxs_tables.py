#!/usr/bin/env python3
"""Write tests/golden/iq2xxs_tables.json from the reference's three copies of the
IQ2_XXS codebook, read as text (nothing of the reference is executed).

The three copies are src/iquant.lisp:25-114 (#x... literals and the decimal
ksigns list), src/cuda/ds4f.cu:656-731 and src/metal/ds4f.metal:20-86
(0x...ULL literals).  All three must agree before the fixture is written.

Run in the build container only:  python tests/golden/make_iq2xxs_tables.py
"""
import json
import os
import re
import sys

REF = os.environ.get("ILLATIO_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))


def lisp_tables(path):
    text = open(path).read()
    gstart = text.index("+iq2xxs-grid+")
    gend = text.index("+ksigns-iq2xs+")
    grid = [int(h, 16) for h in re.findall(r"#x([0-9a-fA-F]{16})", text[gstart:gend])]
    send = text.index("+iq2xxs-signs+", gend)
    body = text[gend:send]
    body = body[body.index(":initial-contents"):]
    signs = [int(d) for d in re.findall(r"\b(\d{1,3})\b", body)]
    return grid, signs


def c_tables(path):
    text = open(path).read()
    grid = [int(h, 16) for h in re.findall(r"0x([0-9a-fA-F]{16})(?:ULL|ull|UL|ul)?", text)]
    # the grid is the first run of 256 sixteen-digit literals
    grid = grid[:256]
    m = re.search(r"ksigns[^=]*=\s*\{([^}]*)\}", text, re.S)
    signs = [int(x, 0) for x in re.findall(r"0x[0-9a-fA-F]+|\b\d+\b", m.group(1))] if m else None
    return grid, signs


def main():
    lg, ls = lisp_tables(os.path.join(REF, "src/iquant.lisp"))
    assert len(lg) == 256 and len(ls) == 128, (len(lg), len(ls))
    for rel in ("src/cuda/ds4f.cu", "src/metal/ds4f.metal"):
        cg, cs = c_tables(os.path.join(REF, rel))
        assert cg == lg, f"grid differs in {rel}"
        if cs is not None:
            assert cs[:128] == ls, f"ksigns differs in {rel}"
    out = {"source": "modus-lisp/illatio src/iquant.lisp:25-114 (= src/cuda/ds4f.cu:656-731 = src/metal/ds4f.metal:20-86)",
           "iq2xxs_grid": [f"{g:016x}" for g in lg], "ksigns_iq2xs": ls}
    with open(os.path.join(HERE, "iq2xxs_tables.json"), "w") as f:
        json.dump(out, f, indent=0)
    print("wrote iq2xxs_tables.json:", len(lg), "grid entries,", len(ls), "sign patterns")


if __name__ == "__main__":
    sys.exit(main())
