#!/usr/bin/env python3
"""Writes ojk_iq_grids.h: the codebooks of the GGUF grid formats (IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS, IQ3_S, IQ1_S /
IQ1_M) in packed form, and tests/golden/iq_grid_digests.json: an FNV-1a-64 of every codebook as its publisher spells
it (little-endian bytes of the u64 / u32 entries), which the test suite recomputes from the packed header.

The codebooks are constants of the file format (ggml-common.h: iq2xxs_grid, iq2xs_grid, iq2s_grid, iq3xxs_grid,
iq3s_grid, iq1s_grid); the reference carries them at crates/ojas-core/src/iq_tables.rs:28-622.  Every entry is a
short vector over a tiny alphabet, so an entry packs into 16 bits:

    IQ2_XXS / IQ2_XS / IQ2_S   8 magnitudes from {8, 25, 43}            digit j (0..2) in bits 2j
    IQ1_S (and IQ1_M)          8 values from {-1, 0, +1}                digit j = value + 1 in bits 2j
    IQ3_XXS                    4 magnitudes from {4, 12, .., 52, 62}    level j (0..7) in bits 3j
    IQ3_S                      4 magnitudes from {1, 3, .., 15}         level j (0..7) in bits 3j

which is an eighth to a quarter of the published size (11.5 KB for all six instead of 59 KB) — small enough that a
workgroup expands the table it needs into LDS, or decodes an entry with two v_perm_b32 against a register-held
alphabet.  Usage:  make_iq_grids.py <file with the published tables, C or Rust syntax>
"""
import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.abspath(os.path.join(HERE, "..", "..", ".."))

TABLES = {  # published name -> (our name, entries, bytes per entry, alphabet, bits per digit)
    "iq2xxs_grid": ("iq2xxs", 256, 8, [8, 25, 43], 2),
    "iq2xs_grid": ("iq2xs", 512, 8, [8, 25, 43], 2),
    "iq2s_grid": ("iq2s", 1024, 8, [8, 25, 43], 2),
    "iq3xxs_grid": ("iq3xxs", 256, 4, [4, 12, 20, 28, 36, 44, 52, 62], 3),
    "iq3s_grid": ("iq3s", 512, 4, [1, 3, 5, 7, 9, 11, 13, 15], 3),
    "iq1s_grid": ("iq1s", 2048, 8, [0xFF, 0x00, 0x01], 2),
}


def fnv1a64(data: bytes) -> int:
    h = 0xCBF29CE484222325
    for b in data:
        h = ((h ^ b) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def published(text: str, name: str, entries: int):
    m = re.search(r"\b%s\b[^=;{\[]*(?::\s*\[[^\]]*\])?\s*(?:\[[^\]]*\])?\s*=\s*[\[{](.*?)[\]}]\s*;" % name, text, re.S | re.I)
    if not m:
        raise SystemExit("table %s not found" % name)
    vals = [int(v, 0) for v in re.findall(r"0x[0-9a-fA-F]+|\d+", m.group(1))]
    if len(vals) != entries:
        raise SystemExit("table %s: %d entries, expected %d" % (name, len(vals), entries))
    return vals


def main():
    if len(sys.argv) != 2:
        raise SystemExit(__doc__)
    text = open(sys.argv[1]).read()
    digests, out = {}, []
    out.append("// Codebooks of the GGUF grid formats in packed form: one 16-bit word per entry, digit j of an entry in bits\n"
               "// 2j (alphabets of three: IQ2_* magnitudes {8, 25, 43}; IQ1_* values {-1, 0, +1}) or 3j (alphabets of eight:\n"
               "// IQ3_XXS magnitudes {4, 12, .., 52, 62}; IQ3_S magnitudes {1, 3, .., 15}).  Written by make_iq_grids.py from\n"
               "// the tables the format's publisher ships (ggml-common.h; the reference: crates/ojas-core/src/iq_tables.rs:28-622).\n"
               "// Plain C and HIP both include this file; OJK_GRID_CONST names the storage class.\n"
               "#pragma once\n#ifndef OJK_GRID_CONST\n#define OJK_GRID_CONST static const\n#endif\n")
    for pub, (ours, entries, nb, alphabet, bits) in TABLES.items():
        vals = published(text, pub.upper() if pub.upper() in text else pub, entries)
        raw = b"".join(v.to_bytes(nb, "little") for v in vals)
        digests[ours] = {"entries": entries, "entry_bytes": nb, "fnv1a64": "0x%016x" % fnv1a64(raw)}
        packed = []
        for v in vals:
            word = 0
            for j in range(nb):
                word |= alphabet.index((v >> (8 * j)) & 0xFF) << (bits * j)
            assert word < 65536
            packed.append(word)
        out.append("OJK_GRID_CONST unsigned short ojk_%s_grid_pk[%d] = {" % (ours, entries))
        for i in range(0, entries, 16):
            out.append("    " + ", ".join("0x%04x" % p for p in packed[i:i + 16]) + ",")
        out.append("};\n")
    open(os.path.join(HERE, "ojk_iq_grids.h"), "w").write("\n".join(out))
    json.dump({"about": "FNV-1a-64 over the little-endian bytes of each published codebook (u64 or u32 entries in order); "
                        "written by ojas-engine_amd/csrc/kernels/make_iq_grids.py", "tables": digests},
              open(os.path.join(ROOT, "tests", "golden", "iq_grid_digests.json"), "w"), indent=1)
    print("wrote ojk_iq_grids.h and tests/golden/iq_grid_digests.json")


if __name__ == "__main__":
    main()
