"""Writes tests/golden/bc1_match_tables.json: SHA-256 digests of the two single-colour endpoint
tables of the reference's BC1 encoder (c_ColorMatch5bit / c_ColorMatch6bit,
src/shaders/BlockCompressCommon.hlsli:40-78), each taken over its 256 entries as little-endian
uint16.  The tables themselves are not stored: the checker regenerates them from their published
rule and the test compares digests (and the literal values, where the reference is present).

Run here, where /root/reference is mounted:  python tests/golden/make_bc1_table_digest.py"""
import hashlib
import json
import os
import re

import numpy as np

REFERENCE = "/root/reference/src/shaders/BlockCompressCommon.hlsli"


def reference_tables(path=REFERENCE):
    text = open(path).read()
    out = []
    for name in ("c_ColorMatch5bit", "c_ColorMatch6bit"):
        body = re.search(name + r"\[256\]\s*=\s*\{([^}]*)\}", text).group(1)
        values = [int(v, 16) for v in re.findall(r"0x[0-9a-fA-F]+", body)]
        assert len(values) == 256
        out.append(np.array(values, dtype="<u2"))
    return out


def digest(table):
    return hashlib.sha256(np.asarray(table, dtype="<u2").tobytes()).hexdigest()


if __name__ == "__main__":
    five, six = reference_tables()
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "bc1_match_tables.json"), "w") as f:
        json.dump({"source": "src/shaders/BlockCompressCommon.hlsli:40-78", "sha256_five_bit": digest(five), "sha256_six_bit": digest(six)}, f, indent=1)
        f.write("\n")
