"""Writes tests/golden/bc_tables.json: SHA-256 digests of the constant tables of the reference's block
compressors, so that the checker's tables - which are regenerated from their rule (BC1 single-colour
endpoint pairs) or typed from the format specification (BC7 partitions and anchors) - can be compared
with the reference's where the reference itself is not present.  Only digests are stored.

  BC1: c_ColorMatch5bit / c_ColorMatch6bit, src/shaders/BlockCompressCommon.hlsli:40-78, 256 entries each
       as little-endian uint16.
  BC7: c_Partitions2_Subset0/1, c_Partitions3_Subset0/1/2 (bit t set = texel t belongs to the subset) and
       c_Partitions2_Anchor1, c_Partitions3_Anchor1/2, src/shaders/CompressBC7.hlsl:32-122; masks as
       little-endian uint32 [partition][subset], anchors as uint8 [table][partition].

Run here, where /root/reference is mounted:  python tests/golden/make_bc_table_digests.py"""
import hashlib
import json
import os
import re

import numpy as np

REFERENCE = "/root/reference/src/shaders"


def _array(text, name, count):
    body = re.search(name + r"\[%d\]\s*=\s*\{([^}]*)\}" % count, text).group(1)
    values = [int(v, 0) for v in re.findall(r"0x[0-9a-fA-F]+|\d+", body)]
    assert len(values) == count, (name, len(values))
    return values


def reference_bc1_tables(root=REFERENCE):
    text = open(os.path.join(root, "BlockCompressCommon.hlsli")).read()
    return [np.array(_array(text, name, 256), dtype="<u2") for name in ("c_ColorMatch5bit", "c_ColorMatch6bit")]


def reference_bc7_tables(root=REFERENCE):
    """(two[64][2], three[64][3], anchors[3][64])"""
    text = open(os.path.join(root, "CompressBC7.hlsl")).read()
    two = np.array([_array(text, "c_Partitions2_Subset%d" % s, 64) for s in range(2)], dtype="<u4").T.copy()
    three = np.array([_array(text, "c_Partitions3_Subset%d" % s, 64) for s in range(3)], dtype="<u4").T.copy()
    anchors = np.array([_array(text, name, 64) for name in ("c_Partitions2_Anchor1", "c_Partitions3_Anchor1", "c_Partitions3_Anchor2")], dtype=np.uint8)
    return two, three, anchors


def digest(array):
    return hashlib.sha256(np.ascontiguousarray(array).tobytes()).hexdigest()


if __name__ == "__main__":
    five, six = reference_bc1_tables()
    two, three, anchors = reference_bc7_tables()
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "bc_tables.json"), "w") as f:
        json.dump({"bc1": {"source": "src/shaders/BlockCompressCommon.hlsli:40-78", "sha256_five_bit": digest(five), "sha256_six_bit": digest(six)},
                   "bc7": {"source": "src/shaders/CompressBC7.hlsl:32-122", "sha256_two_subsets": digest(two), "sha256_three_subsets": digest(three),
                           "sha256_anchors": digest(anchors)}}, f, indent=1)
        f.write("\n")
