#!/usr/bin/env python3
"""Writes tests/golden/ntex_reference_json.json: the JSON chunk of a small NTC file after a round
trip through the reference's OWN parser and serialiser (oracle/_ref/libntc_ref_file.so =
src/JsonFileFormat.cpp + src/JsonSerialization.cpp of LibNTC 0.9.2, compiled by oracle/Makefile).
Run in a container that has the reference tree:

    make -C oracle && python tests/golden/make_ntex_fixture.py

The fixture is data only (one JSON text); it lets the loader test run against the reference's
spelling of a document where the reference tree is absent.
"""
import ctypes as C
import importlib
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import ntex_writer as nw  # noqa: E402
import test_ntc_file as t  # noqa: E402


def main():
    lib = t.ref_file_lib()
    if lib is None:
        sys.exit("oracle/_ref/libntc_ref_file.so is not built")
    ntc = importlib.import_module("rtxntc-library_amd")
    case = t.make_case(ntc)
    data = t.file_of(case, 64, 32, 2, 8, 8, textures=t.TEXTURES, channel_color_spaces=["sRGB"] * 3 + [None] * 5)
    text, _ = nw.split_container(data)
    out, err = C.create_string_buffer(1 << 16), C.create_string_buffer(1024)
    rc = lib.ntc_ref_reserialize_json(text.encode(), out, 1 << 16, err, 1024)
    if rc != 0:
        sys.exit(f"reference parser/serialiser failed ({rc}): {err.value.decode()}")
    with open(os.path.join(HERE, "ntex_reference_json.json"), "w") as f:
        json.dump({"source": "json::SerializeDocument(json::ParseDocument(writer output)), LibNTC 0.9.2",
                   "reference_json": out.value.decode()}, f, indent=1)
    print("wrote ntex_reference_json.json,", len(out.value), "bytes of JSON")


if __name__ == "__main__":
    main()
