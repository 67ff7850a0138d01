#!/usr/bin/env python3
"""Writes tests/golden/ref_layout.json and ref_geometry.json from the reference's OWN host
code (oracle/_ref/libntc_ref_host.so = src/WeightLayout.cpp + src/FeatureGridMath.cpp of
LibNTC 0.9.2, compiled by oracle/Makefile).  Run in a container that has the reference tree:

    make -C oracle && python tests/golden/make_ref_fixtures.py

The fixtures are data only (offsets, sizes, grid dimensions); they let the layout and
geometry checks run where the reference tree is absent.
"""
import ctypes as C
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle_lib  # noqa: E402

CASES = [(4096, 4096, 13, 2), (4096, 4096, 13, 4), (2048, 1024, 12, 3), (1000, 600, 10, 5), (512, 512, 1, 1),
         (64, 64, 7, 6), (8192, 8192, 14, 2), (300, 200, 4, 2), (16, 16, 5, 4), (2048, 2048, 12, 1), (4096, 2048, 1, 2)]


def main():
    ref = oracle_lib.load_ref()
    if ref is None:
        sys.exit("oracle/_ref/libntc_ref_host.so is not built")
    layout = {}
    for name, weight_type in (("GenericInt8", 1), ("GenericFP8", 2)):
        out = (C.c_uint64 * 25)()
        assert ref.ntc_ref_weight_layout(weight_type, out) == 0
        layout[name] = {
            "weightOffset": list(out[0:4]), "scaleOffset": list(out[4:8]), "biasOffset": list(out[8:12]),
            "bufferSize": out[12], "weightSize": list(out[13:17]), "scaleSize": list(out[17:21]), "biasSize": list(out[21:25]),
        }
    geo = (C.c_int * 8)()
    ref.ntc_ref_mlp_geometry(geo)
    layout["mlp"] = {"layerInputs": [geo[2 * i] for i in range(4)], "layerOutputs": [geo[2 * i + 1] for i in range(4)]}
    with open(os.path.join(HERE, "ref_layout.json"), "w") as f:
        json.dump(layout, f, indent=1)

    cases = []
    for (w, h, mips, gs) in CASES:
        n = min(ref.ntc_ref_num_neural_mips(w, h, gs), ref.ntc_ref_lod_to_neural_lod(mips - 1, gs, 8) + 2)
        nlods = [ref.ntc_ref_lod_to_neural_lod(m, gs, n) for m in range(mips)]
        cases.append({
            "width": w, "height": h, "mips": mips, "gridSizeScale": gs, "numNeuralMips": n,
            "neuralLod": nlods,
            "hrDims": [[ref.ntc_ref_grid_dimension(w, nl, gs), ref.ntc_ref_grid_dimension(h, nl, gs)] for nl in nlods],
            "latentBytes16": ref.ntc_ref_quantized_latents_size(w, h, mips, gs, 16),
            "latentBytes8": ref.ntc_ref_quantized_latents_size(w, h, mips, gs, 8),
        })
    with open(os.path.join(HERE, "ref_geometry.json"), "w") as f:
        json.dump({"cases": cases}, f, indent=1)
    print("wrote ref_layout.json, ref_geometry.json")


if __name__ == "__main__":
    main()
