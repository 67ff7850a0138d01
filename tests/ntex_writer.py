"""Writer of NTC texture-set files ("NTEX" containers) for the loader tests.

Test infrastructure.  Written from the container description in the reference
(src/JsonFileFormat.h:26-218 for the header and the JSON schema, src/TextureSet.cpp:498-716 and
src/BinaryChunkBuilder.cpp:56-191 for the order and alignment of the views): a 40-byte header,
the JSON chunk with a terminating zero, padding to 4 bytes, then the binary chunk in which every
view starts on a 4-byte boundary.  The reference's own loader front end (oracle/_ref) accepts
these files; tests/test_ntc_file.py checks that.
"""
import json
import math
import struct

import numpy as np

SIGNATURE = 0x5845544E
CONTAINER_VERSION = 0x100
SCHEMA_VERSION = 3
SHARED_MIPS = [2, 3, 3, 3, 4, 4]
LAYER_WIDTHS_092 = [(48, 64), (64, 48), (48, 32), (32, 16)]     # include/libntc/shaders/InferenceConstants.h:26-40


def lod_to_neural(lod, grid_scale, neural_lods):
    return max(0, min((lod - SHARED_MIPS[grid_scale - 1] + 2) & ~1, neural_lods - 2))


def grid_dim(dim, nlod, grid_scale):
    return max((dim // grid_scale) >> nlod, 1)


def neural_lod_count(width, height, mips, grid_scale):
    min_grid = int(np.float32(min(width, height)) / np.float32(grid_scale))
    count = max(2, int(1.0 + math.floor(math.log2(min_grid)))) & ~1
    return min(count, lod_to_neural(mips - 1, grid_scale, 8) + 2)


class ViewTable:
    def __init__(self):
        self.views, self.chunks, self.size = [], [], 0

    def add(self, data, extra=None):
        data = bytes(data)
        view = {"offset": self.size, "storedSize": len(data)}
        if extra:
            view.update(extra)
        self.views.append(view)
        self.chunks.append(data + b"\0" * (-len(data) % 4))
        self.size += len(self.chunks[-1])
        return len(self.views) - 1

    def blob(self):
        return b"".join(self.chunks)


def split_int8_blob(blob, widths=LAYER_WIDTHS_092):
    """(weights, scales, biases) per layer from a GenericInt8 blob (src/WeightLayout.cpp:42-49)."""
    blob = np.asarray(blob, dtype=np.uint8)
    w_sizes = [i * o for i, o in widths]
    outs = [o for _, o in widths]
    at = 0
    weights, scales, biases = [], [], []
    for n in w_sizes:
        weights.append(blob[at: at + n]); at += n
    for o in outs:
        scales.append(blob[at: at + 4 * o]); at += 4 * o
    for o in outs:
        biases.append(blob[at: at + 4 * o]); at += 4 * o
    assert at == blob.size
    return weights, scales, biases


def split_fp8_blob(blob, widths=LAYER_WIDTHS_092):
    """(weights per layer, output-layer scales, biases per layer) from a GenericFP8 blob (src/WeightLayout.cpp:51-71):
    all matrices, then the fp16 biases of the three e4m3 layers, then the output layer's fp32 scales and int32 biases."""
    blob = np.asarray(blob, dtype=np.uint8)
    at = 0
    weights, biases = [], []
    for i, o in widths:
        weights.append(blob[at: at + i * o]); at += i * o
    for _, o in widths[:-1]:
        biases.append(blob[at: at + 2 * o]); at += 2 * o
    out = widths[-1][1]
    scales = blob[at: at + 4 * out]; at += 4 * out
    biases.append(blob[at: at + 4 * out]); at += 4 * out
    assert at == blob.size
    return weights, scales, biases


def write_ntex(width, height, channels, mips, grid_scale, features, latents, int8_blob, textures=(),
               fp8_version=True, fp8_blob=None, layer_widths=None, layer_data=None, channel_color_spaces=None,
               extra_document_fields=None, mutate=None, json_indent=None, mode_buffers=()):
    """Returns the bytes of an NTC file.

    latents: the quantised latent buffer, u16 layers neural LOD after neural LOD.
    int8_blob: GenericInt8 blob for the 48-64-48-32-16 network (ignored when layer_data is given).
    layer_widths / layer_data: store narrower hidden layers: widths [(in, out)] x 4 and
        data [(weights int8 [out, in], scales f32 [out], biases i32 [out])] x 4.
    mutate(document): last-minute edits of the JSON document (for malformed-file tests).
    mode_buffers: BC7 mode maps to store: (texture index, mip level, bytes, extra view fields or None).
    """
    latents = np.ascontiguousarray(latents).view(np.uint8)
    table = ViewTable()
    widths = layer_widths or LAYER_WIDTHS_092
    if layer_data is None:
        w, s, b = split_int8_blob(int8_blob)
        layer_data = list(zip(w, s, b))
    int8_layers = []
    for (n_in, n_out), (w, s, b) in zip(widths, layer_data):
        int8_layers.append({
            "inputChannels": n_in, "outputChannels": n_out,
            "weightView": table.add(np.ascontiguousarray(w).view(np.uint8)),
            "scaleView": table.add(np.ascontiguousarray(s).view(np.uint8)),
            "biasView": table.add(np.ascontiguousarray(b).view(np.uint8)),
            "weightType": "Int8", "scaleType": "Float32", "biasType": "Int32"})
    versions = [{"layers": int8_layers, "activation": "HGELUClamp", "weightLayout": "RowMajor"}]
    if fp8_version:   # e4m3 hidden layers with fp16 biases and no scales; int8 output layer (src/TextureSet.cpp:561-590)
        rng = np.random.default_rng(7)
        fp8_layers = []
        # the pieces of a GenericFP8 blob (src/WeightLayout.cpp:51-71) when one is given, else arbitrary bytes
        pieces = split_fp8_blob(fp8_blob) if fp8_blob is not None else None
        for index, (n_in, n_out) in enumerate(LAYER_WIDTHS_092):
            last = index == 3
            weights = pieces[0][index] if pieces else rng.integers(0, 120, n_in * n_out, dtype=np.uint8)
            layer = {"inputChannels": n_in, "outputChannels": n_out, "weightView": table.add(weights)}
            if last:
                scales = pieces[1] if pieces else np.ones(n_out, np.float32).view(np.uint8)
                layer.update({"weightType": "Int8", "scaleType": "Float32", "biasType": "Int32", "scaleView": table.add(scales)})
            else:
                layer.update({"weightType": "FloatE4M3", "biasType": "Float16"})
            layer["biasView"] = table.add(pieces[2][index] if pieces else np.zeros(n_out, np.int32 if last else np.float16).view(np.uint8))
            fp8_layers.append(layer)
        versions.append({"layers": fp8_layers, "activation": "HGELUClamp", "weightLayout": "RowMajor"})

    layers = (features + 3) // 4
    neural_lods = neural_lod_count(width, height, mips, grid_scale)
    latent_images, at = [], 0
    for nlod in range(neural_lods):
        gw, gh = grid_dim(width, nlod, grid_scale), grid_dim(height, nlod, grid_scale)
        views = []
        for _ in range(layers):
            views.append(table.add(latents[at: at + gw * gh * 2]))
            at += gw * gh * 2
        latent_images.append({"width": gw, "height": gh, "layerViews": views})
    assert at == latents.size, (at, latents.size)

    color_mips = []
    for m in range(mips):
        nlod = lod_to_neural(m, grid_scale, neural_lods)
        mw, mh = max(width >> m, 1), max(height >> m, 1)
        scale = np.float32(0.5) * max(np.float32(grid_dim(width, nlod, grid_scale)) / np.float32(mw),
                                      np.float32(grid_dim(height, nlod, grid_scale)) / np.float32(mh))
        lod = max(-1.0, min(1.0, 0.25 * math.log2(float(scale))))
        color_mips.append({"width": mw, "height": mh, "latentMip": nlod, "positionLod": lod, "positionScale": float(scale)})

    textures = [dict(t) for t in textures]
    for texture_index, mip_level, data, extra in mode_buffers:
        textures[texture_index].setdefault("bcModeBuffers", []).append({"mipLevel": mip_level, "view": table.add(data, extra)})

    document = {
        "schemaVersion": SCHEMA_VERSION, "width": width, "height": height, "numChannels": channels, "numColorMips": mips,
        "latentShape": {"numFeatures": features},
        "mlpVersions": versions,
        "textures": [dict(t) for t in textures],
        "channels": [({"colorSpace": cs} if cs else {}) for cs in (channel_color_spaces or [None] * channels)],
        "latents": latent_images,
        "colorMips": color_mips,
    }
    if extra_document_fields:
        document.update(extra_document_fields)
    document["views"] = table.views
    if mutate:
        mutate(document)
    return pack_container(json.dumps(document, indent=json_indent), table.blob())


def pack_container(json_text, binary, signature=SIGNATURE, version=CONTAINER_VERSION, binary_size=None):
    text = json_text.encode("ascii") + b"\0"
    json_offset = 40
    binary_offset = (json_offset + len(text) + 3) & ~3
    header = struct.pack("<IIQQQQ", signature, version, json_offset, len(text), binary_offset,
                         len(binary) if binary_size is None else binary_size)
    return header + text + b"\0" * (binary_offset - json_offset - len(text)) + binary


def split_container(data):
    """(json text, binary chunk) of a file written by pack_container."""
    _, _, json_offset, json_size, binary_offset, binary_size = struct.unpack("<IIQQQQ", data[:40])
    return data[json_offset: json_offset + json_size - 1].decode("ascii"), data[binary_offset: binary_offset + binary_size]
