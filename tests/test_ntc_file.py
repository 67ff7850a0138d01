"""Loading NTC files ("NTEX" containers) through the C++ host layer.

What pins what:
 * tests/ntex_writer.py is checked against the REFERENCE'S OWN loader front end where that was
   built (oracle/_ref/libntc_ref_file.so: LoadFileHeadersFromStream + DeserializeTextureSetDesc +
   the JSON parser/serialiser of LibNTC, compiled from the reference tree): its files are accepted
   and yield the same descriptor and latent shape the host layer derives; malformed variants are
   refused with the same status by both.
 * tests/golden/ntex_reference_json.json holds a JSON chunk as the reference's serialiser writes
   it (made by tests/golden/make_ntex_fixture.py); the host layer loads a file built around it.
 * End to end on the GPU: file -> CreateCompressedTextureSetFromMemory -> Decompress -> ReadChannels
   equals the CPU checker on the same latents and weights.
"""
import ctypes as C
import json
import os
import struct

import numpy as np
import pytest

import ntex_writer as nw
import oracle_lib
from cases import ref_case
from test_host_api import run_exe

HERE = os.path.dirname(os.path.abspath(__file__))
REF_FILE_LIB = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "libntc_ref_file.so")
STATUS = {"Ok": 0, "CudaUnavailable": 3, "FileUnavailable": 4, "FileUnrecognized": 5, "FileIncompatible": 6, "Unsupported": 8,
          "IOError": 13, "OutOfRange": 16}

TEXTURES = [
    {"name": "albedo", "firstChannel": 0, "numChannels": 3, "channelFormat": "UNORM8", "rgbColorSpace": "sRGB", "bcFormat": "BC7"},
    {"name": "normal \"ts\"", "firstChannel": 3, "numChannels": 2, "channelFormat": "UNORM16"},
    {"name": "height", "firstChannel": 7, "numChannels": 1, "channelFormat": "FLOAT32", "alphaColorSpace": "HLG"},
]


def ref_file_lib():
    if not os.path.exists(REF_FILE_LIB):
        return None
    lib = C.CDLL(REF_FILE_LIB)
    lib.ntc_ref_parse_file.restype = C.c_int
    lib.ntc_ref_parse_file.argtypes = [C.c_char_p, C.c_uint64, C.POINTER(C.c_int), C.POINTER(C.c_uint64), C.c_char_p, C.c_int]
    lib.ntc_ref_reserialize_json.restype = C.c_int
    lib.ntc_ref_reserialize_json.argtypes = [C.c_char_p, C.c_char_p, C.c_int, C.c_char_p, C.c_int]
    return lib


def ref_parse(lib, data):
    out, out64, msg = (C.c_int * 10)(), (C.c_uint64 * 2)(), C.create_string_buffer(1024)
    status = lib.ntc_ref_parse_file(data, len(data), out, out64, msg, 1024)
    return status, list(out), list(out64), msg.value.decode()


def host_load(tmp_path, data, dims=None, device=0, name="case.ntc"):
    path = tmp_path / name
    path.write_bytes(data)
    out = run_exe("load", path, device, *(dims or ()))
    lines = out.splitlines()
    status = int(lines[0].split()[1])
    message = lines[1][len("message "):]
    info = {ln.split()[0]: ln.split(" ", 1)[1] for ln in lines[2:] if " " in ln and not ln.startswith("texture")}
    info["textures"] = [ln[len("texture "):] for ln in lines[2:] if ln.startswith("texture ")]
    return status, message, info


def make_case(ntc, width=64, height=32, mips=None, grid_scale=2, features=8, channels=8, seed=5):
    mips = mips or ntc.presets.full_mip_count(width, height)
    return ref_case(ntc, ntc.presets.spec_ref092(features), width, height, mips, grid_scale, channels,
                    ntc.abi.OUT_FP16_PLANAR_PAIRS, seed, scale_log2_range=(-17.0, -12.0))


def file_of(case, width, height, grid_scale, features, channels, **kw):
    return nw.write_ntex(width, height, channels, len(case.mips), grid_scale, features, case.latents, case.weights, **kw)


@pytest.mark.parametrize("shape", [(64, 32, 2, 8), (256, 256, 4, 16), (100, 60, 3, 12), (16, 16, 1, 4), (512, 128, 6, 16)])
def test_writer_files_are_accepted_by_the_reference_front_end_and_by_the_host_layer(ntc, tmp_path, shape):
    width, height, grid_scale, features = shape
    case = make_case(ntc, width, height, None, grid_scale, features)
    data = file_of(case, width, height, grid_scale, features, 8, textures=TEXTURES)
    lib = ref_file_lib()
    if lib is not None:
        status, out, out64, msg = ref_parse(lib, data)
        assert status == 0, msg
        assert out[:6] == [width, height, 8, len(case.mips), grid_scale, features]
        assert out[9] == 3 and out[8] == len(case.mips)
        text, binary = nw.split_container(data)
        assert out64[1] == len(binary)
    # host layer without a device: everything validates, the upload is what fails
    status, message, info = host_load(tmp_path, data)
    assert status == STATUS["CudaUnavailable"], message
    status, message, info = host_load(tmp_path, data, dims=(width, height, 8, len(case.mips)))
    assert status == STATUS["CudaUnavailable"], message
    assert info["desc"] == f"{width} {height} 8 {len(case.mips)}"
    assert info["shape"] == f"{grid_scale} {features}"
    assert info["sizes"] == f"{case.latents.nbytes} 9472"
    assert info["textures"] == ["albedo|0|3|UNORM8|7|1|0", 'normal "ts"|3|2|UNORM16|0|0|0', "height|7|1|FLOAT32|0|0|2"]
    assert info["mask"] == "0x9f"
    # file footprint of every latent layer (include/libntc/ntc.h:577-581): offsets from the start of the file,
    # in the order the views were written, each one layer of u16 cells
    text, binary = nw.split_container(data)
    doc = json.loads(text)
    chunk_offset = len(data) - len(binary)
    rows = [ln.split()[1:] for ln in run_exe("load", tmp_path / "case.ntc", 0, width, height, 8, len(case.mips)).splitlines() if ln.startswith("latent ")]
    expected = []
    for level, image in enumerate(doc["latents"]):
        assert len(image["layerViews"]) == (features + 3) // 4
        for layer, view_index in enumerate(image["layerViews"]):
            view = doc["views"][view_index]
            size = image["width"] * image["height"] * 2
            assert view["storedSize"] == size
            expected.append([str(v) for v in (level, layer, view["offset"] + chunk_offset, size, 0, size, 0, image["width"], image["height"], image["width"] * 2)])
    assert rows == expected and len(rows) > 0


def malformed_variants(ntc):
    """(name, file bytes, expected status name).  Each breaks one rule the reference checks in
    LoadFileHeadersFromStream / ParseDocument / DeserializeTextureSetDesc."""
    case = make_case(ntc)
    good = file_of(case, 64, 32, 2, 8, 8)
    text, binary = nw.split_container(good)
    doc = json.loads(text)

    def with_doc(edit):
        d = json.loads(text)
        edit(d)
        return nw.pack_container(json.dumps(d), binary)

    yield "truncated header", good[:30], "IOError"
    yield "bad signature", nw.pack_container(text, binary, signature=0x12345678), "FileUnrecognized"
    yield "bad container version", nw.pack_container(text, binary, version=0x101), "FileUnrecognized"
    yield "binary chunk beyond the end", nw.pack_container(text, binary, binary_size=len(binary) + 4), "FileUnrecognized"
    yield "json syntax", nw.pack_container(text[:-1], binary), "FileUnrecognized"
    yield "schema version", with_doc(lambda d: d.update(schemaVersion=2)), "FileUnrecognized"
    yield "missing width", with_doc(lambda d: d.pop("width")), "FileUnrecognized"
    yield "width is a string", with_doc(lambda d: d.update(width="64")), "FileUnrecognized"
    yield "width is a double", with_doc(lambda d: d.update(width=64.5)), "FileUnrecognized"
    yield "negative height", with_doc(lambda d: d.update(height=-32)), "FileUnrecognized"
    yield "null field", with_doc(lambda d: d.update(numColorMips=None)), "FileUnrecognized"
    yield "unknown enum", with_doc(lambda d: d["mlpVersions"][0]["layers"][0].update(weightType="Int4")), "FileUnrecognized"
    yield "enum as integer", with_doc(lambda d: d["mlpVersions"][0].update(weightLayout=0)), "FileUnrecognized"
    yield "missing view size", with_doc(lambda d: d["views"][0].pop("storedSize")), "FileUnrecognized"
    yield "views is an object", with_doc(lambda d: d.update(views={})), "FileUnrecognized"
    yield "zero channels", with_doc(lambda d: d.update(numChannels=0)), "OutOfRange"
    yield "too many channels", with_doc(lambda d: d.update(numChannels=17)), "OutOfRange"
    yield "odd feature count", with_doc(lambda d: d["latentShape"].update(numFeatures=6)), "OutOfRange"
    yield "grid scale out of range", with_doc(lambda d: d["latents"][0].update(width=4, height=2)), "OutOfRange"


def test_malformed_files_same_status_as_the_reference_front_end(ntc, tmp_path):
    lib = ref_file_lib()
    for name, data, expected in malformed_variants(ntc):
        status, message, _ = host_load(tmp_path, data)
        assert status == STATUS[expected], (name, status, message)
        assert message, name
        if lib is not None:
            ref_status, _, _, ref_message = ref_parse(lib, data)
            assert ref_status == status, (name, ref_status, ref_message, status, message)


def test_random_document_damage_same_status_as_the_reference_front_end(ntc, tmp_path):
    """Seeded damage to the JSON document (values replaced by extremes or other types, members and elements
    removed): whenever the reference's front end (LoadFileHeadersFromStream + its document parser, built from
    the reference's own sources) refuses a file, the host layer refuses it with the same status, and nearly
    always with the same complaint, position and quoted text included (a streaming reader reports the first
    fault in the order of the text, the host layer the first in the order of its schema: with two faults in one
    object whose members are out of schema order the two could pick different ones)."""
    lib = ref_file_lib()
    if lib is None:
        pytest.skip("the reference's host-only sources are not built on this machine")
    import random
    case = make_case(ntc)
    text, binary = nw.split_container(file_of(case, 64, 32, 2, 8, 8, textures=TEXTURES))
    values = [0, -1, 1, 2 ** 31 - 1, 2 ** 31, 2 ** 32 - 1, 2 ** 32, 2 ** 63, 10 ** 30, 0.5, 1e308, 65535, 17,
              "x", "", None, True, [], {}, [1], {"a": 1}]

    def slots(node):
        if isinstance(node, dict):
            for key, value in list(node.items()):
                yield node, key
                yield from slots(value)
        elif isinstance(node, list):
            for index, value in enumerate(node):
                yield node, index
                yield from slots(value)

    rnd = random.Random(2024)
    refused = same_text = 0
    for i in range(120):
        doc = json.loads(text)
        for _ in range(rnd.randint(1, 2)):
            owner, key = rnd.choice(list(slots(doc)))
            if rnd.random() < 0.25:
                del owner[key]
            else:
                owner[key] = rnd.choice(values)
        data = nw.pack_container(json.dumps(doc), binary)
        ref_status, _, _, ref_message = ref_parse(lib, data)
        status, message, _ = host_load(tmp_path, data)
        if ref_status != 0:
            refused += 1
            assert status == ref_status, (i, ref_status, ref_message, status, message)
            same_text += ref_message == message
        else:
            assert status != 0          # no device here: at best everything validates and the upload fails
    assert refused >= 60 and same_text >= 0.98 * refused, (refused, same_text)


def test_header_sums_that_wrap_are_refused(ntc, tmp_path):
    """Chunk offset + size past 2^64: the reference adds the two without a check, finds the (wrapped) end inside
    the file and goes on to allocate a chunk of that size, so it is not asked here; the host layer refuses."""
    import struct
    case = make_case(ntc)
    good = bytearray(file_of(case, 64, 32, 2, 8, 8))
    for field, value in ((16, 2 ** 64 - 40), (32, 2 ** 64 - 1), (8, 2 ** 64 - 8), (24, 2 ** 64 - 64)):
        data = bytearray(good)
        struct.pack_into("<Q", data, field, value & (2 ** 64 - 1))
        if field in (8, 24):                                     # an offset: give it a size that wraps the sum back into the file
            struct.pack_into("<Q", data, field + 8, (100 - value) & (2 ** 64 - 1))
        status, message, _ = host_load(tmp_path, bytes(data))
        assert status == STATUS["FileUnrecognized"], (field, status, message)
        assert "64-bit offset range" in message or "File incomplete" in message, message


def test_semantic_errors_of_the_metadata_stage(ntc, tmp_path):
    """Rules of LoadMetadataFromStream / ValidateMLP / ValidateBufferView / LoadFromStreamPostHeader
    (src/TextureSetMetadata.cpp:434-581,978-1135, src/TextureSet.cpp:154-196); the reference needs a
    CUDA context to reach them, so only the host layer is exercised."""
    case = make_case(ntc)
    good = file_of(case, 64, 32, 2, 8, 8)
    text, binary = nw.split_container(good)

    def load(edit, dims=None, binary_chunk=binary):
        d = json.loads(text)
        edit(d)
        return host_load(tmp_path, nw.pack_container(json.dumps(d), binary_chunk), dims)

    checks = [
        (lambda d: d.update(mlpVersions=[]), "File doesn't contain MLP information"),
        (lambda d: d["mlpVersions"][0]["layers"].pop(), "MLP with 3 layers"),
        (lambda d: d["mlpVersions"][0].update(weightLayout="ColumnMajor"), "Only row-major"),
        (lambda d: d["mlpVersions"][0].pop("weightLayout"), "Only row-major"),
        (lambda d: d["mlpVersions"][0]["layers"][1].update(biasType="Float16"), "Only Int8 weights + Float32 scale + Int32 bias"),
        (lambda d: d["mlpVersions"][0]["layers"][0].update(inputChannels=32), "layer 0 with 32 inputs and 64 outputs"),
        (lambda d: d["mlpVersions"][0]["layers"][3].update(outputChannels=8), "layer 3 with 32 inputs and 8 outputs"),
        (lambda d: d["mlpVersions"][0]["layers"][1].update(outputChannels=64), "layer 1 with 64 inputs and 64 outputs"),
        (lambda d: d["mlpVersions"][0]["layers"][2].update(weightView=999), "Invalid view index 999"),
        (lambda d: d["views"][0].update(offset=2), "is not 4-byte aligned"),
        (lambda d: d["views"][0].update(storedSize=100), "is less than minimum expected size"),
        (lambda d: d["views"][-1].update(storedSize=10 ** 9), "outside of the chunk size"),
        (lambda d: d["latents"][0]["layerViews"].pop(), "Expected 2 layers, got 1"),
        (lambda d: d.update(channels=d["channels"][:-1]), "texture channels while 8 are expected"),
        (lambda d: d["colorMips"][1].pop("latentMip"), "Color MIP 1 doesn't have a mapping"),
        (lambda d: d["colorMips"][2].pop("positionScale"), "Color MIP 2 doesn't have the positionLod and positionScale"),
        (lambda d: d["colorMips"][1].update(width=31), "Color MIP 1 specifies dimensions of 31x16"),
        (lambda d: d["colorMips"][-1].update(latentMip=0), "specifies latent image index 0, but it is expected to be 2"),
        (lambda d: d["latents"][1].update(width=9), "Neural MIP 1 dimensions (9x8) don't match the expected dimensions (16x8)"),
        (lambda d: d.pop("latentShape"), "does not describe a latent shape"),
    ]
    for edit, fragment in checks:
        status, message, _ = load(edit)
        assert status == STATUS["FileUnrecognized"], (fragment, status, message)
        assert fragment in message, (fragment, message)

    status, message, _ = load(lambda d: d["views"][d["latents"][0]["layerViews"][0]].update(compression="GDeflate", uncompressedSize=10 ** 6))
    assert status == STATUS["Unsupported"] and "GDeflate" in message
    # a file with the FP8 version of the MLP only is a valid file (src/TextureSetMetadata.cpp:763-781): without a
    # device the load ends, like that of the complete file, at the first upload
    status, message, _ = load(lambda d: d.update(mlpVersions=d["mlpVersions"][1:]))
    assert status == STATUS["CudaUnavailable"], message
    # an existing set of other dimensions refuses the file
    status, message, _ = load(lambda d: None, dims=(64, 64, 8, 7))
    assert status == STATUS["FileIncompatible"] and "dimensions do not match" in message
    out = run_exe("load", tmp_path / "does_not_exist.ntc", 0)
    assert out.splitlines()[0] == "status 4 FileUnavailable" and "Cannot open file" in out.splitlines()[1]


def test_unknown_members_whitespace_and_escapes_are_tolerated(ntc, tmp_path):
    case = make_case(ntc)
    textures = [{"name": "tab\there", "firstChannel": 0, "numChannels": 4, "futureField": [1, {"a": None}, "x"]}]
    data = file_of(case, 64, 32, 2, 8, 8, textures=textures, json_indent=2,
                   extra_document_fields={"generator": {"name": "test", "version": [1, 2, 3.5e0], "flags": [True, False, None]}})
    lib = ref_file_lib()
    if lib is not None:
        assert ref_parse(lib, data)[0] == 0
    status, message, info = host_load(tmp_path, data, dims=(64, 32, 8, len(case.mips)))
    assert status == STATUS["CudaUnavailable"], message
    assert info["textures"] == ["tab\there|0|4|UNORM8|0|0|0"]


def test_bc7_mode_maps_stored_in_a_file(ntc, tmp_path):
    """bcModeBuffers of a texture (src/TextureSetMetadata.cpp:470-476, src/TextureMetadata.cpp:151-213): maps
    stored as they are come back from GetBC7ModeBuffer, one stored with GDeflate is described by its
    footprint only; the reference's front end accepts the same file."""
    case = make_case(ntc)                                           # 64 x 32: mip 0 is 16 x 8 blocks, mip 1 8 x 4
    rng = np.random.default_rng(11)
    map0 = rng.integers(0, 256, ((16 * 8 * 9 + 31) // 32) * 4, dtype=np.uint8)
    map1 = rng.integers(0, 256, ((8 * 4 * 9 + 31) // 32) * 4, dtype=np.uint8)
    packed = rng.integers(0, 256, 20, dtype=np.uint8)
    buffers = [(0, 0, map0.tobytes(), None), (0, 1, map1.tobytes(), None),
               (0, 2, packed.tobytes(), {"compression": "GDeflate", "uncompressedSize": 12, "crc32": 1234})]
    data = file_of(case, 64, 32, 2, 8, 8, textures=TEXTURES, mode_buffers=buffers)
    lib = ref_file_lib()
    if lib is not None:
        assert ref_parse(lib, data)[0] == 0
    path = tmp_path / "modes.ntc"
    path.write_bytes(data)
    out = run_exe("load", path, 0, 64, 32, 8, len(case.mips))
    rows = [ln.split()[1:] for ln in out.splitlines() if ln.startswith("modes ")]
    text, binary = nw.split_container(data)
    doc = json.loads(text)
    chunk_offset = len(data) - len(binary)
    views = [doc["views"][b["view"]] for b in doc["textures"][0]["bcModeBuffers"]]

    def digest(a):
        total = 0
        for byte in a.tolist():
            total = (total * 131 + byte) % (1 << 64)
        return total
    assert rows == [
        ["0", "0", str(views[0]["offset"] + chunk_offset), str(map0.size), "0", str(map0.size), str(map0.size), str(digest(map0))],
        ["0", "1", str(views[1]["offset"] + chunk_offset), str(map1.size), "0", str(map1.size), str(map1.size), str(digest(map1))],
        ["0", "2", str(views[2]["offset"] + chunk_offset), "20", "1", "12", "0", "0"]], rows
    # a view index that does not exist is a malformed file
    broken = file_of(case, 64, 32, 2, 8, 8, textures=TEXTURES, mode_buffers=buffers[:1],
                     mutate=lambda d: d["textures"][0]["bcModeBuffers"][0].update(view=999))
    status, message, _ = host_load(tmp_path, broken, dims=(64, 32, 8, len(case.mips)))
    assert status == STATUS["FileUnrecognized"] and "Invalid view index" in message


GOLDEN_JSON = os.path.join(HERE, "golden", "ntex_reference_json.json")


def test_host_layer_reads_json_as_the_reference_serialises_it(ntc, tmp_path):
    """The fixture is the JSON chunk of the (64, 32, gs 2, 8 features, 3 textures) file after a
    round trip through the reference's own parser and serialiser."""
    with open(GOLDEN_JSON) as f:
        fixture = json.load(f)
    case = make_case(ntc)
    data = file_of(case, 64, 32, 2, 8, 8, textures=TEXTURES, channel_color_spaces=["sRGB"] * 3 + [None] * 5)
    text, binary = nw.split_container(data)
    lib = ref_file_lib()
    if lib is not None:     # the fixture is still what the reference writes for this document
        out, err = C.create_string_buffer(1 << 16), C.create_string_buffer(1024)
        assert lib.ntc_ref_reserialize_json(text.encode(), out, 1 << 16, err, 1024) == 0, err.value
        assert out.value.decode() == fixture["reference_json"]
    assert json.loads(fixture["reference_json"]) == json.loads(text)      # same document, the reference's spelling
    status, message, info = host_load(tmp_path, nw.pack_container(fixture["reference_json"], binary), dims=(64, 32, 8, len(case.mips)))
    assert status == STATUS["CudaUnavailable"], message
    assert info["shape"] == "2 8" and len(info["textures"]) == 3
    assert info["colorspaces"] == "1 1 1 0 0 0 0 0"


def pixels_from_planar(planar_u16, width, height, channels):
    return planar_u16.reshape(height, channels // 2, width, 2).transpose(0, 2, 1, 3).reshape(-1)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(256, 128, 2, 16, 10), (100, 60, 3, 12, 8), (64, 64, 1, 4, 16)])
def test_gpu_decode_of_a_file_matches_the_checker(ntc, oracle, tmp_path, shape):
    width, height, grid_scale, features, channels = shape
    case = make_case(ntc, width, height, None, grid_scale, features, channels, seed=21)
    data = file_of(case, width, height, grid_scale, features, channels, textures=TEXTURES)
    path = tmp_path / "set.ntc"
    path.write_bytes(data)
    prefix = str(tmp_path / "out")
    out = run_exe("decodefile", path, prefix)
    assert "host decodefile OK" in out
    assert f"desc {width} {height} {channels} {len(case.mips)}" in out and f"shape {grid_scale} {features}" in out
    host = case.host_set()
    host.decode(threads=8)
    for m, mip in enumerate(case.mips):
        planar = np.ascontiguousarray(host.output[mip.outOffset: mip.outOffset + mip.width * mip.height * channels * 2].view(np.uint16))
        got = np.fromfile(f"{prefix}_mip{m}.bin", dtype=np.uint16)
        assert np.array_equal(got, pixels_from_planar(planar, mip.width, mip.height, channels)), f"mip {m}"


@pytest.mark.gpu
def test_gpu_narrow_hidden_layers_are_expanded(ntc, oracle, tmp_path):
    """A file whose hidden layers are narrower than the decoder's (48-32-24-16 instead of
    48-64-48-32): weights land in the top-left corner of zero matrices, missing scales are 1,
    missing biases 0 (src/TextureSetMetadata.cpp:661-761).  The checker decodes the expanded blob."""
    width, height, grid_scale, features, channels = 128, 64, 2, 16, 6
    spec = ntc.presets.spec_ref092(features)
    rng = np.random.default_rng(33)
    narrow = [(48, 32), (32, 24), (24, 16), (16, 16)]
    full = nw.LAYER_WIDTHS_092
    layer_data, blob_w, blob_s, blob_b = [], [], [], []
    for (n_in, n_out), (f_in, f_out) in zip(narrow, full):
        w = rng.integers(-127, 128, (n_out, n_in)).astype(np.int8)
        s = np.exp2(rng.uniform(-15.0, -11.0, n_out)).astype(np.float32)
        b = rng.integers(-20000, 20000, n_out).astype(np.int32)
        layer_data.append((w, s, b))
        big = np.zeros((f_out, f_in), dtype=np.int8)
        big[:n_out, :n_in] = w
        blob_w.append(big.reshape(-1).view(np.uint8))
        blob_s.append(np.concatenate([s, np.ones(f_out - n_out, np.float32)]).view(np.uint8))
        blob_b.append(np.concatenate([b, np.zeros(f_out - n_out, np.int32)]).view(np.uint8))
    expanded = np.concatenate(blob_w + blob_s + blob_b)
    assert expanded.size == 9472
    mips = ntc.presets.full_mip_count(width, height)
    case = ref_case(ntc, spec, width, height, mips, grid_scale, channels, ntc.abi.OUT_FP16_PLANAR_PAIRS, 34, weights=expanded)
    data = nw.write_ntex(width, height, channels, mips, grid_scale, features, case.latents, None, layer_widths=narrow, layer_data=layer_data)
    path = tmp_path / "narrow.ntc"
    path.write_bytes(data)
    prefix = str(tmp_path / "narrow")
    assert "host decodefile OK" in run_exe("decodefile", path, prefix)
    host = case.host_set()
    host.decode(threads=8)
    for m, mip in enumerate(case.mips):
        planar = np.ascontiguousarray(host.output[mip.outOffset: mip.outOffset + mip.width * mip.height * channels * 2].view(np.uint16))
        got = np.fromfile(f"{prefix}_mip{m}.bin", dtype=np.uint16)
        assert np.array_equal(got, pixels_from_planar(planar, mip.width, mip.height, channels)), f"mip {m}"


def test_metadata_only_loading(ntc, tmp_path):
    """CreateTextureSetMetadataFromStream (include/libntc/ntc.h:1158-1163, src/Context.cpp:263-293): the file's
    description of the set without its latents and without a device - also for files whose latent layers are
    stored with GDeflate, which a full load refuses; the footprints then carry the compression type."""
    width, height, grid_scale, features = 64, 32, 2, 8
    case = make_case(ntc, width, height, None, grid_scale, features)
    data = file_of(case, width, height, grid_scale, features, 8, textures=TEXTURES, channel_color_spaces=["sRGB"] * 3 + [None] * 4 + ["HLG"])
    path = tmp_path / "plain.ntc"
    path.write_bytes(data)

    def parse(out):
        lines = out.splitlines()
        return int(lines[0].split()[1]), lines[1], lines[2:]

    status, message, lines = parse(run_exe("metadata", path))
    assert status == STATUS["Ok"], message
    # the same description a full load gives (which fails at the upload here, after everything was parsed)
    loaded = run_exe("load", path, 0, width, height, 8, len(case.mips)).splitlines()[2:]
    assert [ln for ln in lines if not ln.startswith(("weights", "inference"))] == loaded
    weights = np.frombuffer(case.weights, np.uint8)
    digest = 0
    for b in weights.tolist():
        digest = (digest * 131 + b) % (1 << 64)
    assert f"weights {weights.size} {digest}" in lines
    inference = [ln for ln in lines if ln.startswith("inference ")][0].split()
    # TEXTURES claims channels 0-4 and 7; the storage colour spaces of the channels, two bits each
    spaces = [int(v) for v in [ln for ln in lines if ln.startswith("colorspaces")][0].split()[1:]]
    assert inference[1] == "0x9f" and int(inference[3]) == len(case.mips)
    assert int(inference[2], 16) == sum(v << (2 * c) for c, v in enumerate(spaces)) == 0b10_00_00_00_00_01_01_01
    text, binary = nw.split_container(data)
    doc = json.loads(text)
    for token, mip in zip(inference[4:], doc["colorMips"]):
        neural, scale, lod = token.split(":")
        assert int(neural) == mip["latentMip"] and float(scale) == mip["positionScale"] and float(lod) == mip["positionLod"]

    # latent layers marked as GDeflate streams: described, not read
    for view_index in doc["latents"][0]["layerViews"]:
        view = doc["views"][view_index]
        view.update(compression="GDeflate", uncompressedSize=view["storedSize"], crc32=12345)
    packed = tmp_path / "packed.ntc"
    packed.write_bytes(nw.pack_container(json.dumps(doc), binary))
    status, message, _ = host_load(tmp_path, packed.read_bytes(), name="packed_full.ntc")
    assert status == STATUS["Unsupported"], message
    status, message, lines = parse(run_exe("metadata", packed))
    assert status == STATUS["Ok"], message
    rows = [ln.split()[1:] for ln in lines if ln.startswith("latent ")]
    layers = (features + 3) // 4
    assert [r[4] for r in rows] == ["1"] * layers + ["0"] * (len(rows) - layers)      # compression type per layer
    assert [r[6] for r in rows[:layers]] == ["12345"] * layers
