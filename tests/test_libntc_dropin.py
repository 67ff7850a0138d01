"""libntc.so as a drop-in for LibNTC: tests/libntc_dropin_test.cpp includes nothing but LibNTC's own
<libntc/ntc.h> (compiled against it where it lies in the LibNTC tree), links libntc.so and drives it the way
an SDK tool does.

 * no GPU: every virtual of every interface is called once through the interface pointers - a class whose
   vtable did not follow the header's declaration order (or lacked the virtual ITextureSetMetadata base)
   would crash or answer with the wrong status; the library exports every free function the header declares;
 * GPU: CreateContext -> CreateCompressedTextureSetFromMemory -> Decompress(stats, useInt8Weights = true)
   -> ReadChannels gives, byte for byte, what the CPU checker decodes from the same latents and weights.
"""
import os
import re
import subprocess

import numpy as np
import pytest

from cases import Case
from test_ntc_file import TEXTURES, file_of, make_case, pixels_from_planar

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
EXE = os.path.join(HERE, "libntc_dropin_test")
LIB = os.path.join(ROOT, "rtxntc-library_amd", "host", "libntc.so")
REFERENCE_HEADER = "/root/reference/include/libntc/ntc.h"


def run_dropin(*args, env=None):
    if not os.path.exists(EXE):
        pytest.fail(f"{EXE} is not built; run __graft_entry__.build() (make -C tests)")
    full_env = dict(os.environ)
    full_env.pop("LIBNTC_ALLOW_TEXTURE_SETS_WITHOUT_DEVICE", None)
    full_env.update(env or {})
    out = subprocess.run([EXE, *map(str, args)], capture_output=True, text=True, timeout=300, env=full_env)
    assert out.returncode == 0, f"libntc_dropin_test {args[0]} failed:\n{out.stdout}\n{out.stderr}"
    return out.stdout


def small_file(ntc, tmp_path):
    case = make_case(ntc)                                          # 64 x 32, 7 mips, grid scale 2, 8 features, 8 channels
    path = tmp_path / "set.ntc"
    path.write_bytes(file_of(case, 64, 32, 2, 8, 8, textures=TEXTURES))
    return case, path


@pytest.mark.parametrize("sets_without_device", [False, True])
def test_every_virtual_of_the_reference_interfaces_answers(ntc, tmp_path, sets_without_device):
    _, path = small_file(ntc, tmp_path)
    env = {"LIBNTC_ALLOW_TEXTURE_SETS_WITHOUT_DEVICE": "1"} if sets_without_device else {}
    out = run_dropin("walk", path, env={**env, "HIP_VISIBLE_DEVICES": "", "ROCR_VISIBLE_DEVICES": ""})
    assert "libntc drop-in walk OK" in out
    assert ("(with texture sets" in out) == sets_without_device


def test_library_exports_the_free_functions_of_the_reference_header():
    """Every NTC_API function of include/libntc/ntc.h:1307-1391, by its unmangled name."""
    exported = subprocess.run(["nm", "-D", "--defined-only", LIB], capture_output=True, text=True, check=True).stdout
    names = {line.split()[-1] for line in exported.splitlines() if line.strip()}
    if os.path.exists(REFERENCE_HEADER):
        text = open(REFERENCE_HEADER).read()
        text = text[text.index('extern "C"'):]
        declared = set(re.findall(r"NTC_API\s+[\w:\s\*]+?\b(\w+)\s*\(", text))
    else:                                                          # the list as of interface version 0x25121500
        declared = {"GetInterfaceVersion", "GetLibraryVersion", "CreateContext", "DestroyContext", "GetLastErrorMessage", "StatusToString",
                    "ChannelFormatToString", "BlockCompressedFormatToString", "ColorSpaceToString", "InferenceWeightTypeToString",
                    "CompressionTypeToString", "GetBytesPerPixelComponent", "LossToPSNR", "EstimateCompressedTextureSetSize",
                    "GetKnownLatentShapeCount", "EnumerateKnownLatentShapes", "PickLatentShape", "GetLatentShapeBitsPerPixel",
                    "DecodeImageDifferenceResult", "GetBC7ModeBufferSize", "MakeBC7ModeBuffer", "GetGDeflateHeaderSize"}
    assert len(declared) >= 22
    missing = sorted(declared - names)
    assert not missing, f"libntc.so does not export {missing}"


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(256, 128, 2, 16, 10), (100, 60, 3, 12, 8)])
def test_gpu_decode_through_the_reference_header_equals_the_checker(ntc, oracle, tmp_path, shape):
    width, height, grid_scale, features, channels = shape
    case = make_case(ntc, width, height, None, grid_scale, features, channels, seed=41)
    path = tmp_path / "set.ntc"
    path.write_bytes(file_of(case, width, height, grid_scale, features, channels, textures=TEXTURES))
    prefix = str(tmp_path / "out")
    out = run_dropin("decode", path, prefix, 1)
    assert f"libntc drop-in decode OK: {width} x {height}, {channels} channels, {len(case.mips)} mips, Int8 weights" in out
    host = case.host_set()
    host.decode(threads=8)
    for m, mip in enumerate(case.mips):
        planar = np.ascontiguousarray(host.output[mip.outOffset: mip.outOffset + mip.width * mip.height * channels * 2].view(np.uint16))
        got = np.fromfile(f"{prefix}_mip{m}.bin", dtype=np.uint16)
        assert np.array_equal(got, pixels_from_planar(planar, mip.width, mip.height, channels)), f"mip {m}"


@pytest.mark.gpu
def test_gpu_decode_with_the_default_fp8_weights_equals_the_checker(ntc, oracle, tmp_path):
    """Decompress(stats) with useInt8Weights left at its default decodes with the file's FP8 version of the network
    (src/TextureSet.cpp:1664-1682,1812,1826); the checker's FP8 network on the same blob gives the same bytes, and
    the Int8 version of the same file still decodes to ITS bytes."""
    width, height, grid_scale, features, channels = 128, 96, 2, 16, 10
    case = make_case(ntc, width, height, None, grid_scale, features, channels, seed=43)
    spec_fp8 = ntc.presets.spec_ref092_fp8(features)
    fp8_blob = ntc.synth.make_fp8_weights(spec_fp8, 44)
    path = tmp_path / "set.ntc"
    path.write_bytes(file_of(case, width, height, grid_scale, features, channels, textures=TEXTURES, fp8_blob=fp8_blob))
    for use_int8, name in ((0, "FP8"), (1, "Int8")):
        prefix = str(tmp_path / f"out{use_int8}")
        out = run_dropin("decode", path, prefix, use_int8)
        assert f"{name} weights" in out
        checker = case if use_int8 else Case(ntc, spec_fp8, case.mips, case.latents.nbytes, channels, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=0,
                                               latents=case.latents, weights=fp8_blob)
        host = checker.host_set()
        host.decode(threads=8)
        for m, mip in enumerate(case.mips):
            planar = np.ascontiguousarray(host.output[mip.outOffset: mip.outOffset + mip.width * mip.height * channels * 2].view(np.uint16))
            got = np.fromfile(f"{prefix}_mip{m}.bin", dtype=np.uint16)
            assert np.array_equal(got, pixels_from_planar(planar, mip.width, mip.height, channels)), (name, m)
