"""Free functions of the host interface (reference include/libntc/ntc.h:1307-1391,
src/PublicFunctions.cpp): enum names, known latent shapes, size estimate, BC7 mode bitmap.

Pins: the reference's own table of known shapes lists a bit rate next to every shape, and its
bits-per-pixel formula must reproduce that rate (two facts of the reference that check each
other); the size estimate is the latent size of the reference's own FeatureGridMath (oracle/_ref)
plus the 9472-byte Int8 network; the BC7 bitmap is checked on blocks built bit by bit from the BC7
mode table (mode = number of leading zero bits of the block, partition bits after the mode bit)."""
import ctypes as C
import math
import os

import numpy as np
import pytest

HOST_LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "rtxntc-library_amd", "host", "libntc.so")


class LatentShape(C.Structure):
    _fields_ = [("gridSizeScale", C.c_int), ("numFeatures", C.c_int)]


class TextureSetDesc(C.Structure):
    _fields_ = [("width", C.c_int), ("height", C.c_int), ("channels", C.c_int), ("mips", C.c_int)]


class VersionInfo(C.Structure):
    _fields_ = [("major", C.c_int), ("minor", C.c_int), ("point", C.c_int), ("branch", C.c_char_p), ("commitHash", C.c_char_p)]


@pytest.fixture(scope="module")
def host():
    lib = C.CDLL(HOST_LIB)
    for name in ("StatusToString", "ChannelFormatToString", "BlockCompressedFormatToString", "ColorSpaceToString",
                 "InferenceWeightTypeToString", "CompressionTypeToString", "GetLastErrorMessage"):
        getattr(lib, name).restype = C.c_char_p
    lib.GetLibraryVersion.restype = VersionInfo
    lib.GetLatentShapeBitsPerPixel.restype = C.c_float
    lib.GetLatentShapeBitsPerPixel.argtypes = [C.POINTER(LatentShape)]
    lib.EnumerateKnownLatentShapes.argtypes = [C.c_int, C.POINTER(C.c_float), C.POINTER(LatentShape)]
    lib.PickLatentShape.argtypes = [C.c_float, C.POINTER(C.c_float), C.POINTER(LatentShape)]
    lib.EstimateCompressedTextureSetSize.argtypes = [C.POINTER(TextureSetDesc), C.POINTER(LatentShape), C.POINTER(C.c_size_t)]
    lib.DecodeImageDifferenceResult.restype = C.c_double
    lib.DecodeImageDifferenceResult.argtypes = [C.c_uint64]
    lib.GetBC7ModeBufferSize.restype = C.c_size_t
    lib.MakeBC7ModeBuffer.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t]
    lib.GetGDeflateHeaderSize.restype = C.c_size_t
    lib.GetGDeflateHeaderSize.argtypes = [C.c_size_t]
    lib.LossToPSNR.restype = C.c_float
    lib.LossToPSNR.argtypes = [C.c_float]
    return lib


OK, OUT_OF_RANGE, INVALID_ARGUMENT = 0, 16, 10


def test_enum_names(host):
    assert [host.StatusToString(i) for i in (0, 3, 8, 16, 18)] == [b"Ok", b"CudaUnavailable", b"Unsupported", b"OutOfRange", b"UnknownError"]
    assert host.StatusToString(77) == b"77"                       # unknown values print as numbers
    assert [host.ChannelFormatToString(i) for i in range(6)] == [b"UNKNOWN", b"UNORM8", b"UNORM16", b"FLOAT16", b"FLOAT32", b"UINT32"]
    assert [host.BlockCompressedFormatToString(i) for i in range(8)] == [b"None"] + [b"BC%d" % i for i in range(1, 8)]
    assert [host.ColorSpaceToString(i) for i in range(3)] == [b"Linear", b"sRGB", b"HLG"]
    assert [host.InferenceWeightTypeToString(i) for i in range(4)] == [b"Unknown", b"GenericInt8", b"GenericFP8", b"CoopVecFP8"]
    assert [host.CompressionTypeToString(i) for i in range(2)] == [b"None", b"GDeflate"]
    assert host.ColorSpaceToString(9) == b"9"
    version = host.GetLibraryVersion()
    assert (version.major, version.minor, version.point) == (0, 9, 2) and version.branch and version.commitHash is not None
    assert host.GetInterfaceVersion() == 0x25121500
    assert host.GetGDeflateHeaderSize(1 << 20) == 0
    assert math.isinf(host.LossToPSNR(0.0)) and abs(host.LossToPSNR(0.01) - 20.0) < 1e-5


def test_known_latent_shapes(host):
    count = host.GetKnownLatentShapeCount()
    assert count == 9
    rates = []
    for i in range(count):
        bpp, shape = C.c_float(), LatentShape()
        assert host.EnumerateKnownLatentShapes(i, bpp, shape) == OK
        # the rate the table lists is the rate the formula gives for the shape, to the table's two decimals
        assert abs(host.GetLatentShapeBitsPerPixel(shape) - bpp.value) < 0.006, (i, bpp.value)
        # and the formula itself: layers * 16 bits * 1.25 (two neural LODs are read together) per gridSizeScale^2 texels
        layers = (shape.numFeatures + 3) // 4
        assert abs(host.GetLatentShapeBitsPerPixel(shape) - layers * 16 * 1.25 / shape.gridSizeScale ** 2) < 1e-5
        assert 1 <= shape.gridSizeScale <= 6 and shape.numFeatures in (4, 8, 12, 16)
        rates.append(bpp.value)
    assert rates == sorted(rates)
    bpp, shape = C.c_float(), LatentShape()
    assert host.EnumerateKnownLatentShapes(-1, bpp, shape) == OUT_OF_RANGE
    assert host.EnumerateKnownLatentShapes(count, bpp, shape) == OUT_OF_RANGE
    assert b"must be 0-8" in host.GetLastErrorMessage()

    # PickLatentShape: nearest known rate when within 25 % of the request (brute force over the table)
    for request in np.concatenate([np.linspace(0.5, 30.0, 400), np.array(rates, dtype=np.float64)]):
        request = float(np.float32(request))
        want = None
        for r in rates:
            diff = abs(np.float32(r) - np.float32(request))
            if diff < np.float32(request) * np.float32(0.25) and (want is None or diff < abs(np.float32(want) - np.float32(request))):
                want = r
        status = host.PickLatentShape(request, bpp, shape)
        if want is None:
            assert status == OUT_OF_RANGE, request
        else:
            assert status == OK and bpp.value == want, (request, bpp.value, want)
            assert abs(host.GetLatentShapeBitsPerPixel(shape) - want) < 0.006
    assert host.PickLatentShape(0.0, bpp, shape) == OUT_OF_RANGE
    assert host.PickLatentShape(-3.0, bpp, shape) == OUT_OF_RANGE
    assert host.PickLatentShape(20.0, bpp, shape) == OK and (shape.gridSizeScale, shape.numFeatures) == (2, 16)


def test_estimate_compressed_size_against_reference_geometry(host):
    """latent bytes from the reference's own FeatureGridMath + the Int8 network (8192 weights,
    160 outputs x (fp32 scale + fp32 bias) = 9472 bytes, src/PublicFunctions.cpp:372-376).  The
    literal sizes were printed by the reference's CalculateQuantizedLatentsSize (oracle/_ref); the
    library itself is asked again when it is there."""
    import oracle_lib
    ref = oracle_lib.load_ref()
    golden = {(4096, 4096, 13, 2, 16): 44738560, (2048, 1024, 12, 4, 12): 1048560, (1000, 600, 5, 3, 8): 353500,
              (512, 512, 1, 6, 4): 17978, (37, 91, 3, 1, 16): 35352, (8192, 8192, 14, 2, 16): 178954240}
    for (w, h, mips, gs, features), latent_bytes in golden.items():
        size = C.c_size_t()
        desc, shape = TextureSetDesc(w, h, 3, mips), LatentShape(gs, features)
        assert host.EstimateCompressedTextureSetSize(desc, shape, size) == OK
        assert size.value == latent_bytes + 9472, (w, h, mips, gs, features)
        if ref is not None:
            assert ref.ntc_ref_quantized_latents_size(w, h, mips, gs, features) == latent_bytes
    size = C.c_size_t()
    assert host.EstimateCompressedTextureSetSize(TextureSetDesc(0, 4, 3, 1), LatentShape(2, 16), size) == OUT_OF_RANGE
    assert host.EstimateCompressedTextureSetSize(TextureSetDesc(64, 64, 3, 1), LatentShape(7, 16), size) == OUT_OF_RANGE
    assert host.EstimateCompressedTextureSetSize(TextureSetDesc(64, 64, 3, 1), LatentShape(2, 10), size) == OUT_OF_RANGE


def test_decode_image_difference_result(host):
    assert host.DecodeImageDifferenceResult(1 << 48) == 1.0
    assert host.DecodeImageDifferenceResult(0) == 0.0
    assert host.DecodeImageDifferenceResult(3 << 46) == 0.75
    assert host.DecodeImageDifferenceResult((1 << 64) - 1) == float((1 << 64) - 1) * 2.0 ** -48


PARTITION_BITS = [4, 6, 6, 6, 3, 2, 0, 6]      # bits after the mode bit that the bitmap keeps (mode 4: rotation + index selector, mode 5: rotation)


def bc7_block(mode, partition, rng):
    """A 16-byte block whose first bits are `mode` zeros, a one, then the partition bits (LSB first)."""
    value = (1 << mode) | (partition << (mode + 1))
    used = mode + 1 + PARTITION_BITS[mode]
    rest = int(rng.integers(0, 1 << 62)) << used
    word = (value | rest) & ((1 << 128) - 1)
    return word.to_bytes(16, "little")


def test_bc7_mode_buffer(host):
    rng = np.random.default_rng(5)
    wb, hb = 7, 5
    pitch = wb * 16 + 32                                          # padded rows
    data = bytearray(rng.integers(0, 256, hb * pitch, dtype=np.uint8).tobytes())
    want = []
    for row in range(hb):
        for col in range(wb):
            i = row * wb + col
            mode = i % 8 if i != 3 else 0
            partition = int(rng.integers(0, 1 << PARTITION_BITS[mode])) if PARTITION_BITS[mode] else 0
            if i == 3:
                partition = 0                                     # mode 0, partition 0 is stored as 0x1BF
            data[row * pitch + col * 16: row * pitch + col * 16 + 16] = bc7_block(mode, partition, rng)
            want.append(((mode << 6) | partition) or 0x1BF)
    size = host.GetBC7ModeBufferSize(wb, hb)
    assert size == ((wb * hb * 9 + 31) // 32) * 4
    out = (C.c_uint8 * size)()
    src = (C.c_uint8 * len(data)).from_buffer(data)
    assert host.MakeBC7ModeBuffer(wb, hb, src, len(data), pitch, out, size) == OK
    bits = int.from_bytes(bytes(out), "little")
    got = [(bits >> (9 * i)) & 0x1FF for i in range(wb * hb)]
    assert got == want
    assert bits >> (9 * wb * hb) == 0
    # a block of zeros (no mode bit in the first dword) counts as the reserved mode 7
    zero = (C.c_uint8 * 16)()
    one = (C.c_uint8 * 4)()
    assert host.MakeBC7ModeBuffer(1, 1, zero, 16, 16, one, 4) == OK and int.from_bytes(bytes(one), "little") == 7 << 6
    # argument checks
    assert host.MakeBC7ModeBuffer(wb, hb, None, len(data), pitch, out, size) == INVALID_ARGUMENT
    assert host.MakeBC7ModeBuffer(wb, hb, src, len(data), pitch, None, size) == INVALID_ARGUMENT
    assert host.MakeBC7ModeBuffer(wb, hb, src, len(data), wb * 16 - 16, out, size) == INVALID_ARGUMENT
    assert host.MakeBC7ModeBuffer(wb, hb, src, len(data), pitch + 8, out, size) == INVALID_ARGUMENT
    assert host.MakeBC7ModeBuffer(wb, hb, src, len(data) - pitch, pitch, out, size) == INVALID_ARGUMENT
    assert host.MakeBC7ModeBuffer(wb, hb, src, len(data), pitch, out, size - 4) == INVALID_ARGUMENT
    assert b"mode buffer" in host.GetLastErrorMessage()
