"""ctypes view of include/ntc_hip.h: the structs, the loader and the error type.

The shared library is built in-tree (csrc/libntc_hip.so) by __graft_entry__.build();
loading fails loudly when it is missing - there is no CPU decode path in this package.
"""
import ctypes as C
import os

MAX_MIPS = 16
MAX_CHANNELS = 16
MLP_LAYERS = 4

GRID_BILINEAR, GRID_CONCAT2X2 = 0, 1
WEIGHTS_INT8, WEIGHTS_FP8, WEIGHTS_FP8_SCALED = 0, 1, 2
OUT_FP16_PLANAR_PAIRS, OUT_FP16_PIXELS, OUT_UNORM8_PIXELS = 0, 1, 2

ERR_INVALID_ARG, ERR_UNSUPPORTED, ERR_NO_DEVICE, ERR_NOT_INITIALIZED = -1, -2, -3, -4


class DecoderSpec(C.Structure):
    _fields_ = [
        ("hrFeatures", C.c_int32), ("hrBits", C.c_int32), ("hrMode", C.c_int32), ("hrFeatureSlots", C.c_int32),
        ("lrFeatures", C.c_int32), ("lrBits", C.c_int32), ("lrMode", C.c_int32), ("lrFeatureSlots", C.c_int32),
        ("posEncWaves", C.c_int32), ("lodInputs", C.c_int32), ("inputChannels", C.c_int32),
        ("hiddenChannels", C.c_int32 * (MLP_LAYERS - 1)), ("outputChannels", C.c_int32), ("weightType", C.c_int32),
    ]

    def layer_inputs(self, layer):
        return self.inputChannels if layer == 0 else self.hiddenChannels[layer - 1]

    def layer_outputs(self, layer):
        return self.outputChannels if layer == MLP_LAYERS - 1 else self.hiddenChannels[layer]

    def hr_inputs(self):
        return (4 if self.hrMode == GRID_CONCAT2X2 else 1) * self.hrFeatureSlots

    def lr_inputs(self):
        return (4 if self.lrMode == GRID_CONCAT2X2 else 1) * self.lrFeatureSlots

    def copy(self):
        out = DecoderSpec()
        C.memmove(C.byref(out), C.byref(self), C.sizeof(DecoderSpec))
        return out


class WeightLayout(C.Structure):
    _fields_ = [
        ("weightOffset", C.c_uint32 * MLP_LAYERS), ("scaleOffset", C.c_uint32 * MLP_LAYERS),
        ("biasOffset", C.c_uint32 * MLP_LAYERS), ("bufferSize", C.c_uint32),
    ]


class MipDesc(C.Structure):
    _fields_ = [
        ("width", C.c_int32), ("height", C.c_int32), ("hrWidth", C.c_int32), ("hrHeight", C.c_int32),
        ("lrWidth", C.c_int32), ("lrHeight", C.c_int32), ("positionScale", C.c_float), ("positionLod", C.c_float),
        ("hrOffset", C.c_uint64), ("lrOffset", C.c_uint64), ("outOffset", C.c_uint64), ("outRowPitch", C.c_uint64),
    ]


class TextureSet(C.Structure):
    _fields_ = [
        ("spec", DecoderSpec), ("numMips", C.c_int32), ("numChannels", C.c_int32),
        ("outputFormat", C.c_int32), ("outPixelStride", C.c_int32),
        ("latents", C.c_void_p), ("weights", C.c_void_p), ("output", C.c_void_p),
        ("latentsBytes", C.c_uint64), ("weightsBytes", C.c_uint64), ("outputBytes", C.c_uint64),
        ("mips", MipDesc * MAX_MIPS),
        ("queryLatents", C.c_void_p), ("queryLatentsBytes", C.c_uint64),
    ]


class ReadChannels(C.Structure):
    _fields_ = [
        ("planarPairs", C.c_void_p), ("planarBytes", C.c_uint64), ("width", C.c_int32), ("height", C.c_int32),
        ("setChannels", C.c_int32), ("firstChannel", C.c_int32), ("numChannels", C.c_int32),
        ("dst", C.c_void_p), ("dstBytes", C.c_uint64), ("format", C.c_int32), ("useDithering", C.c_int32),
        ("pixelStride", C.c_uint64), ("rowPitch", C.c_uint64),
        ("srcColorSpaces", C.c_uint8 * 16), ("dstColorSpaces", C.c_uint8 * 16),
        ("dstWidth", C.c_int32), ("dstHeight", C.c_int32),
    ]


class WriteChannels(C.Structure):
    _fields_ = [
        ("src", C.c_void_p), ("srcBytes", C.c_uint64), ("format", C.c_int32), ("verticalFlip", C.c_int32),
        ("pixelStride", C.c_uint64), ("rowPitch", C.c_uint64), ("planarPairs", C.c_void_p), ("planarBytes", C.c_uint64),
        ("width", C.c_int32), ("height", C.c_int32), ("setChannels", C.c_int32), ("firstChannel", C.c_int32),
        ("numChannels", C.c_int32), ("reserved", C.c_int32),
        ("srcColorSpaces", C.c_uint8 * 16), ("dstColorSpaces", C.c_uint8 * 16),
        ("srcWidth", C.c_int32), ("srcHeight", C.c_int32),
    ]


class Image(C.Structure):
    _fields_ = [
        ("data", C.c_void_p), ("bytes", C.c_uint64), ("pixelStride", C.c_uint64), ("rowPitch", C.c_uint64),
        ("width", C.c_int32), ("height", C.c_int32), ("format", C.c_int32), ("numChannels", C.c_int32),
    ]


class ImageDifference(C.Structure):
    _fields_ = [
        ("a", Image), ("b", Image),
        ("left", C.c_int32), ("top", C.c_int32), ("width", C.c_int32), ("height", C.c_int32),
        ("alphaThreshold", C.c_float), ("useAlphaThreshold", C.c_int32), ("useMSLE", C.c_int32), ("outputOffset", C.c_uint32),
        ("output", C.c_void_p), ("outputBytes", C.c_uint64),
    ]


class BlockCompress(C.Structure):
    _fields_ = [
        ("src", Image), ("srcLeft", C.c_int32), ("srcTop", C.c_int32), ("widthInBlocks", C.c_int32), ("heightInBlocks", C.c_int32),
        ("dstFormat", C.c_int32), ("dstOffsetX", C.c_int32), ("dstOffsetY", C.c_int32), ("alphaThreshold", C.c_float),
        ("dst", C.c_void_p), ("dstBytes", C.c_uint64), ("dstRowPitch", C.c_uint64),
        ("modeBuffer", C.c_void_p), ("modeBufferBytes", C.c_uint64), ("modeBufferByteOffset", C.c_uint64),
        ("modeMapWidthInBlocks", C.c_int32), ("modeMapHeightInBlocks", C.c_int32), ("modeMapOffsetX", C.c_int32), ("modeMapOffsetY", C.c_int32),
    ]


class Query(C.Structure):
    _fields_ = [("u", C.c_float), ("v", C.c_float), ("mip", C.c_int32)]


FORMAT_UNORM8, FORMAT_UNORM16, FORMAT_FLOAT16, FORMAT_FLOAT32, FORMAT_UINT32 = 1, 2, 3, 4, 5


class NtcHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"ntc_hip error {code}: {message}")
        self.code = code
        self.message = message


# Every symbol include/ntc_hip.h declares: (name, restype, argtypes)
EXPORTS = [
    ("ntc_hip_init", C.c_int, [C.c_int]),
    ("ntc_hip_shutdown", None, []),
    ("ntc_hip_last_error", C.c_char_p, []),
    ("ntc_hip_device_info", C.c_int, [C.c_char_p, C.c_size_t, C.POINTER(C.c_int)]),
    ("ntc_hip_device_clock", C.c_int, [C.POINTER(C.c_int)]),
    ("ntc_hip_alloc", C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    ("ntc_hip_free", C.c_int, [C.c_void_p]),
    ("ntc_hip_upload", C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    ("ntc_hip_download", C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    ("ntc_hip_memset", C.c_int, [C.c_void_p, C.c_int, C.c_size_t]),
    ("ntc_hip_synchronize", C.c_int, []),
    ("ntc_hip_weight_layout", C.c_int, [C.POINTER(DecoderSpec), C.POINTER(WeightLayout)]),
    ("ntc_hip_grid_bytes", C.c_uint64, [C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    ("ntc_hip_decode", C.c_int, [C.POINTER(TextureSet), C.c_int32]),
    ("ntc_hip_decode_static", C.c_int, [C.POINTER(TextureSet), C.c_int32]),
    ("ntc_hip_decode_timed", C.c_int, [C.POINTER(TextureSet), C.c_int32, C.c_int32, C.POINTER(C.c_float)]),
    ("ntc_hip_timer_begin", C.c_int, []),
    ("ntc_hip_timer_end", C.c_int, [C.POINTER(C.c_float)]),
    ("ntc_hip_decode_queries", C.c_int, [C.POINTER(TextureSet), C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64]),
    ("ntc_hip_decode_queries_timed", C.c_int, [C.POINTER(TextureSet), C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64,
                                               C.c_int32, C.POINTER(C.c_float)]),
    ("ntc_hip_query_latents_bytes", C.c_uint64, [C.POINTER(TextureSet)]),
    ("ntc_hip_build_query_latents", C.c_int, [C.POINTER(TextureSet), C.c_void_p, C.c_uint64]),
    ("ntc_hip_read_channels", C.c_int, [C.POINTER(ReadChannels)]),
    ("ntc_hip_write_channels", C.c_int, [C.POINTER(WriteChannels)]),
    ("ntc_hip_image_loss", C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int32, C.c_int32, C.c_int32, C.c_uint32, C.c_int32, C.c_int32,
                                     C.POINTER(C.c_float)]),
    ("ntc_hip_image_difference", C.c_int, [C.POINTER(ImageDifference)]),
    ("ntc_hip_block_compress", C.c_int, [C.POINTER(BlockCompress)]),
    ("ntc_hip_resize_planar", C.c_int, [C.c_void_p, C.c_uint64, C.c_int32, C.c_int32, C.c_void_p, C.c_uint64, C.c_int32, C.c_int32,
                                        C.c_int32, C.c_void_p]),
    ("ntc_hip_selftest_mfma", C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    ("ntc_hip_selftest_mfma_f16", C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32]),
    ("ntc_hip_selftest_fp8_activation", C.c_int, [C.c_void_p, C.c_int32, C.c_void_p]),
]

# The context forms: ntc_hip_ctx_<name>(context, same arguments); ntc_hip_create / ntc_hip_destroy.
_CONTEXT_FORMS = ["device_info", "device_clock", "alloc", "free", "upload", "download", "memset", "synchronize", "decode",
                  "decode_static", "decode_timed", "timer_begin", "timer_end", "build_query_latents", "decode_queries", "decode_queries_timed", "read_channels",
                  "write_channels", "image_loss", "resize_planar", "image_difference", "block_compress"]
_BY_NAME = {name: (restype, argtypes) for name, restype, argtypes in EXPORTS}
EXPORTS += [("ntc_hip_ctx_" + n, _BY_NAME["ntc_hip_" + n][0], [C.c_void_p] + _BY_NAME["ntc_hip_" + n][1]) for n in _CONTEXT_FORMS]
EXPORTS += [("ntc_hip_create", C.c_int, [C.c_int, C.POINTER(C.c_void_p)]), ("ntc_hip_destroy", None, [C.c_void_p])]

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libntc_hip.so")
_lib = None


def load_library():
    """Loads csrc/libntc_hip.so and types every export.  Raises if the library is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is not built; run __graft_entry__.build() (make -C rtxntc-library_amd/csrc)")
        lib = C.CDLL(LIB_PATH)
        for name, restype, argtypes in EXPORTS:
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(code):
    if code != 0:
        raise NtcHipError(code, load_library().ntc_hip_last_error().decode("utf-8", "replace"))
