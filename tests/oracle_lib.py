"""ctypes bindings of the CPU checker (oracle/libntc_oracle.so) and, when it was built, of
the reference's own host-only sources (oracle/_ref/libntc_ref_host.so).  Test-side only."""
import ctypes as C
import importlib
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_PATH = os.path.join(ROOT, "oracle", "libntc_oracle.so")
REF_PATH = os.path.join(ROOT, "oracle", "_ref", "libntc_ref_host.so")

_abi = importlib.import_module("rtxntc-library_amd").abi
_oracle = None
_ref = None


def load_oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_PATH):
            raise ImportError(f"{ORACLE_PATH} is not built; run make -C oracle")
        lib = C.CDLL(ORACLE_PATH)
        lib.ntc_oracle_weight_layout.restype = C.c_int
        lib.ntc_oracle_weight_layout.argtypes = [C.POINTER(_abi.DecoderSpec), C.POINTER(_abi.WeightLayout)]
        lib.ntc_oracle_float_to_half.restype = C.c_uint16
        lib.ntc_oracle_float_to_half.argtypes = [C.c_float]
        lib.ntc_oracle_half_to_float.restype = C.c_float
        lib.ntc_oracle_half_to_float.argtypes = [C.c_uint16]
        lib.ntc_oracle_output_to_half.restype = C.c_uint16
        lib.ntc_oracle_output_to_half.argtypes = [C.c_float]
        lib.ntc_oracle_half_to_unorm8.restype = C.c_uint8
        lib.ntc_oracle_half_to_unorm8.argtypes = [C.c_uint16]
        lib.ntc_oracle_hgelu_quantize.restype = C.c_int
        lib.ntc_oracle_hgelu_quantize.argtypes = [C.c_float]
        lib.ntc_oracle_unpack_field.restype = C.c_int
        lib.ntc_oracle_unpack_field.argtypes = [C.c_uint16, C.c_int, C.c_int]
        lib.ntc_oracle_e4m3_times_512.restype = C.c_int32
        lib.ntc_oracle_e4m3_times_512.argtypes = [C.c_uint8]
        lib.ntc_oracle_layer_int8.restype = None
        lib.ntc_oracle_layer_int8.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        lib.ntc_oracle_quantize_value.restype = C.c_uint32
        lib.ntc_oracle_quantize_value.argtypes = [C.c_float, C.c_int]
        lib.ntc_oracle_encode_position.restype = None
        lib.ntc_oracle_encode_position.argtypes = [C.c_float, C.c_float, C.c_float, C.c_int, C.c_int, C.c_void_p]
        lib.ntc_oracle_bilinear_footprint.restype = None
        lib.ntc_oracle_bilinear_footprint.argtypes = [C.c_float, C.c_float, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        lib.ntc_oracle_decode_texel.restype = C.c_int
        lib.ntc_oracle_decode_texel.argtypes = [C.POINTER(_abi.TextureSet), C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        lib.ntc_oracle_ref_geometry.restype = C.c_int
        lib.ntc_oracle_ref_geometry.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(_abi.MipDesc), C.POINTER(C.c_uint64)]
        lib.ntc_oracle_decode.restype = C.c_double
        lib.ntc_oracle_decode.argtypes = [C.POINTER(_abi.TextureSet), C.c_int]
        lib.ntc_oracle_decode_rows.restype = C.c_double
        lib.ntc_oracle_decode_rows.argtypes = [C.POINTER(_abi.TextureSet), C.c_int, C.c_int, C.c_int, C.c_int]
        lib.ntc_oracle_decode_queries.restype = C.c_int
        lib.ntc_oracle_decode_queries.argtypes = [C.POINTER(_abi.TextureSet), C.c_void_p, C.c_uint64, C.c_void_p, C.c_int]
        lib.ntc_oracle_write_channels.restype = C.c_int
        lib.ntc_oracle_write_channels.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_uint64, C.c_uint64, C.c_void_p,
                                                  C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        lib.ntc_oracle_read_channels_ex.restype = C.c_int
        lib.ntc_oracle_read_channels_ex.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int,
                                                    C.c_uint64, C.c_uint64, C.c_int, C.c_void_p, C.c_void_p]
        lib.ntc_oracle_write_channels_ex.restype = C.c_int
        lib.ntc_oracle_write_channels_ex.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_uint64, C.c_uint64, C.c_void_p,
                                                     C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        lib.ntc_oracle_dither_float.restype = C.c_float
        lib.ntc_oracle_dither_float.argtypes = [C.c_uint32, C.c_int]
        lib.ntc_oracle_image_loss.restype = None
        lib.ntc_oracle_image_loss.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_uint32, C.c_void_p]
        lib.ntc_oracle_read_channels_resized.restype = C.c_int
        lib.ntc_oracle_read_channels_resized.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int,
                                                         C.c_uint64, C.c_uint64, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        lib.ntc_oracle_write_channels_resized.restype = C.c_int
        lib.ntc_oracle_write_channels_resized.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_uint64, C.c_uint64, C.c_int, C.c_int, C.c_void_p,
                                                          C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        lib.ntc_oracle_resize_planar.restype = None
        lib.ntc_oracle_resize_planar.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
        lib.ntc_oracle_block_compress.restype = C.c_int
        lib.ntc_oracle_block_compress.argtypes = [C.c_void_p]
        lib.ntc_oracle_bc6_log2.restype = C.c_float
        lib.ntc_oracle_bc6_log2.argtypes = [C.c_float]
        lib.ntc_oracle_bc6_exp2.restype = C.c_float
        lib.ntc_oracle_bc6_exp2.argtypes = [C.c_float]
        lib.ntc_oracle_bc7_tables.restype = None
        lib.ntc_oracle_bc7_tables.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        lib.ntc_oracle_bc1_match_tables.restype = None
        lib.ntc_oracle_bc1_match_tables.argtypes = [C.c_void_p, C.c_void_p]
        lib.ntc_oracle_image_difference.restype = None
        lib.ntc_oracle_image_difference.argtypes = [C.c_void_p, C.c_void_p]
        lib.ntc_oracle_image_loss_masked.restype = None
        lib.ntc_oracle_image_loss_masked.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_uint32, C.c_int, C.c_int, C.c_void_p]
        lib.ntc_oracle_read_channels.restype = C.c_int
        lib.ntc_oracle_read_channels.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                                 C.c_int, C.c_uint64, C.c_uint64]
        _oracle = lib
    return _oracle


def load_ref():
    """The reference's own host code, or None when oracle/_ref was not built."""
    global _ref
    if _ref is None and os.path.exists(REF_PATH):
        lib = C.CDLL(REF_PATH)
        lib.ntc_ref_weight_layout.restype = C.c_int
        lib.ntc_ref_weight_layout.argtypes = [C.c_int, C.POINTER(C.c_uint64)]
        lib.ntc_ref_mlp_geometry.restype = None
        lib.ntc_ref_mlp_geometry.argtypes = [C.POINTER(C.c_int)]
        for name in ("ntc_ref_lod_to_neural_lod", "ntc_ref_grid_dimension", "ntc_ref_num_neural_mips"):
            getattr(lib, name).restype = C.c_int
            getattr(lib, name).argtypes = [C.c_int, C.c_int, C.c_int]
        lib.ntc_ref_quantized_latents_size.restype = C.c_uint64
        lib.ntc_ref_quantized_latents_size.argtypes = [C.c_int] * 5
        _ref = lib
    return _ref


class HostSet:
    """A texture set whose latents / weights / output live in numpy arrays (for the oracle)."""

    FILL = 0xCD   # bytes the decoder must leave alone keep this pattern (same fill as the device buffer)

    def __init__(self, ntc, spec, mips, num_channels, output_format, latents, weights, output_bytes, pixel_stride=0):
        self.latents = np.ascontiguousarray(latents)
        self.weights = np.ascontiguousarray(weights)
        self.output = np.full(output_bytes, self.FILL, dtype=np.uint8)
        self.desc = ntc.make_texture_set(
            spec, mips, num_channels, output_format,
            self.latents.ctypes.data, self.latents.nbytes, self.weights.ctypes.data, self.weights.nbytes,
            self.output.ctypes.data, self.output.nbytes, pixel_stride)

    def decode(self, threads=8):
        t = load_oracle().ntc_oracle_decode(self.desc, threads)
        assert t >= 0
        return t
