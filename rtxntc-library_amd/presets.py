"""Decoder specs and mip-chain geometry.

ref092  : the geometry compiled into the mounted LibNTC 0.9.2
          (include/libntc/shaders/InferenceConstants.h:26-40; both grids bilinear, 4-bit).
cfg01   : 2x2-concat high-res grid of 8 x 2-bit features + bilinear low-res grid of
          16 x 4-bit features + 12 positional inputs = 60 -> 64, MLP 64-48-32, 16 outputs.
cfg2    : same high-res grid, 12 low-res features (56 -> 64 inputs), MLP 48-48-32.
cfg3    : both grids bilinear 16 x 4-bit, MLP 64-64-64, hidden-layer weights stored as FP8 e4m3.
"""
import math

import numpy as np

from . import abi


def make_spec(hr, lr, lod_inputs, input_channels, hidden, weight_type=abi.WEIGHTS_INT8):
    s = abi.DecoderSpec()
    s.hrFeatures, s.hrBits, s.hrMode, s.hrFeatureSlots = hr
    s.lrFeatures, s.lrBits, s.lrMode, s.lrFeatureSlots = lr
    s.posEncWaves = 3
    s.lodInputs = lod_inputs
    s.inputChannels = input_channels
    for i, h in enumerate(hidden):
        s.hiddenChannels[i] = h
    s.outputChannels = 16
    s.weightType = weight_type
    return s


def spec_ref092(num_features=16):
    return make_spec((num_features, 4, abi.GRID_BILINEAR, 16), (num_features, 4, abi.GRID_BILINEAR, 16), 2, 48, (64, 48, 32))


def spec_ref092_fp8(num_features=16):
    """The same decoder with the FP8 version of the network (GenericFP8 weight blob)."""
    s = spec_ref092(num_features)
    s.weightType = abi.WEIGHTS_FP8
    return s


def spec_cfg01():
    return make_spec((8, 2, abi.GRID_CONCAT2X2, 8), (16, 4, abi.GRID_BILINEAR, 16), 0, 64, (64, 48, 32))


def spec_cfg2():
    return make_spec((8, 2, abi.GRID_CONCAT2X2, 8), (12, 4, abi.GRID_BILINEAR, 12), 0, 64, (48, 48, 32))


def spec_cfg3():
    """Wide decoder with e4m3 hidden-layer weights: both grids bilinear 16 x 4-bit, (lod, lod), 48 -> 64-64-64 -> 16."""
    return make_spec((16, 4, abi.GRID_BILINEAR, 16), (16, 4, abi.GRID_BILINEAR, 16), 2, 48, (64, 64, 64),
                     abi.WEIGHTS_FP8_SCALED)


def grid_bytes(width, height, features, bits):
    per_word = 16 // bits
    return width * height * 2 * ((features + per_word - 1) // per_word)


def full_mip_count(width, height):
    return int(math.floor(math.log2(max(width, height)))) + 1


def _position_constants(hr_w, hr_h, w, h):
    # reference src/TextureSet.cpp:456-461, in fp32
    ws = np.float32(hr_w) / np.float32(w)
    hs = np.float32(hr_h) / np.float32(h)
    scale = np.float32(0.5) * max(ws, hs)
    lod = max(np.float32(-1.0), min(np.float32(1.0), np.float32(0.25) * np.float32(np.log2(scale))))
    return float(scale), float(lod)


def mips_private_grids(spec, width, height, num_mips, hr_div=2, lr_div=4):
    """Per-mip private latent grids: HR (W/hr_div)x(H/hr_div), LR (W/lr_div)x(H/lr_div), min 1.

    Returns (list of MipDesc without output offsets, total latent bytes).  Grids are laid out
    mip after mip, HR grid then LR grid.
    """
    mips, cursor = [], 0
    for m in range(num_mips):
        d = abi.MipDesc()
        d.width, d.height = max(width >> m, 1), max(height >> m, 1)
        d.hrWidth, d.hrHeight = max(d.width // hr_div, 1), max(d.height // hr_div, 1)
        d.lrWidth, d.lrHeight = max(d.width // lr_div, 1), max(d.height // lr_div, 1)
        d.positionScale, d.positionLod = _position_constants(d.hrWidth, d.hrHeight, d.width, d.height)
        d.hrOffset = cursor
        cursor += grid_bytes(d.hrWidth, d.hrHeight, spec.hrFeatures, spec.hrBits)
        d.lrOffset = cursor
        cursor += grid_bytes(d.lrWidth, d.lrHeight, spec.lrFeatures, spec.lrBits)
        mips.append(d)
    return mips, cursor


_SHARED_MIPS = (2, 3, 3, 3, 4, 4)  # reference src/FeatureGridMath.cpp:51-53


def mips_ref092(spec, width, height, num_mips, grid_size_scale):
    """Neural-LOD geometry of LibNTC 0.9.2 (src/FeatureGridMath.cpp:47-77,
    src/FeatureGridHost.cpp:27-58, src/TextureSet.cpp:441-463,1816-1817)."""
    assert 1 <= grid_size_scale <= 6
    shared = _SHARED_MIPS[grid_size_scale - 1]

    def lod_to_neural(lod, neural_lods):
        return max(0, min(((lod - shared + 2) & ~1), neural_lods - 2))

    def grid_dim(dim, nlod):
        return max((dim // grid_size_scale) >> nlod, 1)

    min_grid = int(np.float32(min(width, height)) / np.float32(grid_size_scale))
    num_neural = max(2, int(1.0 + math.floor(math.log2(min_grid)))) & ~1
    num_neural = min(num_neural, lod_to_neural(num_mips - 1, 8) + 2)
    layers = (spec.hrFeatures + 3) // 4
    offsets = [0]
    for n in range(num_neural):
        offsets.append(offsets[-1] + grid_dim(width, n) * grid_dim(height, n) * 2 * layers)
    mips = []
    for m in range(num_mips):
        nlod = lod_to_neural(m, num_neural)
        d = abi.MipDesc()
        d.width, d.height = max(width >> m, 1), max(height >> m, 1)
        d.hrWidth, d.hrHeight = grid_dim(width, nlod), grid_dim(height, nlod)
        d.lrWidth, d.lrHeight = max(d.hrWidth >> 1, 1), max(d.hrHeight >> 1, 1)
        d.positionScale, d.positionLod = _position_constants(d.hrWidth, d.hrHeight, d.width, d.height)
        d.hrOffset, d.lrOffset = offsets[nlod], offsets[nlod + 1]
        mips.append(d)
    return mips, offsets[-1]


def assign_output_offsets(mips, num_channels, output_format, pixel_stride=None):
    """Packs the mips one after another in the output buffer.  Returns (pixel stride, total bytes).

    Planar pairs follow the reference's mip offsets (src/TextureSet.cpp:88-101): mip m starts
    at sum of earlier mips' texel counts x even channel count.
    """
    cursor = 0
    if output_format == abi.OUT_FP16_PLANAR_PAIRS:
        c2 = (num_channels + 1) & ~1
        for d in mips:
            d.outOffset, d.outRowPitch = cursor, 0
            cursor += d.width * d.height * c2 * 2
        return 0, cursor
    bpc = 1 if output_format == abi.OUT_UNORM8_PIXELS else 2
    stride = pixel_stride if pixel_stride is not None else num_channels * bpc
    for d in mips:
        d.outOffset, d.outRowPitch = cursor, d.width * stride
        cursor += d.height * d.outRowPitch
        cursor = (cursor + 15) & ~15
    return stride, cursor
