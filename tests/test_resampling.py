"""Resampling copies: ReadChannels / WriteChannels at a size other than the mip's, and GenerateMips
(reference SetupBilinearFilter, CopyImageKernel, ResizeMultichannelImageKernel:
src/ImageProcessing.cu:24-72,178-265; src/TextureSet.cpp:1121-1142).

The checker is pinned by a numpy float64 statement of the filter (clamped position, bilinear weights)
and by exact cases; the kernels must equal the checker bit for bit (same fp32 operations)."""
import ctypes as C

import numpy as np
import pytest

from test_host_api import random_user_image, run_exe, BPC

FMT_DTYPE = {1: np.uint8, 2: np.uint16, 3: np.float16, 4: np.float32, 5: np.uint32}


def random_planar(rng, width, height, channels, wild=True):
    """Halves in the internal layout: values in [0, 1.2), and with `wild` also negative and large ones
    and the ends of the half range."""
    n = width * height * channels
    vals = rng.uniform(0.0, 1.2, n)
    if wild:
        pick = rng.random(n)
        vals = np.where(pick < 0.2, rng.standard_normal(n) * 300, vals)
        vals = np.where(pick > 0.98, np.sign(rng.standard_normal(n)) * 65504.0, vals)
    return vals.astype(np.float16).view(np.uint16)


def planar_to_pixels(planar_u16, width, height, channels):
    """[h][w][c] float64 view of an image in the internal layout."""
    return planar_u16.view(np.float16).reshape(height, channels // 2, width, 2).transpose(0, 2, 1, 3).reshape(height, width, channels).astype(np.float64)


def np_resample(src, dst_w, dst_h):
    """float64 bilinear resampling of [h][w][c] with the reference's position rule."""
    src_h, src_w = src.shape[:2]
    x = np.clip((np.arange(dst_w) + 0.5) / dst_w * src_w - 0.5, 0, src_w - 1)
    y = np.clip((np.arange(dst_h) + 0.5) / dst_h * src_h - 0.5, 0, src_h - 1)
    x0, y0 = np.floor(x).astype(int), np.floor(y).astype(int)
    fx, fy = (x - x0)[None, :, None], (y - y0)[:, None, None]
    x1, y1 = np.minimum(x0 + 1, src_w - 1), np.minimum(y0 + 1, src_h - 1)
    top = src[y0][:, x0] * (1 - fx) + src[y0][:, x1] * fx
    bottom = src[y1][:, x0] * (1 - fx) + src[y1][:, x1] * fx
    return top * (1 - fy) + bottom * fy


def oracle_resize(oracle, src, sw, sh, dw, dh, channels, spaces=None):
    dst = np.zeros(dw * dh * channels, dtype=np.uint16)
    cs = None if spaces is None else np.asarray(spaces, dtype=np.uint8).ctypes.data
    oracle.ntc_oracle_resize_planar(src.ctypes.data, sw, sh, dst.ctypes.data, dw, dh, channels, cs)
    return dst


def test_checker_resize_against_numpy(oracle):
    rng = np.random.default_rng(3)
    channels = 6
    for (sw, sh), (dw, dh) in (((64, 48), (32, 24)), ((37, 21), (18, 10)), ((5, 3), (2, 1)), ((16, 16), (40, 25)), ((9, 9), (9, 9)), ((1, 1), (4, 4))):
        src = random_planar(rng, sw, sh, channels, wild=False)
        got = planar_to_pixels(oracle_resize(oracle, src, sw, sh, dw, dh, channels), dw, dh, channels)
        want = np_resample(planar_to_pixels(src, sw, sh, channels), dw, dh)
        # fp32 position and blend, result rounded to half
        assert np.allclose(got, want, rtol=2e-3, atol=2e-3), ((sw, sh), (dw, dh), np.abs(got - want).max())
    # exact: a 2x reduction is the four texels of each block times 1/4, added in the order (x0,y0), (x1,y0), (x0,y1), (x1,y1)
    sw, sh = 32, 20
    src = random_planar(rng, sw, sh, channels)
    src[src == 0x7BFF] = 0x7800                              # keep the sums finite: four times 65504 / 4 rounds past the half range
    src[src == 0xFBFF] = 0xF800
    px = planar_to_pixels(src, sw, sh, channels).astype(np.float32)
    a, b, c, d = px[0::2, 0::2], px[0::2, 1::2], px[1::2, 0::2], px[1::2, 1::2]
    quarter = np.float32(0.25)
    want = (((a * quarter + b * quarter) + c * quarter) + d * quarter).astype(np.float16)
    got = oracle_resize(oracle, src, sw, sh, sw // 2, sh // 2, channels)
    assert np.array_equal(planar_to_pixels(got, sw // 2, sh // 2, channels), want.astype(np.float64))
    # exact: same size = copy; a constant image stays constant at any size
    assert np.array_equal(oracle_resize(oracle, src, sw, sh, sw, sh, channels), src)
    flat = np.full(sw * sh * channels, np.float16(0.375).view(np.uint16), dtype=np.uint16)
    assert np.all(oracle_resize(oracle, flat, sw, sh, 13, 7, channels) == np.float16(0.375).view(np.uint16))
    # sRGB storage: filtered in linear light, i.e. not the same as filtering the stored values
    spaces = [1] * 16
    src = random_planar(rng, sw, sh, channels, wild=False)
    linear = oracle_resize(oracle, src, sw, sh, sw // 2, sh // 2, channels)
    srgb = oracle_resize(oracle, src, sw, sh, sw // 2, sh // 2, channels, spaces)
    assert not np.array_equal(linear, srgb)
    stored = planar_to_pixels(src, sw, sh, channels)
    lin = np.where(stored <= 0.04045, stored / 12.92, ((np.abs(stored) + 0.055) / 1.055) ** 2.4)
    mean = np_resample(lin, sw // 2, sh // 2)
    back = np.where(mean <= 0.0031308, mean * 12.92, 1.055 * np.abs(mean) ** (1 / 2.4) - 0.055)
    assert np.allclose(planar_to_pixels(srgb, sw // 2, sh // 2, channels), back, rtol=3e-3, atol=3e-3)


def test_checker_resized_copies_agree_with_the_plain_ones(oracle):
    """Same-size calls of the resampling functions equal the 1:1 functions; resampled reads equal a
    planar resize followed by a 1:1 read when the format does not round (FLOAT32)."""
    rng = np.random.default_rng(4)
    w, h, channels = 23, 11, 8
    planar = random_planar(rng, w, h, channels, wild=False)
    for fmt in (1, 2, 3, 4):
        stride, pitch = BPC[fmt] * channels, BPC[fmt] * channels * w + 4 * BPC[fmt]
        plain = np.full(h * pitch, 0xEE, dtype=np.uint8)
        resized = plain.copy()
        assert oracle.ntc_oracle_read_channels(planar.ctypes.data, w, h, channels, 0, channels, plain.ctypes.data, fmt, stride, pitch) == 0
        assert oracle.ntc_oracle_read_channels_resized(planar.ctypes.data, w, h, channels, 0, channels, resized.ctypes.data, fmt, stride, pitch, w, h, 0, None, None) == 0
        assert np.array_equal(plain, resized), fmt
        back_plain = np.zeros(w * h * channels, dtype=np.uint16)
        back_resized = back_plain.copy()
        assert oracle.ntc_oracle_write_channels(plain.ctypes.data, fmt, 1, stride, pitch, back_plain.ctypes.data, w, h, channels, 0, channels) == 0
        assert oracle.ntc_oracle_write_channels_resized(plain.ctypes.data, fmt, 1, stride, pitch, w, h, back_resized.ctypes.data, w, h, channels, 0, channels, None, None) == 0
        assert np.array_equal(back_plain, back_resized), fmt
    dw, dh = 9, 14
    out = np.zeros(dw * dh * channels, dtype=np.float32)
    assert oracle.ntc_oracle_read_channels_resized(planar.ctypes.data, w, h, channels, 0, channels, out.ctypes.data, 4, 4 * channels, 4 * channels * dw, dw, dh, 0, None, None) == 0
    want = np_resample(planar_to_pixels(planar, w, h, channels), dw, dh)
    assert np.allclose(out.reshape(dh, dw, channels), want, rtol=1e-5, atol=1e-6)
    # and the write direction: FLOAT32 image of another size into the internal layout, flipped
    img = rng.random((dh, dw, channels)).astype(np.float32)
    got = np.zeros(w * h * channels, dtype=np.uint16)
    assert oracle.ntc_oracle_write_channels_resized(img.ctypes.data, 4, 1, 4 * channels, 4 * channels * dw, dw, dh, got.ctypes.data, w, h, channels, 0, channels, None, None) == 0
    want = np_resample(img.astype(np.float64), w, h)[::-1]
    assert np.allclose(planar_to_pixels(got, w, h, channels), want, rtol=2e-3, atol=1e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [1, 2, 3, 4, 5])
def test_gpu_resampled_copies_match_checker(ntc, device, oracle, fmt):
    rng = np.random.default_rng(40 + fmt)
    w, h, channels = 203, 61, 10
    planar = random_planar(rng, w, h, channels)
    d_planar = device.upload(planar)
    for (dw, dh), first, count, dither in (((101, 30), 0, 10, 0), ((64, 64), 3, 4, 1), ((300, 77), 9, 1, 0), ((1, 1), 0, 3, 0)):
        stride = BPC[fmt] * (count + 1)
        pitch = stride * dw + 2 * BPC[fmt]
        d_dst = device.upload(np.full(dh * pitch, 0xEE, dtype=np.uint8))
        rc = ntc.abi.ReadChannels()
        rc.planarPairs, rc.planarBytes, rc.width, rc.height, rc.setChannels = d_planar.ptr, d_planar.nbytes, w, h, channels
        rc.firstChannel, rc.numChannels, rc.dst, rc.dstBytes, rc.format = first, count, d_dst.ptr, d_dst.nbytes, fmt
        rc.pixelStride, rc.rowPitch, rc.dstWidth, rc.dstHeight, rc.useDithering = stride, pitch, dw, dh, dither
        ntc.abi.check(device.lib.ntc_hip_read_channels(rc))
        device.synchronize()
        want = np.full(dh * pitch, 0xEE, dtype=np.uint8)
        assert oracle.ntc_oracle_read_channels_resized(planar.ctypes.data, w, h, channels, first, count, want.ctypes.data, fmt, stride, pitch, dw, dh, dither, None, None) == 0
        assert np.array_equal(d_dst.download(), want), (fmt, dw, dh, first, count)
    # write direction
    for (sw, sh), first, count, flip in (((406, 122), 0, 10, 0), ((57, 200), 2, 5, 1), ((2, 3), 9, 1, 0)):
        img, _, stride, pitch = random_user_image(rng, fmt, sw, sh, count, 2 * BPC[fmt])
        start = np.full(w * h * channels, 0x1234, dtype=np.uint16)
        d_src, d_dst = device.upload(img), device.upload(start)
        wc = ntc.abi.WriteChannels()
        wc.src, wc.srcBytes, wc.format, wc.verticalFlip, wc.pixelStride, wc.rowPitch = d_src.ptr, d_src.nbytes, fmt, flip, stride, pitch
        wc.planarPairs, wc.planarBytes = d_dst.ptr, d_dst.nbytes
        wc.width, wc.height, wc.setChannels, wc.firstChannel, wc.numChannels, wc.srcWidth, wc.srcHeight = w, h, channels, first, count, sw, sh
        ntc.abi.check(device.lib.ntc_hip_write_channels(wc))
        device.synchronize()
        want = start.copy()
        assert oracle.ntc_oracle_write_channels_resized(img.ctypes.data, fmt, flip, stride, pitch, sw, sh, want.ctypes.data, w, h, channels, first, count, None, None) == 0
        assert np.array_equal(d_dst.download().view(np.uint16), want), (fmt, sw, sh, first, count, flip)
    # argument checks: one of the two sizes missing; image smaller than the stated size
    rc.dstWidth, rc.dstHeight = 5, 0
    assert device.lib.ntc_hip_read_channels(rc) == ntc.abi.ERR_INVALID_ARG
    wc.srcWidth, wc.srcHeight = 4000, 4000
    assert device.lib.ntc_hip_write_channels(wc) == ntc.abi.ERR_INVALID_ARG


@pytest.mark.gpu
def test_gpu_resize_planar_matches_checker(ntc, device, oracle):
    rng = np.random.default_rng(46)
    channels = 16
    for (sw, sh), (dw, dh), spaces in (((256, 128), (128, 64), None), ((255, 127), (127, 63), None), ((3, 5), (1, 2), None), ((64, 64), (100, 30), None)):
        src = random_planar(rng, sw, sh, channels)
        d_src, d_dst = device.upload(src), device.upload(np.zeros(dw * dh * channels, dtype=np.uint16))
        ntc.abi.check(device.lib.ntc_hip_resize_planar(d_src.ptr, d_src.nbytes, sw, sh, d_dst.ptr, d_dst.nbytes, dw, dh, channels, None))
        device.synchronize()
        assert np.array_equal(d_dst.download().view(np.uint16), oracle_resize(oracle, src, sw, sh, dw, dh, channels)), ((sw, sh), (dw, dh))
    # sRGB storage: transfer functions come from each side's math library, one half ulp of slack
    sw, sh, dw, dh = 128, 64, 64, 32
    src = random_planar(rng, sw, sh, channels, wild=False)
    spaces = np.array([1, 0, 2, 1] * 4, dtype=np.uint8)
    d_src, d_dst = device.upload(src), device.upload(np.zeros(dw * dh * channels, dtype=np.uint16))
    ntc.abi.check(device.lib.ntc_hip_resize_planar(d_src.ptr, d_src.nbytes, sw, sh, d_dst.ptr, d_dst.nbytes, dw, dh, channels, spaces.ctypes.data))
    device.synchronize()
    got = d_dst.download().view(np.uint16).astype(np.int32)
    want = oracle_resize(oracle, src, sw, sh, dw, dh, channels, spaces).astype(np.int32)
    assert np.abs(got - want).max() <= 1
    assert device.lib.ntc_hip_resize_planar(d_src.ptr, d_src.nbytes, sw, sh, d_src.ptr, d_src.nbytes, dw, dh, channels, None) == ntc.abi.ERR_INVALID_ARG
    assert device.lib.ntc_hip_resize_planar(d_src.ptr, d_src.nbytes - 2, sw, sh, d_dst.ptr, d_dst.nbytes, dw, dh, channels, None) == ntc.abi.ERR_INVALID_ARG


@pytest.mark.gpu
def test_host_layer_generate_mips(ntc, oracle, tmp_path):
    """WriteChannels from an image of twice the size of mip 0, GenerateMips, and the reference page of
    every mip against the checker's chain of resamplings (channel 1 stored as sRGB)."""
    w, h, channels, mips = 48, 20, 6, 5
    rng = np.random.default_rng(47)
    image = rng.random((2 * h, 2 * w, channels)).astype(np.float32)
    path = tmp_path / "image.bin"
    image.tofile(path)
    prefix = str(tmp_path / "out")
    assert "host genmips OK" in run_exe("genmips", w, h, channels, mips, path, prefix)
    spaces = np.zeros(16, dtype=np.uint8)
    spaces[1] = 1
    linear = np.zeros(16, dtype=np.uint8)
    level = np.zeros(w * h * channels, dtype=np.uint16)
    assert oracle.ntc_oracle_write_channels_resized(image.ctypes.data, 4, 0, 4 * channels, 4 * channels * 2 * w, 2 * w, 2 * h, level.ctypes.data,
                                                    w, h, channels, 0, channels, linear.ctypes.data, spaces.ctypes.data) == 0
    mw, mh = w, h
    for mip in range(mips):
        got = np.fromfile(f"{prefix}_mip{mip}.bin", dtype=np.uint16).astype(np.int32)
        want = level.reshape(mh, channels // 2, mw, 2).transpose(0, 2, 1, 3).reshape(-1).astype(np.int32)
        slack = np.where(np.arange(got.size) % channels == 1, 1 + mip, 0)    # the sRGB channel: one half ulp per pass through the transfer functions
        assert np.all(np.abs(got - want) <= slack), mip
        nw, nh = max(mw // 2, 1), max(mh // 2, 1)
        level = oracle_resize(oracle, level, mw, mh, nw, nh, channels, spaces)
        mw, mh = nw, nh
