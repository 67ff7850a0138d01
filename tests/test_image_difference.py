"""Image-difference pass (reference src/shaders/ImageDifference.hlsl behind
IContext::MakeImageDifferenceComputePass): per-channel MSE / MSLE of a rectangle of two images,
accumulated as 16.48 fixed point.

The checker is pinned by numpy float64 statements of the definition (to the fp32 accumulation
error) and by cases whose fixed-point result is exact; the GPU must equal the checker bit for bit
in MSE mode (same fp32 operations in the same order) and to 1e-5 in MSLE mode (device logf)."""
import ctypes as C

import numpy as np
import pytest

BPC = {1: 1, 2: 2, 3: 2, 4: 4, 5: 4}
DTYPE = {1: np.uint8, 2: np.uint16, 3: np.float16, 4: np.float32, 5: np.uint32}


def make_image(rng, fmt, width, height, channels, pad_pixels=0, pad_rows=0, other=None, noise=0.05):
    """(raw bytes as uint8 array, float64 values [h][w][4] with defaults 0,0,0,1, pixelStride, rowPitch)."""
    if fmt in (1, 2):
        top = 255 if fmt == 1 else 65535
        if other is None:
            codes = rng.integers(0, top + 1, (height, width, channels))
        else:
            codes = np.clip(np.rint(other[:, :, :channels] * top + rng.normal(0, noise * top, (height, width, channels))), 0, top)
        stored = codes.astype(DTYPE[fmt])
        values = stored.astype(np.float32) / np.float32(top)
    elif fmt == 5:
        stored = rng.integers(0, 6, (height, width, channels)).astype(np.uint32)
        values = stored.astype(np.float32)
    else:
        base = rng.random((height, width, channels)) * 2 - 0.5 if other is None else other[:, :, :channels] + rng.normal(0, noise, (height, width, channels))
        stored = base.astype(DTYPE[fmt])
        values = stored.astype(np.float32)
    stride = BPC[fmt] * (channels + pad_pixels)
    pitch = stride * width + BPC[fmt] * pad_rows
    raw = np.full(height * pitch, 0xA5, dtype=np.uint8)
    rows = np.lib.stride_tricks.as_strided(raw, shape=(height, width, channels * BPC[fmt]), strides=(pitch, stride, 1))
    rows[...] = stored.view(np.uint8).reshape(height, width, channels * BPC[fmt])
    full = np.zeros((height, width, 4), dtype=np.float64)
    full[:, :, 3] = 1.0
    full[:, :, :channels] = values.astype(np.float64)
    return raw, full, stride, pitch


def fill_image(abi_image, ptr, nbytes, stride, pitch, width, height, fmt, channels):
    abi_image.data, abi_image.bytes, abi_image.pixelStride, abi_image.rowPitch = ptr, nbytes, stride, pitch
    abi_image.width, abi_image.height, abi_image.format, abi_image.numChannels = width, height, fmt, channels


def np_difference(va, vb, left, top, width, height, alpha_threshold=None, msle=False):
    a = va[top: top + height, left: left + width]
    b = vb[top: top + height, left: left + width]
    diff = np.log(np.abs(a) + 1) - np.log(np.abs(b) + 1) if msle else a - b
    if alpha_threshold is not None:
        transparent = (a[:, :, 3] < np.float32(alpha_threshold)) & (b[:, :, 3] < np.float32(alpha_threshold))
        diff = diff.copy()
        diff[transparent, :3] = 0
    return (diff ** 2).mean(axis=(0, 1))


def decode(fixed):
    return np.array([float(v) * 2.0 ** -48 for v in fixed])


def oracle_difference(ntc, oracle, raw_a, raw_b, desc_a, desc_b, extent, alpha_threshold=None, msle=False, start=(0, 0, 0, 0)):
    p = ntc.abi.ImageDifference()
    fill_image(p.a, raw_a.ctypes.data, raw_a.nbytes, *desc_a)
    fill_image(p.b, raw_b.ctypes.data, raw_b.nbytes, *desc_b)
    p.left, p.top, p.width, p.height = extent
    p.alphaThreshold = 0.0 if alpha_threshold is None else alpha_threshold
    p.useAlphaThreshold, p.useMSLE = int(alpha_threshold is not None), int(msle)
    out = (C.c_uint64 * 4)(*start)
    oracle.ntc_oracle_image_difference(C.byref(p), out)
    return list(out)


def test_checker_against_numpy(ntc, oracle):
    rng = np.random.default_rng(11)
    w, h = 200, 150
    for fmt, channels in ((1, 4), (2, 4), (3, 4), (4, 4), (1, 3), (4, 2), (5, 4)):
        raw_a, va, stride, pitch = make_image(rng, fmt, w, h, channels, pad_pixels=1, pad_rows=3)
        raw_b, vb, _, _ = make_image(rng, fmt, w, h, channels, pad_pixels=1, pad_rows=3, other=va)
        desc = (stride, pitch, w, h, fmt, channels)
        for extent in ((0, 0, w, h), (5, 7, 130, 100), (199, 149, 1, 1), (64, 0, 64, 64)):
            got = decode(oracle_difference(ntc, oracle, raw_a, raw_b, desc, desc, extent))
            want = np_difference(va, vb, *extent)
            assert np.allclose(got, want, rtol=2e-5, atol=2.0 ** -47), (fmt, channels, extent, got, want)
        for thr in (0.3, 0.9):
            got = decode(oracle_difference(ntc, oracle, raw_a, raw_b, desc, desc, (3, 2, 150, 120), alpha_threshold=thr))
            want = np_difference(va, vb, 3, 2, 150, 120, alpha_threshold=thr)
            assert np.allclose(got, want, rtol=2e-5, atol=2.0 ** -47), (fmt, channels, thr)
        if fmt != 5:
            got = decode(oracle_difference(ntc, oracle, raw_a, raw_b, desc, desc, (0, 0, w, h), msle=True))
            assert np.allclose(got, np_difference(va, vb, 0, 0, w, h, msle=True), rtol=1e-4, atol=2.0 ** -40), (fmt, channels)


def test_checker_fixed_point_is_exact_on_dyadic_cases(ntc, oracle):
    """All differences 1 (codes 0 against 255): every 64 x 64 workgroup adds 4096 / (W * H), and the
    16.48 result is exactly 1 whatever the number of workgroups; an identical image adds nothing;
    a second pass adds to what the buffer holds."""
    for w, h in ((64, 64), (128, 64), (256, 128), (32, 16)):
        a = np.zeros(w * h * 4, dtype=np.uint8)
        b = np.full(w * h * 4, 255, dtype=np.uint8)
        desc = (4, 4 * w, w, h, 1, 4)
        out = oracle_difference(ntc, oracle, a, b, desc, desc, (0, 0, w, h))
        assert out == [1 << 48] * 4, (w, h, out)
        assert oracle_difference(ntc, oracle, a, a, desc, desc, (0, 0, w, h)) == [0, 0, 0, 0]
        again = oracle_difference(ntc, oracle, a, b, desc, desc, (0, 0, w, h), start=(5, 1 << 48, 0, 7))
        assert again == [(1 << 48) + 5, 2 << 48, 1 << 48, (1 << 48) + 7]
    # a quarter of the pixels differ by 1/2 in one channel (FLOAT32): mse = 1/16 exactly
    w, h = 128, 128
    a = np.zeros((h, w, 4), dtype=np.float32)
    b = a.copy()
    b[::2, ::2, 1] = 0.5
    desc = (16, 16 * w, w, h, 4, 4)
    out = oracle_difference(ntc, oracle, a.reshape(-1).view(np.uint8), b.reshape(-1).view(np.uint8), desc, desc, (0, 0, w, h))
    assert out == [0, 1 << 44, 0, 0]
    # alpha below the threshold in both images: colour differences do not count, alpha still does
    a = np.zeros((h, w, 4), dtype=np.float32)
    b = np.ones((h, w, 4), dtype=np.float32)
    b[:, :, 3] = 0.25
    raw_a, raw_b = a.reshape(-1).view(np.uint8), b.reshape(-1).view(np.uint8)
    assert oracle_difference(ntc, oracle, raw_a, raw_b, desc, desc, (0, 0, w, h), alpha_threshold=0.5) == [0, 0, 0, 1 << 44]
    assert oracle_difference(ntc, oracle, raw_a, raw_b, desc, desc, (0, 0, w, h), alpha_threshold=0.25) == [1 << 48] * 3 + [1 << 44]


def gpu_difference(ntc, device, d_a, d_b, desc_a, desc_b, extent, alpha_threshold=None, msle=False, start=(0, 0, 0, 0), offset=0):
    p = ntc.abi.ImageDifference()
    fill_image(p.a, d_a.ptr, d_a.nbytes, *desc_a)
    fill_image(p.b, d_b.ptr, d_b.nbytes, *desc_b)
    p.left, p.top, p.width, p.height = extent
    p.alphaThreshold = 0.0 if alpha_threshold is None else alpha_threshold
    p.useAlphaThreshold, p.useMSLE = int(alpha_threshold is not None), int(msle)
    buffer = np.zeros(offset // 8 + 4, dtype=np.uint64)
    buffer[offset // 8:] = start
    d_out = device.upload(buffer.view(np.uint8))
    p.output, p.outputBytes, p.outputOffset = d_out.ptr, d_out.nbytes, offset
    ntc.abi.check(device.lib.ntc_hip_image_difference(p))
    device.synchronize()
    return [int(v) for v in d_out.download().view(np.uint64)]


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,channels", [(1, 4), (2, 4), (3, 4), (4, 4), (1, 3), (4, 1), (5, 4)])
def test_gpu_image_difference_matches_checker(ntc, device, oracle, fmt, channels):
    rng = np.random.default_rng(20 + fmt + channels)
    w, h = 333, 270
    raw_a, va, stride, pitch = make_image(rng, fmt, w, h, channels, pad_pixels=1, pad_rows=2)
    raw_b, vb, _, _ = make_image(rng, fmt, w, h, channels, pad_pixels=1, pad_rows=2, other=va)
    desc = (stride, pitch, w, h, fmt, channels)
    d_a, d_b = device.upload(raw_a), device.upload(raw_b)
    for extent, thr in (((0, 0, w, h), None), ((17, 3, 200, 255), None), ((332, 269, 1, 1), None), ((10, 10, 129, 65), 0.5)):
        want = oracle_difference(ntc, oracle, raw_a, raw_b, desc, desc, extent, alpha_threshold=thr, start=(1, 2, 3, 4))
        got = gpu_difference(ntc, device, d_a, d_b, desc, desc, extent, alpha_threshold=thr, start=(1, 2, 3, 4), offset=16)
        assert got[:2] == [0, 0] and got[2:] == want, (fmt, channels, extent, thr)
        assert np.allclose(decode(got[2:]), np_difference(va, vb, *extent, alpha_threshold=thr), rtol=2e-5, atol=2.0 ** -40)
    if fmt != 5:
        got = decode(gpu_difference(ntc, device, d_a, d_b, desc, desc, (0, 0, w, h), msle=True))
        assert np.allclose(got, np_difference(va, vb, 0, 0, w, h, msle=True), rtol=1e-4, atol=2.0 ** -40)


@pytest.mark.gpu
def test_gpu_image_difference_large_and_arguments(ntc, device, oracle):
    """4096 x 4096 RGBA8 against itself plus one changed pixel (exact result), and the argument checks."""
    w, h = 4096, 4096
    rng = np.random.default_rng(31)
    a = rng.integers(0, 256, (h, w, 4), dtype=np.uint8)
    b = a.copy()
    a[1000, 2000] = (0, 0, 0, 0)
    b[1000, 2000] = (255, 0, 255, 0)
    d_a, d_b = device.upload(a.reshape(-1)), device.upload(b.reshape(-1))
    desc = (4, 4 * w, w, h, 1, 4)
    got = gpu_difference(ntc, device, d_a, d_b, desc, desc, (0, 0, w, h))
    assert got == [1 << 24, 0, 1 << 24, 0]                 # 1 / 2^24 pixels differ by exactly 1: 2^-24 in 16.48
    p = ntc.abi.ImageDifference()
    fill_image(p.a, d_a.ptr, d_a.nbytes, *desc)
    fill_image(p.b, d_b.ptr, d_b.nbytes, *desc)
    d_out = device.upload(np.zeros(32, dtype=np.uint8))
    p.output, p.outputBytes = d_out.ptr, d_out.nbytes
    p.left, p.top, p.width, p.height = 0, 0, w, h
    bad = ntc.abi.ERR_INVALID_ARG
    for field, value in (("left", -1), ("width", 0), ("width", w + 1), ("top", 1), ("outputOffset", 4), ("outputOffset", 8)):
        saved = getattr(p, field)
        setattr(p, field, value)
        assert device.lib.ntc_hip_image_difference(p) == bad, (field, value)
        setattr(p, field, saved)
    p.a.format = 9
    assert device.lib.ntc_hip_image_difference(p) == bad
    p.a.format = 1
    p.b.bytes = d_b.nbytes - 1
    assert device.lib.ntc_hip_image_difference(p) == bad
    p.b.bytes = d_b.nbytes
    ntc.abi.check(device.lib.ntc_hip_image_difference(p))
    device.synchronize()
