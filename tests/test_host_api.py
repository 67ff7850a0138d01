"""The C++ host layer (rtxntc-library_amd/host) driven like LibNTC: CreateContext ->
CreateTextureSet -> SetLatentShape / preset -> data -> Decompress -> ReadChannels.
The C++ driver is tests/host_api_test.cpp; comparisons against the CPU checker happen here."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

import oracle_lib
from cases import cfg_case, ref_case

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "host_api_test")


def run_exe(*args):
    if not os.path.exists(EXE):
        pytest.fail(f"{EXE} is not built; run __graft_entry__.build() (make -C tests)")
    out = subprocess.run([EXE, *map(str, args)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, f"host_api_test {args[0]} failed:\n{out.stdout}\n{out.stderr}"
    return out.stdout


def test_host_layer_status_codes_and_state_machine():
    assert "host cpu checks OK" in run_exe("cpu")


def np_read_channels(planar_u16, width, height, set_channels, first, count, fmt, pixel_stride, row_pitch, fill):
    """numpy model of CopyImage's 1:1 branch for the five channel formats."""
    bpc = {1: 1, 2: 2, 3: 2, 4: 4, 5: 4}[fmt]
    img = planar_u16.reshape(height, set_channels // 2, width, 2)
    dst = np.full(height * row_pitch, fill, dtype=np.uint8)
    dst_channels = pixel_stride // bpc
    for ch in range(dst_channels):
        if ch < count:
            c = first + ch
            v = img[:, c // 2, :, c % 2].view(np.float16).astype(np.float32)
        else:
            v = np.full((height, width), 1.0 if ch == 3 else 0.0, dtype=np.float32)
        if fmt in (1, 2):
            scale = np.float32(255.0 if fmt == 1 else 65535.0)
            p = (v * scale).astype(np.float32).astype(np.float64)          # one fp32 rounding, then exact
            r = np.where(p >= 0, np.floor(p + 0.5), np.ceil(p - 0.5))
            out = np.clip(r, 0, scale).astype(np.uint8 if fmt == 1 else np.uint16)
        elif fmt == 3:
            out = np.clip(v, -65504, 65504).astype(np.float16)
        elif fmt == 4:
            out = v
        else:
            out = np.maximum(v, 0).astype(np.uint32)
        raw = np.ascontiguousarray(out).view(np.uint8).reshape(height, width, bpc)
        for y in range(height):
            row = dst[y * row_pitch: y * row_pitch + width * pixel_stride].reshape(width, pixel_stride)
            row[:, ch * bpc:(ch + 1) * bpc] = raw[y]
    return dst


def random_planar(rng, width, height, channels):
    vals = np.concatenate([rng.uniform(-0.2, 1.2, width * height * channels // 2),
                           rng.standard_normal(width * height * channels - width * height * channels // 2) * 300])
    rng.shuffle(vals)
    halves = vals.astype(np.float16).view(np.uint16)
    halves[:8] = np.array([0x0000, 0x8000, 0x3C00, 0x7BFF, 0xFBFF, 0x0001, 0x3800, 0x1C04], dtype=np.uint16)
    return halves


@pytest.mark.parametrize("fmt", [1, 2, 3, 4, 5])
def test_checker_read_channels_against_numpy(oracle, fmt):
    rng = np.random.default_rng(fmt)
    w, h, C_ = 37, 9, 6
    planar = random_planar(rng, w, h, C_)
    bpc = {1: 1, 2: 2, 3: 2, 4: 4, 5: 4}[fmt]
    for first, count, dst_channels in ((0, 6, 6), (1, 3, 4), (4, 1, 1)):
        stride = dst_channels * bpc
        pitch = w * stride + 12
        dst = np.full(h * pitch, 0xEE, dtype=np.uint8)
        assert oracle.ntc_oracle_read_channels(planar.ctypes.data, w, h, C_, first, count, dst.ctypes.data, fmt, stride, pitch) == 0
        want = np_read_channels(planar, w, h, C_, first, count, fmt, stride, pitch, 0xEE)
        assert np.array_equal(dst, want)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [1, 2, 3, 4, 5])
def test_gpu_read_channels_all_formats(ntc, device, oracle, fmt):
    rng = np.random.default_rng(10 + fmt)
    w, h, C_ = 200, 33, 16
    planar = random_planar(rng, w, h, C_)
    d_src = device.upload(planar)
    bpc = {1: 1, 2: 2, 3: 2, 4: 4, 5: 4}[fmt]
    # (the last two: a pixel stride of more than 16 components - every one of them is written, src/ImageProcessing.cu:237-240)
    for first, count, dst_channels in ((0, 16, 16), (5, 3, 4), (15, 1, 1), (2, 7, 7), (0, 16, 21), (3, 2, 64)):
        stride = dst_channels * bpc
        pitch = w * stride + 4 * bpc
        d_dst = device.alloc(h * pitch)
        d_dst.fill(0xEE)
        rc = ntc.abi.ReadChannels()
        rc.planarPairs, rc.planarBytes = d_src.ptr, d_src.nbytes
        rc.width, rc.height, rc.setChannels, rc.firstChannel, rc.numChannels = w, h, C_, first, count
        rc.dst, rc.dstBytes, rc.format, rc.pixelStride, rc.rowPitch = d_dst.ptr, d_dst.nbytes, fmt, stride, pitch
        ntc.abi.check(device.lib.ntc_hip_read_channels(rc))
        device.synchronize()
        want = np.full(h * pitch, 0xEE, dtype=np.uint8)
        assert oracle.ntc_oracle_read_channels(planar.ctypes.data, w, h, C_, first, count, want.ctypes.data, fmt, stride, pitch) == 0
        assert np.array_equal(d_dst.download(), want), (fmt, first, count)


@pytest.mark.gpu
@pytest.mark.parametrize("preset", [0, 1, 2])
def test_host_layer_decode_and_read_back(ntc, oracle, tmp_path, preset):
    w, h, channels = 256, 128, 10
    mips = ntc.presets.full_mip_count(w, h)
    if preset == 0:
        case = ref_case(ntc, ntc.presets.spec_ref092(12), w, h, mips, 2, channels, ntc.abi.OUT_FP16_PLANAR_PAIRS, 71, scale_log2_range=(-17.0, -12.0))
        grid_scale, features = 2, 12
    else:
        spec = ntc.presets.spec_cfg01() if preset == 1 else ntc.presets.spec_cfg2()
        case = cfg_case(ntc, spec, w, h, mips, channels, ntc.abi.OUT_FP16_PLANAR_PAIRS, 72 + preset, scale_log2_range=(-17.0, -12.0))
        grid_scale, features = 0, 0
    lat, wts = tmp_path / "latents.bin", tmp_path / "weights.bin"
    case.latents.tofile(lat)
    case.weights.tofile(wts)
    prefix = str(tmp_path / "out")
    assert "host decode OK" in run_exe("decode", preset, w, h, mips, channels, grid_scale, features, lat, wts, prefix)
    host = case.host_set()
    host.decode(threads=8)
    for m, mip in enumerate(case.mips):
        planar = host.output[mip.outOffset: mip.outOffset + mip.width * mip.height * channels * 2].view(np.uint16)
        planar = np.ascontiguousarray(planar)
        pitch = channels * mip.width + 8
        want = np.full(mip.height * pitch, 0, dtype=np.uint8)        # padded host reads come back zero-filled
        oracle.ntc_oracle_read_channels(planar.ctypes.data, mip.width, mip.height, channels, 0, channels, want.ctypes.data, 1, channels, pitch)
        got = np.fromfile(f"{prefix}_mip{m}_unorm8.bin", dtype=np.uint8)
        assert np.array_equal(got, want), f"preset {preset} mip {m} unorm8"
        want16 = np.zeros(mip.height * mip.width * 8, dtype=np.uint8)
        oracle.ntc_oracle_read_channels(planar.ctypes.data, mip.width, mip.height, channels, 1, 3, want16.ctypes.data, 3, 8, mip.width * 8)
        got16 = np.fromfile(f"{prefix}_mip{m}_rgba16f.bin", dtype=np.uint8)
        assert np.array_equal(got16, want16), f"preset {preset} mip {m} rgba16f"
    # mip 0 again, dithered, channels 0..2 encoded as sRGB: one code of slack for the transfer function
    mip = case.mips[0]
    planar = np.ascontiguousarray(host.output[mip.outOffset: mip.outOffset + w * h * channels * 2].view(np.uint16))
    want = np.zeros(h * w * channels, dtype=np.uint8)
    src_cs = np.zeros(16, dtype=np.uint8)
    dst_cs = np.array([1, 1, 1] + [0] * 13, dtype=np.uint8)
    oracle.ntc_oracle_read_channels_ex(planar.ctypes.data, w, h, channels, 0, channels, want.ctypes.data, 1, channels, channels * w, 1,
                                       src_cs.ctypes.data, dst_cs.ctypes.data)
    got = np.fromfile(f"{prefix}_srgb_dither.bin", dtype=np.uint8)
    assert np.abs(got.astype(int) - want.astype(int)).max() <= 1
    assert np.array_equal(got.reshape(h, w, channels)[:, :, 3:], want.reshape(h, w, channels)[:, :, 3:])     # linear channels: exact


# ---- WriteChannels and the loss statistics of Decompress ------------------------------------------

BPC = {1: 1, 2: 2, 3: 2, 4: 4, 5: 4}


def random_user_image(rng, fmt, width, height, channels, pad):
    """Pitch-linear user image in channel format fmt; returns (bytes, float32 values [h, w, c])."""
    if fmt == 1:
        raw = rng.integers(0, 256, (height, width, channels)).astype(np.uint8)
        vals = (raw.astype(np.float32) / np.float32(255.0)).astype(np.float32)
    elif fmt == 2:
        raw = rng.integers(0, 65536, (height, width, channels)).astype(np.uint16)
        vals = (raw.astype(np.float32) / np.float32(65535.0)).astype(np.float32)
    elif fmt == 3:
        raw = (rng.standard_normal((height, width, channels)) * 50).astype(np.float16)
        vals = raw.astype(np.float32)
    elif fmt == 4:
        raw = (rng.standard_normal((height, width, channels)) * 3).astype(np.float32)
        raw.reshape(-1)[:4] = [1e9, -1e9, 65519.9, 1e-9]                      # saturate, not overflow to Inf
        vals = raw
    else:
        raw = rng.integers(0, 70000, (height, width, channels)).astype(np.uint32)
        vals = raw.astype(np.float32)
    stride = channels * BPC[fmt]
    pitch = width * stride + pad
    img = np.full(height * pitch, 0x5A, dtype=np.uint8)
    for y in range(height):
        img[y * pitch: y * pitch + width * stride] = np.ascontiguousarray(raw[y]).view(np.uint8).reshape(-1)
    return img, vals, stride, pitch


def np_write_channels(planar, vals, set_channels, first, flip):
    """numpy model: clamp to the finite half range, round to half (nearest even), planar pairs."""
    h, w, n = vals.shape
    img = planar.reshape(h, set_channels // 2, w, 2)
    src = vals[::-1] if flip else vals
    halves = np.clip(src, -65504.0, 65504.0).astype(np.float32).astype(np.float16).view(np.uint16)
    for ch in range(n):
        c = first + ch
        img[:, c // 2, :, c % 2] = halves[:, :, ch]


@pytest.mark.parametrize("fmt", [1, 2, 3, 4, 5])
def test_checker_write_channels_against_numpy(oracle, fmt):
    rng = np.random.default_rng(40 + fmt)
    w, h, C_ = 29, 7, 8
    for first, count, flip in ((0, 8, 0), (3, 4, 1), (7, 1, 0)):
        img, vals, stride, pitch = random_user_image(rng, fmt, w, h, count, 6 * BPC[fmt])
        got = np.full(w * h * C_, 0x1234, dtype=np.uint16)
        want = got.copy()
        assert oracle.ntc_oracle_write_channels(img.ctypes.data, fmt, flip, stride, pitch, got.ctypes.data, w, h, C_, first, count) == 0
        np_write_channels(want, vals, C_, first, flip)
        assert np.array_equal(got, want), (fmt, first, count, flip)


def np_image_loss(a, b, width, height, set_channels, mask):
    fa = a.view(np.float16).astype(np.float64).reshape(height, set_channels // 2, width, 2)
    fb = b.view(np.float16).astype(np.float64).reshape(height, set_channels // 2, width, 2)
    out = np.zeros(16)
    for c in range(set_channels):
        if mask >> c & 1:
            out[c] = np.mean((fa[:, c // 2, :, c % 2] - fb[:, c // 2, :, c % 2]) ** 2)
    return out


def test_checker_image_loss_against_numpy(oracle):
    rng = np.random.default_rng(50)
    w, h, C_ = 61, 13, 10
    a = (rng.random(w * h * C_)).astype(np.float16).view(np.uint16)
    b = (rng.random(w * h * C_)).astype(np.float16).view(np.uint16)
    for mask in (0x3FF, 0x155, 0x200, 0):
        got = np.zeros(16, dtype=np.float64)
        oracle.ntc_oracle_image_loss(a.ctypes.data, b.ctypes.data, w, h, C_, mask, got.ctypes.data)
        assert np.allclose(got, np_image_loss(a, b, w, h, C_, mask), rtol=1e-12, atol=0)
        assert all(got[c] == 0 for c in range(16) if not mask >> c & 1)


def np_image_loss_masked(a, b, width, height, set_channels, mask, mask_channel, discard):
    """numpy statement of the loss branch with its mask options (src/Inference.cu:80-84,96-97,107-112).
    Returns (mse[16], the decoded image with its mask channel clamped)."""
    fa = a.view(np.float16).astype(np.float64).reshape(height, set_channels // 2, width, 2).copy()
    fb = b.view(np.float16).astype(np.float64).reshape(height, set_channels // 2, width, 2)
    masked_out = np.zeros((height, width), dtype=bool)
    if mask_channel >= 0:
        plane = fa[:, mask_channel // 2, :, mask_channel % 2]
        fa[:, mask_channel // 2, :, mask_channel % 2] = np.clip(plane, 0.0, 1.0) + 0.0    # + 0.0: -0 -> +0
        if discard:
            masked_out = fb[:, mask_channel // 2, :, mask_channel % 2] == 0
    out = np.zeros(16)
    for c in range(set_channels):
        if mask >> c & 1:
            d = fa[:, c // 2, :, c % 2] - fb[:, c // 2, :, c % 2]
            if c != mask_channel:
                d = np.where(masked_out, 0.0, d)
            out[c] = np.mean(d ** 2)
    return out, fa.astype(np.float16).view(np.uint16).reshape(-1)


def masked_loss_images(rng, w, h, C_, mask_channel):
    """A decoded image whose mask channel leaves [0, 1] (and holds -0), and a reference whose mask
    channel is zero (+0 or -0) on about a third of the texels."""
    a = (rng.random(w * h * C_) * 1.5 - 0.25).astype(np.float16).view(np.uint16).copy()
    b = rng.random(w * h * C_).astype(np.float16).view(np.uint16).copy()
    av = a.reshape(h, C_ // 2, w, 2)
    bv = b.reshape(h, C_ // 2, w, 2)
    pick = rng.random((h, w))
    bv[:, mask_channel // 2, :, mask_channel % 2][pick < 0.2] = 0x0000
    bv[:, mask_channel // 2, :, mask_channel % 2][(pick >= 0.2) & (pick < 0.33)] = 0x8000
    av[:, mask_channel // 2, :, mask_channel % 2][rng.random((h, w)) < 0.1] = 0x8000
    return a, b


def test_checker_masked_image_loss(oracle):
    rng = np.random.default_rng(51)
    w, h, C_ = 45, 17, 8
    for mask_channel in (3, 6):
        a, b = masked_loss_images(rng, w, h, C_, mask_channel)
        for discard in (0, 1):
            for mask in (0xFF, 0x0F, 1 << mask_channel):
                got, work = np.zeros(16), a.copy()
                oracle.ntc_oracle_image_loss_masked(work.ctypes.data, b.ctypes.data, w, h, C_, mask, mask_channel, discard, got.ctypes.data)
                want, clamped = np_image_loss_masked(a, b, w, h, C_, mask, mask_channel, discard)
                assert np.allclose(got, want, rtol=1e-12, atol=0)
                assert np.array_equal(work, clamped)
                assert not np.array_equal(work, a)
                # clamping is idempotent and changes the mask channel only
                again, work2 = np.zeros(16), work.copy()
                oracle.ntc_oracle_image_loss_masked(work2.ctypes.data, b.ctypes.data, w, h, C_, mask, mask_channel, discard, again.ctypes.data)
                assert np.array_equal(work2, work) and np.array_equal(again, got)
                other = np.ones(C_, dtype=bool); other[mask_channel] = False
                assert np.array_equal(work.reshape(h, C_ // 2, w, 2).transpose(0, 2, 1, 3).reshape(h, w, C_)[:, :, other],
                                      a.reshape(h, C_ // 2, w, 2).transpose(0, 2, 1, 3).reshape(h, w, C_)[:, :, other])
    # special cases: no mask channel = the plain loss; a reference mask without zeros = discard has no
    # effect; a reference mask of zeros = only the mask channel counts
    a, b = masked_loss_images(rng, w, h, C_, 2)
    plain, got = np.zeros(16), np.zeros(16)
    oracle.ntc_oracle_image_loss(a.ctypes.data, b.ctypes.data, w, h, C_, 0xFF, plain.ctypes.data)
    work = a.copy()
    oracle.ntc_oracle_image_loss_masked(work.ctypes.data, b.ctypes.data, w, h, C_, 0xFF, -1, 1, got.ctypes.data)
    assert np.array_equal(got, plain) and np.array_equal(work, a)
    bv = b.reshape(h, C_ // 2, w, 2)
    bv[:, 1, :, 0] = np.float16(0.5).view(np.uint16)
    keep, drop = np.zeros(16), np.zeros(16)
    work = a.copy()
    oracle.ntc_oracle_image_loss_masked(work.ctypes.data, b.ctypes.data, w, h, C_, 0xFF, 2, 0, keep.ctypes.data)
    oracle.ntc_oracle_image_loss_masked(work.ctypes.data, b.ctypes.data, w, h, C_, 0xFF, 2, 1, drop.ctypes.data)
    assert np.array_equal(keep, drop)
    bv[:, 1, :, 0] = 0
    oracle.ntc_oracle_image_loss_masked(work.ctypes.data, b.ctypes.data, w, h, C_, 0xFF, 2, 1, drop.ctypes.data)
    assert drop[2] > 0 and not np.delete(drop, 2).any()


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [1, 2, 3, 4, 5])
def test_gpu_write_channels_all_formats(ntc, device, oracle, fmt):
    rng = np.random.default_rng(60 + fmt)
    w, h, C_ = 203, 31, 16
    for first, count, flip in ((0, 16, 0), (5, 3, 1), (15, 1, 0), (2, 7, 1)):
        img, _, stride, pitch = random_user_image(rng, fmt, w, h, count, 4 * BPC[fmt])
        start = np.full(w * h * C_, 0x1234, dtype=np.uint16)
        d_src, d_dst = device.upload(img), device.upload(start)
        wc = ntc.abi.WriteChannels()
        wc.src, wc.srcBytes, wc.format, wc.verticalFlip, wc.pixelStride, wc.rowPitch = d_src.ptr, d_src.nbytes, fmt, flip, stride, pitch
        wc.planarPairs, wc.planarBytes = d_dst.ptr, d_dst.nbytes
        wc.width, wc.height, wc.setChannels, wc.firstChannel, wc.numChannels = w, h, C_, first, count
        ntc.abi.check(device.lib.ntc_hip_write_channels(wc))
        device.synchronize()
        want = start.copy()
        assert oracle.ntc_oracle_write_channels(img.ctypes.data, fmt, flip, stride, pitch, want.ctypes.data, w, h, C_, first, count) == 0
        assert np.array_equal(d_dst.download().view(np.uint16), want), (fmt, first, count, flip)
    # a source image shorter than height * rowPitch is refused before any launch
    wc.srcBytes = h * pitch - pitch
    assert device.lib.ntc_hip_write_channels(wc) == ntc.abi.ERR_INVALID_ARG


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 1, 2), (67, 5, 6), (512, 300, 16), (2048, 2048, 12)])
def test_gpu_image_loss_against_checker(ntc, device, oracle, shape):
    w, h, C_ = shape
    rng = np.random.default_rng(w)
    a = rng.random(w * h * C_).astype(np.float16).view(np.uint16)
    b = (a.view(np.float16).astype(np.float32) + rng.standard_normal(w * h * C_).astype(np.float32) * 0.05).astype(np.float16).view(np.uint16)
    d_a, d_b = device.upload(a), device.upload(b)
    for mask in ((1 << C_) - 1, 0x5 & ((1 << C_) - 1), 0):
        got = (C.c_float * 16)()
        ntc.abi.check(device.lib.ntc_hip_image_loss(d_a.ptr, d_b.ptr, d_a.nbytes, w, h, C_, mask, -1, 0, got))
        want = np.zeros(16, dtype=np.float64)
        oracle.ntc_oracle_image_loss(a.ctypes.data, b.ctypes.data, w, h, C_, mask, want.ctypes.data)
        # double accumulation on both sides; the result is rounded to float once
        assert np.allclose(np.array(got[:], dtype=np.float64), want, rtol=2e-7, atol=0), (shape, mask)
    assert np.array_equal(d_a.download().view(np.uint16), a)        # without a mask channel the decoded image is only read
    assert device.lib.ntc_hip_image_loss(d_a.ptr, d_b.ptr, d_a.nbytes - 2, w, h, C_, 1, -1, 0, got) == ntc.abi.ERR_INVALID_ARG
    assert device.lib.ntc_hip_image_loss(d_a.ptr, d_b.ptr, d_a.nbytes, w, h, C_, 1, C_, 0, got) == ntc.abi.ERR_INVALID_ARG
    assert device.lib.ntc_hip_image_loss(d_a.ptr, d_a.ptr, d_a.nbytes, w, h, C_, 1, 0, 0, got) == ntc.abi.ERR_INVALID_ARG   # overlap


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 1, 2), (67, 5, 6), (515, 300, 16)])
def test_gpu_masked_image_loss_against_checker(ntc, device, oracle, shape):
    """Alpha-mask options of the loss branch: the decoded mask channel is clamped in place (bit-exact
    against the checker), masked-out texels count on the mask channel only."""
    w, h, C_ = shape
    rng = np.random.default_rng(w + 1)
    for mask_channel in sorted({0, C_ - 1, C_ // 2}):
        a, b = masked_loss_images(rng, w, h, C_, mask_channel)
        for discard in (0, 1):
            mask = (1 << C_) - 1
            d_a, d_b = device.upload(a), device.upload(b)
            got = (C.c_float * 16)()
            ntc.abi.check(device.lib.ntc_hip_image_loss(d_a.ptr, d_b.ptr, d_a.nbytes, w, h, C_, mask, mask_channel, discard, got))
            want, work = np.zeros(16), a.copy()
            oracle.ntc_oracle_image_loss_masked(work.ctypes.data, b.ctypes.data, w, h, C_, mask, mask_channel, discard, want.ctypes.data)
            assert np.array_equal(d_a.download().view(np.uint16), work), (shape, mask_channel, discard)
            assert np.allclose(np.array(got[:], dtype=np.float64), want, rtol=2e-7, atol=0), (shape, mask_channel, discard)


def parse_stats(text, tag, mips):
    lines = {ln.split()[1]: [float(v) for v in ln.split()[2:]] for ln in text.splitlines() if ln.startswith(tag + " ")}
    return lines["overall"][0], np.array(lines["mips"][:mips]), np.array(lines["channels"])


@pytest.mark.gpu
@pytest.mark.parametrize("separate", [0, 1])
def test_host_layer_loss_statistics(ntc, oracle, tmp_path, separate):
    """Decompress(&stats) after WriteChannels: per-channel / per-mip / overall MSE combined as
    src/TextureSet.cpp:1833-1892 does, over the channels the registered textures claim."""
    w, h, channels = 128, 64, 8
    mips = ntc.presets.full_mip_count(w, h)
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), w, h, mips, channels, ntc.abi.OUT_FP16_PLANAR_PAIRS, 91, scale_log2_range=(-17.0, -12.0))
    lat, wts = tmp_path / "latents.bin", tmp_path / "weights.bin"
    case.latents.tofile(lat)
    case.weights.tofile(wts)
    host = case.host_set()
    host.decode(threads=8)
    rng = np.random.default_rng(92)
    prefix = str(tmp_path / "ref")
    mask = 0x37                                     # textures on channels 0..2 and 4..5
    valid = [c for c in range(channels) if mask >> c & 1]
    mse = np.zeros((mips, 16))
    pixels = np.array([m.width * m.height for m in case.mips], dtype=np.float64)
    planes = []
    for m, mip in enumerate(case.mips):
        decoded = np.ascontiguousarray(host.output[mip.outOffset: mip.outOffset + mip.width * mip.height * channels * 2].view(np.uint16))
        ref = rng.random((mip.height, mip.width, channels)).astype(np.float32)
        ref.tofile(f"{prefix}_mip{m}.bin")
        ref_planar = np.zeros(mip.width * mip.height * channels, dtype=np.uint16)
        np_write_channels(ref_planar, ref, channels, 0, False)
        mse[m] = np_image_loss(decoded, ref_planar, mip.width, mip.height, channels, mask)
        planes.append((decoded, ref_planar))
    out = run_exe("loss", 1, w, h, mips, channels, 0, 0, lat, wts, prefix, separate)
    assert "host loss OK" in out
    overall, per_mip, per_channel = parse_stats(out, "first", mips)
    want_mip = mse[:, valid].mean(axis=1)
    assert np.allclose(per_mip, want_mip, rtol=1e-6)
    assert np.allclose(per_channel, (mse * pixels[:, None]).sum(axis=0) / pixels.sum(), rtol=1e-6)
    assert np.isclose(overall, (want_mip * pixels).sum() / pixels.sum(), rtol=1e-6)
    assert all(per_channel[c] == 0 for c in range(16) if c not in valid)
    overall2, per_mip2, _ = parse_stats(out, "second", mips)
    if separate:    # the reference image survives the decode: same numbers again
        assert overall2 == overall and np.array_equal(per_mip2, per_mip)
    else:           # shared page: the first decode overwrote the reference image (as in the reference library)
        assert overall2 == 0 and not per_mip2.any()

    def pixels_of(planar):
        return planar.reshape(h, channels // 2, w, 2).transpose(0, 2, 1, 3).reshape(-1)
    decoded0, ref0 = planes[0]
    page_ref = np.fromfile(prefix + "_page_reference.bin", dtype=np.uint16)
    page_out = np.fromfile(prefix + "_page_output.bin", dtype=np.uint16)
    assert np.array_equal(page_out, pixels_of(decoded0))
    assert np.array_equal(page_ref, pixels_of(ref0 if separate else decoded0))


@pytest.mark.gpu
@pytest.mark.parametrize("preset", [0, 1])
def test_host_layer_shuffle_inference_outputs(ntc, tmp_path, preset):
    """ShuffleInferenceOutputs permutes the rows of the output layer in the weights that
    GetInferenceWeights returns (src/TextureSetMetadata.cpp:305-432).  Checked through the decoder:
    with the shuffled blob as the set's weights, channel ch decodes to what channel
    mapping[ch].channelIndex decoded to before, bit for bit; constants come out as
    round(c * 2^16) / 2^16; undefined channels as zero; a permutation and its inverse restore the blob."""
    w, h, channels = 96, 64, 16
    if preset == 0:
        case = ref_case(ntc, ntc.presets.spec_ref092(16), w, h, 1, 2, channels, ntc.abi.OUT_FP16_PLANAR_PAIRS, 95, scale_log2_range=(-17.0, -12.0))
    else:
        case = cfg_case(ntc, ntc.presets.spec_cfg01(), w, h, 1, channels, ntc.abi.OUT_FP16_PLANAR_PAIRS, 96, scale_log2_range=(-17.0, -12.0))
    lat, wts = tmp_path / "latents.bin", tmp_path / "weights.bin"
    case.latents.tofile(lat)
    case.weights.tofile(wts)
    assert "host shuffle OK" in run_exe("shuffle", preset, w, h, channels, 2, 16, lat, wts)


@pytest.mark.gpu
def test_host_layer_image_difference():
    assert "host image difference OK" in run_exe("imagediff")


@pytest.mark.gpu
@pytest.mark.parametrize("with_stats", [1, 0])
def test_host_layer_mask_channel(ntc, oracle, tmp_path, with_stats):
    """SetMaskChannelIndex (include/libntc/ntc.h:936-940): Decompress clamps the decoded mask channel to
    [0, 1] whenever textures are registered, and with discardMaskedOutPixels the loss of the other
    channels skips texels whose reference mask is zero (src/Inference.cu:80-112)."""
    w, h, channels, mask_channel = 96, 40, 8, 5
    mips = ntc.presets.full_mip_count(w, h)
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), w, h, mips, channels, ntc.abi.OUT_FP16_PLANAR_PAIRS, 93, scale_log2_range=(-17.0, -12.0))
    lat, wts = tmp_path / "latents.bin", tmp_path / "weights.bin"
    case.latents.tofile(lat)
    case.weights.tofile(wts)
    host = case.host_set()
    host.decode(threads=8)
    rng = np.random.default_rng(94)
    prefix = str(tmp_path / "ref")
    mask = 0x37
    valid = [c for c in range(channels) if mask >> c & 1]
    mse = np.zeros((mips, 16))
    pixels = np.array([m.width * m.height for m in case.mips], dtype=np.float64)
    clamped0 = decoded0 = None
    for m, mip in enumerate(case.mips):
        decoded = np.ascontiguousarray(host.output[mip.outOffset: mip.outOffset + mip.width * mip.height * channels * 2].view(np.uint16))
        ref = rng.random((mip.height, mip.width, channels)).astype(np.float32)
        ref[:, :, mask_channel][rng.random((mip.height, mip.width)) < 0.3] = 0.0
        ref.tofile(f"{prefix}_mip{m}.bin")
        ref_planar = np.zeros(mip.width * mip.height * channels, dtype=np.uint16)
        np_write_channels(ref_planar, ref, channels, 0, False)
        mse[m], clamped = np_image_loss_masked(decoded, ref_planar, mip.width, mip.height, channels, mask, mask_channel, True)
        if m == 0:
            decoded0, clamped0 = decoded, clamped
    assert not np.array_equal(decoded0, clamped0)       # the decoded mask channel does leave [0, 1]
    out = run_exe("loss", 1, w, h, mips, channels, 0, 0, lat, wts, prefix, 1, mask_channel, 1, with_stats)
    assert "host loss OK" in out
    page_out = np.fromfile(prefix + "_page_output.bin", dtype=np.uint16)
    assert np.array_equal(page_out, clamped0.reshape(h, channels // 2, w, 2).transpose(0, 2, 1, 3).reshape(-1))
    if with_stats:
        overall, per_mip, per_channel = parse_stats(out, "first", mips)
        want_mip = mse[:, valid].mean(axis=1)
        assert np.allclose(per_mip, want_mip, rtol=1e-6)
        assert np.allclose(per_channel, (mse * pixels[:, None]).sum(axis=0) / pixels.sum(), rtol=1e-6)
        assert np.isclose(overall, (want_mip * pixels).sum() / pixels.sum(), rtol=1e-6)


# ---- colour spaces and dithering in ReadChannels / WriteChannels -----------------------------------

def jenkins(a):
    """Robert Jenkins' 32-bit integer hash as HashBasedRNG seeds with it (src/CudaUtils.h:147-157)."""
    m = 0xFFFFFFFF
    a = ((a + 0x7ed55d16) + (a << 12)) & m
    a = ((a ^ 0xc761c23c) ^ (a >> 19)) & m
    a = ((a + 0x165667b1) + (a << 5)) & m
    a = ((a + 0xd3a2646c) ^ (a << 9)) & m
    a = ((a + 0xfd7046c5) + (a << 3)) & m
    a = ((a ^ 0xb55a4f09) ^ (a >> 16)) & m
    return a


def dither_model(linear_index, draw):
    """Draw `draw` of HashBasedRNG: its Murmur3Hash() is MurmurHash3_x86_32 of the 4-byte counter
    (starting at 1) with the Jenkins-hashed pixel index as seed -- computed here with scikit-learn's
    implementation of that hash."""
    from sklearn.utils import murmurhash3_32
    h = murmurhash3_32((draw + 1).to_bytes(4, "little"), seed=jenkins(linear_index), positive=True)
    return np.uint32((h & 0x7FFFFF) | 0x3F800000).view(np.float32) - np.float32(1.0)


def test_checker_dither_generator_is_murmur3_of_the_counter(oracle):
    for index in (0, 1, 2, 77, 4095, 123456789, 0xFFFFFFFF):
        for draw in range(5):
            assert oracle.ntc_oracle_dither_float(index, draw) == dither_model(index, draw), (index, draw)


def srgb_encode(v):
    v = np.asarray(v, dtype=np.float64)
    return np.where(v <= 0.0031308, v * 12.92, 1.055 * np.power(np.maximum(v, 1e-30), 1 / 2.4) - 0.055)


def srgb_decode(v):
    v = np.asarray(v, dtype=np.float64)
    return np.where(v <= 0.04045, v / 12.92, np.power((np.maximum(v, 0) + 0.055) / 1.055, 2.4))


def hlg_encode(v):
    v = np.asarray(v, dtype=np.float64)
    e = np.abs(v)
    return np.sign(v) * np.where(e < 1, 0.5 * np.sqrt(e), 0.17883277 * np.log(np.maximum(e - 0.28466892, 1e-30)) + 0.55991073)


def hlg_decode(v):
    v = np.asarray(v, dtype=np.float64)
    h = np.abs(v)
    return np.sign(v) * np.where(h < 0.5, 4 * h * h, np.exp((h - 0.55991073) / 0.17883277) + 0.28466892)


ENCODE = {0: lambda v: np.asarray(v, dtype=np.float64), 1: srgb_encode, 2: hlg_encode}
DECODE = {0: lambda v: np.asarray(v, dtype=np.float64), 1: srgb_decode, 2: hlg_decode}


def unit_planar(rng, width, height, channels):
    return rng.uniform(0.0, 1.0, width * height * channels).astype(np.float16).view(np.uint16)


def test_checker_color_spaces_and_dithering_against_float64_models(oracle):
    """UNORM8 reads: storage colour space -> linear -> requested colour space, plus dithering; the
    float64 model must agree to one code (the transfer functions are float32 in the checker)."""
    rng = np.random.default_rng(70)
    w, h, C_ = 33, 6, 4
    planar = unit_planar(rng, w, h, C_)
    values = planar.view(np.float16).astype(np.float64).reshape(h, C_ // 2, w, 2).transpose(0, 2, 1, 3).reshape(h, w, C_)
    for src_cs, dst_cs, dither in ((0, 1, 0), (1, 0, 0), (2, 0, 0), (0, 2, 0), (1, 2, 1), (0, 0, 1)):
        got = np.zeros(h * w * C_, dtype=np.uint8)
        src = np.full(16, src_cs, dtype=np.uint8)
        dst = np.full(16, dst_cs, dtype=np.uint8)
        assert oracle.ntc_oracle_read_channels_ex(planar.ctypes.data, w, h, C_, 0, C_, got.ctypes.data, 1, C_, w * C_, dither,
                                                  src.ctypes.data, dst.ctypes.data) == 0
        want = ENCODE[dst_cs](DECODE[src_cs](values))
        if dither:
            noise = np.array([[[float(dither_model(x + y * w, ch)) - 0.5 for ch in range(C_)] for x in range(w)] for y in range(h)])
            want = want + noise / 255.0
        want = np.clip(np.floor(want * 255.0 + 0.5), 0, 255)
        assert np.abs(got.reshape(h, w, C_).astype(np.float64) - want).max() <= 1, (src_cs, dst_cs, dither)
        if src_cs == 0 and dst_cs == 0:       # no transcendental involved: the model is exact up to float32 rounding at ties
            assert (got.reshape(h, w, C_) != want).mean() < 0.01


def gpu_read_ex(ntc, device, planar, w, h, C_, first, count, fmt, stride, pitch, dither, src_cs, dst_cs):
    d_src = device.upload(planar)
    d_dst = device.alloc(h * pitch)
    d_dst.fill(0xEE)
    rc = ntc.abi.ReadChannels()
    rc.planarPairs, rc.planarBytes = d_src.ptr, d_src.nbytes
    rc.width, rc.height, rc.setChannels, rc.firstChannel, rc.numChannels = w, h, C_, first, count
    rc.dst, rc.dstBytes, rc.format, rc.pixelStride, rc.rowPitch = d_dst.ptr, d_dst.nbytes, fmt, stride, pitch
    rc.useDithering = dither
    for i in range(16):
        rc.srcColorSpaces[i], rc.dstColorSpaces[i] = src_cs[i], dst_cs[i]
    ntc.abi.check(device.lib.ntc_hip_read_channels(rc))
    device.synchronize()
    return d_dst.download()


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [1, 2, 3, 4])
def test_gpu_read_channels_dithering_is_bit_exact(ntc, device, oracle, fmt):
    """Linear colour spaces: the noise generator is integer arithmetic and the rest IEEE float32."""
    rng = np.random.default_rng(80 + fmt)
    w, h, C_ = 301, 17, 8
    planar = unit_planar(rng, w, h, C_)
    zeros = np.zeros(16, dtype=np.uint8)
    for first, count, dst_channels in ((0, 8, 8), (2, 3, 4)):
        stride = dst_channels * BPC[fmt]
        pitch = w * stride + 8
        got = gpu_read_ex(ntc, device, planar, w, h, C_, first, count, fmt, stride, pitch, 1, zeros, zeros)
        want = np.full(h * pitch, 0xEE, dtype=np.uint8)
        assert oracle.ntc_oracle_read_channels_ex(planar.ctypes.data, w, h, C_, first, count, want.ctypes.data, fmt, stride, pitch, 1,
                                                  zeros.ctypes.data, zeros.ctypes.data) == 0
        assert np.array_equal(got, want), (fmt, first)
    if fmt == 1:      # the noise does something: about a quarter of the codes move against the undithered read
        plain = gpu_read_ex(ntc, device, planar, w, h, C_, 0, 8, 1, 8, w * 8, 0, zeros, zeros)
        noisy = gpu_read_ex(ntc, device, planar, w, h, C_, 0, 8, 1, 8, w * 8, 1, zeros, zeros)
        moved = (plain != noisy).mean()
        assert 0.15 < moved < 0.35 and np.abs(plain.astype(int) - noisy.astype(int)).max() == 1


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [1, 2, 3, 4])
def test_gpu_read_channels_color_spaces_within_one_code(ntc, device, oracle, fmt):
    """sRGB / HLG: powf, expf, logf, sqrtf come from different math libraries on the two sides, so
    the comparison allows 1 code of UNORM8, 3 of UNORM16, 1 ulp of fp16, 4e-6 relative in fp32."""
    rng = np.random.default_rng(90 + fmt)
    w, h, C_ = 257, 9, 6
    planar = unit_planar(rng, w, h, C_)
    src_cs = np.array([0, 1, 2, 0, 1, 2] + [0] * 10, dtype=np.uint8)
    dst_cs = np.array([1, 0, 0, 2, 2, 1] + [0] * 10, dtype=np.uint8)
    stride = C_ * BPC[fmt]
    pitch = w * stride
    got = gpu_read_ex(ntc, device, planar, w, h, C_, 0, C_, fmt, stride, pitch, 0, src_cs, dst_cs)
    want = np.zeros(h * pitch, dtype=np.uint8)
    assert oracle.ntc_oracle_read_channels_ex(planar.ctypes.data, w, h, C_, 0, C_, want.ctypes.data, fmt, stride, pitch, 0,
                                              src_cs.ctypes.data, dst_cs.ctypes.data) == 0
    if fmt == 1:
        assert np.abs(got.astype(int) - want.astype(int)).max() <= 1 and (got != want).mean() < 0.01
    elif fmt == 2:
        assert np.abs(got.view(np.uint16).astype(int) - want.view(np.uint16).astype(int)).max() <= 3
    elif fmt == 3:
        assert np.abs(got.view(np.int16).astype(int) - want.view(np.int16).astype(int)).max() <= 1
    else:
        a, b = got.view(np.float32).astype(np.float64), want.view(np.float32).astype(np.float64)
        assert np.all(np.abs(a - b) <= 4e-6 * np.abs(b) + 1e-9)


@pytest.mark.gpu
def test_gpu_write_channels_color_spaces_within_one_ulp(ntc, device, oracle):
    rng = np.random.default_rng(95)
    w, h, C_ = 130, 11, 6
    img, _, stride, pitch = random_user_image(rng, 1, w, h, C_, 4)
    src_cs = np.array([1, 1, 2, 0, 0, 2] + [0] * 10, dtype=np.uint8)
    dst_cs = np.array([0, 2, 0, 1, 2, 2] + [0] * 10, dtype=np.uint8)
    start = np.zeros(w * h * C_, dtype=np.uint16)
    d_src, d_dst = device.upload(img), device.upload(start)
    wc = ntc.abi.WriteChannels()
    wc.src, wc.srcBytes, wc.format, wc.verticalFlip, wc.pixelStride, wc.rowPitch = d_src.ptr, d_src.nbytes, 1, 0, stride, pitch
    wc.planarPairs, wc.planarBytes = d_dst.ptr, d_dst.nbytes
    wc.width, wc.height, wc.setChannels, wc.firstChannel, wc.numChannels = w, h, C_, 0, C_
    for i in range(16):
        wc.srcColorSpaces[i], wc.dstColorSpaces[i] = src_cs[i], dst_cs[i]
    ntc.abi.check(device.lib.ntc_hip_write_channels(wc))
    device.synchronize()
    want = start.copy()
    assert oracle.ntc_oracle_write_channels_ex(img.ctypes.data, 1, 0, stride, pitch, want.ctypes.data, w, h, C_, 0, C_,
                                               src_cs.ctypes.data, dst_cs.ctypes.data) == 0
    got = d_dst.download().view(np.int16).astype(int)
    assert np.abs(got - want.view(np.int16).astype(int)).max() <= 1
    wc.dstColorSpaces[3] = 9
    assert device.lib.ntc_hip_write_channels(wc) == ntc.abi.ERR_INVALID_ARG
