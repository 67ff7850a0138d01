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
    for first, count, dst_channels in ((0, 16, 16), (5, 3, 4), (15, 1, 1), (2, 7, 7)):
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
