"""BC1 / BC2 / BC3 block compression (reference src/shaders/CompressBC1.hlsl, CompressBC2.hlsl,
CompressBC3.hlsl and the BC1_* / BC2_* functions of BlockCompressCommon.hlsli).

What pins the checker:
  * its single-colour endpoint tables, regenerated from their published rule, equal the reference's
    literal tables (digest fixture; the literal values too where the reference is present);
  * the format's standard decoder (numpy, below): blocks a BC1 block can hold exactly must decode
    exactly or nearly so, transparent texels must decode transparent, and on smooth and noisy blocks
    the encoder must beat a plain bounding-box encoder written here independently;
  * BC2 alpha against its closed form, BC3 alpha against the BC4 encoder of the same values.
The float operation order inside the encoder (the shader compiler is free to fuse and reorder) is
not pinned by anything: parity with a compiled shader is to a few blocks' choice of equally good
encodings, not bit for bit.  The kernel must equal the checker bit for bit."""
import ctypes as C
import hashlib
import json
import os

import numpy as np
import pytest

from test_image_difference import fill_image

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def compress(ntc, oracle_or_none, device, image, fmt, channels, dst_format, blocks_x, blocks_y, left=0, top=0, off_x=0, off_y=0,
             pitch=None, threshold=1.0 / 255.0, fill=0xEE, hook=None):
    """image: [h][w][channels] of the format's dtype.  Through the checker (device None) or the kernel.
    hook(params, upload) may set further fields; upload(array) gives the address of a copy the callee can read.
    Returns uint64 [rows][pitch / 8]."""
    h, w = image.shape[:2]
    raw = np.ascontiguousarray(image).view(np.uint8).reshape(-1)
    per = 8 if dst_format in (1, 4) else 16
    pitch = pitch or (off_x + blocks_x) * per
    dst = np.full((off_y + blocks_y) * pitch, fill, dtype=np.uint8)
    p = ntc.abi.BlockCompress()
    stride = image.strides[1]
    p.srcLeft, p.srcTop, p.widthInBlocks, p.heightInBlocks, p.dstFormat = left, top, blocks_x, blocks_y, dst_format
    p.dstOffsetX, p.dstOffsetY, p.dstBytes, p.dstRowPitch, p.alphaThreshold = off_x, off_y, dst.nbytes, pitch, threshold
    keep = []
    if device is None:
        fill_image(p.src, raw.ctypes.data, raw.nbytes, stride, stride * w, w, h, fmt, channels)
        p.dst = dst.ctypes.data
        if hook:
            hook(p, lambda a: (keep.append(np.ascontiguousarray(a)), keep[-1].ctypes.data)[1])
        assert oracle_or_none.ntc_oracle_block_compress(C.byref(p)) == 0
        return dst.view(np.uint64).reshape(off_y + blocks_y, pitch // 8)
    d_src, d_dst = device.upload(raw), device.upload(dst)
    fill_image(p.src, d_src.ptr, d_src.nbytes, stride, stride * w, w, h, fmt, channels)
    p.dst = d_dst.ptr
    if hook:
        hook(p, lambda a: (keep.append(device.upload(np.ascontiguousarray(a).view(np.uint8).reshape(-1))), keep[-1].ptr)[1])
    ntc.abi.check(device.lib.ntc_hip_block_compress(p))
    device.synchronize()
    return d_dst.download().view(np.uint64).reshape(off_y + blocks_y, pitch // 8)


def image_of_blocks(blocks):
    """blocks: [n][16][4] floats -> float32 image [4][4 n][4], blocks side by side."""
    n = blocks.shape[0]
    image = np.zeros((4, 4 * n, 4), dtype=np.float32)
    for i in range(n):
        image[:, 4 * i: 4 * i + 4] = blocks[i].reshape(4, 4, 4)
    return image


def encode_bc1(ntc, oracle, blocks, threshold=1.0 / 255.0):
    return compress(ntc, oracle, None, image_of_blocks(blocks), 4, 4, 1, blocks.shape[0], 1, threshold=threshold)[0]


def expand565(w):
    return np.array([((w >> 11) & 31) / 31.0, ((w >> 5) & 63) / 63.0, (w & 31) / 31.0])


def bc1_decode(block):
    """16 RGBA texels of one BC1 block, as the format defines them."""
    block = int(block)
    w0, w1, bits = block & 0xFFFF, (block >> 16) & 0xFFFF, block >> 32
    c0, c1 = expand565(w0), expand565(w1)
    if w0 > w1:
        palette = [np.append(c0, 1), np.append(c1, 1), np.append((2 * c0 + c1) / 3, 1), np.append((c0 + 2 * c1) / 3, 1)]
    else:
        palette = [np.append(c0, 1), np.append(c1, 1), np.append((c0 + c1) / 2, 1), np.zeros(4)]
    return np.array([palette[(bits >> (2 * t)) & 3] for t in range(16)])


def test_checker_single_colour_tables_equal_the_reference(oracle):
    five, six = np.zeros(256, dtype="<u2"), np.zeros(256, dtype="<u2")
    oracle.ntc_oracle_bc1_match_tables(five.ctypes.data, six.ctypes.data)
    golden = json.load(open(os.path.join(GOLDEN, "bc_tables.json")))["bc1"]
    assert hashlib.sha256(five.tobytes()).hexdigest() == golden["sha256_five_bit"]
    assert hashlib.sha256(six.tobytes()).hexdigest() == golden["sha256_six_bit"]
    reference = "/root/reference/src/shaders/BlockCompressCommon.hlsli"
    if os.path.exists(reference):
        import importlib.util
        spec = importlib.util.spec_from_file_location("make_bc_table_digests", os.path.join(GOLDEN, "make_bc_table_digests.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        ref5, ref6 = mod.reference_bc1_tables()
        assert np.array_equal(five, ref5) and np.array_equal(six, ref6)
    # what the tables are for: the 1/3 : 2/3 mix of the pair reproduces the value to within 1 (of 255), 2 at worst
    for table, bits in ((five, 5), (six, 6)):
        a, b = (table & 0xFF).astype(int), (table >> 8).astype(int)
        ex = (lambda v: (v << 3) | (v >> 2)) if bits == 5 else (lambda v: (v << 2) | (v >> 4))
        shown = (2 * ex(a) + ex(b)) / 3.0
        err = np.abs(shown - np.arange(256))
        assert err.max() <= (2.0 if bits == 5 else 1.0) and err.mean() < 0.7


def test_checker_constant_blocks(ntc, oracle):
    """One opaque colour: every texel decodes to the same colour, each component within 2.6 / 255 of
    the input (half a step from rounding the mean, up to 1.33 from the table, the rest from the
    table's integer endpoint expansion against the format's exact one)."""
    rng = np.random.default_rng(1)
    colours = np.concatenate([rng.random((60, 3)), [[0, 0, 0], [1, 1, 1], [1, 0, 0.5], [0.2, 0.2, 0.2]]])
    blocks = np.ones((len(colours), 16, 4))
    blocks[:, :, :3] = colours[:, None, :]
    out = encode_bc1(ntc, oracle, blocks)
    for block, colour in zip(out, colours):
        dec = bc1_decode(block)
        assert np.all(dec[:, 3] == 1.0)
        assert np.abs(dec[:, :3] - dec[0, :3]).max() < 1e-12
        assert np.abs(dec[0, :3] - colour).max() <= 2.6 / 255.0, (hex(int(block)), colour, dec[0])


def test_checker_two_colour_blocks_that_bc1_holds_exactly(ntc, oracle):
    """Texels drawn from two 5:6:5 colours: a BC1 block can hold them exactly, and the encoder finds
    that block (or one within a rounding step of it) almost always."""
    rng = np.random.default_rng(2)
    blocks, worst = [], []
    for _ in range(80):
        w = rng.integers(0, 65536, 2)
        ends = np.array([expand565(int(w[0])), expand565(int(w[1]))])
        pick = rng.integers(0, 2, 16)
        pick[:2] = [0, 1]
        b = np.ones((16, 4))
        b[:, :3] = ends[pick]
        blocks.append(b)
    blocks = np.array(blocks)
    out = encode_bc1(ntc, oracle, blocks)
    errors = np.array([np.abs(bc1_decode(o)[:, :3] - b[:, :3]).max() for o, b in zip(out, blocks)])
    assert (errors < 1e-6).mean() > 0.7, (errors < 1e-6).mean()
    assert np.quantile(errors, 0.95) < 0.04, np.sort(errors)[-8:]


def box_encoder_error(block):
    """Squared error of a plain encoder: bounding-box corners along the luminance order rounded to
    5:6:5, nearest of the four colours per texel."""
    rgb = block[:, :3]
    lum = rgb @ np.array([0.299, 0.587, 0.114])
    lo, hi = rgb[lum.argmin()], rgb[lum.argmax()]
    q = lambda c: np.array([np.rint(c[0] * 31) / 31, np.rint(c[1] * 63) / 63, np.rint(c[2] * 31) / 31])
    lo, hi = q(lo), q(hi)
    palette = np.array([hi, lo, (2 * hi + lo) / 3, (hi + 2 * lo) / 3])
    d = ((rgb[:, None, :] - palette[None]) ** 2).sum(axis=2)
    return d.min(axis=1).sum()


def test_checker_quality_against_a_plain_encoder(ntc, oracle):
    rng = np.random.default_rng(3)
    blocks = []
    xs, ys = np.meshgrid(np.arange(4), np.arange(4))
    for i in range(120):
        base, gx, gy = rng.random(3), rng.normal(0, 0.04, 3), rng.normal(0, 0.04, 3)
        rgb = base[None, None] + xs[..., None] * gx + ys[..., None] * gy + rng.normal(0, rng.choice([0.0, 0.01, 0.05]), (4, 4, 3))
        b = np.ones((16, 4))
        b[:, :3] = np.clip(rgb, 0, 1).reshape(16, 3)
        blocks.append(b)
    for i in range(20):
        b = np.ones((16, 4))
        b[:, :3] = rng.random((16, 3))
        blocks.append(b)
    blocks = np.array(blocks)
    out = encode_bc1(ntc, oracle, blocks)
    ours = np.array([((bc1_decode(o)[:, :3] - b[:, :3]) ** 2).sum() for o, b in zip(out, blocks)])
    plain = np.array([box_encoder_error(b) for b in blocks])
    assert ours.sum() < 0.75 * plain.sum(), (ours.sum(), plain.sum())
    assert (ours <= plain + 1e-4).mean() > 0.85, (ours <= plain + 1e-4).mean()
    psnr = lambda e: 10 * np.log10(1.0 / (e.mean() / 48 + 1e-12))
    print("PSNR ours / plain, smooth blocks: %.2f / %.2f dB" % (psnr(ours[:120]), psnr(plain[:120])))
    assert psnr(ours[:120]) > psnr(plain[:120]) + 1.0


def test_checker_transparency(ntc, oracle):
    rng = np.random.default_rng(4)
    # all texels transparent: the all-transparent block
    b = np.zeros((1, 16, 4))
    b[0, :, :3] = rng.random((16, 3))
    assert int(encode_bc1(ntc, oracle, b)[0]) == 0xFFFFFFFF00000000
    # some transparent: those decode to transparent black, the rest stay opaque and close
    blocks = []
    for _ in range(40):
        blk = np.ones((16, 4))
        base = rng.random(3)
        blk[:, :3] = np.clip(base + rng.normal(0, 0.03, (16, 3)), 0, 1)
        holes = rng.random(16) < 0.3
        holes[0], holes[1] = True, False
        blk[holes, 3] = 0.0
        blocks.append(blk)
    blocks = np.array(blocks)
    out = encode_bc1(ntc, oracle, blocks)
    for o, blk in zip(out, blocks):
        dec = bc1_decode(o)
        holes = blk[:, 3] == 0
        assert np.all(dec[holes, 3] == 0) and np.all(dec[~holes, 3] == 1), hex(int(o))
        assert np.abs(dec[~holes, :3] - blk[~holes, :3]).max() < 0.12
    # the threshold decides what counts as transparent
    blk = np.ones((1, 16, 4)) * 0.5
    blk[0, :8, 3] = 0.3
    low = bc1_decode(encode_bc1(ntc, oracle, blk, threshold=0.1)[0])
    high = bc1_decode(encode_bc1(ntc, oracle, blk, threshold=0.4)[0])
    assert np.all(low[:, 3] == 1) and np.all(high[:8, 3] == 0) and np.all(high[8:, 3] == 1)


def test_checker_bc2_bc3_and_geometry(ntc, oracle):
    rng = np.random.default_rng(5)
    w, h = 22, 13
    image = rng.random((h, w, 4)).astype(np.float32) * 1.2 - 0.1
    image[:, :, :3] = (0.5 + 0.4 * np.sin(np.arange(w)[None, :, None] / 3.0 + np.arange(h)[:, None, None] / 5.0 + np.arange(3))).astype(np.float32)
    image[3, 5, 3] = np.nan
    bx, by = 6, 4
    bc2 = compress(ntc, oracle, None, image, 4, 4, 2, bx, by, off_x=1, off_y=2, pitch=(1 + bx) * 16 + 32)
    assert np.all(bc2[:2] == 0xEEEEEEEEEEEEEEEE) and np.all(bc2[:, :2] == 0xEEEEEEEEEEEEEEEE) and np.all(bc2[:, 2 + 2 * bx:] == 0xEEEEEEEEEEEEEEEE)
    bc2 = bc2[2:, 2: 2 + 2 * bx]
    bc3 = compress(ntc, oracle, None, image, 4, 4, 3, bx, by)
    assert np.array_equal(bc2[:, 1::2], bc3[:, 1::2])                       # same colour blocks
    # colour blocks ignore alpha: the same as BC1 of the image made opaque
    opaque = image.copy()
    opaque[:, :, 3] = 1.0
    bc1 = compress(ntc, oracle, None, opaque, 4, 4, 1, bx, by)
    inside = (slice(0, 3), slice(0, 5))                                     # blocks wholly inside the image
    # (outside the image BC1 reads alpha 0 where BC2 / BC3 force 1)
    assert np.array_equal(bc1[inside], bc3[:, 1::2][inside])
    # BC2 alpha: 4 bits per texel, rint(saturate(a) * 15)
    padded = np.zeros((by * 4, bx * 4), dtype=np.float32)
    padded[:h, :w] = np.clip(np.nan_to_num(image[:, :, 3], nan=0.0), 0, 1)
    want = np.rint(padded * np.float32(15.0)).astype(np.uint64)
    for j in range(by):
        for i in range(bx):
            nib = want[4 * j: 4 * j + 4, 4 * i: 4 * i + 4].reshape(-1)
            assert int(bc2[j, 2 * i]) == sum(int(v) << (4 * t) for t, v in enumerate(nib))
    # BC3 alpha = BC4 of the alpha channel
    alpha_image = np.ascontiguousarray(image[:, :, 3:4])
    bc4 = compress(ntc, oracle, None, alpha_image, 4, 1, 4, bx, by)
    assert np.array_equal(bc3[:, 0::2], bc4)
    # a sub-rectangle equals the same blocks of the full encode
    part = compress(ntc, oracle, None, image, 4, 4, 1, 2, 2, left=8, top=4)
    full = compress(ntc, oracle, None, image, 4, 4, 1, bx, by)
    assert np.array_equal(part, full[1:3, 2:4])
    # images with fewer channels: missing colour channels read 0, missing alpha reads 1
    rg = np.ascontiguousarray(image[:, :, :2])
    as_rgba = np.zeros_like(image)
    as_rgba[:, :, :2], as_rgba[:, :, 3] = rg, 1.0
    assert np.array_equal(compress(ntc, oracle, None, rg, 4, 2, 1, 5, 3), compress(ntc, oracle, None, as_rgba, 4, 4, 1, 5, 3))


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,dst_format", [(1, 1), (4, 1), (3, 2), (1, 3), (4, 3), (2, 1)])
def test_gpu_colour_block_compress_matches_checker(ntc, device, oracle, fmt, dst_format):
    rng = np.random.default_rng(100 * fmt + dst_format)
    w, h, channels = 203, 90, 4
    xs, ys = np.meshgrid(np.arange(w), np.arange(h))
    smooth = 0.5 + 0.4 * np.sin(xs[..., None] / np.array([7.0, 11.0, 5.0, 13.0]) + ys[..., None] / np.array([9.0, 4.0, 17.0, 6.0]))
    noisy = smooth + rng.normal(0, 0.05, smooth.shape) * (rng.random((h, w, 1)) < 0.5)
    noisy[rng.random((h, w)) < 0.02] = 0.0
    noisy[rng.random((h, w)) < 0.02] = 1.0
    noisy[:, :, 3] = np.where(rng.random((h, w)) < 0.15, 0.0, np.clip(noisy[:, :, 3] + 0.4, 0, 1))        # holes, mostly opaque
    noisy[40:60, 100:140, 3] = 1.0                                                                       # an opaque region
    noisy[60:80, 20:60] = noisy[60, 20]                                                                  # a constant region
    noisy[10:20, 150:170, :3] = np.where(rng.random((10, 20, 1)) < 0.5, [0.2, 0.8, 0.4], [0.7, 0.1, 0.9])   # two colours
    if fmt == 1:
        image = np.clip(np.rint(noisy * 255), 0, 255).astype(np.uint8)
    elif fmt == 2:
        image = np.clip(np.rint(noisy * 65535), 0, 65535).astype(np.uint16)
    else:
        wild = noisy * 1.3 - 0.15                                                                        # values outside [0, 1]
        image = wild.astype(np.float16 if fmt == 3 else np.float32)
        image[44:48, 60:64, :3] = np.where(rng.random((4, 4, 3)) < 0.5, -0.0, 0.0)                          # signed zeros
        if fmt == 4:
            image[5, 7, 1] = np.nan
            image[33, 90, 3] = np.nan
            image[70, 130, 0] = np.inf
    blocks_x, blocks_y = (w + 3) // 4, (h + 3) // 4
    per = 8 if dst_format == 1 else 16
    for left, top, bx, by, off_x, off_y, threshold in ((0, 0, blocks_x, blocks_y, 0, 0, 1.0 / 255.0), (8, 12, 20, 9, 3, 1, 0.5)):
        pitch = (off_x + bx) * per + 16
        want = compress(ntc, oracle, None, image, fmt, channels, dst_format, bx, by, left, top, off_x, off_y, pitch, threshold)
        got = compress(ntc, None, device, image, fmt, channels, dst_format, bx, by, left, top, off_x, off_y, pitch, threshold)
        bad = np.argwhere(got != want)
        assert bad.size == 0, (fmt, dst_format, len(bad), bad[:3], [hex(int(got[tuple(b)])) for b in bad[:3]], [hex(int(want[tuple(b)])) for b in bad[:3]])


@pytest.mark.gpu
def test_gpu_colour_block_compress_three_channel_source_and_arguments(ntc, device, oracle):
    rng = np.random.default_rng(7)
    image = rng.integers(0, 256, (32, 48, 3), dtype=np.uint8)
    for dst_format in (1, 2, 3):
        want = compress(ntc, oracle, None, image, 1, 3, dst_format, 12, 8)
        got = compress(ntc, None, device, image, 1, 3, dst_format, 12, 8)
        assert np.array_equal(got, want)
    p = ntc.abi.BlockCompress()
    d_src = device.upload(image.reshape(-1))
    d_dst = device.upload(np.zeros(12 * 8 * 16, dtype=np.uint8))
    fill_image(p.src, d_src.ptr, d_src.nbytes, 3, 3 * 48, 48, 32, 1, 3)
    p.widthInBlocks, p.heightInBlocks, p.dst, p.dstBytes, p.dstRowPitch = 12, 8, d_dst.ptr, d_dst.nbytes, 12 * 16
    for dst_format, status in ((0, ntc.abi.ERR_INVALID_ARG), (8, ntc.abi.ERR_INVALID_ARG), (-1, ntc.abi.ERR_INVALID_ARG)):
        p.dstFormat = dst_format
        assert device.lib.ntc_hip_block_compress(p) == status
    p.dstFormat, p.dstBytes = 3, 12 * 8 * 16 - 1
    assert device.lib.ntc_hip_block_compress(p) == ntc.abi.ERR_INVALID_ARG
    p.dstFormat, p.dstBytes, p.dstRowPitch = 1, 12 * 8 * 8, 12 * 8
    ntc.abi.check(device.lib.ntc_hip_block_compress(p))
    device.synchronize()
