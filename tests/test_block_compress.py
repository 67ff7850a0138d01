"""BC4 / BC5 block compression (reference src/shaders/CompressBC4.hlsl, CompressBC5.hlsl and the
BC4_* functions of BlockCompressCommon.hlsli): the pass that follows decode when textures are handed
to a renderer block-compressed.

The checker is pinned through the format's standard decoder (numpy): blocks that a BC4 block can
hold exactly must decode exactly, random blocks must come close to the best block a brute-force
search over all endpoint pairs finds, and the refinement never ends worse than it started.  The
kernel must equal the checker bit for bit."""
import ctypes as C

import numpy as np
import pytest

from test_image_difference import fill_image


def bc4_palette(e0, e1):
    """Palette of a BC4 block as the format defines it (real-valued interpolation)."""
    p = np.zeros(8)
    p[0], p[1] = e0, e1
    if e0 > e1:
        for k in range(2, 8):
            p[k] = ((8 - k) * e0 + (k - 1) * e1) / 7.0
    else:
        for k in range(2, 6):
            p[k] = ((6 - k) * e0 + (k - 1) * e1) / 5.0
        p[6], p[7] = 0.0, 255.0
    return p


def bc4_decode(block):
    """16 values in [0, 255] of one 64-bit BC4 block."""
    block = int(block)
    pal = bc4_palette(block & 0xFF, (block >> 8) & 0xFF)
    return np.array([pal[(block >> (16 + 3 * t)) & 7] for t in range(16)])


def oracle_bc(ntc, oracle, image, fmt, channels, dst_format, blocks_x, blocks_y, left=0, top=0, off_x=0, off_y=0, pitch=None, fill=0xEE):
    """image: [h][w][channels] array of the format's dtype.  Returns the destination as uint64 [rows][pitch / 8]."""
    h, w = image.shape[:2]
    raw = np.ascontiguousarray(image).view(np.uint8).reshape(-1)
    per = 8 if dst_format == 4 else 16
    pitch = pitch or (off_x + blocks_x) * per
    dst = np.full((off_y + blocks_y) * pitch, fill, dtype=np.uint8)
    p = ntc.abi.BlockCompress()
    stride = image.strides[1]
    fill_image(p.src, raw.ctypes.data, raw.nbytes, stride, stride * w, w, h, fmt, channels)
    p.srcLeft, p.srcTop, p.widthInBlocks, p.heightInBlocks, p.dstFormat = left, top, blocks_x, blocks_y, dst_format
    p.dstOffsetX, p.dstOffsetY, p.dst, p.dstBytes, p.dstRowPitch = off_x, off_y, dst.ctypes.data, dst.nbytes, pitch
    assert oracle.ntc_oracle_block_compress(C.byref(p)) == 0
    return dst.view(np.uint64).reshape(off_y + blocks_y, pitch // 8)


def encode_blocks(ntc, oracle, values):
    """values: [n][16] integers 0..255 -> n BC4 blocks (through a UNORM8 image of n blocks side by side)."""
    n = values.shape[0]
    image = np.zeros((4, 4 * n, 1), dtype=np.uint8)
    for i in range(n):
        image[:, 4 * i: 4 * i + 4, 0] = values[i].reshape(4, 4)
    return oracle_bc(ntc, oracle, image, 1, 1, 4, n, 1)[0]


def block_error(block, values):
    return float(((bc4_decode(block) - values) ** 2).sum())


def block_error_integer_palette(block, v):
    """Squared error measured as the encoder measures it: integer palette with the +3 / +2 rounding bias."""
    block = int(block)
    e0, e1 = block & 0xFF, (block >> 8) & 0xFF
    pal = [e0, e1] + ([((7 - k) * e0 + k * e1 + 3) // 7 for k in range(1, 7)] if e0 > e1
                      else [((5 - k) * e0 + k * e1 + 2) // 5 for k in range(1, 5)] + [0, 255])
    return float(sum((pal[(block >> (16 + 3 * t)) & 7] - int(v[t])) ** 2 for t in range(16)))


def start_error(v):
    """Squared error of the eight-value palette the encoder starts from (integer palette)."""
    lo, hi = int(v.min()), int(v.max())
    e0 = 255 if hi == 255 else hi - (hi - lo) // 34
    e1 = 0 if lo == 0 else lo + (hi - lo) // 34
    pal = np.array([e0, e1] + ([((7 - k) * e0 + k * e1 + 3) // 7 for k in range(1, 7)] if e0 > e1
                               else [((5 - k) * e0 + k * e1 + 2) // 5 for k in range(1, 5)] + [0, 255]))
    return float(((pal[None, :] - v[:, None]) ** 2).min(axis=1).sum())


def test_checker_blocks_that_bc4_holds_exactly(ntc, oracle):
    """Constant blocks and blocks whose values are the extremes 0 / 255 plus the eight-value start
    palette's own entries decode exactly.  (Two arbitrary values need not: when the refinement ends on
    a repeated assignment the reference keeps the error from before the last refit for its comparison
    with the six-value candidate, hlsli:734-738,785-788, and that is mirrored.)"""
    rng = np.random.default_rng(1)
    cases = [np.full(16, v) for v in (0, 1, 7, 128, 254, 255)]
    for _ in range(20):
        cases.append(rng.choice([0, 255], 16))
    values = np.array(cases)
    blocks = encode_blocks(ntc, oracle, values)
    for block, want in zip(blocks, values):
        assert np.array_equal(bc4_decode(block), want), (hex(int(block)), want)
    # two values, ramps: at most the error of the start palette, and exact far more often than not
    cases = []
    for _ in range(60):
        a, b = sorted(rng.choice(256, 2, replace=False))
        cases.append(rng.choice([a, b], 16))
    for _ in range(40):
        step = int(rng.integers(1, 37))
        lo = int(rng.integers(0, 256 - 7 * step))
        cases.append(lo + step * rng.integers(0, 8, 16))
    values = np.array(cases)
    blocks = encode_blocks(ntc, oracle, values)
    errors = np.array([block_error_integer_palette(b, v) for b, v in zip(blocks, values)])
    starts = np.array([start_error(v) for v in values])
    assert np.all(errors <= starts)
    assert (errors[:60] == 0).mean() > 0.5


def best_possible_error(values):
    """Smallest squared error over every endpoint pair (both palettes), nearest entry per texel."""
    e0, e1 = np.meshgrid(np.arange(256.0), np.arange(256.0), indexing="ij")
    k = np.arange(2, 8)[None, None, :]
    eight = ((8 - k) * e0[..., None] + (k - 1) * e1[..., None]) / 7.0
    k6 = np.arange(2, 6)[None, None, :]
    six = np.concatenate([((6 - k6) * e0[..., None] + (k6 - 1) * e1[..., None]) / 5.0,
                          np.zeros((256, 256, 1)), np.full((256, 256, 1), 255.0)], axis=2)
    pal = np.where((e0 > e1)[..., None], eight, six)
    pal = np.concatenate([e0[..., None], e1[..., None], pal], axis=2)       # [256][256][8]
    err = np.zeros((256, 256))
    for v in values:
        err += ((pal - v) ** 2).min(axis=2)
    return err.min()


def test_checker_quality_against_brute_force(ntc, oracle):
    rng = np.random.default_rng(2)
    blocks_values = []
    for _ in range(32):
        base, slope_x, slope_y = rng.integers(0, 200), rng.integers(-12, 13), rng.integers(-12, 13)
        xs, ys = np.meshgrid(np.arange(4), np.arange(4))
        v = base + slope_x * xs + slope_y * ys + rng.normal(0, rng.choice([0.5, 3, 10]), (4, 4))
        blocks_values.append(np.clip(np.rint(v), 0, 255).reshape(-1).astype(np.int64))
    for _ in range(8):
        blocks_values.append(rng.integers(0, 256, 16))                      # noise
    values = np.array(blocks_values)
    blocks = encode_blocks(ntc, oracle, values)
    ratios = np.array([(block_error(b, v) + 4.0) / (best_possible_error(v) + 4.0) for b, v in zip(blocks, values)])
    assert np.median(ratios) < 1.2 and np.quantile(ratios, 0.9) < 2.0, (np.median(ratios), np.quantile(ratios, 0.9), ratios.max())


def test_checker_refinement_never_ends_worse_than_it_starts(ntc, oracle):
    """The encoder keeps the best block it has seen, so its error is at most that of the start
    endpoints of the eight-value palette (extremes moved inwards by range / 34, 0 and 255 kept).
    Measured with the integer palette the encoder itself uses, so the bound is exact."""
    rng = np.random.default_rng(3)
    values = rng.integers(0, 256, (300, 16))
    values[:100] = np.clip(values[:100] // 8 + 100, 0, 255)                 # narrow ranges too
    blocks = encode_blocks(ntc, oracle, values)
    for block, v in zip(blocks, values):
        assert block_error_integer_palette(block, v) <= start_error(v), (hex(int(block)), v)


def test_checker_block_geometry_and_inputs(ntc, oracle):
    rng = np.random.default_rng(4)
    w, h = 22, 13                                                           # not multiples of 4: the rest reads as 0
    image = rng.random((h, w, 3)).astype(np.float32) * 1.4 - 0.2            # values outside [0, 1] saturate
    image[2, 3, 0] = np.nan                                                 # a NaN counts as 0
    blocks_x, blocks_y = 6, 4
    out = oracle_bc(ntc, oracle, image, 4, 3, 5, blocks_x, blocks_y, off_x=1, off_y=2, pitch=(1 + blocks_x) * 16 + 32)
    assert np.all(out[:2] == 0xEEEEEEEEEEEEEEEE) and np.all(out[:, :2] == 0xEEEEEEEEEEEEEEEE) and np.all(out[:, 2 + 2 * blocks_x:] == 0xEEEEEEEEEEEEEEEE)
    padded = np.zeros((blocks_y * 4, blocks_x * 4, 2))
    sat = np.clip(np.nan_to_num(image[:, :, :2], nan=0.0), 0, 1)
    padded[:h, :w] = np.rint(sat.astype(np.float32) * np.float32(255.0))
    for by in range(blocks_y):
        for bx in range(blocks_x):
            for c in range(2):
                want = padded[4 * by: 4 * by + 4, 4 * bx: 4 * bx + 4, c].reshape(-1)
                got = bc4_decode(out[2 + by, 2 + 2 * bx + c])
                rng_ = want.max() - want.min()
                assert np.abs(got - want).max() <= rng_ / 14.0 + 2.0, (by, bx, c)
    # a sub-rectangle equals the same blocks of the full encode
    full = oracle_bc(ntc, oracle, image, 4, 3, 4, blocks_x, blocks_y)
    part = oracle_bc(ntc, oracle, image, 4, 3, 4, 2, 2, left=8, top=4)
    assert np.array_equal(part, full[1:3, 2:4])
    p = ntc.abi.BlockCompress()
    p.dstFormat = 8
    assert oracle.ntc_oracle_block_compress(C.byref(p)) == -1


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,dst_format", [(1, 4), (1, 5), (3, 5), (4, 4), (2, 5)])
def test_gpu_block_compress_matches_checker(ntc, device, oracle, fmt, dst_format):
    rng = np.random.default_rng(10 * fmt + dst_format)
    w, h, channels = 203, 90, 4
    xs, ys = np.meshgrid(np.arange(w), np.arange(h))
    smooth = 0.5 + 0.4 * np.sin(xs[..., None] / np.array([7.0, 11.0, 5.0, 13.0]) + ys[..., None] / np.array([9.0, 4.0, 17.0, 6.0]))
    noisy = smooth + rng.normal(0, 0.05, smooth.shape) * (rng.random((h, w, 1)) < 0.5)
    noisy[rng.random((h, w)) < 0.02] = 0.0
    noisy[rng.random((h, w)) < 0.02] = 1.0
    if fmt == 1:
        image = np.clip(np.rint(noisy * 255), 0, 255).astype(np.uint8)
    elif fmt == 2:
        image = np.clip(np.rint(noisy * 65535), 0, 65535).astype(np.uint16)
    else:
        image = noisy.astype(np.float16 if fmt == 3 else np.float32)
    blocks_x, blocks_y = (w + 3) // 4, (h + 3) // 4
    per = 8 if dst_format == 4 else 16
    for left, top, bx, by, off_x, off_y in ((0, 0, blocks_x, blocks_y, 0, 0), (8, 12, 20, 9, 3, 1)):
        pitch = (off_x + bx) * per + 16
        want = oracle_bc(ntc, oracle, image, fmt, channels, dst_format, bx, by, left, top, off_x, off_y, pitch)
        d_src = device.upload(np.ascontiguousarray(image).view(np.uint8).reshape(-1))
        d_dst = device.upload(np.full((off_y + by) * pitch, 0xEE, dtype=np.uint8))
        p = ntc.abi.BlockCompress()
        fill_image(p.src, d_src.ptr, d_src.nbytes, image.strides[1], image.strides[1] * w, w, h, fmt, channels)
        p.srcLeft, p.srcTop, p.widthInBlocks, p.heightInBlocks, p.dstFormat = left, top, bx, by, dst_format
        p.dstOffsetX, p.dstOffsetY, p.dst, p.dstBytes, p.dstRowPitch = off_x, off_y, d_dst.ptr, d_dst.nbytes, pitch
        ntc.abi.check(device.lib.ntc_hip_block_compress(p))
        device.synchronize()
        got = d_dst.download().view(np.uint64).reshape(off_y + by, pitch // 8)
        bad = np.argwhere(got != want)
        assert bad.size == 0, (fmt, dst_format, len(bad), bad[:3], [hex(int(got[tuple(b)])) for b in bad[:3]], [hex(int(want[tuple(b)])) for b in bad[:3]])
    # argument checks
    p.dstFormat = 9
    assert device.lib.ntc_hip_block_compress(p) == ntc.abi.ERR_INVALID_ARG
    p.dstFormat = dst_format
    p.dstBytes = (off_y + by - 1) * pitch + (off_x + bx) * per - 1      # one byte short of the last block
    assert device.lib.ntc_hip_block_compress(p) == ntc.abi.ERR_INVALID_ARG
    p.dstBytes = d_dst.nbytes
    p.dstRowPitch = pitch - 4
    assert device.lib.ntc_hip_block_compress(p) == ntc.abi.ERR_INVALID_ARG


def test_unorm_quotient_shortcut_is_exact():
    """The kernels turn UNORM8 / UNORM16 texels into floats with q = k * r, q + fma(-q, d, k) * r (r = 1 / d
    rounded) instead of a division; that is the correctly rounded k / d for every k (exact rationals here)."""
    from fractions import Fraction

    def rn32(value):
        f = np.float32(float(value))
        candidates = [f, np.nextafter(f, np.float32(np.inf)), np.nextafter(f, np.float32(-np.inf))]
        return min(candidates, key=lambda c: (abs(Fraction(float(c)) - value), int(np.float32(c).view(np.uint32)) & 1))
    for d in (255, 65535):
        r = np.float32(1.0) / np.float32(d)
        ks = range(d + 1) if d == 255 else list(range(0, 65536, 7)) + [65535, 65534, 32768, 32767, 1, 2, 3]
        for k in ks:
            q = np.float32(k) * r
            rem = rn32(Fraction(float(-q)) * d + k)
            q2 = rn32(Fraction(float(rem)) * Fraction(float(r)) + Fraction(float(q)))
            assert q2 == np.float32(k) / np.float32(d), (d, k)

