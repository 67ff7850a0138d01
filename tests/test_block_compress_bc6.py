"""BC6H (unsigned) block compression (reference src/shaders/CompressBC6.hlsl).

What pins the checker:
  * its deterministic log2 / exp2 (the shader uses the hardware's approximations) against numpy's;
  * a BC6H decoder written here from the format specification (numpy) for the three modes the encoder
    emits - 10-bit one-subset (mode 11), 7-bit base + 6-bit deltas (mode 2), 9-bit base + 5-bit deltas
    (mode 6): constant blocks decode to within the endpoint quantisation step, smooth blocks to about
    a percent, two-region blocks choose the two-subset modes and decode well, out-of-range texels are
    clamped;
  * the partitions are the first 32 of the BC7 table (checked against the reference there).
Float operation order and the transcendental functions differ from a compiled shader by construction:
parity with its exact blocks is unpinned.  The kernel must equal the checker bit for bit."""
import numpy as np
import pytest

from test_block_compress_color import compress
from test_block_compress_bc7 import tables  # noqa: F401  (fixture)

W3 = [0, 9, 18, 27, 37, 46, 55, 64]
W4 = [0, 4, 9, 13, 17, 21, 26, 30, 34, 38, 43, 47, 51, 55, 60, 64]


def field(bits, *positions):
    """Assembles a value from single bit positions, lowest bit first."""
    return sum(((bits >> p) & 1) << i for i, p in enumerate(positions))


def rng_bits(bits, start, count):
    return (bits >> start) & ((1 << count) - 1)


def sext(v, n):
    return v - (1 << n) if v & (1 << (n - 1)) else v


def unquantize(x, n):
    if x == 0:
        return 0
    if x == (1 << n) - 1:
        return 0xFFFF
    return ((x << 16) + 0x8000) >> n


def bc6_decode(lo, hi, tables):
    """-> (mode, partition, 16 RGB texels as float32), unsigned BC6H as the format defines it."""
    two, _, anchors = tables
    bits = int(lo) | (int(hi) << 64)
    if bits & 3 == 1:                                     # mode 2: 7.666
        mode, base, delta = 2, 7, 6
        rw, gw, bw = rng_bits(bits, 5, 7), rng_bits(bits, 15, 7), rng_bits(bits, 25, 7)
        rx, gx, bx = rng_bits(bits, 35, 6), rng_bits(bits, 45, 6), rng_bits(bits, 55, 6)
        ry, rz = rng_bits(bits, 65, 6), rng_bits(bits, 71, 6)
        gy = field(bits, 41, 42, 43, 44, 24, 2)
        gz = field(bits, 51, 52, 53, 54, 3, 4)
        by = field(bits, 61, 62, 63, 64, 14, 22)
        bz = field(bits, 12, 13, 23, 32, 34, 33)
    elif bits & 31 == 0x0E:                               # mode 6: 9.555
        mode, base, delta = 6, 9, 5
        rw, gw, bw = rng_bits(bits, 5, 9), rng_bits(bits, 15, 9), rng_bits(bits, 25, 9)
        rx, gx, bx = rng_bits(bits, 35, 5), rng_bits(bits, 45, 5), rng_bits(bits, 55, 5)
        ry, rz = rng_bits(bits, 65, 5), rng_bits(bits, 71, 5)
        gy = field(bits, 41, 42, 43, 44, 24)
        gz = field(bits, 51, 52, 53, 54, 40)
        by = field(bits, 61, 62, 63, 64, 14)
        bz = field(bits, 50, 60, 70, 76, 34)
    else:
        assert bits & 31 == 0x03, hex(bits & 31)          # mode 11: 10.10, one subset
        ends = np.array([[rng_bits(bits, 5 + 10 * (3 * e + c), 10) for c in range(3)] for e in range(2)])
        unq = np.vectorize(lambda v: unquantize(int(v), 10))(ends)
        out, at = [], 65
        for t in range(16):
            n = 3 if t == 0 else 4
            w = W4[rng_bits(bits, at, n)]
            at += n
            out.append(((64 - w) * unq[0] + w * unq[1] + 32) >> 6)
        assert at == 128
        return 11, 0, ((np.array(out) * 31) >> 6).astype(np.uint16).view(np.float16).astype(np.float32)
    partition = rng_bits(bits, 77, 5)
    mask = (1 << base) - 1
    w = np.array([rw, gw, bw])
    ends = [w] + [(w + np.array([sext(a, delta), sext(b, delta), sext(c, delta)])) & mask for a, b, c in ((rx, gx, bx), (ry, gy, by), (rz, gz, bz))]
    unq = [np.array([unquantize(int(v), base) for v in e]) for e in ends]
    anchor = int(anchors[0, partition])
    out, at = [], 82
    for t in range(16):
        n = 2 if t in (0, anchor) else 3
        wt = W3[rng_bits(bits, at, n)]
        at += n
        s = (int(two[partition, 1]) >> t) & 1
        out.append(((64 - wt) * unq[2 * s] + wt * unq[2 * s + 1] + 32) >> 6)
    assert at == 128
    return mode, partition, ((np.array(out) * 31) >> 6).astype(np.uint16).view(np.float16).astype(np.float32)


def image_of_blocks(blocks):
    n = blocks.shape[0]
    image = np.zeros((4, 4 * n, 3), dtype=np.float32)
    for i in range(n):
        image[:, 4 * i: 4 * i + 4] = blocks[i].reshape(4, 4, 3)
    return image


def encode_bc6(ntc, oracle, blocks):
    return compress(ntc, oracle, None, image_of_blocks(blocks), 4, 3, 6, blocks.shape[0], 1).reshape(-1, 2)


def test_checker_log2_and_exp2(oracle):
    rng = np.random.default_rng(1)
    xs = np.concatenate([np.exp2(rng.uniform(-140, 127, 4000)), [1.0, 2.0, 0.5, 1.4142135, 1.4142137, 65505.0, 1e-45, 1.1754944e-38, 3.4e38]]).astype(np.float32)
    got = np.array([oracle.ntc_oracle_bc6_log2(float(x)) for x in xs])
    want = np.log2(xs.astype(np.float64))
    assert np.abs(got - want).max() <= 4e-7 * np.maximum(1.0, np.abs(want)).max()
    assert np.all(np.abs(got - want) <= 2.5e-7 * np.maximum(1.0, np.abs(want)))
    assert oracle.ntc_oracle_bc6_log2(0.0) == -np.inf and np.isnan(oracle.ntc_oracle_bc6_log2(-1.0)) and oracle.ntc_oracle_bc6_log2(np.inf) == np.inf
    assert oracle.ntc_oracle_bc6_log2(1.0) == 0.0 and oracle.ntc_oracle_bc6_log2(8.0) == 3.0
    ys = np.concatenate([rng.uniform(-149, 127.99, 4000), [0.0, 1.0, -1.0, 0.5, -0.5, 16.0, -126.0, -126.5, -149.0, 127.5]]).astype(np.float32)
    got = np.array([oracle.ntc_oracle_bc6_exp2(float(y)) for y in ys], dtype=np.float64)
    want = np.exp2(ys.astype(np.float64))
    normal = want >= 1.2e-38
    assert np.all(np.abs(got[normal] - want[normal]) <= 3e-7 * want[normal])
    assert np.all(np.abs(got[~normal] - want[~normal]) <= 1.5e-45 + 3e-7 * want[~normal])
    assert oracle.ntc_oracle_bc6_exp2(0.0) == 1.0 and oracle.ntc_oracle_bc6_exp2(10.0) == 1024.0 and oracle.ntc_oracle_bc6_exp2(-3.0) == 0.125
    assert oracle.ntc_oracle_bc6_exp2(128.0) == np.inf and oracle.ntc_oracle_bc6_exp2(-151.0) == 0.0 and np.isnan(oracle.ntc_oracle_bc6_exp2(np.nan))


def test_checker_bc6_constant_blocks_and_clamping(ntc, oracle, tables):
    rng = np.random.default_rng(2)
    colours = np.concatenate([np.exp2(rng.uniform(-6, 12, (40, 3))), [[0, 0, 0], [1, 1, 1], [65504, 65504, 65504], [0.5, 0, 1000.0]]]).astype(np.float32)
    blocks = np.repeat(colours[:, None, :], 16, axis=1)
    out = encode_bc6(ntc, oracle, blocks)
    for (lo, hi), colour in zip(out, colours):
        mode, _, dec = bc6_decode(lo, hi, tables)
        assert np.all(dec == dec[0])
        # 10-bit endpoints: 31 half codes per step, i.e. 3.1 % of the value (plus half a smallest step near 0)
        assert np.all(np.abs(dec[0] - colour) <= 0.032 * colour + 2e-3), (mode, colour, dec[0])
    # values a BC6H block cannot hold are clamped: negatives and NaN to 0, anything above to 65504
    wild = np.repeat(np.array([[-5.0, np.nan, 1e9], [np.inf, -np.inf, 3.0]], dtype=np.float32)[:, None, :], 16, axis=1)
    clamped = np.repeat(np.array([[0.0, 0.0, 65504.0], [65504.0, 0.0, 3.0]], dtype=np.float32)[:, None, :], 16, axis=1)
    assert np.array_equal(encode_bc6(ntc, oracle, wild), encode_bc6(ntc, oracle, clamped))


def sample_blocks(rng, tables, n_each=40):
    two = tables[0]
    xs, ys = np.meshgrid(np.arange(4), np.arange(4))

    def smooth():
        a = np.exp2(rng.uniform(-3, 8, 3))
        b = a * np.exp2(rng.uniform(-1.5, 1.5, 3))
        t = (xs * rng.normal(0, 0.12) + ys * rng.normal(0, 0.12) + rng.random()).reshape(16, 1)
        t = t - np.floor(t)
        return (a + (b - a) * t) * (1 + rng.normal(0, 0.002, (16, 3)))
    blocks, kinds = [], []
    for _ in range(n_each):
        blocks.append(smooth()); kinds.append("smooth")
    for kind, factors in (("two regions, near", [0.6, 1.6]), ("two regions, far", [0.1, 8.0])):
        for _ in range(n_each):
            a = smooth()
            c = a[::-1] * rng.choice(factors) * np.exp2(rng.uniform(-0.2, 0.2, 3))
            p = rng.integers(0, 32)
            pick = np.array([(int(two[p, 1]) >> t) & 1 for t in range(16)], dtype=bool)
            blocks.append(np.where(pick[:, None], a, c)); kinds.append(kind)
    for _ in range(n_each):
        blocks.append(np.exp2(rng.uniform(-2, 6, (16, 3)))); kinds.append("noise")
    return np.array(blocks, dtype=np.float32), np.array(kinds)


def test_checker_bc6_quality_and_modes(ntc, oracle, tables):
    rng = np.random.default_rng(3)
    blocks, kinds = sample_blocks(rng, tables)
    out = encode_bc6(ntc, oracle, blocks)
    modes, errors = [], []
    for (lo, hi), b in zip(out, blocks):
        mode, _, dec = bc6_decode(lo, hi, tables)
        assert np.all(np.isfinite(dec))
        modes.append(mode)
        errors.append(np.mean(np.log2((dec + 1.0) / (b + 1.0)) ** 2))
    modes, errors = np.array(modes), np.array(errors)
    report = {k: (float(np.sqrt(errors[kinds == k].mean())), sorted(set(modes[kinds == k].tolist()))) for k in dict.fromkeys(kinds)}
    print(report)
    # root mean squared log2 error: 0.04 is 2.8 % of the value (a 4-bit ramp over a factor of up to 2.8)
    assert np.sqrt(errors[kinds == "smooth"].mean()) < 0.04
    assert np.sqrt(errors[kinds == "two regions, near"].mean()) < 0.08
    assert np.sqrt(errors[kinds == "two regions, far"].mean()) < 0.2       # only the coarse 7-bit mode reaches that far
    assert np.isin(modes[kinds == "two regions, near"], [2, 6]).mean() > 0.7
    assert np.isin(modes[kinds == "two regions, far"], [2]).mean() > 0.4
    assert set(modes.tolist()) == {2, 6, 11}


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [4, 3, 1])
def test_gpu_bc6_matches_checker(ntc, device, oracle, fmt):
    rng = np.random.default_rng(600 + fmt)
    w, h = 131, 58
    xs, ys = np.meshgrid(np.arange(w), np.arange(h))
    base = np.exp2(3 * np.sin(xs[..., None] / np.array([7.0, 11.0, 5.0]) + ys[..., None] / np.array([9.0, 4.0, 17.0])) + 2)
    image = base * (1 + rng.normal(0, 0.05, base.shape) * (rng.random((h, w, 1)) < 0.5))
    edges = (xs // 3 + ys // 5) % 2 == 0
    image[edges] *= 0.05                                                     # hard edges inside blocks
    image[20:28, 8:40] = image[20, 8]                                        # a constant region
    image[30:34, 50:90] = 0.0
    if fmt == 1:
        image = np.clip(np.rint(image * 4), 0, 255).astype(np.uint8)         # low dynamic range input works too
    else:
        image = image.astype(np.float16 if fmt == 3 else np.float32)
        image[44:48, 60:64] = np.where(rng.random((4, 4, 3)) < 0.5, -0.0, 0.0)             # signed zeros
        if fmt == 4:
            image[5, 7, 1], image[33, 90, 2], image[40, 3, 0], image[41, 100, 1] = np.nan, np.inf, -3.0, 1e7
    blocks_x, blocks_y = (w + 3) // 4, (h + 3) // 4
    for left, top, bx, by, off_x, off_y in ((0, 0, blocks_x, blocks_y, 0, 0), (8, 12, 15, 7, 3, 1)):
        pitch = (off_x + bx) * 16 + 16
        want = compress(ntc, oracle, None, image, fmt, 3, 6, bx, by, left, top, off_x, off_y, pitch)
        got = compress(ntc, None, device, image, fmt, 3, 6, bx, by, left, top, off_x, off_y, pitch)
        bad = np.argwhere(got != want)
        assert bad.size == 0, (fmt, len(bad), bad[:3], [hex(int(got[tuple(b)])) for b in bad[:3]], [hex(int(want[tuple(b)])) for b in bad[:3]])
