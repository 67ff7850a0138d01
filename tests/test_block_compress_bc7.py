"""BC7 block compression (reference src/shaders/CompressBC7.hlsl; mode buffer:
MakeBC7ModeBuffer, src/PublicFunctions.cpp:476-558).

What pins the checker:
  * its partition and anchor tables, typed from the format specification, equal the reference's
    (digest fixture; the literal values too where the reference is present);
  * a BC7 decoder written here from the format specification (numpy): every block the encoder
    emits must be a valid block that decodes close to its source - constant colours and exact alpha
    0 / 1 to within a code, smooth and two-region blocks far better than BC1 does, and the error
    the decoder measures must be the smallest among the candidates the modes offer only in the
    sense the tests state (the search is the reference's heuristic, not exhaustive);
  * the single-mode path against the full search: re-encoding every block with the mode and
    partition the full search chose must give the same block.
The float operation order inside the encoder is a stated choice (the shader compiler is free to fuse
and reorder): parity with a compiled shader's exact blocks is unpinned.  The kernel must equal the
checker bit for bit."""
import hashlib
import json
import os

import numpy as np
import pytest

from test_block_compress_color import GOLDEN, compress, encode_bc1, bc1_decode

# (subsets, partition bits, rotation bits, index-selection bit, colour bits, alpha bits, per-endpoint p-bit,
#  shared p-bit, index bits, second index bits): Table of the BPTC specification
MODES = [(3, 4, 0, 0, 4, 0, 1, 0, 3, 0), (2, 6, 0, 0, 6, 0, 0, 1, 3, 0), (3, 6, 0, 0, 5, 0, 0, 0, 2, 0), (2, 6, 0, 0, 7, 0, 1, 0, 2, 0),
         (1, 0, 2, 1, 5, 6, 0, 0, 2, 3), (1, 0, 2, 0, 7, 8, 0, 0, 2, 2), (1, 0, 0, 0, 7, 7, 1, 0, 4, 0), (2, 6, 0, 0, 5, 5, 1, 0, 2, 0)]
WEIGHTS = {2: [0, 21, 43, 64], 3: [0, 9, 18, 27, 37, 46, 55, 64], 4: [0, 4, 9, 13, 17, 21, 26, 30, 34, 38, 43, 47, 51, 55, 60, 64]}


@pytest.fixture(scope="module")
def tables(oracle):
    two, three, anchors = np.zeros((64, 2), dtype="<u4"), np.zeros((64, 3), dtype="<u4"), np.zeros((3, 64), dtype=np.uint8)
    oracle.ntc_oracle_bc7_tables(two.ctypes.data, three.ctypes.data, anchors.ctypes.data)
    return two, three, anchors


class BitReader:
    def __init__(self, lo, hi):
        self.value, self.at = int(lo) | (int(hi) << 64), 0

    def get(self, n):
        v = (self.value >> self.at) & ((1 << n) - 1)
        self.at += n
        return v


def bc7_decode(lo, hi, tables):
    """-> (mode, partition, 16 RGBA texels as integers 0..255), as the format defines them."""
    two, three, anchors = tables
    r = BitReader(lo, hi)
    mode = 0
    while mode < 8 and r.get(1) == 0:
        mode += 1
    assert mode < 8, "reserved mode"
    ns, pb, rb, isb, cb, ab, epb, spb, ib, ib2 = MODES[mode]
    partition, rotation, index_selection = r.get(pb), r.get(rb), r.get(isb)
    ends = np.zeros((2 * ns, 4), dtype=np.int64)
    for c in range(3):
        for e in range(2 * ns):
            ends[e, c] = r.get(cb)
    for e in range(2 * ns):
        ends[e, 3] = r.get(ab) if ab else 0
    cbits, abits = cb, ab
    if epb:
        for e in range(2 * ns):
            p = r.get(1)
            ends[e, :3] = (ends[e, :3] << 1) | p
            if ab:
                ends[e, 3] = (ends[e, 3] << 1) | p
        cbits, abits = cb + 1, (ab + 1 if ab else 0)
    if spb:
        for s in range(ns):
            p = r.get(1)
            ends[2 * s: 2 * s + 2, :3] = (ends[2 * s: 2 * s + 2, :3] << 1) | p
        cbits = cb + 1
    ends[:, :3] = (ends[:, :3] << (8 - cbits)) | (ends[:, :3] >> (2 * cbits - 8))
    if ab:
        ends[:, 3] = (ends[:, 3] << (8 - abits)) | (ends[:, 3] >> (2 * abits - 8))
    else:
        ends[:, 3] = 255
    if ns == 1:
        subset = np.zeros(16, dtype=int)
        anchor_of = [0]
    elif ns == 2:
        subset = np.array([1 if (int(two[partition, 1]) >> t) & 1 else 0 for t in range(16)])
        anchor_of = [0, int(anchors[0, partition])]
    else:
        subset = np.array([2 if (int(three[partition, 2]) >> t) & 1 else (1 if (int(three[partition, 1]) >> t) & 1 else 0) for t in range(16)])
        anchor_of = [0, int(anchors[1, partition]), int(anchors[2, partition])]
    first = [r.get(ib - 1 if t == anchor_of[subset[t]] else ib) for t in range(16)]
    second = [r.get(ib2 - 1 if t == 0 else ib2) for t in range(16)] if ib2 else None
    assert r.at == 128, (mode, r.at)
    out = np.zeros((16, 4), dtype=np.int64)
    for t in range(16):
        e0, e1 = ends[2 * subset[t]], ends[2 * subset[t] + 1]
        if second is None:
            w = WEIGHTS[ib][first[t]]
            out[t] = ((64 - w) * e0 + w * e1 + 32) >> 6
        else:
            colour_w = WEIGHTS[ib2][second[t]] if index_selection else WEIGHTS[ib][first[t]]
            alpha_w = WEIGHTS[ib][first[t]] if index_selection else WEIGHTS[ib2][second[t]]
            out[t, :3] = ((64 - colour_w) * e0[:3] + colour_w * e1[:3] + 32) >> 6
            out[t, 3] = ((64 - alpha_w) * e0[3] + alpha_w * e1[3] + 32) >> 6
        if rotation:
            out[t, rotation - 1], out[t, 3] = out[t, 3], out[t, rotation - 1]
    return mode, partition | (rotation if rb else 0) | (index_selection << 2 if isb else 0), out


def image_of_blocks(blocks):
    n = blocks.shape[0]
    image = np.zeros((4, 4 * n, 4), dtype=np.float32)
    for i in range(n):
        image[:, 4 * i: 4 * i + 4] = blocks[i].reshape(4, 4, 4)
    return image


def encode_bc7(ntc, oracle, blocks, mode_buffer=None, map_size=None, map_offset=(0, 0)):
    """blocks: [n][16][4] floats -> [n][2] uint64"""
    image = image_of_blocks(blocks)
    out = compress_bc7(ntc, oracle, None, image, 4, 4, blocks.shape[0], 1, mode_buffer=mode_buffer, map_size=map_size, map_offset=map_offset)
    return out.reshape(-1, 2)


def compress_bc7(ntc, oracle, device, image, fmt, channels, blocks_x, blocks_y, mode_buffer=None, map_size=None, map_offset=(0, 0), byte_offset=0, **kw):
    def hook(p, upload):
        if mode_buffer is not None:
            p.modeBuffer, p.modeBufferBytes, p.modeBufferByteOffset = upload(mode_buffer), mode_buffer.nbytes, byte_offset
            p.modeMapWidthInBlocks, p.modeMapHeightInBlocks = map_size or (blocks_x, blocks_y)
            p.modeMapOffsetX, p.modeMapOffsetY = map_offset
    return compress(ntc, oracle, device, image, fmt, channels, 7, blocks_x, blocks_y, hook=hook, **kw)


def pack_mode_buffer(entries, byte_offset=0):
    """9 bits per entry, little-endian bit order, size rounded up to 4 bytes (MakeBC7ModeBuffer)."""
    n = len(entries)
    out = np.zeros(byte_offset + (((n * 9 + 31) >> 5) << 2), dtype=np.uint8)
    for i, e in enumerate(entries):
        for b in range(9):
            if (int(e) >> b) & 1:
                out[byte_offset + ((i * 9 + b) >> 3)] |= 1 << ((i * 9 + b) & 7)
    return out


def entry_of(mode, partition):
    e = (mode << 6) | partition
    return 0x1BF if e == 0 else e


def sample_blocks(rng, tables, n_each=24):
    """Opaque smooth, opaque two-region, opaque three-region, noisy, translucent, with alpha 0 / 1 extremes."""
    xs, ys = np.meshgrid(np.arange(4), np.arange(4))
    blocks, kinds = [], []

    def smooth():
        # colours along one line of colour space (what one pair of endpoints can hold), slightly perturbed
        a, b = rng.random(4), rng.random(4)
        t = (xs * rng.normal(0, 0.12) + ys * rng.normal(0, 0.12) + rng.random()).reshape(16, 1)
        return np.clip(a + (b - a) * (t - np.floor(t)) + rng.normal(0, 0.004, (16, 4)), 0, 1)
    for _ in range(n_each):
        b = smooth(); b[:, 3] = 1.0
        blocks.append(b); kinds.append("smooth")
    two, three, _ = tables
    for _ in range(n_each):                                      # regions shaped like one of the format's partitions
        a, c = smooth(), smooth()
        p = rng.integers(0, 64)
        pick = np.array([(int(two[p, 1]) >> t) & 1 for t in range(16)], dtype=bool)
        b = np.where(pick[:, None], a, c); b[:, 3] = 1.0
        blocks.append(b); kinds.append("two regions")
    for _ in range(n_each):
        a, c, d = smooth(), smooth(), smooth()
        p = rng.integers(0, 64)
        region = np.array([2 if (int(three[p, 2]) >> t) & 1 else (1 if (int(three[p, 1]) >> t) & 1 else 0) for t in range(16)])
        b = np.choose(region[:, None], [a, c, d]); b[:, 3] = 1.0
        blocks.append(b); kinds.append("three regions")
    for _ in range(n_each):
        b = rng.random((16, 4)); b[:, 3] = 1.0
        blocks.append(b); kinds.append("noise")
    for _ in range(n_each):
        blocks.append(smooth()); kinds.append("translucent")
    for _ in range(n_each):
        b = smooth()
        b[:, 3] = rng.choice([0.0, 1.0], 16)
        blocks.append(b); kinds.append("alpha 0 / 1")
    for _ in range(n_each):
        b = smooth()
        b[:, :3] = b[0, :3]                                      # constant colour, alpha varies
        blocks.append(b); kinds.append("alpha only")
    return np.array(blocks), kinds


def test_checker_bc7_tables_equal_the_reference(tables):
    two, three, anchors = tables
    golden = json.load(open(os.path.join(GOLDEN, "bc_tables.json")))["bc7"]
    assert hashlib.sha256(two.tobytes()).hexdigest() == golden["sha256_two_subsets"]
    assert hashlib.sha256(three.tobytes()).hexdigest() == golden["sha256_three_subsets"]
    assert hashlib.sha256(anchors.tobytes()).hexdigest() == golden["sha256_anchors"]
    if os.path.exists("/root/reference/src/shaders/CompressBC7.hlsl"):
        import importlib.util
        spec = importlib.util.spec_from_file_location("make_bc_table_digests", os.path.join(GOLDEN, "make_bc_table_digests.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        ref2, ref3, ref_anchors = mod.reference_bc7_tables()
        assert np.array_equal(two, ref2) and np.array_equal(three, ref3) and np.array_equal(anchors, ref_anchors)
    # what the format requires of them: subsets partition the block, texel 0 is in subset 0, anchors lie in their subsets
    assert np.all((two[:, 0] | two[:, 1]) == 0xFFFF) and np.all((two[:, 0] & two[:, 1]) == 0) and np.all(two[:, 0] & 1)
    assert np.all((three[:, 0] | three[:, 1] | three[:, 2]) == 0xFFFF) and np.all(three[:, 0] & 1)
    assert np.all((three[:, 0] & three[:, 1]) == 0) and np.all((three[:, 0] & three[:, 2]) == 0) and np.all((three[:, 1] & three[:, 2]) == 0)
    for p in range(64):
        assert (int(two[p, 1]) >> int(anchors[0, p])) & 1 and (int(three[p, 1]) >> int(anchors[1, p])) & 1 and (int(three[p, 2]) >> int(anchors[2, p])) & 1


def test_checker_bc7_constant_and_extreme_blocks(ntc, oracle, tables):
    rng = np.random.default_rng(1)
    colours = np.concatenate([rng.integers(0, 256, (40, 4)), [[0, 0, 0, 255], [255, 255, 255, 255], [0, 0, 0, 0], [255, 0, 128, 0], [17, 17, 17, 255]]])
    colours[:20, 3] = 255
    blocks = np.repeat((colours / 255.0)[:, None, :], 16, axis=1)
    out = encode_bc7(ntc, oracle, blocks)
    for (lo, hi), colour in zip(out, colours):
        mode, _, dec = bc7_decode(lo, hi, tables)
        assert np.all(dec == dec[0]), (mode, dec)
        assert np.abs(dec[0] - colour).max() <= 1, (mode, colour, dec[0])
        if colour[3] in (0, 255):
            assert dec[0, 3] == colour[3], (mode, colour, dec[0])


def test_checker_bc7_quality_and_modes(ntc, oracle, tables):
    rng = np.random.default_rng(2)
    blocks, kinds = sample_blocks(rng, tables)
    out = encode_bc7(ntc, oracle, blocks)
    modes, errors = [], []
    for (lo, hi), b in zip(out, blocks):
        mode, _, dec = bc7_decode(lo, hi, tables)
        modes.append(mode)
        errors.append(((dec / 255.0 - b) ** 2).sum())
    modes, errors, kinds = np.array(modes), np.array(errors), np.array(kinds)
    psnr = lambda e: 10 * np.log10(1.0 / (e.mean() / 64 + 1e-12))
    report = {k: (round(float(psnr(errors[kinds == k])), 1), sorted(set(modes[kinds == k].tolist()))) for k in dict.fromkeys(kinds)}
    print(report)
    assert psnr(errors[kinds == "smooth"]) > 43 and psnr(errors[kinds == "two regions"]) > 39 and psnr(errors[kinds == "three regions"]) > 35
    assert psnr(errors[kinds == "translucent"]) > 41 and psnr(errors[kinds == "alpha only"]) > 45 and psnr(errors[kinds == "alpha 0 / 1"]) > 36
    # opaque blocks keep alpha at 255; blocks with alpha never use the opaque-only modes
    for (lo, hi), b, mode in zip(out, blocks, modes):
        if np.all(b[:, 3] == 1.0):
            assert np.all(bc7_decode(lo, hi, tables)[2][:, 3] == 255)
        else:
            assert mode >= 4
    # alpha exactly 0 / 1 stays exact where the whole block has only those two values
    for (lo, hi), b in zip(out[kinds == "alpha 0 / 1"], blocks[kinds == "alpha 0 / 1"]):
        dec = bc7_decode(lo, hi, tables)[2]
        assert np.array_equal(dec[:, 3], (b[:, 3] * 255).astype(int))
    # partitioned modes are what region blocks need; every family of modes occurs somewhere
    assert np.isin(modes[kinds == "two regions"], [0, 1, 2, 3, 7]).mean() > 0.6
    assert np.isin(modes[kinds == "three regions"], [0, 2]).mean() > 0.3
    assert len(set(modes.tolist())) >= 6, set(modes.tolist())
    # BC7 against BC1 on the opaque blocks: a small fraction of its error
    opaque = np.isin(kinds, ["smooth", "two regions", "three regions"])
    bc1 = encode_bc1(ntc, oracle, blocks[opaque])
    bc1_errors = np.array([((bc1_decode(o)[:, :3] - b[:, :3]) ** 2).sum() for o, b in zip(bc1, blocks[opaque])])
    assert errors[opaque].sum() < 0.2 * bc1_errors.sum(), (errors[opaque].sum(), bc1_errors.sum())


def test_checker_bc7_single_mode_equals_full_search(ntc, oracle, tables):
    """The mode buffer path computes the chosen mode exactly as the full search does, so encoding each
    block again with the (mode, partition) the full search ended on gives the same block; entries of 0
    and blocks outside the mode map give the marker block."""
    rng = np.random.default_rng(3)
    blocks, _ = sample_blocks(rng, tables, n_each=12)
    full = encode_bc7(ntc, oracle, blocks)
    entries = []
    for lo, hi in full:
        mode, partition, _ = bc7_decode(lo, hi, tables)
        entries.append(entry_of(mode, partition))
    again = encode_bc7(ntc, oracle, blocks, mode_buffer=pack_mode_buffer(entries))
    assert np.array_equal(again, full), np.argwhere(again != full)[:4]
    # forcing another mode still gives valid blocks of that mode that decode sensibly
    for forced in range(8):
        part = 5 if forced in (0, 1, 2, 3, 7) else (6 if forced == 4 else 2 if forced == 5 else 0)
        out = encode_bc7(ntc, oracle, blocks[:8], mode_buffer=pack_mode_buffer([entry_of(forced, part)] * 8))
        for (lo, hi), b in zip(out, blocks[:8]):
            mode, partition, dec = bc7_decode(lo, hi, tables)
            assert mode == forced and partition == part
            assert np.abs(dec[:, :3] / 255.0 - b[:, :3]).max() < 0.35
    # a map offset selects other entries; outside the map and zero entries: the marker block
    marker = np.array([0x0001f00000f80004, 0x1f9e00003ff0001f], dtype=np.uint64)
    shifted = encode_bc7(ntc, oracle, blocks[:4], mode_buffer=pack_mode_buffer([0] + entries[:2]), map_size=(3, 1), map_offset=(1, 0))
    assert np.array_equal(shifted[0], full[0]) and np.array_equal(shifted[1], full[1])
    assert np.array_equal(shifted[2], marker) and np.array_equal(shifted[3], marker)
    zero = encode_bc7(ntc, oracle, blocks[:2], mode_buffer=pack_mode_buffer([0, entries[1]]))
    assert np.array_equal(zero[0], marker) and np.array_equal(zero[1], full[1])
    mode, _, dec = bc7_decode(marker[0], marker[1], tables)        # the marker is a valid block: black, red, green, blue squares
    assert sorted(set(map(tuple, dec.tolist()))) == [(0, 0, 0, 255), (0, 0, 255, 255), (0, 255, 0, 255), (255, 0, 0, 255)]


def gpu_image(rng, w, h):
    xs, ys = np.meshgrid(np.arange(w), np.arange(h))
    smooth = 0.5 + 0.4 * np.sin(xs[..., None] / np.array([7.0, 11.0, 5.0, 13.0]) + ys[..., None] / np.array([9.0, 4.0, 17.0, 6.0]))
    noisy = smooth + rng.normal(0, 0.05, smooth.shape) * (rng.random((h, w, 1)) < 0.5)
    noisy[rng.random((h, w)) < 0.02] = 0.0
    noisy[rng.random((h, w)) < 0.02] = 1.0
    noisy[:, : w // 2, 3] = 1.0                                              # left half opaque: modes 0-3 take part
    noisy[:, w // 2:, 3] = np.where(rng.random((h, w - w // 2)) < 0.2, 0.0, np.clip(noisy[:, w // 2:, 3] + 0.3, 0, 1))
    edges = (xs // 3 + ys // 5) % 2 == 0                                     # hard edges inside blocks
    noisy[edges, :3] = 1.0 - noisy[edges, :3]
    noisy[h // 2: h // 2 + 8, 8:40] = noisy[h // 2, 8]                       # a constant region
    return noisy


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [1, 4, 3, 2])
def test_gpu_bc7_matches_checker(ntc, device, oracle, tables, fmt):
    rng = np.random.default_rng(700 + fmt)
    w, h = 131, 58
    noisy = gpu_image(rng, w, h)
    if fmt == 1:
        image = np.clip(np.rint(noisy * 255), 0, 255).astype(np.uint8)
    elif fmt == 2:
        image = np.clip(np.rint(noisy * 65535), 0, 65535).astype(np.uint16)
    else:
        image = (noisy * 1.2 - 0.1).astype(np.float16 if fmt == 3 else np.float32)
        image[:, : w // 2, 3] = 1.0
        image[44:48, 60:64, :3] = np.where(rng.random((4, 4, 3)) < 0.5, -0.0, 0.0)     # signed zeros
        if fmt == 4:
            image[5, 7, 1] = np.nan
            image[33, 90, 3] = np.nan
    blocks_x, blocks_y = (w + 3) // 4, (h + 3) // 4
    for left, top, bx, by, off_x, off_y in ((0, 0, blocks_x, blocks_y, 0, 0), (8, 12, 15, 7, 3, 1)):
        pitch = (off_x + bx) * 16 + 16
        want = compress_bc7(ntc, oracle, None, image, fmt, 4, bx, by, left=left, top=top, off_x=off_x, off_y=off_y, pitch=pitch)
        got = compress_bc7(ntc, None, device, image, fmt, 4, bx, by, left=left, top=top, off_x=off_x, off_y=off_y, pitch=pitch)
        bad = np.argwhere(got != want)
        assert bad.size == 0, (fmt, len(bad), bad[:3], [hex(int(got[tuple(b)])) for b in bad[:3]], [hex(int(want[tuple(b)])) for b in bad[:3]])
    # the same through a mode buffer made from the full search's blocks (offset inside a larger buffer and map)
    full = compress_bc7(ntc, oracle, None, image, fmt, 4, blocks_x, blocks_y).reshape(blocks_y, blocks_x, 2)
    entries = np.zeros((blocks_y + 2, blocks_x + 3), dtype=np.int64)
    for y in range(blocks_y):
        for x in range(blocks_x):
            mode, partition, _ = bc7_decode(full[y, x, 0], full[y, x, 1], tables)
            entries[y + 2, x + 3] = entry_of(mode, partition)
    entries[4, 6] = 0                                                         # one block without an entry
    buffer = pack_mode_buffer(entries.reshape(-1), byte_offset=8)
    args = dict(mode_buffer=buffer, map_size=(blocks_x + 3, blocks_y + 2), map_offset=(3, 2), byte_offset=8)
    want = compress_bc7(ntc, oracle, None, image, fmt, 4, blocks_x, blocks_y, **args).reshape(blocks_y, blocks_x, 2)
    got = compress_bc7(ntc, None, device, image, fmt, 4, blocks_x, blocks_y, **args).reshape(blocks_y, blocks_x, 2)
    assert np.array_equal(got, want), np.argwhere(got != want)[:4]
    same = np.all(want == full, axis=2)
    expected_to_differ = np.zeros_like(same)
    expected_to_differ[2, 3] = True                                           # the block without an entry
    if image.dtype.kind == "f":                                               # blocks with a NaN texel: every error is NaN, the
        for y, x in np.argwhere(np.isnan(image.astype(np.float32)).any(axis=2)):    # full search's pick depends on its order
            same[y // 4, x // 4] = False
            expected_to_differ[y // 4, x // 4] = True
    assert np.array_equal(~same, expected_to_differ), np.argwhere(~same != expected_to_differ)


@pytest.mark.gpu
def test_gpu_bc7_arguments(ntc, device, oracle):
    from test_image_difference import fill_image
    rng = np.random.default_rng(9)
    image = rng.integers(0, 256, (16, 32, 4), dtype=np.uint8)
    d_src = device.upload(image.reshape(-1))
    d_dst = device.upload(np.zeros(8 * 4 * 16, dtype=np.uint8))
    d_modes = device.upload(pack_mode_buffer([entry_of(6, 0)] * 32))
    p = ntc.abi.BlockCompress()
    fill_image(p.src, d_src.ptr, d_src.nbytes, 4, 4 * 32, 32, 16, 1, 4)
    p.widthInBlocks, p.heightInBlocks, p.dst, p.dstBytes, p.dstRowPitch, p.dstFormat = 8, 4, d_dst.ptr, d_dst.nbytes, 8 * 16, 7
    p.modeBuffer, p.modeBufferBytes, p.modeMapWidthInBlocks, p.modeMapHeightInBlocks = d_modes.ptr, d_modes.nbytes, 8, 4
    ntc.abi.check(device.lib.ntc_hip_block_compress(p))
    p.modeBufferBytes = d_modes.nbytes - 4                                   # the map no longer fits
    assert device.lib.ntc_hip_block_compress(p) == ntc.abi.ERR_INVALID_ARG
    p.modeBufferBytes, p.modeBufferByteOffset = d_modes.nbytes, 2            # not a multiple of 4
    assert device.lib.ntc_hip_block_compress(p) == ntc.abi.ERR_INVALID_ARG
    p.modeBufferByteOffset, p.modeMapWidthInBlocks = 0, 0
    assert device.lib.ntc_hip_block_compress(p) == ntc.abi.ERR_INVALID_ARG
    p.modeMapWidthInBlocks = 8
    device.synchronize()
