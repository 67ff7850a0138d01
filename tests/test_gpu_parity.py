"""GPU parity: the HIP decoder, called through the C ABI, against the CPU checker on the
same seeded inputs.  Integer/byte work: every output byte must be equal."""
import ctypes as C

import numpy as np
import pytest

from cases import cfg_case, ref_case, first_mismatch

pytestmark = pytest.mark.gpu

# scale range that keeps layer outputs inside the active part of HGELU (|x| of a few units)
# instead of saturating it, so rounding in the requantiser is exercised
ACTIVE = (-17.0, -12.0)


def run_both(device, case):
    host = case.host_set()
    host.decode(threads=8)
    dset = case.device_set(device)
    device.decode([dset])
    device.synchronize()
    got = case.d_output.download()
    return host.output, got


def assert_equal_bytes(expected, got, what):
    mm = first_mismatch(expected, got)
    assert mm is None, f"{what}: {mm[1]} of {expected.size} bytes differ, first at {mm[0]}: oracle {mm[2]} gpu {mm[3]}"


def test_mfma_operand_layout(device):
    rng = np.random.default_rng(5)
    a = rng.integers(-128, 128, size=(16, 64), dtype=np.int8)
    b = rng.integers(-128, 128, size=(64, 16), dtype=np.int8)
    d = np.zeros((16, 16), dtype=np.int32)
    from importlib import import_module
    abi = import_module("rtxntc-library_amd").abi
    abi.check(device.lib.ntc_hip_selftest_mfma(a.ctypes.data, b.ctypes.data, d.ctypes.data))
    assert np.array_equal(d, a.astype(np.int64) @ b.astype(np.int64))


@pytest.mark.parametrize("depth", [16, 32])
def test_mfma_f16_integer_sums_are_exact(device, depth):
    """The fp16 matrix instruction with integer-valued operands: layout, and exactness of the fp32
    accumulation while every partial sum stays below 2^24 -- including accumulator inputs that
    leave only a few units of headroom, positive and negative."""
    from importlib import import_module
    abi = import_module("rtxntc-library_amd").abi
    rng = np.random.default_rng(6 + depth)
    for trial in range(8):
        a = rng.integers(-127, 128, size=(16, depth))
        b = rng.integers(-15, 241, size=(depth, 16))
        if trial == 1:                                   # worst case magnitudes, all one sign
            a[:], b[:] = 127, 240
        if trial == 2:
            a[:], b[:] = -127, 240
        room = (1 << 24) - 1 - np.abs(a).sum(axis=1, keepdims=True) * 240
        c = rng.integers(-room, room + 1, size=(16, 16))
        if trial in (1, 3):
            c = np.broadcast_to(room, (16, 16)).copy()      # the sum ends exactly at 2^24 - 1 ...
        if trial in (2, 4):
            c = -np.broadcast_to(room, (16, 16)).copy()     # ... or at -(2^24 - 1) for all-negative rows
        exact = a @ b + c
        assert np.abs(exact).max() < (1 << 24)
        ah, bh = a.astype(np.float16), b.astype(np.float16)
        cf, d = c.astype(np.float32), np.zeros((16, 16), dtype=np.float32)
        assert np.array_equal(ah.astype(np.int64), a) and np.array_equal(cf.astype(np.int64), c)
        abi.check(device.lib.ntc_hip_selftest_mfma_f16(ah.ctypes.data, bh.ctypes.data, cf.ctypes.data, d.ctypes.data, depth))
        assert np.array_equal(d.astype(np.int64), exact), (depth, trial)


@pytest.mark.parametrize("depth", [16, 32])
def test_mfma_f16_takes_subnormal_operands_exactly(device, depth):
    """The form the decode kernel uses: activations n in [-15, 240] enter as the fp16 SUBNORMALS n * 2^-24
    (bit pattern |n|, sign bit for negatives) and the accumulator starts at bias * 2^-24.  The instruction must
    neither flush them nor lose a bit: the result times 2^24 is the integer sum, to the last unit of headroom."""
    from importlib import import_module
    abi = import_module("rtxntc-library_amd").abi
    rng = np.random.default_rng(60 + depth)
    for trial in range(8):
        a = rng.integers(-127, 128, size=(16, depth))
        n = rng.integers(-15, 241, size=(depth, 16))
        if trial == 1:
            a[:], n[:] = 127, 240
        if trial == 2:
            a[:], n[:] = -127, 240
        if trial == 5:
            n[:] = rng.integers(-1, 2, size=n.shape)     # the smallest subnormals and both zeros
        room = (1 << 24) - 1 - np.abs(a).sum(axis=1, keepdims=True) * 240
        c = rng.integers(-room, room + 1, size=(16, 16))
        if trial in (1, 3):
            c = np.broadcast_to(room, (16, 16)).copy()
        if trial in (2, 4):
            c = -np.broadcast_to(room, (16, 16)).copy()
        exact = a @ n + c
        ah = a.astype(np.float16)
        bits = np.abs(n).astype(np.uint16) | np.where(n <= 0, 0x8000, 0).astype(np.uint16)    # zero enters as -0
        bh = np.ascontiguousarray(bits.view(np.float16))
        assert np.array_equal(bh.astype(np.float64) * 2.0 ** 24, n)
        cf = (c.astype(np.float64) * 2.0 ** -24).astype(np.float32)
        assert np.array_equal(cf.astype(np.float64) * 2.0 ** 24, c)
        d = np.zeros((16, 16), dtype=np.float32)
        abi.check(device.lib.ntc_hip_selftest_mfma_f16(ah.ctypes.data, bh.ctypes.data, cf.ctypes.data, d.ctypes.data, depth))
        assert np.array_equal(d.astype(np.float64) * 2.0 ** 24, exact), (depth, trial)


@pytest.mark.parametrize("scale_range", [(-10.0, -4.0), ACTIVE])
def test_cfg0_plumbing_512_fp16(ntc, device, scale_range):
    """The plumbing configuration: 512x512, one mip, 8 channels, 64-48-32 int8, fp16 planar output."""
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), 512, 512, 1, 8, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=0,
                    scale_log2_range=scale_range)
    expected, got = run_both(device, case)
    assert_equal_bytes(expected, got, "cfg0")


@pytest.mark.parametrize("fmt", ["planar", "fp16px", "unorm8"])
def test_cfg1_shape_small_full_mip_chain(ntc, device, fmt):
    """Config 1's shape at 256x256: full mip chain down to 1x1, 16 channels, all output formats."""
    f = {"planar": ntc.abi.OUT_FP16_PLANAR_PAIRS, "fp16px": ntc.abi.OUT_FP16_PIXELS, "unorm8": ntc.abi.OUT_UNORM8_PIXELS}[fmt]
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), 256, 256, 9, 16, f, seed=11, scale_log2_range=ACTIVE)
    expected, got = run_both(device, case)
    assert_equal_bytes(expected, got, f"cfg1-small {fmt}")


@pytest.mark.parametrize("w,h,ch", [(100, 36, 7), (67, 5, 16), (1, 1, 3), (130, 130, 10), (16, 300, 1)])
def test_ragged_sizes_and_channel_counts(ntc, device, w, h, ch):
    """Non-power-of-two sizes (the general fp32 sampling path), tile tails, odd channel counts."""
    for f in (ntc.abi.OUT_FP16_PLANAR_PAIRS, ntc.abi.OUT_FP16_PIXELS, ntc.abi.OUT_UNORM8_PIXELS):
        case = cfg_case(ntc, ntc.presets.spec_cfg01(), w, h, ntc.presets.full_mip_count(w, h), ch, f, seed=w * 31 + h,
                        scale_log2_range=ACTIVE)
        expected, got = run_both(device, case)
        # includes padding and dropped channels: both sides start from the same fill pattern
        assert_equal_bytes(expected, got, f"ragged {w}x{h}x{ch} fmt {f}")


@pytest.mark.parametrize("features,grid_scale", [(16, 2), (8, 4), (12, 3), (4, 1)])
def test_ref092_geometry(ntc, device, features, grid_scale):
    """The mounted LibNTC 0.9.2 decoder: both grids bilinear 4-bit, shared neural LODs, (lod, lod) inputs."""
    spec = ntc.presets.spec_ref092(features)
    case = ref_case(ntc, spec, 192, 128, 8, grid_scale, 10, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=features,
                    scale_log2_range=ACTIVE)
    expected, got = run_both(device, case)
    assert_equal_bytes(expected, got, f"ref092 f{features} gs{grid_scale}")


def test_cfg2_batch_of_sets(ntc, device):
    """Config 2's shape, small: several sets with their own weights and latents in one launch."""
    spec = ntc.presets.spec_cfg2()
    cases = [cfg_case(ntc, spec, 128, 128, 8, 12, ntc.abi.OUT_UNORM8_PIXELS, seed=100 + i, scale_log2_range=ACTIVE)
             for i in range(5)]
    hosts = [c.host_set() for c in cases]
    for hset in hosts:
        hset.decode(threads=8)
    dsets = [c.device_set(device) for c in cases]
    device.decode(dsets)
    device.synchronize()
    for i, (c, hset) in enumerate(zip(cases, hosts)):
        assert_equal_bytes(hset.output, c.d_output.download(), f"cfg2 set {i}")


def test_cfg3_batch_with_set_boundaries_inside_a_workgroups_share(ntc, device):
    """More tiles than resident workgroups can take a few at a time: every workgroup owns a share of ten tiles, its
    two wave quartets walk one half each of the part that uses one set's weights, and sets begin in the middle of
    shares.  Tile counts per set that are odd and even."""
    sizes = [(512, 384), (320, 200), (448, 512), (64, 700), (512, 512), (384, 320)]
    spec = ntc.presets.spec_cfg3()
    cases = [cfg_case(ntc, spec, w, h, ntc.presets.full_mip_count(w, h), 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=500 + i,
                      scale_log2_range=(-17.0, -13.0)) for i, (w, h) in enumerate(sizes)]
    hosts = [c.host_set() for c in cases]
    for hset in hosts:
        hset.decode(threads=8)
    device.decode([c.device_set(device) for c in cases])
    device.synchronize()
    for i, (c, hset) in enumerate(zip(cases, hosts)):
        assert_equal_bytes(hset.output, c.d_output.download(), f"cfg3 batch, set {i}")


def test_cfg3_fp8_batch_of_sets(ntc, device):
    """Several e4m3 sets with their own weights in one launch.  A workgroup of that decoder works on two tiles at
    a time as long as both use the staged weights; every set has an odd number of tiles (353) and a workgroup's
    share is four tiles, so shares straddle set boundaries at either parity."""
    spec = ntc.presets.spec_cfg3()
    cases = [cfg_case(ntc, spec, 256, 256, 9, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=300 + i, scale_log2_range=ACTIVE)
             for i in range(5)]
    assert sum(((m.width + 63) // 64) * ((m.height + 3) // 4) for m in cases[0].mips) == 353
    hosts = [c.host_set() for c in cases]
    for hset in hosts:
        hset.decode(threads=8)
    dsets = [c.device_set(device) for c in cases]
    device.decode(dsets)
    device.synchronize()
    for i, (c, hset) in enumerate(zip(cases, hosts)):
        assert_equal_bytes(hset.output, c.d_output.download(), f"cfg3 set {i}")


@pytest.mark.parametrize("w,h,mips,fmt", [(256, 256, 1, "planar"), (128, 64, 8, "unorm8"), (90, 70, 4, "fp16px")])
def test_cfg3_fp8_weights(ntc, device, w, h, mips, fmt):
    """Config 3's shape: wide 64-64-64 decoder whose hidden-layer weights are FP8 e4m3 with a per-channel
    fp32 scale.  The device evaluates the e4m3 dot products exactly (integer planes of 512 w: three on the int8
    MFMA for layer 0, two on the fp16 MFMA for layers 1 and 2), so the comparison is byte equality - inside the
    1e-3 / 1 LSB bound with room to spare."""
    f = {"planar": ntc.abi.OUT_FP16_PLANAR_PAIRS, "fp16px": ntc.abi.OUT_FP16_PIXELS, "unorm8": ntc.abi.OUT_UNORM8_PIXELS}[fmt]
    for scales in ((-17.0, -13.0), (-10.0, -4.0)):
        case = cfg_case(ntc, ntc.presets.spec_cfg3(), w, h, mips, 16, f, seed=w + mips, scale_log2_range=scales)
        expected, got = run_both(device, case)
        assert_equal_bytes(expected, got, f"cfg3 fp8 {w}x{h} {fmt} {scales}")
        if fmt == "planar":
            a, b = expected.view(np.float16).astype(np.float32), got.view(np.float16).astype(np.float32)
            assert np.max(np.abs(a - b)) <= 1e-3              # the bound the FP8 variant is specified to


def test_cfg3_fp8_extreme_weights(ntc, device):
    """Every hidden weight at +-448 (the largest e4m3) and the e4m3 subnormals, inputs saturating: int32
    accumulators near their limits on both sides must match the checker's wrapped arithmetic."""
    spec = ntc.presets.spec_cfg3()
    layout = ntc.synth.weight_layout(spec)
    blob = ntc.synth.make_weights(spec, 3, scale_log2_range=(-20.0, -18.0))
    w = blob[:layout.weightOffset[3]]
    pattern = np.array([0x7E, 0xFE, 0x01, 0x81, 0x7E, 0x7E, 0x08, 0xF7], dtype=np.uint8)
    w[:] = np.resize(pattern, w.size)
    case = cfg_case(ntc, spec, 64, 64, 1, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=19, weights=blob)
    expected, got = run_both(device, case)
    assert_equal_bytes(expected, got, "cfg3 fp8 extreme")


@pytest.mark.parametrize("slack", [-1, 0, 1, 1 << 20])
def test_cfg3_fp8_fp16_layer_path_boundary(ntc, device, slack):
    """Layers 1 and 2 of the e4m3 decoder run as two fp16 planes only while the int32 accumulator that defines
    the result cannot wrap: |bias| + 128 * sum|512 w| < 2^31 for every channel.  One channel per layer is put
    just inside (slack -1), on and past that limit, with both signs of the bias, so the fp16 planes, the
    three-plane int8 form and the switch between them all face the checker's wrapping arithmetic."""
    import np_decoder
    spec = ntc.presets.spec_cfg3()
    layout = ntc.synth.weight_layout(spec)
    for sign in (1, -1):
        blob = ntc.synth.make_weights(spec, 60 + slack % 5, scale_log2_range=(-30.0, -22.0), bias_sigma=1e-7)
        bias = blob[layout.biasOffset[0]:layout.bufferSize].view(np.int32)
        inside = True
        for layer, row in ((1, 7), (2, 42)):
            w = blob[layout.weightOffset[layer]: layout.weightOffset[layer] + 64 * 64].reshape(64, 64)
            row_abs = np.abs(np_decoder.e4m3_times_512(w)).sum(axis=1)
            magnitude = (1 << 31) + slack - 128 * int(row_abs[row])     # |bias| + 128*sum|512 w| = 2^31 + slack
            magnitude = min(magnitude, (1 << 31) - 1)                     # (an int32 cannot hold more)
            assert 0 < magnitude
            bias[64 * layer + row] = sign * magnitude
            limits = np.abs(bias[64 * layer: 64 * layer + 64].astype(np.int64)) + 128 * row_abs
            assert ((limits >= 1 << 31) == (np.arange(64) == row)).all() if magnitude + 128 * int(row_abs[row]) >= 1 << 31 else (limits < 1 << 31).all()
            inside = inside and bool((limits < 1 << 31).all())
        assert inside == (slack < 0)
        case = cfg_case(ntc, spec, 128, 64, 3, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=61, weights=blob)
        expected, got = run_both(device, case)
        assert_equal_bytes(expected, got, f"cfg3 fp16 path boundary, slack {slack}, sign {sign}")


def test_extreme_weights_saturate_cleanly(ntc, device):
    """All-(-127)/127 weights with the largest scale and huge biases: accumulators near their
    extremes, activations pinned at both ends of the quantiser."""
    spec = ntc.presets.spec_cfg01()
    layout = ntc.synth.weight_layout(spec)
    blob = ntc.synth.make_weights(spec, 3, scale_log2_range=(-4.0, -4.0))
    w = blob[:layout.scaleOffset[0]].view(np.int8)
    w[:] = np.where(np.arange(w.size) % 3 == 0, -127, 127)
    bias = blob[layout.biasOffset[0]:layout.bufferSize].view(np.int32)
    bias[::2] = 2 ** 30
    bias[1::2] = -(2 ** 30)
    case = cfg_case(ntc, spec, 64, 64, 1, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=9, weights=blob)
    expected, got = run_both(device, case)
    assert_equal_bytes(expected, got, "extreme weights")


@pytest.mark.parametrize("slack", [-1, 0, 1, 4096])
def test_fp16_layer_path_boundary(ntc, device, slack):
    """Layers 1..3 run on the fp16 matrix instruction only while |bias - 113*sum(W)| + 240*sum|W| stays
    below 2^24 for every channel; one channel is put exactly at (slack = -1: just inside), on and just
    past that limit, with both signs, so both code paths and the switch between them face the checker."""
    spec = ntc.presets.spec_cfg01()
    layout = ntc.synth.weight_layout(spec)
    for sign in (1, -1):
        blob = ntc.synth.make_weights(spec, 40 + slack % 7, scale_log2_range=(-22.0, -21.0))
        ins, outs = [64, 64, 48, 32], [64, 48, 32, 16]
        bias = blob[layout.biasOffset[0]:layout.bufferSize].view(np.int32)
        for layer, row in ((1, 5), (2, 17), (3, 9)):
            w = blob[layout.weightOffset[layer]: layout.weightOffset[layer] + ins[layer] * outs[layer]].view(np.int8).reshape(outs[layer], ins[layer])
            total, total_abs = int(w[row].astype(np.int64).sum()), int(np.abs(w[row].astype(np.int64)).sum())
            shifted = sign * ((1 << 24) + slack - 240 * total_abs)        # |shifted| + 240*sum|W| = 2^24 + slack
            bias[sum(outs[:layer]) + row] = shifted + 113 * total
        case = cfg_case(ntc, spec, 128, 64, 3, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=50, weights=blob)
        expected, got = run_both(device, case)
        assert_equal_bytes(expected, got, f"fp16 path boundary, slack {slack}, sign {sign}")


@pytest.mark.parametrize("spec_name", ["spec_cfg01", "spec_cfg2"])
def test_layer0_conversion_shortcut_boundary(ntc, device, spec_name):
    """Layer 0's int32 accumulators are read as floats through a magic-number start value while every bias of the
    layer is at most 3 100 000 in magnitude (|acc| < 2^22); one bias at the limit and one just past it, with both
    signs, send a set through either form of the layer."""
    spec = getattr(ntc.presets, spec_name)()
    layout = ntc.synth.weight_layout(spec)
    for value in (3100000, 3100001, -3100000, -3100001):
        blob = ntc.synth.make_weights(spec, 90 + abs(value) % 5, scale_log2_range=(-22.0, -21.0))
        bias = blob[layout.biasOffset[0]:layout.bufferSize].view(np.int32)
        bias[7] = value
        bias[40] = -value // 2
        case = cfg_case(ntc, spec, 128, 64, 3, 12, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=91, weights=blob)
        expected, got = run_both(device, case)
        assert_equal_bytes(expected, got, f"layer-0 conversion shortcut, bias {value}")


def test_outputs_beyond_the_fp16_range_become_zero(ntc, device):
    """Large output scales: network outputs pass 65520 in magnitude, which the contract stores as 0
    (Inference.cu:125-126).  The weights still qualify for the fp16 form of layers 1..3, but not for
    its unchecked stores; the checker must agree byte for byte and zeros must actually occur."""
    spec = ntc.presets.spec_cfg01()
    blob = ntc.synth.make_weights(spec, 77, scale_log2_range=(-2.0, 1.0))
    case = cfg_case(ntc, spec, 256, 128, 4, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=78, weights=blob)
    expected, got = run_both(device, case)
    assert_equal_bytes(expected, got, "overflowing outputs")
    halves = np.asarray(expected).view(np.uint16)
    assert (halves == 0).mean() > 0.01 and (np.abs(halves.view(np.float16).astype(np.float32)) > 30000).mean() > 0.01


@pytest.mark.parametrize("fmt_name", ["OUT_UNORM8_PIXELS", "OUT_FP16_PIXELS"])
def test_stores_of_chosen_output_values(ntc, device, fmt_name):
    """Output layer with zero weights: every texel's channel c is bias[c] * 2^-11, so the stores see chosen
    values - the unorm8 tie 1/2 (-> 128), values next to the half-integers of v * 255, the clamps at 0 and 255,
    and halves that need rounding.  The checker must agree and the tie must come out as 128."""
    spec = ntc.presets.spec_cfg01()
    layout = ntc.synth.weight_layout(spec)
    blob = ntc.synth.make_weights(spec, 5, scale_log2_range=ACTIVE)
    last = ntc.abi.MLP_LAYERS - 1
    n_in, n_out = spec.layer_inputs(last), spec.layer_outputs(last)
    blob[layout.weightOffset[last]:layout.weightOffset[last] + n_in * n_out] = 0
    blob[layout.scaleOffset[last]:layout.scaleOffset[last] + 4 * n_out] = np.full(n_out, 2.0 ** -11, dtype=np.float32).view(np.uint8)
    #          1/2   just below / above   0.5/255 region       1    >1    <0    0   1/255-ish   odd 11-bit patterns
    biases = [1024, 1023, 1025, 4, 5, 3, 2048, 4096, -512, 0, 8, 9, 2047, 1365, 683, 1]
    blob[layout.biasOffset[last]:layout.biasOffset[last] + 4 * n_out] = np.array(biases, dtype=np.int32).view(np.uint8)
    fmt = getattr(ntc.abi, fmt_name)
    case = cfg_case(ntc, spec, 96, 40, 2, 16, fmt, seed=6, weights=blob)
    expected, got = run_both(device, case)
    assert_equal_bytes(expected, got, f"chosen outputs, {fmt_name}")
    if fmt == ntc.abi.OUT_UNORM8_PIXELS:
        first = np.asarray(expected).view(np.uint8)[:16].tolist()
        assert first[0] == 128 and first[6] == 255 and first[7] == 255 and first[8] == 0 and first[9] == 0
        assert first[1] == 127 and first[2] == 128           # 0.49951 * 255 = 127.38, 0.50049 * 255 = 127.62


@pytest.mark.parametrize("fmt_name,shift,row_pad,stride", [
    ("OUT_FP16_PIXELS", 2, 0, 32), ("OUT_FP16_PIXELS", 0, 2, 32), ("OUT_FP16_PIXELS", 0, 0, 34), ("OUT_FP16_PIXELS", 4, 4, 36),
    ("OUT_FP16_PIXELS", 8, 8, 40),
    ("OUT_UNORM8_PIXELS", 1, 0, 16), ("OUT_UNORM8_PIXELS", 0, 3, 16), ("OUT_UNORM8_PIXELS", 0, 0, 17), ("OUT_UNORM8_PIXELS", 2, 2, 18),
    ("OUT_UNORM8_PIXELS", 4, 4, 20)])
def test_pixel_layouts_with_and_without_vector_stores(ntc, device, fmt_name, shift, row_pad, stride):
    """A lane's four channels go out as one store only where the mip's start, row pitch and pixel stride are all
    multiples of the group's size (8 bytes of fp16, 4 of unorm8); any other layout takes the channel-by-channel
    stores.  Starts, pitches and strides off those multiples, one at a time and together, and a padded layout on
    them; every byte of the buffer - the gaps keep their fill pattern - against the checker."""
    fmt = getattr(ntc.abi, fmt_name)
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), 96, 40, 3, 16, fmt, seed=77, scale_log2_range=ACTIVE, pixel_stride=stride)
    cursor = shift
    for d in case.mips:                                    # re-place the mips: shifted starts, padded rows
        d.outOffset, d.outRowPitch = cursor, d.width * stride + row_pad
        cursor = ((cursor + d.height * d.outRowPitch + 15) & ~15) + shift
    case.output_bytes = cursor + 16
    expected, got = run_both(device, case)
    assert_equal_bytes(expected, got, f"{fmt_name} start {shift} pad {row_pad} stride {stride}")


def test_decode_is_idempotent_and_timed_variant_matches(ntc, device):
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), 320, 200, 4, 16, ntc.abi.OUT_UNORM8_PIXELS, seed=21, scale_log2_range=ACTIVE)
    dset = case.device_set(device)
    device.decode([dset])
    device.synchronize()
    first = case.d_output.download().copy()
    ms = device.decode_timed([dset], 3)
    assert ms > 0
    assert np.array_equal(first, case.d_output.download())


def test_timer_spans_the_calls_between_its_two_ends(ntc, device):
    """ntc_hip_timer_begin / _end: device time of whatever was queued between them.  A span around five decodes is
    at least as long as five decodes timed back to back by ntc_hip_decode_timed (it also holds the table uploads
    between them) and of the same order; an end without a begin is an error, and so is a second end."""
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), 1024, 1024, 5, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=22)
    dsets = device.pack_sets([case.device_set(device)])
    for _ in range(20):
        device.decode(dsets)
    device.synchronize()
    each = min(device.decode_timed(dsets, 5) for _ in range(3))
    device.timer_begin()
    for _ in range(5):
        device.decode(dsets)
    span = device.timer_end()
    assert 0.8 * 5 * each < span < 5 * each * 3 + 1.0, (each, span)
    with pytest.raises(ntc.NtcHipError) as e:
        device.timer_end()
    assert e.value.code == ntc.abi.ERR_INVALID_ARG and "timer_begin" in e.value.message
    device.timer_begin()
    assert device.timer_end() >= 0.0                         # an empty span


def test_argument_errors_are_reported(ntc, device):
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), 64, 64, 1, 8, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=1)
    dset = case.device_set(device)
    dset.latentsBytes = 16
    with pytest.raises(ntc.NtcHipError) as e:
        device.decode([dset])
    assert e.value.code == ntc.abi.ERR_INVALID_ARG and "latent" in e.value.message
    dset = case.device_set(device)
    dset.spec.hiddenChannels[0] = 32
    with pytest.raises(ntc.NtcHipError) as e:
        device.decode([dset])
    assert e.value.code in (ntc.abi.ERR_UNSUPPORTED, ntc.abi.ERR_INVALID_ARG)


def test_offsets_that_would_wrap_are_rejected(ntc, device):
    """Offsets and pitches near 2^64 must not slip through a wrapped sum."""
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), 64, 64, 1, 8, ntc.abi.OUT_UNORM8_PIXELS, seed=1)
    for field, value in (("hrOffset", (1 << 64) - 2), ("lrOffset", (1 << 64) - 2), ("outOffset", (1 << 64) - 4), ("outRowPitch", 1 << 62)):
        dset = case.device_set(device)
        setattr(dset.mips[0], field, value)
        with pytest.raises(ntc.NtcHipError) as e:
            device.decode([dset])
        assert e.value.code == ntc.abi.ERR_INVALID_ARG, field


def test_pixel_rows_beyond_4_gib_are_rejected(ntc, device):
    """A texel's place inside its row is a 32-bit offset in the kernel: a width and pixel stride whose product
    passes 2^32 must be refused, not wrapped."""
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), 8192, 4, 1, 8, ntc.abi.OUT_UNORM8_PIXELS, seed=1)
    dset = case.device_set(device)
    dset.outPixelStride = 1 << 19                         # 8191 * 2^19 + 8 = 4 GiB - 2^19 + 8: still fine, were the buffer that large
    dset.mips[0].outRowPitch = 8192 << 19
    with pytest.raises(ntc.NtcHipError) as e:
        device.decode([dset])
    assert e.value.code == ntc.abi.ERR_INVALID_ARG and "output buffer" in e.value.message
    dset.outPixelStride = 1 << 20                         # 8191 * 2^20 passes 2^32
    dset.mips[0].outRowPitch = 8192 << 20
    with pytest.raises(ntc.NtcHipError) as e:
        device.decode([dset])
    assert e.value.code == ntc.abi.ERR_INVALID_ARG and "4 GiB" in e.value.message


def test_fill_any_alignment(ntc, device):
    """ntc_hip_memset is a kernel: every alignment of start and end, bytes outside untouched."""
    rng = np.random.default_rng(5)
    base = rng.integers(0, 256, 4096, dtype=np.uint8)
    for start, count, value in ((0, 4096, 0), (1, 1, 7), (3, 13, 255), (5, 27, 1), (16, 16, 9), (15, 17, 3), (31, 1000, 0xAB), (8, 4080, 0x55), (2, 3, 4)):
        buf = device.upload(base)
        ntc.abi.check(device.lib.ntc_hip_memset(buf.ptr + start, value, count))
        device.synchronize()
        want = base.copy()
        want[start:start + count] = value
        assert np.array_equal(buf.download(), want), (start, count)
    big = device.alloc((1 << 26) + 5)
    big.fill(0x11)
    ntc.abi.check(device.lib.ntc_hip_memset(big.ptr + 3, 0xEE, (1 << 26) - 1))
    device.synchronize()
    got = big.download()
    assert np.all(got[:3] == 0x11) and np.all(got[3:(1 << 26) + 2] == 0xEE) and np.all(got[(1 << 26) + 2:] == 0x11)
