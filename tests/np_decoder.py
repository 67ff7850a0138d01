"""An independent numpy restatement of the int8 decode contract, whole mips at a time.

Test infrastructure.  It exists to pin the C++ checker (oracle/ntc_oracle.cpp) end to end:
it is written from the reference text separately (vectorised, integer GEMMs in int64,
explicit float32 arithmetic, its own fused-multiply-add built from float64 with
round-to-odd), so an indexing, ordering or rounding mistake in one of the two shows up as a
difference.  Reference lines are cited where each step comes from.
"""
import numpy as np

F32 = np.float32


def fma32(a, b, c):
    """fl32(a*b + c) with ONE rounding, for float32 arrays.

    a*b is exact in float64 (48-bit product).  The float64 sum is corrected to round-to-odd
    using the exact TwoSum error, after which rounding to float32 equals a single rounding.
    """
    a = np.asarray(a, dtype=F32).astype(np.float64)
    b = np.asarray(b, dtype=F32).astype(np.float64)
    c = np.asarray(c, dtype=F32).astype(np.float64)
    p = a * b
    s = p + c
    bb = s - p
    err = (p - (s - bb)) + (c - bb)                      # exact error of the addition
    bits = s.view(np.int64) if isinstance(s, np.ndarray) else np.float64(s).view(np.int64)
    s = np.array(s, dtype=np.float64, ndmin=1)
    err = np.array(err, dtype=np.float64, ndmin=1)
    bits = s.view(np.int64)
    need = (err != 0) & ((bits & 1) == 0)
    # move one ulp toward the true value when the kept mantissa is even: makes it odd
    toward = np.where(err > 0, np.inf, -np.inf)
    s = np.where(need, np.nextafter(s, toward), s)
    return s.astype(F32)


def unpack_grid(words, width, height, features, bits):
    """[layers*h*w] u16 -> [h, w, features] codes.  Feature i of a layer at bits [bits*i, +bits)
    (reference src/Quantizer.cu:519-523,568-571)."""
    per = 16 // bits
    layers = (features + per - 1) // per
    planes = np.asarray(words[: layers * height * width], dtype=np.uint16).reshape(layers, height, width)
    out = np.zeros((height, width, features), dtype=np.int32)
    for f in range(features):
        out[:, :, f] = (planes[f // per] >> np.uint16(bits * (f % per))) & np.uint16((1 << bits) - 1)
    return out


def footprint(coord_count, size, grid):
    """Per texel index: (i0, i1, d) along one axis (reference src/FeatureGridDevice.h:33-57)."""
    idx = np.arange(coord_count, dtype=F32)
    u = (idx + F32(0.5)) / F32(size)                       # src/Inference.cu:52-53
    p = u * F32(grid) - F32(0.5)
    b = np.floor(p)
    d = (p - b).astype(F32)
    bi = b.astype(np.int64)
    bi = np.where(bi < 0, bi + grid, bi)
    return bi % grid, (bi + 1) % grid, d


def sample_grid(codes, mode, slots, width, height, bits):
    """[H, W, inputs] int8 network inputs from one grid for a whole mip."""
    gh, gw, features = codes.shape
    x0, x1, dx = footprint(width, width, gw)
    y0, y1, dy = footprint(height, height, gh)
    code_scale = 255 // ((1 << bits) - 1)
    taps = [codes[np.ix_(y0, x0)], codes[np.ix_(y0, x1)], codes[np.ix_(y1, x0)], codes[np.ix_(y1, x1)]]
    if mode == 1:   # 2x2 concat: a00, a01, a10, a11 (src/FeatureGridDevice.h:67-70)
        out = np.zeros((height, width, 4 * slots), dtype=np.int8)
        for t, tap in enumerate(taps):
            out[:, :, t * slots: t * slots + features] = (tap * code_scale - 128).astype(np.int8)
        return out
    dxn, dyn = F32(1) - dx, F32(1) - dy
    w00 = (dyn[:, None] * dxn[None, :]).astype(F32)
    w10 = (dyn[:, None] * dx[None, :]).astype(F32)
    w01 = (dy[:, None] * dxn[None, :]).astype(F32)
    w11 = (dy[:, None] * dx[None, :]).astype(F32)
    # note: reference multiplies dx-term first (dxn*dyn etc.); products of two floats commute exactly
    out = np.zeros((height, width, slots), dtype=np.int8)
    for f in range(features):
        q = [tap[:, :, f].astype(F32) for tap in taps]
        t = (w00 * q[0]).astype(F32)
        t = fma32(w10, q[1], t).reshape(height, width)
        t = fma32(w01, q[2], t).reshape(height, width)
        t = fma32(w11, q[3], t).reshape(height, width)
        v = (t * F32(code_scale)).astype(F32)
        out[:, :, f] = (np.floor(v).astype(np.int32) - 128).astype(np.int8)    # Inference.hlsli:80-82
    return out


def positional(width, height, scale, lod, waves, lod_inputs):
    """Inference.hlsli:89-120.  int(float) truncates toward zero."""
    px = (np.arange(width, dtype=F32) * F32(scale)).astype(F32)
    py = (np.arange(height, dtype=F32) * F32(scale)).astype(F32)
    out = np.zeros((height, width, 4 * waves + lod_inputs), dtype=np.int8)

    def enc(p):
        fr = (p - np.floor(p)).astype(F32)
        e = (fr * F32(2) - F32(1)).astype(F32)
        return np.trunc((e * F32(127.5)).astype(F32)).astype(np.int32).astype(np.int8)

    for w in range(waves):
        out[:, :, 4 * w + 0] = enc(px)[None, :]
        out[:, :, 4 * w + 1] = enc(py)[:, None]
        out[:, :, 4 * w + 2] = enc((px + F32(0.25)).astype(F32))[None, :]
        out[:, :, 4 * w + 3] = enc((py + F32(0.25)).astype(F32))[:, None]
        px = (px * F32(2)).astype(F32)
        py = (py * F32(2)).astype(F32)
    if lod_inputs:
        out[:, :, 4 * waves:] = np.int8(int(np.trunc(F32(lod) * F32(127.5))))
    return out


def hgelu_quantize(x):
    """Inference.hlsli:123-131 on float32 arrays -> int8."""
    x = np.asarray(x, dtype=F32)
    t = fma32(x, F32(0.333333), F32(0.5)).reshape(x.shape)
    t = np.minimum(np.maximum(t, F32(0)), F32(1))
    y = (np.minimum(x, F32(3)) * t).astype(F32)
    r = np.rint((y * F32(80)).astype(F32))                 # rint = round-half-even
    return (r.astype(np.int32) - 113).astype(np.int8)


def e4m3_times_512(byte_array):
    """OCP e4m3 bytes -> the exact integers 512*value, from the format definition:
    (-1)^s * 2^(e-7) * (1 + m/8) for e > 0, (-1)^s * 2^-6 * (m/8) for e = 0; NaN patterns -> 0."""
    b = np.asarray(byte_array).view(np.uint8).astype(np.int64)
    sgn, e, m = b >> 7, (b >> 3) & 15, b & 7
    val = np.where(e > 0, np.ldexp(1.0 + m / 8.0, e - 7), np.ldexp(m / 8.0, -6)) * 512.0
    out = np.where(sgn == 1, -val, val)
    out = np.where((b & 0x7F) == 0x7F, 0.0, out)
    assert np.array_equal(out, np.rint(out))
    return out.astype(np.int64)


def decode_mip(spec, layout, blob, latents_u16, mip):
    """Returns (inputs int8 [H,W,IN], outputs float32 [H,W,16]) for one colour mip."""
    W, H = mip.width, mip.height
    hr_words = latents_u16[mip.hrOffset // 2:]
    lr_words = latents_u16[mip.lrOffset // 2:]
    hr = unpack_grid(hr_words, mip.hrWidth, mip.hrHeight, spec.hrFeatures, spec.hrBits)
    lr = unpack_grid(lr_words, mip.lrWidth, mip.lrHeight, spec.lrFeatures, spec.lrBits)
    parts = [
        sample_grid(hr, spec.hrMode, spec.hrFeatureSlots, W, H, spec.hrBits),
        sample_grid(lr, spec.lrMode, spec.lrFeatureSlots, W, H, spec.lrBits),
        positional(W, H, mip.positionScale, mip.positionLod, spec.posEncWaves, spec.lodInputs),
    ]
    used = sum(p.shape[2] for p in parts)
    inputs = np.zeros((H, W, spec.inputChannels), dtype=np.int8)
    inputs[:, :, :used] = np.concatenate(parts, axis=2)
    act = inputs.reshape(-1, spec.inputChannels).astype(np.int64)
    out = None
    for layer in range(4):
        n_in, n_out = spec.layer_inputs(layer), spec.layer_outputs(layer)
        w = blob[layout.weightOffset[layer]: layout.weightOffset[layer] + n_in * n_out].view(np.int8).reshape(n_out, n_in)
        if spec.weightType == 2 and layer < 3:
            w = e4m3_times_512(w)
        scale = blob[layout.scaleOffset[layer]: layout.scaleOffset[layer] + 4 * n_out].view(np.float32)
        bias = blob[layout.biasOffset[layer]: layout.biasOffset[layer] + 4 * n_out].view(np.int32)
        acc = act @ w.astype(np.int64).T + bias.astype(np.int64)             # Inference.hlsli:148-162
        acc32 = acc.astype(np.int32)
        assert np.array_equal(acc32.astype(np.int64), acc), "accumulator left int32 range"
        r = (acc32.astype(F32) * scale[None, :]).astype(F32)                 # Inference.hlsli:164-165
        if layer == 3:
            out = r
        else:
            act = hgelu_quantize(r).astype(np.int64)
    return inputs, out.reshape(H, W, 16)


# ---- the FP8 network (include/libntc/shaders/InferenceCoopVec.hlsli:22-124,127-160,235-398) -------------------

E4M3_POSITIVE = np.array([(m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7) for e in range(16) for m in range(8)][:127])


def round_to_e4m3(values):
    """Nearest e4m3 value of each float (brute force over the 127 non-negative values, ties to the even
    code, everything from 448 up saturates at 448); NaN -> 0."""
    v = np.asarray(values, dtype=np.float64)
    a = np.abs(np.nan_to_num(v, nan=0.0, posinf=1e9, neginf=-1e9))
    hi = np.clip(np.searchsorted(E4M3_POSITIVE, a, side="left"), 1, 126)     # E4M3_POSITIVE[hi-1] <= a <= E4M3_POSITIVE[hi] inside the range
    lo = hi - 1
    d_lo, d_hi = a - E4M3_POSITIVE[lo], E4M3_POSITIVE[hi] - a
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))
    r = np.where(pick_hi, E4M3_POSITIVE[hi], E4M3_POSITIVE[lo])
    r = np.where(a >= 448.0, 448.0, r)
    return np.copysign(r, np.where(np.isnan(v), 0.0, v))


def hgelu_half(x16):
    """NtcHGELUClamp_Forward_CoopVec (hlsli:150-153) on float16 arrays, every operation rounded to half once."""
    x = np.asarray(x16, dtype=np.float16).astype(np.float64)
    third = np.float64(np.float16(1.0 / 3.0))
    with np.errstate(over="ignore", invalid="ignore"):
        t = (x * third + 0.5).astype(np.float16).astype(np.float64)          # exact in float64, one rounding
        t = np.clip(t, 0.0, 1.0)
        y = (np.clip(x, -3.0, 3.0) * t).astype(np.float16)
    return np.where(np.isnan(x), np.float16(0), y)


def fp8_inputs(spec, latents_u16, mip):
    """[H, W, 48] float16: the network's input vector before its e4m3 reading (hlsli:22-107)."""
    W, H = mip.width, mip.height
    out = np.zeros((H, W, spec.inputChannels), dtype=np.float16)
    for base, words, gw, gh, features in ((0, latents_u16[mip.hrOffset // 2:], mip.hrWidth, mip.hrHeight, spec.hrFeatures),
                                          (spec.hrFeatureSlots, latents_u16[mip.lrOffset // 2:], mip.lrWidth, mip.lrHeight, spec.lrFeatures)):
        codes = unpack_grid(words, gw, gh, features, 4)
        x0, x1, dx = footprint(W, W, gw)
        y0, y1, dy = footprint(H, H, gh)
        taps = [codes[np.ix_(y0, x0)], codes[np.ix_(y0, x1)], codes[np.ix_(y1, x0)], codes[np.ix_(y1, x1)]]
        dxn, dyn = F32(1) - dx, F32(1) - dy
        w = [(dyn[:, None] * dxn[None, :]).astype(F32), (dyn[:, None] * dx[None, :]).astype(F32),
             (dy[:, None] * dxn[None, :]).astype(F32), (dy[:, None] * dx[None, :]).astype(F32)]
        for f in range(features):
            q = [tap[:, :, f].astype(F32) for tap in taps]
            t = (w[0] * q[0]).astype(F32)
            for i in (1, 2, 3):
                t = fma32(w[i], q[i], t).reshape(H, W)
            out[:, :, base + f] = fma32(t, F32(2.0 / 15.0), F32(-1)).reshape(H, W).astype(np.float16)
    at = spec.hrFeatureSlots + spec.lrFeatureSlots
    px = (np.arange(W, dtype=F32) * F32(mip.positionScale)).astype(F32)
    py = (np.arange(H, dtype=F32) * F32(mip.positionScale)).astype(F32)

    def enc(p):
        return (((p - np.floor(p)).astype(F32) * F32(2)).astype(F32) - F32(1)).astype(F32).astype(np.float16)

    for _ in range(spec.posEncWaves):
        out[:, :, at + 0] = enc(px)[None, :]
        out[:, :, at + 1] = enc(py)[:, None]
        out[:, :, at + 2] = enc((px + F32(0.25)).astype(F32))[None, :]
        out[:, :, at + 3] = enc((py + F32(0.25)).astype(F32))[:, None]
        px, py, at = (px * F32(2)).astype(F32), (py * F32(2)).astype(F32), at + 4
    out[:, :, at: at + spec.lodInputs] = np.float16(F32(mip.positionLod))
    return out


def layer_e4m3(w_bytes, bias16, a):
    """Layer outputs (float16) from e4m3 weights [out, in], fp16 biases and e4m3-valued inputs a [n, in]: the
    exact dot product in three parts by the bits of |512 w|, added in fp32 as ((s2 + s1) + s0) + bias."""
    w512 = e4m3_times_512(w_bytes)
    a512 = np.rint(np.asarray(a, dtype=np.float64) * 512.0).astype(np.int64)
    assert np.array_equal(a512 / 512.0, np.asarray(a, dtype=np.float64))
    mag, sign = np.abs(w512), np.sign(w512)
    parts = []
    for shift, unit in ((0, -18), (7, -11), (14, -4)):
        plane = sign * ((mag >> shift) & (127 if shift < 14 else 0xFFFF))
        s_int = a512 @ plane.T
        assert np.abs(s_int).max(initial=0) < (1 << 24)
        parts.append(np.ldexp(s_int.astype(np.float64), unit).astype(F32))
    with np.errstate(over="ignore"):
        r = ((parts[2] + parts[1]).astype(F32) + parts[0]).astype(F32)
        r = (r + np.asarray(bias16, dtype=np.float16).astype(F32)[None, :]).astype(F32)
        return r.astype(np.float16)


def decode_mip_fp8(spec, layout, blob, latents_u16, mip):
    """Outputs float32 [H, W, 16] of one colour mip through the FP8 network (NtcEvaluateMLP_CoopVec_FP8)."""
    H, W = mip.height, mip.width
    a = round_to_e4m3(fp8_inputs(spec, latents_u16, mip).reshape(-1, spec.inputChannels).astype(np.float64))
    q = None
    for layer in range(3):
        n_in, n_out = spec.layer_inputs(layer), spec.layer_outputs(layer)
        w = blob[layout.weightOffset[layer]: layout.weightOffset[layer] + n_in * n_out].reshape(n_out, n_in)
        bias = blob[layout.biasOffset[layer]: layout.biasOffset[layer] + 2 * n_out].view(np.float16)
        y = hgelu_half(layer_e4m3(w, bias, a))
        if layer < 2:
            a = round_to_e4m3(y.astype(np.float64))
        else:
            q = np.rint(80.0 * y.astype(np.float64) - 113.0).astype(np.int64)     # exact in float64, one rounding
            assert q.min() >= -128 and q.max() <= 127
    n_in = spec.layer_inputs(3)
    w = blob[layout.weightOffset[3]: layout.weightOffset[3] + n_in * 16].view(np.int8).reshape(16, n_in).astype(np.int64)
    scale = blob[layout.scaleOffset[3]: layout.scaleOffset[3] + 64].view(np.float32)
    bias = blob[layout.biasOffset[3]: layout.biasOffset[3] + 64].view(np.int32).astype(np.int64)
    acc = (q @ w.T + bias).astype(np.int32)
    return (acc.astype(F32) * scale[None, :]).astype(F32).reshape(H, W, 16)


def to_half_bits(outputs):
    h = np.asarray(outputs, dtype=F32).astype(np.float16)        # IEEE round-to-nearest-even
    bits = h.view(np.uint16).copy()
    bits[(bits & 0x7C00) == 0x7C00] = 0                          # IsHalfSpecial -> 0, src/Inference.cu:125-126
    return bits


def half_bits_to_unorm8(bits):
    v = bits.view(np.float16).astype(np.float64) * 255.0         # exact
    r = np.where(v >= 0, np.floor(v + 0.5), np.ceil(v - 0.5))    # roundf, exact in float64
    return np.clip(r, 0, 255).astype(np.uint8)                   # src/ImageProcessing.cu:146-149


def store_mip(out_bytes, mip, outputs, num_channels, output_format, pixel_stride):
    """Writes one mip's outputs into the flat output byte array per the three layouts."""
    H, W = mip.height, mip.width
    hb = to_half_bits(outputs)
    if output_format == 0:   # planar pairs, src/RegressionKernels.h:36-45
        c2 = (num_channels + 1) & ~1
        img = out_bytes[mip.outOffset: mip.outOffset + H * W * c2 * 2].view(np.uint16).reshape(H, c2 // 2, W, 2)
        for ch in range(c2):
            img[:, ch // 2, :, ch % 2] = hb[:, :, ch]
        return
    bpc = 1 if output_format == 2 else 2
    vals = hb if output_format == 1 else half_bits_to_unorm8(hb)
    for y in range(H):
        row = out_bytes[mip.outOffset + y * mip.outRowPitch: mip.outOffset + y * mip.outRowPitch + W * pixel_stride]
        px = row.reshape(W, pixel_stride)[:, : num_channels * bpc]
        px[:] = np.ascontiguousarray(vals[y, :, :num_channels]).view(np.uint8).reshape(W, num_channels * bpc)
