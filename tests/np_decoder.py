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
