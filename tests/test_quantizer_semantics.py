"""What scale and bias in an int8 weight blob MEAN.

The decoder only sees the blob; the reference's encoder-side quantiser
(QuantizeColumnInt8, src/Quantizer.cu:88-208) defines how a float layer (weights w, bias b, inputs in
[-1, 1] quantised by tin::InputQuant, hidden activations quantised by ActHGELUClamp to steps of 1/80
starting at -15/80) turns into (W_q, scale, bias_i32).  This test restates that quantiser in numpy,
quantises random float layers with it, and checks that the checker's integer layer
    r = float(bias_i32 + sum W_q * a) * scale                       (Inference.hlsli:148-165)
reproduces the float layer evaluated on the de-quantised operands,
    r = b + sum w~ * a~,   a~ = a/127.5 (inputs) or (a + 113)/80 (hidden activations),
to within the rounding of the stored bias (half a scale step).  A dropped -113 offset, a wrong
activation step or input scale, a bias added after scaling, or a transposed weight matrix all fail it.
"""
import numpy as np
import pytest


def quantize_layer_int8(w, b, input_layer):
    """w: float32 [in][out], b: float32 [out] -> (W_q int8 [out][in], scale f32 [out], bias_i32 [out], w~ [in][out])."""
    n_in, n_out = w.shape
    wq = np.zeros((n_out, n_in), dtype=np.int8)
    scale = np.zeros(n_out, dtype=np.float32)
    bias_i = np.zeros(n_out, dtype=np.int32)
    w_deq = np.zeros_like(w)
    for c in range(n_out):
        col = w[:, c].astype(np.float32)
        limit = np.float32(max(abs(col.max()), abs(col.min())))                # Quantizer.cu:99-111
        q = np.float32(127.5) * col / limit
        q = np.where(q >= 0, np.floor(q + 0.5), np.ceil(q - 0.5))              # round(): half away from zero
        q = np.clip(q, -127, 127)                                              # Quantizer.cu:116-131
        wq[c] = q.astype(np.int8)
        w_deq[:, c] = (q * limit / np.float32(127.5)).astype(np.float32)
        layer_scale = limit / np.float32(127.5)
        layer_bias = np.float32(b[c])
        if input_layer:
            layer_scale = layer_scale / np.float32(127.5)                      # tin::InputQuant::scale, :157-160
        else:
            layer_scale = layer_scale * np.float32(3.1875 / 255)               # ActHGELUClamp::step = 1/80
            layer_bias = layer_bias - np.float32(int(q.sum()) * -113) * layer_scale      # :163-164
        scale[c] = layer_scale
        t = np.float64(layer_bias) / np.float64(layer_scale)
        bias_i[c] = int(np.floor(t + 0.5) if t >= 0 else np.ceil(t - 0.5))     # roundf, :202
    return wq, scale, bias_i, w_deq


@pytest.mark.parametrize("n_in,n_out,input_layer", [(64, 64, True), (48, 64, True), (64, 48, False), (48, 32, False), (32, 16, False)])
def test_integer_layer_equals_dequantised_float_layer(oracle, n_in, n_out, input_layer):
    rng = np.random.default_rng(n_in * 100 + n_out)
    w = (rng.standard_normal((n_in, n_out)) * 0.3).astype(np.float16).astype(np.float32)
    b = (rng.standard_normal(n_out) * 0.2).astype(np.float16).astype(np.float32)
    wq, scale, bias_i, w_deq = quantize_layer_int8(w, b, input_layer)
    assert np.abs(wq).max() == 127
    for trial in range(50):
        if input_layer:
            a = rng.integers(-127, 128, n_in).astype(np.int8)
            a_real = a.astype(np.float64) / 127.5
        else:
            a = rng.integers(-128, 128, n_in).astype(np.int8)
            a_real = (a.astype(np.float64) + 113) / 80.0
            assert a_real.min() >= -15 / 80 and a_real.max() <= 3.0
        r = np.zeros(n_out, dtype=np.float32)
        wq_c, scale_c, bias_c = np.ascontiguousarray(wq), np.ascontiguousarray(scale), np.ascontiguousarray(bias_i)
        oracle.ntc_oracle_layer_int8(wq_c.ctypes.data, scale_c.ctypes.data, bias_c.ctypes.data, n_in, n_out, a.ctypes.data, r.ctypes.data)
        want = b.astype(np.float64) + a_real @ w_deq.astype(np.float64)
        tol = 0.5 * scale.astype(np.float64) * 1.001 + 2e-6 * (1 + np.abs(want))
        assert np.all(np.abs(r.astype(np.float64) - want) <= tol), (trial, np.abs(r - want).max(), tol.min())
