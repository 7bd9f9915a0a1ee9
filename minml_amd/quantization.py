"""Host-side preparation of an int8 layer, mirroring the reference's src/layers/quantization.cpp and quantization.hpp (it runs once per
layer on the host there as well): AffineTransform (:20-55 of the header), quantize (quantization.cpp:39-43) and
quantize_weights(..., "per_first_dim", 8) (:55-93). Every step is evaluated in float32 in the reference's order, so the integers and
the per-channel constants that come out are the reference's.
"""
import numpy as np

_f = np.float32


def round_half_away(x):
    """std::round on float32: halves away from zero (numpy's round goes to even)."""
    x = np.asarray(x, _f)
    return np.copysign(np.floor(np.abs(x) + _f(0.5)), x).astype(_f)


def quantize(x, bits=8):
    """clamp(round(x), -2^(bits-1), 2^(bits-1) - 1) as int32 (quantization.cpp:39-43)."""
    limit = _f(1 << (bits - 1))
    return np.maximum(-limit, np.minimum(limit - _f(1.0), round_half_away(x))).astype(np.int32)


def quantize_tensor(x, transform):
    """Real values -> int8 with the inverse of `transform` = (scale, shift): q = quantize(x * (1 / scale) + (-shift / scale))
    (AffineTransform::get_inverse, quantization.hpp:44-47, applied as one multiplication and one addition, :39-43)."""
    scale, shift = _f(transform[0]), _f(transform[1])
    inv_scale, inv_shift = _f(1.0) / scale, -shift / scale
    t = np.asarray(x, _f) * inv_scale
    return quantize(t + inv_shift).astype(np.int8)


def quantize_weights(weights, bias, input_transform, bits=8):
    """Per-output-channel symmetric weights: (int8 weights of the same shape, fp32 channel scales [Cout], fp32 bias [Cout]).
    channel_scale = 127 / max|w|; q = quantize(w * channel_scale); scales = s_in / channel_scale; bias' = shift_in / channel_scale * sum(q) + b."""
    w = np.ascontiguousarray(weights, _f)
    rows = w.reshape(w.shape[0], -1)
    s_in, shift_in = _f(input_transform[0]), _f(input_transform[1])
    channel_scale = (_f((1 << (bits - 1)) - 1) / np.abs(rows).max(axis=1)).astype(_f)
    q = quantize(rows * channel_scale[:, None], bits)
    scales = (s_in / channel_scale).astype(_f)
    b = np.zeros(w.shape[0], _f) if bias is None else np.asarray(bias, _f)
    folded = ((shift_in / channel_scale).astype(_f) * q.sum(axis=1).astype(_f)).astype(_f) + b
    return q.astype(np.int8).reshape(w.shape), scales, folded.astype(_f)


def symmetric_transform(max_abs, bits=8):
    """Per-tensor symmetric activation quantisation: scale = max|x| / 127, shift 0."""
    return (float(_f(max(float(max_abs), 1e-30)) / _f((1 << (bits - 1)) - 1)), 0.0)
