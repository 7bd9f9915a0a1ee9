"""The oracle's int8 layer against the reference itself: quantize_weights (src/layers/quantization.cpp:55-93) and the integer branch of
Conv2D::forward (src/layers/Conv2D.cpp:240-308), recorded from the compiled reference by tests/golden/make_int8_fixtures.py
(kernel sizes 1 / 3 / 5, with and without residual, int8 and fp32 outputs, all activations, asymmetric input quantisation so that the
padding value and the folded bias are not trivial). Bit for bit, the fp32 outputs included."""
import os

import numpy as np
import pytest

import oracle as O

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_int8_conv2d.npz")


def cases():
    data = np.load(PATH)
    names = sorted({k.split("/")[0] for k in data.files})
    return data, names


DATA, NAMES = cases()


def unpack(name):
    spec = [int(v) for v in DATA[name + "/spec"]]
    qd = [float(v) for v in DATA[name + "/qd"]]
    return spec, (qd[0], qd[1]), (qd[2], qd[3]), (qd[4], qd[5])


def test_fixture_covers_the_branch():
    specs = [unpack(n)[0] for n in NAMES]
    assert {s[5] for s in specs} == {1, 3, 5}
    assert {s[6] for s in specs} >= {0, 1, 2, 3, 5}
    assert {bool(s[7]) for s in specs} == {True, False} and {bool(s[8]) for s in specs} == {True, False}
    assert any(unpack(n)[1][1] != 0.0 for n in NAMES)  # a shifted input: input_zero != 0, folded bias != bias


@pytest.mark.parametrize("name", NAMES)
def test_quantize_weights_equals_reference(name):
    _, in_qd, _, _ = unpack(name)
    q, scales, folded = O.quantize_weights(DATA[name + "/weights"], DATA[name + "/bias"], in_qd)
    assert np.array_equal(q, DATA[name + "/q"])
    assert np.array_equal(scales.view(np.uint32), DATA[name + "/scales"].view(np.uint32))
    assert np.array_equal(folded.view(np.uint32), DATA[name + "/folded_bias"].view(np.uint32))
    if in_qd[1] != 0.0:
        assert not np.array_equal(folded, DATA[name + "/bias"])


@pytest.mark.parametrize("name", NAMES)
def test_int8_conv2d_forward_equals_reference(name):
    spec, in_qd, out_qd, ext_qd = unpack(name)
    has_ext, int8_out, act = bool(spec[7]), bool(spec[8]), spec[6]
    ext = DATA[name + "/ext"] if has_ext else None
    got = O.int8_conv2d_forward(DATA[name + "/x"], in_qd, DATA[name + "/q"], DATA[name + "/scales"], DATA[name + "/folded_bias"],
                                O.INT8 if int8_out else O.FLOAT32, out_qd, ext, ext_qd, act)
    want = DATA[name + "/y"]
    if int8_out:
        assert np.array_equal(got, want)
    else:
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_host_side_quantization_equals_reference():
    """minml_amd.quantization (the host-side mirror used by the int8 network) against the same reference answers."""
    from minml_amd import quantization as Q

    for name in NAMES:
        _, in_qd, _, _ = unpack(name)
        q, scales, folded = Q.quantize_weights(DATA[name + "/weights"], DATA[name + "/bias"], in_qd)
        assert np.array_equal(q, DATA[name + "/q"])
        assert np.array_equal(np.asarray(scales, np.float32).view(np.uint32), DATA[name + "/scales"].view(np.uint32))
        assert np.array_equal(np.asarray(folded, np.float32).view(np.uint32), DATA[name + "/folded_bias"].view(np.uint32))


def test_cpu_and_device_requantisation_formulas_differ_rarely():
    """The HIP library requantises with the CPU layer's formula (round(x / s) written as x * (1 / s) + (-shift / s)); the reference's
    device kernel writes (x - shift) / s. On accumulators, scales and ranges of the size the 20 x 256 int8 network produces the two
    agree except for a handful of values at a .5 boundary, and never by more than one int8 step."""
    rng = np.random.default_rng(7)
    rows, channels = 225 * 64, 256
    acc = rng.integers(-30000, 30000, (rows, channels), dtype=np.int32)
    scales = (rng.uniform(0.5, 2.0, channels) * 1e-4).astype(np.float32)  # weight scale x input scale
    bias = rng.normal(0.0, 0.05, channels).astype(np.float32)
    ext = rng.integers(-128, 128, (rows, channels), dtype=np.int8)
    total = differing = 0
    for out_qd in ((3.0 / 127.0, 0.0), (0.0237, 0.41), (1.0 / 64.0, -0.25)):
        for use_ext in (False, True):
            e, eq = (ext, (2.5 / 127.0, 0.0)) if use_ext else (None, (1.0, 0.0))
            cpu_form = O.quantized_scale_shift_act(acc, scales, bias, O.INT8, out_qd, e, eq, O.RELU)
            device_form = O.quantized_scale_shift_act_device_form(acc, scales, bias, out_qd, e, eq, O.RELU)
            delta = np.abs(cpu_form.astype(np.int32) - device_form.astype(np.int32))
            assert delta.max() <= 1
            total += delta.size
            differing += int(np.count_nonzero(delta))
    print("requantisation, CPU-layer formula against device-kernel formula: %d of %d outputs differ (by one step)" % (differing, total), flush=True)
    assert differing <= total * 1e-4
