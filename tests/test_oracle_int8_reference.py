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
