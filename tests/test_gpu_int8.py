"""The int8 path on the GPU: int8 x int8 -> int32 GEMM, per-channel requantisation, and the fused int8 convolution, against the CPU
oracle of src/layers/Conv2D.cpp:240-308 — BIT FOR BIT (int32 accumulators, requantised int8 outputs and the fp32 outputs of the
un-fused float tail)."""
import numpy as np
import pytest

import oracle as O
from minml_amd import backend as B
from minml_amd import core as ml
from minml_amd.conv2d import Conv2D
from util import init_for_test, mismatches

pytestmark = pytest.mark.gpu

# the transforms of test/backend/test_quantization.cpp:189-191
IN_QD, OUT_QD, EXT_QD = (0.123, 4.56), (0.078, 0.9), (0.078, -0.9)


def init_for_test_int8(shape, shift):
    """src/utils/testing_util.cpp:36-40: int8(255 * sin(i / 10 + shift) - 128), wrapped like the C conversion."""
    n = int(np.prod(shape))
    i = np.arange(n, dtype=np.float64)
    v = np.trunc(255.0 * np.sin(i / 10.0 + shift) - 128.0).astype(np.int64)
    return ((v + 128) % 256 - 128).astype(np.int8).reshape(shape)


@pytest.mark.parametrize("shape", [(75, 44, 36), (1716, 44, 36), (130, 70, 64), (300, 256, 2304), (33, 5, 20), (64, 64, 16),
                                   (33001, 256, 256), (40000, 72, 128), (32900, 132, 512)])
def test_int8_gemm_exact(ctx, shape):
    M, N, K = shape
    rng = np.random.default_rng(M)
    A = rng.integers(-128, 128, (M, K)).astype(np.int8)
    Bm = rng.integers(-128, 128, (N, K)).astype(np.int8)
    dC = ml.Tensor((M, N), "int32")
    ml.gemm(ctx, "n", "t", dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm), 1.0, 0.0)
    assert mismatches(dC.copyToHost(ctx), O.int8_gemm_nt(A, Bm)) == 0


def test_reference_test_case_conv2D_1x1(ctx):
    """test/backend/test_quantization.cpp:173-240 with its deterministic inputs: 11 x 12 x 13 x 36 -> 44, int8 GEMM then
    quantized_scale_shift_act to int8 and to fp32, ReLU, with an int8 residual."""
    b, h, w, cin, cout = 11, 12, 13, 36, 44
    x = init_for_test_int8((b, h, w, cin), 1.0)
    wt = init_for_test_int8((cout, 1, 1, cin), 0.0)
    bias = init_for_test((cout,), 1.0)
    scales = init_for_test((cout,), 1.0, 0.001)
    ext = init_for_test_int8((b, h, w, cout), 0.0)
    acc = ml.Tensor((b * h * w, cout), "int32")
    ml.gemm(ctx, "n", "t", acc, ml.toDevice(ctx, x.reshape(-1, cin)), ml.toDevice(ctx, wt.reshape(cout, cin)), 1.0, 0.0)
    for code in (O.INT8, O.FLOAT32):
        out = ml.Tensor((b, h, w, cout), code)
        ml.quantized_scale_shift_act(ctx, out, OUT_QD, acc, ml.toDevice(ctx, scales), ml.toDevice(ctx, bias), "relu", ml.toDevice(ctx, ext), EXT_QD)
        want = O.int8_conv2d_forward(x, IN_QD, wt, scales, bias, code, OUT_QD, ext, EXT_QD, O.RELU)
        assert mismatches(out.copyToHost(ctx), want) == 0


@pytest.mark.parametrize("shape,cout,k", [((11, 12, 13, 36), 44, 1), ((3, 12, 13, 32), 44, 5), ((2, 15, 15, 64), 64, 3), ((2, 6, 5, 7), 9, 3),
                                          ((2, 15, 15, 256), 256, 3), ((1, 19, 19, 48), 20, 3), ((2, 9, 9, 16), 130, 1),
                                          ((1, 15, 15, 128), 384, 3), ((1, 15, 15, 128), 320, 3)])
@pytest.mark.parametrize("act", ["relu", "linear"])
def test_int8_convolution_bit_exact(ctx, shape, cout, k, act):
    """Both device routes — the single fused launch and the reference's three calls (im2row with zero-point padding, int8 GEMM,
    requantisation: src/layers/Conv2D.cpp:214-239) — to int8 and to fp32, with and without residual."""
    b, h, w, cin = shape
    rng = np.random.default_rng(cout * k)
    x = rng.integers(-128, 128, shape).astype(np.int8)
    wt = rng.integers(-127, 128, (cout, k, k, cin)).astype(np.int8)
    scales = (rng.random(cout) * 0.002 + 0.0005).astype(np.float32)
    bias = rng.standard_normal(cout).astype(np.float32)
    ext = rng.integers(-128, 128, (b, h, w, cout)).astype(np.int8)
    dx, dw, ds, db, de = (ml.toDevice(ctx, a) for a in (x, wt, scales, bias, ext))
    for use_ext in (True, False):
        for code in (O.INT8, O.FLOAT32):
            want = O.int8_conv2d_forward(x, IN_QD, wt, scales, bias, code, OUT_QD, ext if use_ext else None, EXT_QD, ml.act_of(act))
            dy = ml.Tensor((b, h, w, cout), code)
            ml.quantizedConvForward(ctx, dx, IN_QD, dw, ds, db, dy, OUT_QD, de if use_ext else None, EXT_QD, act)
            assert mismatches(dy.copyToHost(ctx), want) == 0
        layer = Conv2D(ctx, shape, cout, k, act, True, "int8")
        layer.setupQuantization(wt, scales, bias, [IN_QD, EXT_QD], OUT_QD, int8_mode="reference")
        ws = ml.Tensor((max(1, layer.getWorkspaceSize()),), B.DTYPE_INT32)
        dy = ml.Tensor((b, h, w, cout), "int8")
        layer.forward([dx, de] if use_ext else [dx], dy, ws)
        want = O.int8_conv2d_forward(x, IN_QD, wt, scales, bias, O.INT8, OUT_QD, ext if use_ext else None, EXT_QD, ml.act_of(act))
        assert mismatches(dy.copyToHost(ctx), want) == 0


def test_quantized_network_layer_config3(ctx):
    """Config 3's recipe on one residual-block convolution: per-output-channel symmetric int8 weights (scale = max|w| / 127), per-tensor
    symmetric activations (shift 0), int32 accumulation, requantisation with fused bias + ReLU. Quantised parameters come from the
    reference's quantize_weights arithmetic (src/layers/quantization.cpp:55-93)."""
    rng = np.random.default_rng(33)
    cin = cout = 256
    w = (rng.standard_normal((cout, 3, 3, cin)) * np.sqrt(2.0 / (9 * cin))).astype(np.float32)
    bias = (rng.standard_normal(cout) * 0.01).astype(np.float32)
    xf = np.maximum(rng.standard_normal((4, 15, 15, cin)), 0).astype(np.float32)
    in_qd = (float(np.abs(xf).max() / 127.0), 0.0)
    out_qd = (0.05, 0.0)
    q, scales, qb = O.quantize_weights(w, bias, in_qd)
    assert np.array_equal(qb, bias)  # symmetric activations: nothing folded into the bias
    xq = np.clip(np.round(xf / in_qd[0]), -128, 127).astype(np.int8)
    dy = ml.Tensor((4, 15, 15, cout), "int8")
    ml.quantizedConvForward(ctx, ml.toDevice(ctx, xq), in_qd, ml.toDevice(ctx, q), ml.toDevice(ctx, scales), ml.toDevice(ctx, qb), dy, out_qd, None,
                            (1.0, 0.0), "relu")
    want = O.int8_conv2d_forward(xq, in_qd, q, scales, qb, O.INT8, out_qd, None, (1.0, 0.0), O.RELU)
    assert mismatches(dy.copyToHost(ctx), want) == 0
    # and the quantised layer tracks the fp32 layer it came from
    ref = O.conv2d_forward(xf, w, bias, None, O.RELU)
    deq = dy.copyToHost(ctx).astype(np.float32) * out_qd[0]
    assert np.abs(deq - ref).mean() < 0.05


def test_int8_full_size_properties(ctx):
    """Config 3 at full size (B = 1024, 15x15, 256 -> 256, 3x3): positions are independent (a sub-batch reproduces its slice bit for
    bit), a sample of positions matches the oracle, and the sum of all int32 accumulators equals the closed form
    sum_o sum_taps (sum_c w[o,tap,c] * colsum[tap,c]) computed in int64 from column sums of the input."""
    rng = np.random.default_rng(34)
    shape, cout = (1024, 15, 15, 256), 256
    x = rng.integers(-128, 128, shape).astype(np.int8)
    wt = rng.integers(-127, 128, (cout, 3, 3, 256)).astype(np.int8)
    scales = np.full(cout, 1.0, np.float32)
    bias = np.zeros(cout, np.float32)
    qd = (1.0, 0.0)
    dx, dw, ds, db = (ml.toDevice(ctx, a) for a in (x, wt, scales, bias))
    full = ml.Tensor(shape[:3] + (cout,), "float32")
    ml.quantizedConvForward(ctx, dx, qd, dw, ds, db, full, qd, None, qd, "linear")
    got = full.copyToHost(ctx)  # float(acc) exactly, |acc| < 2^24 is not guaranteed, so compare through the oracle and sub-batches
    part = ml.Tensor((8, 15, 15, cout), "float32")
    ml.quantizedConvForward(ctx, dx.view((8, 15, 15, 256), 500 * 225 * 256), qd, dw, ds, db, part, qd, None, qd, "linear")
    assert np.array_equal(part.copyToHost(ctx), got[500:508])
    want = O.int8_conv2d_forward(x[500:502], qd, wt, scales, bias, O.FLOAT32, qd)
    assert np.array_equal(got[500:502], want)
    # checksum of the integer accumulators through the int8 GEMM on the 1x1 view (exact int32), against the closed form
    acc = ml.Tensor((1024 * 225, cout), "int32")
    w1 = np.ascontiguousarray(wt[:, 1, 1, :])
    ml.gemm(ctx, "n", "t", acc, dx.view((1024 * 225, 256)), ml.toDevice(ctx, w1), 1.0, 0.0)
    total = int(acc.copyToHost(ctx).astype(np.int64).sum())
    colsum = x.reshape(-1, 256).astype(np.int64).sum(axis=0)
    assert total == int((w1.astype(np.int64) @ colsum).sum())


@pytest.mark.parametrize("int8_mode", ["fused", "reference"])
def test_quantized_network_bit_exact_per_layer_and_at_the_head(ctx, int8_mode):
    """Configuration 3's recipe on a whole (small) network: activation ranges calibrated with the fp32 network, per-channel int8 weights,
    every layer's int8 output and the fp32 head bit for bit against the oracle's integer branch, in the single-launch form and in the
    reference's three-call form (im2row -> int8 GEMM -> requantisation)."""
    from minml_amd import quantization as Q
    from minml_amd.resnet import QuantizedResNet, calibrate_activations, make_input, make_parameters
    from oracle.cpu_net import CpuQuantizedResNet

    board, planes, channels, blocks, batch = 9, 32, 64, 3, 5
    params = make_parameters(5, planes, channels, blocks)
    ranges = calibrate_activations(ctx, params, board, planes, channels, blocks, batches=6, batch_size=3, seed=5)
    assert len(ranges) == 2 + 2 * blocks and ranges[0] == 1.0 and all(r > 0 for r in ranges)
    net = QuantizedResNet(ctx, batch, board, planes, channels, blocks, params, ranges, int8_mode)
    # the host-side quantisation is the reference's (oracle restatement), bit for bit
    for (w, b), (q, scales, folded, in_qd, _, _) in zip(params, net.host_parameters):
        oq, oscales, ofolded = O.quantize_weights(w, b, in_qd)
        assert np.array_equal(q.reshape(-1), np.asarray(oq).reshape(-1)) and np.array_equal(scales, oscales) and np.array_equal(folded, ofolded)
    x = make_input(77, batch, board, planes)
    xq = Q.quantize_tensor(x, net.transforms[0])
    assert np.array_equal(xq, (x * 127).astype(np.int8))  # binary planes with range 1: scale 1 / 127, so the planes become 0 / 127
    got_layers = []
    net.observer = lambda index, tensor: got_layers.append(tensor.copyToHost(ctx))
    net.setInput(x)
    head = net.forward().copyToHost(ctx)
    want_layers = []
    want_head = CpuQuantizedResNet(net.host_parameters, blocks).forward(xq, want_layers)
    assert len(got_layers) == len(want_layers) == 1 + 2 * blocks
    for index, (got, want) in enumerate(zip(got_layers, want_layers)):
        assert mismatches(got, want) == 0, "layer %d" % index
        assert np.abs(got.astype(np.int32)).max() > 20  # the calibrated ranges are used, not a degenerate all-zero net
    assert np.array_equal(head, want_head)


def test_quantized_network_full_size(ctx):
    """Configuration 3 itself (20 blocks x 256 channels, B = 1024): repeated passes give the same bits, the first positions reproduce a
    batch-4 run of the same network bit for bit (positions are independent), and two of those positions match the oracle's integer
    branch bit for bit at the fp32 head and at the last block's int8 output."""
    from minml_amd import quantization as Q
    from minml_amd.resnet import QuantizedResNet, calibrate_activations, make_input, make_parameters
    from oracle.cpu_net import CpuQuantizedResNet

    board, planes, channels, blocks = 15, 32, 256, 20
    params = make_parameters(1, planes, channels, blocks)
    ranges = calibrate_activations(ctx, params, board, planes, channels, blocks, batches=8, batch_size=4, seed=1)
    x = make_input(1, 1024, board, planes)
    net = QuantizedResNet(ctx, 1024, board, planes, channels, blocks, params, ranges)
    net.setInput(x)
    a = net.forward().copyToHost(ctx)
    assert np.array_equal(a, net.forward().copyToHost(ctx))
    assert np.isfinite(a).all() and np.abs(a).max() > 0
    small = QuantizedResNet(ctx, 4, board, planes, channels, blocks, params, ranges)
    small.setInput(x[:4])
    trunk = []
    small.observer = lambda index, tensor: trunk.append(tensor.copyToHost(ctx)) if index == 2 * blocks else None
    b = small.forward().copyToHost(ctx)
    assert np.array_equal(a[:4], b)
    want_layers = []
    want = CpuQuantizedResNet(small.host_parameters, blocks).forward(Q.quantize_tensor(x[:2], small.transforms[0]), want_layers)
    assert np.array_equal(b[:2], want)
    assert mismatches(trunk[0][:2], want_layers[-1]) == 0


def _reference_int8_cases():
    import os

    data = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_int8_conv2d.npz"))
    return data, sorted({k.split("/")[0] for k in data.files})


_REF8, _REF8_NAMES = _reference_int8_cases()


@pytest.mark.parametrize("name", _REF8_NAMES)
def test_int8_convolution_equals_reference_layer(ctx, name):
    """Both device routes against what the reference's own Conv2D::forward (integer branch, src/layers/Conv2D.cpp:240-308) and
    quantize_weights produced (tests/golden/make_int8_fixtures.py): bit for bit for linear / ReLU, int8 and fp32 outputs; for sigmoid /
    tanh / exp the device's exponential differs from the host libm in the last place, so int8 outputs may differ by one count and fp32
    outputs by 1e-6 relative."""
    spec = [int(v) for v in _REF8[name + "/spec"]]
    qd = [float(v) for v in _REF8[name + "/qd"]]
    b, h, w, cin, cout, k, act, has_ext, int8_out = spec
    in_qd, out_qd, ext_qd = (qd[0], qd[1]), (qd[2], qd[3]), (qd[4], qd[5])
    x, q, scales, folded, want = (_REF8[name + "/" + key] for key in ("x", "q", "scales", "folded_bias", "y"))
    de = ml.toDevice(ctx, _REF8[name + "/ext"]) if has_ext else None
    dx, dw, ds, db = (ml.toDevice(ctx, a) for a in (x, q, scales, folded))
    exact = act in (O.LINEAR, O.RELU)

    def check(got):
        if exact:
            assert mismatches(got, want) == 0
        elif int8_out:
            assert np.abs(got.astype(np.int32) - want.astype(np.int32)).max() <= 1
        else:
            assert np.abs(got - want).max() <= 1e-6 * max(1.0, np.abs(want).max())

    dy = ml.Tensor((b, h, w, cout), "int8" if int8_out else "float32")
    ml.quantizedConvForward(ctx, dx, in_qd, dw, ds, db, dy, out_qd, de, ext_qd, act)
    check(dy.copyToHost(ctx))
    if int8_out:  # the reference's three device calls (im2row with the zero-point padding, int8 GEMM, requantisation)
        layer = Conv2D(ctx, (b, h, w, cin), cout, k, act, True, "int8")
        layer.setupQuantization(q, scales, folded, [in_qd, ext_qd], out_qd, int8_mode="reference")
        ws = ml.Tensor((max(1, layer.getWorkspaceSize()),), B.DTYPE_INT32)
        dy2 = ml.Tensor((b, h, w, cout), "int8")
        layer.forward([dx, de] if has_ext else [dx], dy2, ws)
        check(dy2.copyToHost(ctx))
