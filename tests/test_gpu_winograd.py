"""Winograd F(4x4,3x3) transforms on the GPU against the CPU oracle, through the C-ABI (hip_winograd_*_transform).

The bar: the three transforms reproduce the reference's expression trees, so fp32 results and truncated fp16 results are compared
BIT FOR BIT (ReLU / linear); transcendental activations within the per-layer tolerance (max-abs relative 1e-4 fp32, 1e-2 fp16).
Shapes follow test/backend/test_winograd.cpp:396-513 ({3,9,11,35}, {3,7,11,35}: edge tiles, channel counts that match no vector width)
plus the benchmark's own (15x15 x 256, 19x19)."""
import numpy as np
import pytest

import oracle as O
from minml_amd import core as ml
from util import TOL, max_abs_rel, mismatches, random_tensor
from test_oracle_pins import INPUT_ONES, INPUT_RAMP, OUTPUT_ONES, OUTPUT_RAMP, WEIGHT_NINES, WEIGHT_RAMP, both_channels

pytestmark = pytest.mark.gpu

SHAPES = [((3, 9, 11, 35), 21), ((3, 7, 11, 35), 35), ((2, 15, 15, 32), 64), ((2, 15, 15, 256), 256), ((1, 19, 19, 64), 128), ((1, 4, 4, 2), 2),
          ((2, 3, 2, 1), 1), ((1, 5, 17, 6), 10)]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape,cout", SHAPES)
def test_transforms_bit_exact(ctx, dtype, shape, cout):
    rng = np.random.default_rng(hash((shape, cout)) % 2 ** 31)
    b, h, w, c = shape
    tiles = b * ((h + 3) // 4) * ((w + 3) // 4)
    # weights
    wt = random_tensor(rng, (cout, 3, 3, c), dtype)
    dm = ml.Tensor((36, cout, c), dtype)
    for invert in (False, True):
        ml.winogradWeightTransform(ctx, ml.toDevice(ctx, wt), dm, invert)
        assert mismatches(dm.copyToHost(ctx), O.winograd_weight_transform(wt, invert)) == 0
    # input
    x = random_tensor(rng, shape, dtype)
    dv = ml.Tensor((36, tiles, c), dtype)
    ml.winogradInputTransform(ctx, (cout, 3, 3, c), ml.toDevice(ctx, x), dv)
    assert mismatches(dv.copyToHost(ctx), O.winograd_input_transform(x)) == 0
    # output with every combination of bias / residual, linear and ReLU
    m = random_tensor(rng, (36, tiles, cout), dtype)
    bias = random_tensor(rng, (cout,), dtype)
    ext = random_tensor(rng, (b, h, w, cout), dtype)
    dmm, db, de = ml.toDevice(ctx, m), ml.toDevice(ctx, bias), ml.toDevice(ctx, ext)
    for use_bias in (True, False):
        for use_ext in (True, False):
            for act in (O.LINEAR, O.RELU):
                dy = ml.Tensor((b, h, w, cout), dtype)
                dy.setall(ctx, 7.0)
                ml.winogradOutputTransform(ctx, (cout, 3, 3, cout), dmm, dy, db if use_bias else None, de if use_ext else None, act)
                want = O.winograd_output_transform(m, (b, h, w, cout), bias if use_bias else None, ext if use_ext else None, act)
                assert mismatches(dy.copyToHost(ctx), want) == 0


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("act", [O.SIGMOID, O.TANH, O.LEAKY_RELU, O.EXP])
def test_output_transform_other_activations(ctx, dtype, act):
    rng = np.random.default_rng(act)
    shape, cout = (2, 9, 11, 12), 12
    m = random_tensor(rng, (36, 2 * 3 * 3, cout), dtype, 0.2)
    bias = random_tensor(rng, (cout,), dtype)
    ext = random_tensor(rng, shape, dtype)
    dy = ml.Tensor(shape, dtype)
    ml.winogradOutputTransform(ctx, (cout, 3, 3, cout), ml.toDevice(ctx, m), dy, ml.toDevice(ctx, bias), ml.toDevice(ctx, ext), act)
    assert max_abs_rel(dy.copyToHost(ctx), O.winograd_output_transform(m, shape, bias, ext, act)) <= TOL[dtype]


def test_golden_vectors_through_the_gpu(ctx):
    """The literals of test/backend/test_winograd.cpp:218-323, mean-abs-diff <= 1e-4 as there."""
    for image, expected in ((np.ones((4, 4)), INPUT_ONES), (np.arange(1, 17).reshape(4, 4), INPUT_RAMP)):
        dv = ml.Tensor((36, 1, 2), "float32")
        ml.winogradInputTransform(ctx, (2, 3, 3, 2), ml.toDevice(ctx, both_channels(image)[None]), dv)
        got = dv.copyToHost(ctx)
        for ch in range(2):
            assert np.abs(got[:, 0, ch].reshape(6, 6) - np.array(expected)).mean() <= 1e-4
    for matrices, expected in ((np.ones(36), OUTPUT_ONES), (np.arange(1, 37), OUTPUT_RAMP)):
        dy = ml.Tensor((1, 4, 4, 2), "float32")
        ml.winogradOutputTransform(ctx, (2, 3, 3, 2), ml.toDevice(ctx, both_channels(matrices)[:, None, :]), dy, None, None, "linear")
        got = dy.copyToHost(ctx)
        for ch in range(2):
            assert np.abs(got[0, :, :, ch] - np.array(expected)).mean() <= 1e-4
    for kernel, expected in ((np.full((3, 3), 9.0), WEIGHT_NINES), (np.arange(1, 10).reshape(3, 3), WEIGHT_RAMP)):
        dm = ml.Tensor((36, 1, 2), "float32")
        ml.winogradWeightTransform(ctx, ml.toDevice(ctx, both_channels(kernel)[None]), dm, False)
        got = dm.copyToHost(ctx)
        for ch in range(2):
            assert np.abs(got[:, 0, ch].reshape(6, 6) - np.array(expected)).mean() <= 1e-4


@pytest.mark.parametrize("tag,dtype", [("f32", "float32"), ("f16", "float16")])
def test_reference_fixtures_through_the_gpu(ctx, golden, tag, dtype):
    """Outputs recorded from the reference's compiled CPU backend (tests/golden/make_fixtures.py)."""
    g = golden
    dm = ml.Tensor((36, 13, 19), dtype)
    ml.winogradWeightTransform(ctx, ml.toDevice(ctx, g["wg_w_" + tag]), dm, False)
    assert mismatches(dm.copyToHost(ctx), g["wg_wm_" + tag]) == 0
    ml.winogradWeightTransform(ctx, ml.toDevice(ctx, g["wg_w_" + tag]), dm, True)
    assert mismatches(dm.copyToHost(ctx), g["wg_wm_inverted_" + tag]) == 0
    dv = ml.Tensor((36, 18, 19), dtype)
    ml.winogradInputTransform(ctx, (13, 3, 3, 19), ml.toDevice(ctx, g["wg_x_" + tag]), dv)
    assert mismatches(dv.copyToHost(ctx), g["wg_v_" + tag]) == 0
    dy = ml.Tensor((2, 9, 11, 13), dtype)
    ml.winogradOutputTransform(ctx, (13, 3, 3, 13), ml.toDevice(ctx, g["wg_m_" + tag]), dy, ml.toDevice(ctx, g["wg_bias_" + tag]),
                               ml.toDevice(ctx, g["wg_ext_" + tag]), "relu")
    assert mismatches(dy.copyToHost(ctx), g["wg_y_relu_" + tag]) == 0
    ml.winogradOutputTransform(ctx, (13, 3, 3, 13), ml.toDevice(ctx, g["wg_m_" + tag]), dy, ml.toDevice(ctx, g["wg_bias_" + tag]), None, "linear")
    assert mismatches(dy.copyToHost(ctx), g["wg_y_linear_" + tag]) == 0
    # the GEMM in between, within tolerance (the MFMA accumulation order is the hardware's)
    dmo = ml.Tensor((36, 18, 13), dtype)
    ml.gemmBatched(ctx, "n", "t", dmo, ml.toDevice(ctx, g["wg_v_" + tag]), ml.toDevice(ctx, g["wg_wm_" + tag]))
    assert max_abs_rel(dmo.copyToHost(ctx), g["wg_m_" + tag]) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_full_pipeline_against_direct_convolution(ctx, dtype):
    """test/backend/test_conv2D.cpp:580-629: {3,13,17,35} -> 21 filters, weight transform -> input transform -> gemmBatched('n','t') ->
    output transform with bias, against the direct convolution."""
    rng = np.random.default_rng(11)
    x = random_tensor(rng, (3, 13, 17, 35), dtype)
    w = random_tensor(rng, (21, 3, 3, 35), dtype, 0.1)
    bias = random_tensor(rng, (21,), dtype)
    wm = ml.Tensor((36, 21, 35), dtype)
    ml.winogradWeightTransform(ctx, ml.toDevice(ctx, w), wm, False)
    v = ml.Tensor((36, 3 * 4 * 5, 35), dtype)
    m = ml.Tensor((36, 3 * 4 * 5, 21), dtype)
    ml.winogradInputTransform(ctx, (21, 3, 3, 35), ml.toDevice(ctx, x), v)
    ml.gemmBatched(ctx, "n", "t", m, v, wm, 1.0, 0.0)
    y = ml.Tensor((3, 13, 17, 21), dtype)
    ml.winogradOutputTransform(ctx, (21, 3, 3, 35), m, y, ml.toDevice(ctx, bias), None, "sigmoid")
    got = y.copyToHost(ctx)
    direct = O.conv2d_forward(x, w, bias, None, O.SIGMOID)
    if dtype == "float32":
        assert max_abs_rel(got, direct) <= TOL[dtype]
    else:
        # in fp16 the Winograd algorithm itself (matrices truncated to half between the stages) is what differs from a direct
        # convolution, on the CPU reference as much as here: the tolerance applies against the same algorithm on the CPU, and the
        # distance to the direct convolution is bounded the way the reference bounds it (mean absolute difference)
        pipeline = O.winograd_output_transform(O.gemm(O.winograd_input_transform(x), O.winograd_weight_transform(w)), (3, 13, 17, 21), bias, None,
                                               O.SIGMOID)
        assert max_abs_rel(got, pipeline) <= TOL[dtype]
        assert np.abs(O.from_half(got) - O.from_half(direct)).mean() <= 1e-2


def test_empty_and_full_size_properties(ctx):
    """Empty batch is a no-op; at the benchmark's full size (B = 1024, 15x15, 256 channels, fp16) the transform of a batch equals the
    transforms of its halves (positions are independent), and an all-zero image transforms to zeros."""
    ml.winogradInputTransform(ctx, (8, 3, 3, 8), ml.Tensor((0, 15, 15, 8), "float16"), ml.Tensor((36, 0, 8), "float16"))
    rng = np.random.default_rng(12)
    x = random_tensor(rng, (1024, 15, 15, 256), "float16")
    dx = ml.toDevice(ctx, x)
    full = ml.Tensor((36, 16384, 256), "float16")
    ml.winogradInputTransform(ctx, (256, 3, 3, 256), dx, full)
    got = full.copyToHost(ctx)
    half = ml.Tensor((36, 8192, 256), "float16")
    ml.winogradInputTransform(ctx, (256, 3, 3, 256), dx.view((512, 15, 15, 256), 512 * 225 * 256), half)
    assert np.array_equal(got[:, 8192:], half.copyToHost(ctx))
    sample = O.winograd_input_transform(x[1000:1002])
    assert np.array_equal(got[:, 16000:16032], sample)
    dx.zeroall(ctx)
    ml.winogradInputTransform(ctx, (256, 3, 3, 256), dx, full)
    assert not full.copyToHost(ctx).any()


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape", [(2, 15, 15, 64), (3, 19, 19, 128), (2, 9, 11, 64), (1, 4, 4, 64), (2, 7, 5, 192), (2, 9, 11, 35)])
def test_fused_output_input_transform_bit_exact(ctx, dtype, shape):
    """hip_winograd_output_input_transform against the oracle's output transform followed by its input transform, bit for bit: with
    and without bias / residual, ReLU / linear / a transcendental activation (exact against the GPU's own two-call sequence), with
    y written to memory and with y kept on chip. The last shape (35 channels) takes the entry point's two-kernel route."""
    rng = np.random.default_rng(sum(shape))
    b, h, w, c = shape
    tiles = b * ((h + 3) // 4) * ((w + 3) // 4)
    m = random_tensor(rng, (36, tiles, c), dtype)
    bias = random_tensor(rng, (c,), dtype)
    ext = random_tensor(rng, shape, dtype)
    dm, db, de = ml.toDevice(ctx, m), ml.toDevice(ctx, bias), ml.toDevice(ctx, ext)
    wshape = (c, 3, 3, c)
    for use_bias, use_ext, act in ((True, True, O.RELU), (False, False, O.LINEAR), (True, False, O.RELU), (False, True, O.LINEAR)):
        want_y = O.winograd_output_transform(m, shape, bias if use_bias else None, ext if use_ext else None, act)
        want_v = O.winograd_input_transform(want_y)
        for keep_y in (True, False):
            if not keep_y and c % 64 != 0:
                continue
            dy = ml.Tensor(shape, dtype)
            dy.setall(ctx, 7.0)
            dv = ml.Tensor((36, tiles, c), dtype)
            dv.setall(ctx, float("nan"))
            ml.winogradOutputInputTransform(ctx, wshape, dm, shape, dy if keep_y else None, db if use_bias else None, de if use_ext else None, act, dv)
            assert mismatches(dv.copyToHost(ctx), want_v) == 0
            if keep_y:
                assert mismatches(dy.copyToHost(ctx), want_y) == 0
    # activations that the reference runs as a second pass: identical to the GPU's own two calls
    dy2, dv2 = ml.Tensor(shape, dtype), ml.Tensor((36, tiles, c), dtype)
    ml.winogradOutputTransform(ctx, wshape, dm, dy2, db, de, O.TANH)
    ml.winogradInputTransform(ctx, wshape, dy2, dv2)
    dy3, dv3 = ml.Tensor(shape, dtype), ml.Tensor((36, tiles, c), dtype)
    ml.winogradOutputInputTransform(ctx, wshape, dm, shape, dy3, db, de, O.TANH, dv3)
    assert mismatches(dv3.copyToHost(ctx), dv2.copyToHost(ctx)) == 0
    assert mismatches(dy3.copyToHost(ctx), dy2.copyToHost(ctx)) == 0


@pytest.mark.parametrize("case", [(32, 15, 15, True, True, O.RELU), (64, 13, 16, False, False, O.RELU), (36, 15, 15, True, False, O.LINEAR),
                                  (256, 15, 15, True, True, O.RELU), (8, 15, 15, True, True, O.RELU), (32, 19, 19, True, True, O.RELU)])
def test_whole_layer_launch_is_bit_identical(ctx, case):
    """hip_winograd_layer_forward against the library's own batched product followed by the fused transform, bit for bit (the same MFMA
    sequence per element), with and without residual / stored output, for batches that give the XCDs equal and unequal numbers of chunks.
    The last two cases (batch below 32, 25 tiles per image) take the entry point's two-call route through the output matrices."""
    batch, h, w, use_ext, keep_y, act = case
    c = 256
    rng = np.random.default_rng(batch + h)
    tiles = batch * ((h + 3) // 4) * ((w + 3) // 4)
    shape = (batch, h, w, c)
    wshape = (c, 3, 3, c)
    v = random_tensor(rng, (36, tiles, c), "float16")
    u = random_tensor(rng, (36, c, c), "float16", 0.05)
    bias = random_tensor(rng, (c,), "float16")
    ext = random_tensor(rng, shape, "float16")
    du, db, de = ml.toDevice(ctx, u), ml.toDevice(ctx, bias), ml.toDevice(ctx, ext)
    # reference sequence of this library
    dv, dm = ml.toDevice(ctx, v), ml.Tensor((36, tiles, c), "float16")
    ml.gemmBatched(ctx, "n", "t", dm, dv, du, 1.0, 0.0)
    want_y, want_next = ml.Tensor(shape, "float16"), ml.Tensor((36, tiles, c), "float16")
    ml.winogradOutputInputTransform(ctx, wshape, dm, shape, want_y, db, de if use_ext else None, act, want_next)
    # one launch, next matrices written over the input matrices as the network runner does
    dv2, dm2 = ml.toDevice(ctx, v), ml.Tensor((36, tiles, c), "float16")
    got_y = ml.Tensor(shape, "float16")
    got_y.setall(ctx, 7.0)
    for repeat in range(2):  # the second launch finds the scratch buffer and the counters used
        ml.convertType(ctx, dv2, ml.toDevice(ctx, v))
        ml.winogradLayerForward(ctx, wshape, dv2, du, dm2, shape, got_y if keep_y else None, db, de if use_ext else None, act, dv2)
        assert ml.winogradLayerErrors(ctx) == 0
        assert mismatches(dv2.copyToHost(ctx), want_next.copyToHost(ctx)) == 0
        if keep_y:
            assert mismatches(got_y.copyToHost(ctx), want_y.copyToHost(ctx)) == 0


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_residual_may_alias_the_output(ctx, dtype):
    """y = act(transform + bias + y): the residual tensor is the output tensor itself (an in-place skip connection). Both the stand-alone
    output transform and the fused form read every residual element before they write it."""
    rng = np.random.default_rng(17)
    shape, c = (3, 15, 15, 64), 64
    tiles = 3 * 16
    m = random_tensor(rng, (36, tiles, c), dtype)
    bias = random_tensor(rng, (c,), dtype)
    ext = random_tensor(rng, shape, dtype)
    want_y = O.winograd_output_transform(m, shape, bias, ext, O.RELU)
    dm, db = ml.toDevice(ctx, m), ml.toDevice(ctx, bias)
    y = ml.toDevice(ctx, ext)
    ml.winogradOutputTransform(ctx, (c, 3, 3, c), dm, y, db, y, O.RELU)
    assert mismatches(y.copyToHost(ctx), want_y) == 0
    y = ml.toDevice(ctx, ext)
    nxt = ml.Tensor((36, tiles, c), dtype)
    ml.winogradOutputInputTransform(ctx, (c, 3, 3, c), dm, shape, y, db, y, O.RELU, nxt)
    assert mismatches(y.copyToHost(ctx), want_y) == 0
    assert mismatches(nxt.copyToHost(ctx), O.winograd_input_transform(want_y)) == 0
