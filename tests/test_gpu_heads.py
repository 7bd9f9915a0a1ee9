"""The steps after the convolution trunk on the GPU against the CPU oracle and the reference's fixtures, through the C-ABI: softmax,
global average pooling, batch normalisation in inference mode and its folding.

Tolerances (max-abs relative error per result tensor): fp32 1e-4, fp16 1e-2. The kernels reduce in a different order than the
sequential CPU loops (wavefront shuffles, 8 partial sums per channel), so results agree to rounding, not bit for bit."""
import numpy as np
import pytest

import oracle as O
from minml_amd import core as ml
from util import TOL, max_abs_rel, mismatches, random_tensor, storage

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tag,dtype", [("f32", "float32"), ("f16", "float16")])
def test_heads_against_reference_fixtures(ctx, golden, tag, dtype):
    g = golden
    for key in ("sm", "sm3"):
        x = g[key + "_x_" + tag]
        d = ml.toDevice(ctx, x)
        ml.softmaxForward(ctx, d, d)  # in place, like the reference's own test
        assert max_abs_rel(d.copyToHost(ctx), g[key + "_y_" + tag]) <= TOL[dtype]
    for key in ("gap", "gap7"):
        x = g[key + "_x_" + tag]
        y = ml.Tensor((x.shape[0], x.shape[3]), dtype)
        ml.globalAveragePoolingForward(ctx, 1.0, ml.toDevice(ctx, x), 0.0, y)
        assert max_abs_rel(y.copyToHost(ctx), g[key + "_y_" + tag]) <= TOL[dtype]
    if dtype == "float32":
        for key in ("fd", "fd3"):
            w, b = ml.toDevice(ctx, g[key + "_w"]), ml.toDevice(ctx, g[key + "_b"])
            ml.foldBatchnorm(ctx, w, b, ml.toDevice(ctx, g[key + "_gamma"]), ml.toDevice(ctx, g[key + "_beta"]), ml.toDevice(ctx, g[key + "_stats"]))
            assert max_abs_rel(w.copyToHost(ctx), g[key + "_w_out"]) <= 1e-6
            assert max_abs_rel(b.copyToHost(ctx), g[key + "_b_out"]) <= 1e-6


def test_softmax_known_answer(ctx):
    """test/backend/test_nonlinearity.cpp:48-61 (fp32, 1e-4) and :63-79 (fp16, 1e-3), mean absolute difference."""
    x = np.array([[0.1, -0.9, 2.0, 0.0], [0.3, -1.0, 0.7, -0.1]], np.float32)
    want = np.array([[0.11162444, 0.04106433, 0.74630924, 0.10100197], [0.29114823, 0.07934714, 0.43434212, 0.19516249]], np.float32)
    d = ml.toDevice(ctx, x)
    ml.softmaxForward(ctx, d, d)
    assert np.abs(d.copyToHost(ctx) - want).mean() <= 1e-4
    dh = ml.toDevice(ctx, O.to_half(x))
    ml.softmaxForward(ctx, dh, dh)
    assert np.abs(O.from_half(dh.copyToHost(ctx)) - want).mean() <= 1e-3


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape", [(1024, 225), (4096, 3), (7, 1), (33, 16), (33, 17), (50, 64), (50, 65), (19, 128), (21, 200), (9, 361), (5, 1000),
                                   (3, 1024), (3, 1025), (2, 5000), (6, 2048), (9, 520), (300, 256)])
def test_softmax_shapes(ctx, dtype, shape):
    """Every kernel form: thread per row (up to 16 columns), row in registers (1, 2, 4, 8, 16 values per lane; 1, 2, 4 16-byte vectors per
    lane where the row length is a multiple of the vector), streaming (longer rows)."""
    rng = np.random.default_rng(shape[0] * 7919 + shape[1])
    x = random_tensor(rng, shape, dtype, 4.0)
    y = ml.Tensor(shape, dtype)
    ml.softmaxForward(ctx, y, ml.toDevice(ctx, x))
    got = y.copyToHost(ctx)
    assert max_abs_rel(got, O.softmax_forward(x)) <= TOL[dtype]
    rows = O.as_float(got).astype(np.float64).sum(axis=1)
    assert np.abs(rows - 1.0).max() <= (1e-5 if dtype == "float32" else 2e-3 * max(1.0, shape[1] / 64))
    d = ml.toDevice(ctx, x)
    ml.softmaxForward(ctx, d, d)
    assert mismatches(d.copyToHost(ctx), got) == 0  # in place gives the same bits


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape", [(12, 13, 14, 132), (64, 15, 15, 256), (3, 19, 19, 64), (2, 5, 5, 7), (5, 1, 1, 8), (1, 8, 8, 1), (4, 3, 3, 260),
                                   (2, 7, 7, 1032)])
def test_global_average_pooling_shapes(ctx, dtype, shape):
    """test/backend/test_global_pooling.cpp:493-572 uses [12, 13, 14, 132]; plus channel counts for the 8-, 4- and 1-wide forms and more than
    one channel slab."""
    rng = np.random.default_rng(sum(shape))
    x = random_tensor(rng, shape, dtype)
    y = ml.Tensor((shape[0], shape[3]), dtype)
    ml.globalAveragePoolingForward(ctx, 1.0, ml.toDevice(ctx, x), 0.0, y)
    want = O.global_average_pooling_forward(x)
    scale = float(np.abs(O.as_float(x)).mean())  # means of zero-mean data are small: compare on the scale of the inputs
    assert np.abs(O.as_float(y.copyToHost(ctx)).astype(np.float64) - O.as_float(want)).max() / scale <= TOL[dtype]
    y0 = random_tensor(rng, (shape[0], shape[3]), dtype)
    dy = ml.toDevice(ctx, y0)
    ml.globalAveragePoolingForward(ctx, 0.5, ml.toDevice(ctx, x), -2.0, dy)
    want = O.global_average_pooling_forward(x, 0.5, -2.0, y0)
    assert max_abs_rel(dy.copyToHost(ctx), want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_global_average_pooling_more_images_than_one_grid_dimension_holds(ctx, dtype):
    shape = (65540, 2, 2, 8)
    rng = np.random.default_rng(3)
    x = random_tensor(rng, shape, dtype)
    y = ml.Tensor((shape[0], shape[3]), dtype)
    ml.globalAveragePoolingForward(ctx, 1.0, ml.toDevice(ctx, x), 0.0, y)
    got, want = O.as_float(y.copyToHost(ctx)).astype(np.float64), O.as_float(O.global_average_pooling_forward(x))
    scale = float(np.abs(O.as_float(x)).mean())
    assert np.abs(got - want).max() / scale <= TOL[dtype]
    assert np.abs(got[65535:] - want[65535:]).max() / scale <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape", [(123, 34), (8, 15, 15, 256), (5, 19, 19, 64), (77, 7), (3, 5, 5, 36), (1000, 1), (40, 520)])
def test_batchnorm_inference_shapes(ctx, dtype, shape):
    """The commented-out reference test uses [123, 34] with TANH (test/backend/test_normalization.cpp:537-568); every activation, the
    scaled / accumulating form, absent gamma and bias, and the 8-, 4- and 1-wide kernel forms."""
    rng = np.random.default_rng(sum(shape))
    c = shape[-1]
    x = random_tensor(rng, shape, dtype)
    gamma, bias = storage(rng.standard_normal(c) + 1.5, dtype), random_tensor(rng, (c,), dtype)
    stats = np.stack([rng.standard_normal(c), rng.random(c) + 0.05]).astype(np.float32)
    dx, dg, db, ds = ml.toDevice(ctx, x), ml.toDevice(ctx, gamma), ml.toDevice(ctx, bias), ml.toDevice(ctx, stats)
    for act_name, act in (("linear", O.LINEAR), ("tanh", O.TANH), ("relu", O.RELU), ("sigmoid", O.SIGMOID), ("leaky_relu", O.LEAKY_RELU)):
        y = ml.Tensor(shape, dtype)
        ml.batchnormInference(ctx, 1.0, dx, dg, db, ds, 0.0, y, act_name)
        assert max_abs_rel(y.copyToHost(ctx), O.batchnorm_inference(x, gamma, bias, stats, act)) <= TOL[dtype]
    y0 = random_tensor(rng, shape, dtype)
    dy = ml.toDevice(ctx, y0)
    ml.batchnormInference(ctx, 0.5, dx, dg, db, ds, 2.0, dy, "relu")
    assert max_abs_rel(dy.copyToHost(ctx), O.batchnorm_inference(x, gamma, bias, stats, O.RELU, 0.5, 2.0, y0)) <= TOL[dtype]
    y = ml.Tensor(shape, dtype)
    ml.batchnormInference(ctx, 1.0, dx, None, None, ds, 0.0, y, "linear")
    assert max_abs_rel(y.copyToHost(ctx), O.batchnorm_inference(x, None, None, stats)) <= TOL[dtype]
    ml.batchnormInference(ctx, 1.0, dx, dg, db, ds, 0.0, dx, "linear")  # in place
    assert max_abs_rel(dx.copyToHost(ctx), O.batchnorm_inference(x, gamma, bias, stats)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("wshape", [(256, 3, 3, 256), (10, 33), (3, 3, 12), (1, 1, 1, 64), (64, 5, 5, 3)])
def test_fold_batchnorm_then_convolve(ctx, dtype, wshape):
    """Folded weights against the oracle, and the identity that folding exists for: convolution followed by batch normalisation equals the
    convolution with the folded weights (both on the device)."""
    rng = np.random.default_rng(sum(wshape))
    depthwise = len(wshape) == 3
    c = wshape[-1] if depthwise else wshape[0]
    w, b = random_tensor(rng, wshape, dtype, 0.1), random_tensor(rng, (c,), dtype)
    gamma, beta = storage(rng.standard_normal(c) * 0.2 + 1.0, dtype), random_tensor(rng, (c,), dtype, 0.5)
    stats = np.stack([rng.standard_normal(c) * 0.3, rng.random(c) + 0.5]).astype(np.float32)
    dw, db = ml.toDevice(ctx, w), ml.toDevice(ctx, b)
    ml.foldBatchnorm(ctx, dw, db, ml.toDevice(ctx, gamma), ml.toDevice(ctx, beta), ml.toDevice(ctx, stats))
    fw, fb = O.fold_batchnorm(w, b, gamma, beta, stats)
    tol = 1e-6 if dtype == "float32" else 1e-3  # one truncation step of the fp16 result
    assert max_abs_rel(dw.copyToHost(ctx), fw) <= tol and max_abs_rel(db.copyToHost(ctx), fb) <= tol
    if len(wshape) == 4 and wshape[1] in (1, 3, 5):
        x = random_tensor(rng, (2, 9, 9, wshape[3]), dtype)
        dx = ml.toDevice(ctx, x)
        plain = ml.Tensor((2, 9, 9, c), dtype)
        ml.convolutionImplicitGemmForward(ctx, dx, ml.toDevice(ctx, w), plain, ml.toDevice(ctx, b), None, "linear")
        normed = ml.Tensor((2, 9, 9, c), dtype)
        ml.batchnormInference(ctx, 1.0, plain, ml.toDevice(ctx, gamma), ml.toDevice(ctx, beta), ml.toDevice(ctx, stats), 0.0, normed, "relu")
        folded = ml.Tensor((2, 9, 9, c), dtype)
        ml.convolutionImplicitGemmForward(ctx, dx, dw, folded, db, None, "relu")
        assert max_abs_rel(folded.copyToHost(ctx), normed.copyToHost(ctx)) <= (1e-4 if dtype == "float32" else 2e-2)


def test_heads_reject_bad_arguments(ctx):
    x = ml.Tensor((2, 3, 3, 8), "float32")
    with pytest.raises(ValueError):
        ml.globalAveragePoolingForward(ctx, 1.0, x, 0.0, ml.Tensor((2, 9), "float32"))
    with pytest.raises(ValueError):
        ml.batchnormInference(ctx, 1.0, x, None, None, ml.Tensor((2, 9), "float32"), 0.0, x)
    with pytest.raises(ValueError):
        ml.foldBatchnorm(ctx, ml.Tensor((4, 8), "float32"), ml.Tensor((5,), "float32"), None, None, ml.Tensor((2, 4), "float32"))


def test_full_size_policy_and_value_inputs(ctx):
    """Benchmark-size tensors through size-independent properties: policy rows sum to one and keep their order; pooling is linear and
    reproduces a constant image; batch normalisation with identity statistics is the identity."""
    rng = np.random.default_rng(11)
    logits = random_tensor(rng, (1024, 225), "float16", 3.0)
    d = ml.toDevice(ctx, logits)
    ml.softmaxForward(ctx, d, d)
    p = O.from_half(d.copyToHost(ctx)).astype(np.float64)
    assert np.abs(p.sum(axis=1) - 1.0).max() <= 5e-3
    assert np.array_equal(p.argmax(axis=1), O.from_half(logits).argmax(axis=1))
    x = random_tensor(rng, (1024, 15, 15, 256), "float16")
    dx = ml.toDevice(ctx, x)
    y = ml.Tensor((1024, 256), "float16")
    ml.globalAveragePoolingForward(ctx, 1.0, dx, 0.0, y)
    mean = O.from_half(x).astype(np.float64).mean(axis=(1, 2))
    assert np.abs(O.from_half(y.copyToHost(ctx)) - mean).max() <= 2e-3
    stats = np.stack([np.zeros(256), np.ones(256) - 1e-6]).astype(np.float32)
    out = ml.Tensor(x.shape, "float16")
    ml.batchnormInference(ctx, 1.0, dx, None, None, ml.toDevice(ctx, stats), 0.0, out, "linear")
    assert max_abs_rel(out.copyToHost(ctx), x) <= 1e-3


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_policy_and_value_heads_after_a_trunk(ctx, dtype):
    """The two heads of a board-game network on one trunk output [B, 15, 15, 256], every step on the device against the same chain of
    oracle calls: policy = 1x1 convolution to one plane -> softmax over the 225 squares; value = global average pooling -> Dense 256 ->
    256 with ReLU -> Dense 256 -> 3 -> softmax (Dense rides on gemm_ex, as in the reference's src/layers/Dense.cpp)."""
    rng = np.random.default_rng(21)
    batch, board, c = 64, 15, 256
    trunk = storage(np.maximum(rng.standard_normal((batch, board, board, c)), 0.0), dtype)
    wp, bp = random_tensor(rng, (1, 1, 1, c), dtype, 0.1), random_tensor(rng, (1,), dtype)
    w1, b1 = random_tensor(rng, (c, c), dtype, 0.1), random_tensor(rng, (c,), dtype)
    w2, b2 = random_tensor(rng, (3, c), dtype, 0.1), random_tensor(rng, (3,), dtype)
    dt = ml.toDevice(ctx, trunk)
    # policy
    logits = ml.Tensor((batch, board, board, 1), dtype)
    ml.convolutionImplicitGemmForward(ctx, dt, ml.toDevice(ctx, wp), logits, ml.toDevice(ctx, bp), None, "linear")
    policy = logits.view((batch, board * board))
    ml.softmaxForward(ctx, policy, policy)
    want_logits = O.conv2d_forward(trunk, wp, bp, None, O.LINEAR).reshape(batch, board * board)
    want_policy = O.softmax_forward(want_logits)
    assert max_abs_rel(policy.copyToHost(ctx), want_policy) <= TOL[dtype] * 2  # two chained steps
    # value
    pooled = ml.Tensor((batch, c), dtype)
    ml.globalAveragePoolingForward(ctx, 1.0, dt, 0.0, pooled)
    hidden = ml.Tensor((batch, c), dtype)
    ml.gemm_ex(ctx, hidden, 1.0, "n", pooled, "t", ml.toDevice(ctx, w1), 0.0, None, ml.toDevice(ctx, b1), "relu")
    out = ml.Tensor((batch, 3), dtype)
    ml.gemm_ex(ctx, out, 1.0, "n", hidden, "t", ml.toDevice(ctx, w2), 0.0, None, ml.toDevice(ctx, b2), "linear")
    ml.softmaxForward(ctx, out, out)
    want = O.global_average_pooling_forward(trunk)
    want = O.gemm(want, w1, bias=b1, act=O.RELU)
    want = O.softmax_forward(O.gemm(want, w2, bias=b2))
    assert max_abs_rel(out.copyToHost(ctx), want) <= TOL[dtype] * 4  # four chained steps
    assert np.abs(O.as_float(out.copyToHost(ctx)).astype(np.float64).sum(axis=1) - 1.0).max() <= (1e-5 if dtype == "float32" else 3e-3)
