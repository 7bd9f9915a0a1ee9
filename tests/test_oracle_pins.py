"""Pins of the CPU oracle that do not need the reference: golden vectors lifted from the reference's tests, closed forms, brute force on
tiny inputs and independent numpy evaluations. A dropped term, a wrong sign or index, or a transposed operand fails at least one."""
import numpy as np
import pytest

import oracle as O
from util import init_for_test, values

# ---- literals of test/backend/test_winograd.cpp:218-323 --------------------------------------------------------------------------
BT = np.array([[1, 0, -1.25, 0, 0.25, 0], [0, 1, 1, -0.25, -0.25, 0], [0, -1, 1, 0.25, -0.25, 0], [0, -1, -0.5, 1, 0.5, 0],
               [0, 1, -0.5, -1, 0.5, 0], [0, 1, 0, -1.25, 0, 0.25]], np.float64)
AT = np.array([[1, 1, 1, 0.25, 0.25, 0], [0, 1, -1, 0.5, -0.5, 0], [0, 1, 1, 1, 1, 0], [0, 1, -1, 2, -2, 2]], np.float64)
G = np.array([[1, 0, 0], [2 / 3, 2 / 3, 2 / 3], [2 / 3, -2 / 3, 2 / 3], [1 / 3, 2 / 3, 4 / 3], [1 / 3, -2 / 3, 4 / 3], [0, 0, 2]], np.float64)

INPUT_ONES = [[1, -1.5, 0, 0, 0, 0.25], [-1.5, 2.25, 0, 0, 0, -0.375], [0] * 6, [0] * 6, [0] * 6, [0.25, -0.375, 0, 0, 0, 0.0625]]
INPUT_RAMP = [[3.5, -4.25, -0.75, -3.0, 1.0, 3.25], [-1.25, 0.375, 1.125, 4.5, -1.5, -3.875], [-3.0, 4.5, 0, 0, 0, -0.75],
              [-12.0, 18.0, 0, 0, 0, -3.0], [4.0, -6.0, 0, 0, 0, 1.0], [10.375, -15.3125, -0.1875, -0.75, 0.25, 3.1875]]
OUTPUT_ONES = [[12.25, 0, 14, 7], [0, 0, 0, 0], [14, 0, 16, 8], [7, 0, 8, 4]]
OUTPUT_RAMP = [[128.625, -5.25, 163.0, 88.5], [-31.5, 0, -36.0, -18.0], [243.0, -6.0, 296.0, 156.0], [163.5, -3.0, 196.0, 102.0]]
WEIGHT_NINES = [[9, 18, 6, 21, 9, 18], [18, 36, 12, 42, 18, 36], [6, 12, 4, 14, 6, 12], [21, 42, 14, 49, 21, 42], [9, 18, 6, 21, 9, 18],
                [18, 36, 12, 42, 18, 36]]
WEIGHT_RAMP = [[1.0, 4.0, 1.3333333333, 5.6666666667, 3.0, 6.0], [8.0, 20.0, 6.6666666667, 25.3333333333, 12.0, 24.0],
               [2.6666666667, 6.6666666667, 2.222222222, 8.4444444444, 4.0, 8.0], [12.3333333333, 29.3333333333, 9.7777777778, 36.5555555556, 17.0, 34.0],
               [7.0, 16.0, 5.3333333333, 19.6666666667, 9.0, 18.0], [14.0, 32.0, 10.6666666667, 39.3333333333, 18.0, 36.0]]


def both_channels(plane):
    return np.repeat(np.asarray(plane, np.float32)[..., None], 2, axis=-1)


@pytest.mark.parametrize("image,expected", [(np.ones((4, 4)), INPUT_ONES), (np.arange(1, 17).reshape(4, 4), INPUT_RAMP)])
def test_input_transform_golden(image, expected):
    x = both_channels(image)[None]  # [1,4,4,2]
    m = O.winograd_input_transform(x)  # [36,1,2]
    for ch in range(2):
        assert np.abs(m[:, 0, ch].reshape(6, 6) - np.array(expected)).mean() <= 1e-4


@pytest.mark.parametrize("matrices,expected", [(np.ones(36), OUTPUT_ONES), (np.arange(1, 37), OUTPUT_RAMP)])
def test_output_transform_golden(matrices, expected):
    m = both_channels(matrices)[:, None, :]  # [36,1,2]
    y = O.winograd_output_transform(m, (1, 4, 4, 2))
    for ch in range(2):
        assert np.abs(y[0, :, :, ch] - np.array(expected)).mean() <= 1e-4


@pytest.mark.parametrize("kernel,expected", [(np.full((3, 3), 9.0), WEIGHT_NINES), (np.arange(1, 10).reshape(3, 3), WEIGHT_RAMP)])
def test_weight_transform_golden(kernel, expected):
    w = both_channels(kernel)[None]  # [1,3,3,2]
    m = O.winograd_weight_transform(w)  # [36,1,2]
    for ch in range(2):
        assert np.abs(m[:, 0, ch].reshape(6, 6) - np.array(expected)).mean() <= 1e-4


def direct_conv64(x, w, bias=None, add=None):
    """baseline_conv2D_forward (test/backend/test_conv2D.cpp:22-59) in float64."""
    b, h, wd, cin = x.shape
    cout, k = w.shape[0], w.shape[1]
    pad = (k - 1) // 2
    xp = np.zeros((b, h + 2 * pad + 1, wd + 2 * pad + 1, cin))
    xp[:, pad:pad + h, pad:pad + wd] = x
    y = np.zeros((b, h, wd, cout))
    for i in range(k):
        for j in range(k):
            y += np.einsum("bhwc,oc->bhwo", xp[:, i:i + h, j:j + wd], w[:, i, j].astype(np.float64))
    if bias is not None:
        y += bias
    if add is not None:
        y += add
    return y


def test_matrix_form_and_closed_form():
    """V = Bt d B, U = G g Gt, Y = At M A in float64 against the oracle, and the whole pipeline against a direct convolution, on a shape
    with edge tiles in both directions and channel counts that are not multiples of anything."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 9, 11, 5)).astype(np.float32)
    w = rng.standard_normal((7, 3, 3, 5)).astype(np.float32)
    v = O.winograd_input_transform(x)
    u = O.winograd_weight_transform(w)
    # matrix form per tile / filter pair
    xp = np.zeros((2, 14, 14, 5))
    xp[:, 1:10, 1:12] = x
    t = 0
    for b in range(2):
        for tx in range(3):
            for ty in range(3):
                d = xp[b, 4 * tx:4 * tx + 6, 4 * ty:4 * ty + 6]  # [6,6,C]
                ref = np.einsum("ij,jkc,lk->ilc", BT, d, BT)
                assert np.abs(v[:, t].reshape(6, 6, 5) - ref).max() <= 1e-5
                t += 1
    ref_u = np.einsum("ij,ojkc,lk->iloc", G, w.astype(np.float64), G)
    assert np.abs(u.reshape(6, 6, 7, 5) - ref_u).max() <= 1e-5
    m = O.gemm(v, u)  # [36, tiles, 7]
    y = O.winograd_output_transform(m, (2, 9, 11, 7))
    want = direct_conv64(x.astype(np.float64), w)
    assert np.abs(y - want).max() / np.abs(want).max() <= 1e-5
    # the same with bias, residual and ReLU fused in the output transform
    bias = rng.standard_normal(7).astype(np.float32)
    add = rng.standard_normal((2, 9, 11, 7)).astype(np.float32)
    y2 = O.winograd_output_transform(m, (2, 9, 11, 7), bias, add, O.RELU)
    want2 = np.maximum(direct_conv64(x.astype(np.float64), w, bias, add), 0)
    assert np.abs(y2 - want2).max() / np.abs(want2).max() <= 1e-5


def test_weight_transform_invert_is_rotation():
    w = init_for_test((3, 3, 3, 4), 0.3)
    assert np.array_equal(O.winograd_weight_transform(w, True), O.winograd_weight_transform(np.ascontiguousarray(w[:, ::-1, ::-1, :])))


def test_zero_padding_equals_zero_extended_image():
    """An edge tile must equal the interior tile of the image extended by zeros."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, 6, 7, 3)).astype(np.float32)
    big = np.zeros((1, 16, 16, 3), np.float32)
    big[:, 4:10, 4:11] = x
    v_small = O.winograd_input_transform(x)  # tiles 2x2
    v_big = O.winograd_input_transform(big)  # tiles 4x4; tile (1..2, 1..2) cover the same pixels
    for tx in range(2):
        for ty in range(2):
            assert np.array_equal(v_small[:, tx * 2 + ty], v_big[:, (tx + 1) * 4 + (ty + 1)])


# ---- fp16 ------------------------------------------------------------------------------------------------------------------------
def test_fp16_roundtrip_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    f = O.from_half(h)
    assert np.array_equal(f[np.isfinite(f)], h.view(np.float16).astype(np.float32)[np.isfinite(f)])  # widening is exact
    back = O.to_half(f)
    not_nan = ~np.isnan(f)
    assert np.array_equal(back[not_nan], h[not_nan])


def test_fp16_narrowing_truncates_toward_zero():
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.standard_normal(20000) * 10, rng.standard_normal(20000) * 1e-4, rng.standard_normal(5000) * 1e-7,
                        [0.0, -0.0, 65504.0, 65519.9, 6.0e-5, 5.9e-8, 1.0009765]]).astype(np.float32)
    got = O.from_half(O.to_half(x)).astype(np.float64)
    xd = x.astype(np.float64)
    assert np.all(np.abs(got) <= np.abs(xd))  # never rounds away from zero
    assert np.all(np.sign(got) * np.sign(xd) >= 0)
    # and it is the closest representable value on that side: the next half away from zero overshoots
    nearest = x.astype(np.float16)
    toward_zero = np.where(np.abs(nearest.astype(np.float64)) > np.abs(xd), np.nextafter(nearest, np.float16(0)), nearest)
    assert np.array_equal(got, toward_zero.astype(np.float64))


# ---- GEMM ------------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("ops", ["nn", "nt", "tn", "tt"])
def test_gemm_against_numpy(ops):
    """test/backend/test_gemms.cpp:31-90 sizes: 23 x 45 x 67 with alpha = 1.1, beta = 0.1."""
    M, N, K = 23, 45, 67
    A = init_for_test((M, K) if ops[0] == "n" else (K, M), 0.0)
    Bm = init_for_test((K, N) if ops[1] == "n" else (N, K), 1.0)
    C = init_for_test((M, N), 2.0)
    a = A if ops[0] == "n" else A.T
    b = Bm if ops[1] == "n" else Bm.T
    want = 1.1 * (a.astype(np.float64) @ b.astype(np.float64)) + 0.1 * C
    got = O.gemm(A, Bm, ops[0], ops[1], alpha=1.1, beta=0.1, C=C)
    assert np.abs(got - want).mean() <= 1e-4
    assert np.abs(got - want).max() / np.abs(want).max() <= 1e-5


def test_gemm_ex_epilogue_order_and_batch_broadcast():
    rng = np.random.default_rng(3)
    A = rng.standard_normal((4, 10, 12)).astype(np.float32)
    Bm = rng.standard_normal((9, 12)).astype(np.float32)  # rank 2: broadcast over the batch
    got = O.gemm(A, Bm)
    want = np.einsum("bmk,nk->bmn", A.astype(np.float64), Bm.astype(np.float64))
    assert np.abs(got - want).max() <= 1e-4
    bias = rng.standard_normal(9).astype(np.float32)
    C = rng.standard_normal((10, 9)).astype(np.float32)
    got = O.gemm(A[0], Bm, alpha=0.5, beta=2.0, C=C, bias=bias, act=O.RELU)
    want = np.maximum(0.5 * (A[0].astype(np.float64) @ Bm.T.astype(np.float64)) + bias + 2.0 * C, 0)
    assert np.abs(got - want).max() <= 1e-4
    # beta == 0 must not read C: NaNs there stay out of the result
    got = O.gemm(A[0], Bm, beta=0.0, C=np.full((10, 9), np.nan, np.float32))
    assert np.isfinite(got).all()


def test_gemm_k_tile_only_changes_rounding():
    rng = np.random.default_rng(4)
    A = (rng.standard_normal((6, 2500)) * 0.1).astype(np.float32)
    Bm = (rng.standard_normal((5, 2500)) * 0.1).astype(np.float32)
    want = A.astype(np.float64) @ Bm.T.astype(np.float64)
    for k_tile in (0, 1024):
        assert np.abs(O.gemm(A, Bm, k_tile=k_tile) - want).max() <= 1e-4


# ---- im2row / convolution -------------------------------------------------------------------------------------------------------
def test_im2row_brute_force():
    """baseline_receptive_fields (test/backend/test_gemm_conv.cpp:17-62): exact equality."""
    x = init_for_test((2, 5, 4, 3), 0.7)
    for k in (3, 5):
        rows = O.im2row(x, k)
        pad = (k - 1) // 2
        for b in range(2):
            for h in range(5):
                for w in range(4):
                    want = []
                    for i in range(-pad, pad + 1):
                        for j in range(-pad, pad + 1):
                            inside = 0 <= h + i < 5 and 0 <= w + j < 4
                            want.extend(x[b, h + i, w + j] if inside else np.zeros(3, np.float32))
                    assert np.array_equal(rows[(b * 5 + h) * 4 + w], np.array(want, np.float32))


@pytest.mark.parametrize("k", [1, 3, 5])
def test_conv2d_against_direct(k):
    rng = np.random.default_rng(k)
    x = rng.standard_normal((2, 6, 7, 5)).astype(np.float32)
    w = (rng.standard_normal((4, k, k, 5)) * 0.3).astype(np.float32)
    bias = rng.standard_normal(4).astype(np.float32)
    add = rng.standard_normal((2, 6, 7, 4)).astype(np.float32)
    got = O.conv2d_forward(x, w, bias, add, O.RELU)
    want = np.maximum(direct_conv64(x.astype(np.float64), w, bias, add), 0)
    assert np.abs(got - want).max() / np.abs(want).max() <= 1e-5


# ---- int8 ------------------------------------------------------------------------------------------------------------------------
def test_quantize_rounds_half_away_and_clamps():
    """quantize() of src/layers/quantization.cpp:39-43 / test/backend/test_quantization.cpp:33-36."""
    cases = {0.5: 1, -0.5: -1, 1.5: 2, 2.5: 3, -2.5: -3, 0.49: 0, 126.5: 127, 127.5: 127, 300.0: 127, -128.5: -128, -1000.0: -128, -127.5: -128}
    for x, want in cases.items():
        assert O.quantize(x) == want


def numpy_int8_conv(x, in_qd, w, scales, bias, out_qd, ext, ext_qd, relu, to_int8):
    """Independent evaluation: integer part in int64 through padding with the zero point, float tail in numpy float32 step by step."""
    b, h, wd, cin = x.shape
    cout, k = w.shape[0], w.shape[1]
    pad = (k - 1) // 2
    zero = int(np.round(np.float32(0.0) * (np.float32(1.0) / np.float32(in_qd[0])) + (-np.float32(in_qd[1]) / np.float32(in_qd[0]))))
    xp = np.full((b, h + 2 * pad, wd + 2 * pad, cin), zero, np.int64)
    xp[:, pad:pad + h, pad:pad + wd] = x
    acc = np.zeros((b, h, wd, cout), np.int64)
    for i in range(k):
        for j in range(k):
            acc += np.einsum("bhwc,oc->bhwo", xp[:, i:i + h, j:j + wd], w[:, i, j].astype(np.int64))
    assert np.abs(acc).max() < 2 ** 31
    tmp = acc.astype(np.float32) * scales.astype(np.float32)
    tmp = tmp + bias.astype(np.float32)
    if ext is not None:
        e = ext.astype(np.float32) * np.float32(ext_qd[0])
        e = e + np.float32(ext_qd[1])
        tmp = tmp + e
    if relu:
        tmp = np.maximum(tmp, np.float32(0))
    if not to_int8:
        return tmp
    q = tmp * (np.float32(1.0) / np.float32(out_qd[0]))
    q = q + (-np.float32(out_qd[1]) / np.float32(out_qd[0]))
    # round half away from zero; the +-0.5 is added in float64, where it is exact for every float32 q in range
    q64 = q.astype(np.float64)
    q64 = np.where(q64 >= 0, np.floor(q64 + 0.5), np.ceil(q64 - 0.5))
    return np.clip(q64, -128, 127).astype(np.int8)


@pytest.mark.parametrize("k,shape", [(1, (11, 12, 13, 36, 44)), (3, (2, 6, 7, 8, 5)), (5, (1, 6, 5, 4, 3))])
def test_int8_conv_against_numpy(k, shape):
    """Transforms of test/backend/test_quantization.cpp:189-191 — (0.123, 4.56), (0.078, 0.9), (0.078, -0.9) — zero point -37."""
    b, h, w, cin, cout = shape
    rng = np.random.default_rng(10 + k)
    x = rng.integers(-128, 128, (b, h, w, cin)).astype(np.int8)
    wt = rng.integers(-127, 128, (cout, k, k, cin)).astype(np.int8)
    scales = (rng.random(cout) * 0.002 + 0.0005).astype(np.float32)
    bias = rng.standard_normal(cout).astype(np.float32)
    ext = rng.integers(-128, 128, (b, h, w, cout)).astype(np.int8)
    in_qd, out_qd, ext_qd = (0.123, 4.56), (0.078, 0.9), (0.078, -0.9)
    got8 = O.int8_conv2d_forward(x, in_qd, wt, scales, bias, O.INT8, out_qd, ext, ext_qd, O.RELU)
    gotf = O.int8_conv2d_forward(x, in_qd, wt, scales, bias, O.FLOAT32, out_qd, ext, ext_qd, O.RELU)
    assert np.array_equal(gotf, numpy_int8_conv(x, in_qd, wt, scales, bias, out_qd, ext, ext_qd, True, False))
    assert np.array_equal(got8, numpy_int8_conv(x, in_qd, wt, scales, bias, out_qd, ext, ext_qd, True, True))
    # without residual, linear
    got8 = O.int8_conv2d_forward(x, in_qd, wt, scales, bias, O.INT8, out_qd, None, (1.0, 0.0), O.LINEAR)
    assert np.array_equal(got8, numpy_int8_conv(x, in_qd, wt, scales, bias, out_qd, None, None, False, True))


def test_int8_identity_transform_is_integer_convolution():
    """scale 1, shift 0 everywhere, unit channel scales, zero bias: the float output is exactly the integer convolution."""
    rng = np.random.default_rng(20)
    x = rng.integers(-5, 6, (1, 5, 5, 4)).astype(np.int8)
    wt = rng.integers(-3, 4, (3, 3, 3, 4)).astype(np.int8)
    got = O.int8_conv2d_forward(x, (1.0, 0.0), wt, np.ones(3, np.float32), np.zeros(3, np.float32), O.FLOAT32, (1.0, 0.0))
    want = direct_conv64(x.astype(np.float64), wt.astype(np.float64))
    assert np.array_equal(got.astype(np.float64), want)
    acc = O.int8_gemm_nt(O.im2row(x, 3), wt.reshape(3, -1))
    assert np.array_equal(acc.reshape(1, 5, 5, 3).astype(np.float64), want)
    same = O.quantized_scale_shift_act(acc, np.ones(3, np.float32), np.zeros(3, np.float32), O.FLOAT32, (1.0, 0.0))
    assert np.array_equal(same.reshape(got.shape), got)


def test_quantize_weights_per_first_dim():
    """src/layers/quantization.cpp:55-93: scale = 127 / max|w| per output filter, bias' = shift_in / cs * sum(q) + b."""
    rng = np.random.default_rng(21)
    w = rng.standard_normal((6, 3, 3, 5)).astype(np.float32)
    b = rng.standard_normal(6).astype(np.float32)
    q, scales, qb = O.quantize_weights(w, b, (0.05, 0.3))
    flat = w.reshape(6, -1)
    cs = np.float32(127.0) / np.abs(flat).max(axis=1)
    assert np.abs(q.reshape(6, -1)).max(axis=1).tolist() == [127] * 6  # the largest weight of every filter maps to +-127
    assert np.allclose(scales, np.float32(0.05) / cs, rtol=1e-6)
    assert np.abs(q.reshape(6, -1) - flat * cs[:, None]).max() <= 0.5 + 1e-4
    assert np.allclose(qb, np.float32(0.3) / cs * q.reshape(6, -1).sum(axis=1) + b, rtol=1e-5, atol=1e-6)
    # symmetric activations (shift 0): the bias is untouched
    _, _, qb0 = O.quantize_weights(w, b, (0.05, 0.0))
    assert np.array_equal(qb0, b)


# ---- element-wise neighbours ------------------------------------------------------------------------------------------------------
def test_unpack_input_bits():
    rng = np.random.default_rng(22)
    packed = rng.integers(0, 2 ** 32, (6, 2), dtype=np.uint64).astype(np.uint32)
    got = O.unpack_input(packed, (2, 3, 40), O.FLOAT32).reshape(6, 40)
    for i in range(6):
        for j in range(40):
            assert got[i, j] == float((int(packed[i, j // 32]) >> (j % 32)) & 1)
    assert np.array_equal(O.from_half(O.unpack_input(packed, (2, 3, 40), O.FLOAT16)).reshape(6, 40), got)


def test_add_bias_act_and_add_tensors():
    x = init_for_test((5, 7), 0.2)
    b = init_for_test((7,), 1.2)
    assert np.allclose(O.add_bias_act(x, b, O.TANH), np.tanh(x.astype(np.float64) + b), atol=1e-6)
    assert np.array_equal(O.add_bias_act(x, b, O.RELU), np.maximum(x + b, 0))
    y = init_for_test((5, 7), 2.2)
    got = O.add_tensors(y, 0.5, x, -2.0, x, 0.0, None, 0.25)
    assert np.allclose(got, 0.5 * x - 2.0 * x + 0.25 * y, atol=1e-6)
    assert np.allclose(values(O.add_tensors(O.to_half(y), 1.0, O.to_half(x), beta=1.0)), x + y, atol=4e-3)


def test_softmax_known_answer_and_invariants():
    """The literal of the reference's own test (test/backend/test_nonlinearity.cpp:22-31, tolerance 1e-4 there), rows that sum to one,
    invariance under a shift of the whole row, and a closed form for two columns (the logistic function)."""
    x = np.array([[0.1, -0.9, 2.0, 0.0], [0.3, -1.0, 0.7, -0.1]], np.float32)
    want = np.array([[0.11162444, 0.04106433, 0.74630924, 0.10100197], [0.29114823, 0.07934714, 0.43434212, 0.19516249]], np.float32)
    assert np.abs(O.softmax_forward(x) - want).max() <= 1e-6
    assert np.abs(O.as_float(O.softmax_forward(O.to_half(x))) - want).max() <= 1e-3  # the reference's fp16 tolerance
    rng = np.random.default_rng(5)
    z = (rng.standard_normal((9, 225)) * 4).astype(np.float32)
    y = O.softmax_forward(z)
    assert np.abs(y.sum(axis=1) - 1.0).max() <= 1e-5 and (y >= 0).all()
    assert np.abs(O.softmax_forward(z + np.float32(7.5)) - y).max() <= 1e-5
    exact = np.exp(z.astype(np.float64) - z.max(axis=1, keepdims=True))
    assert np.abs(y - exact / exact.sum(axis=1, keepdims=True)).max() <= 1e-6
    two = (rng.standard_normal((50, 2)) * 3).astype(np.float32)
    logistic = 1.0 / (1.0 + np.exp(-(two[:, 0].astype(np.float64) - two[:, 1])))
    assert np.abs(O.softmax_forward(two)[:, 0] - logistic).max() <= 1e-6


def test_global_average_pooling_against_numpy():
    """The reference's baseline (test/backend/test_global_pooling.cpp:23-40, tolerance 1e-6 in fp32 / 1e-4 in fp16 there) is a plain mean;
    alpha and beta follow the device form y = alpha * mean + beta * y."""
    rng = np.random.default_rng(6)
    x = rng.standard_normal((4, 13, 14, 36)).astype(np.float32)
    mean = x.astype(np.float64).mean(axis=(1, 2))
    assert np.abs(O.global_average_pooling_forward(x) - mean).max() <= 1e-6
    y0 = rng.standard_normal((4, 36)).astype(np.float32)
    assert np.abs(O.global_average_pooling_forward(x, 0.5, -2.0, y0) - (0.5 * mean - 2.0 * y0)).max() <= 1e-5
    xh = O.to_half(x)
    mean_h = O.from_half(xh).astype(np.float64).mean(axis=(1, 2))
    assert np.abs(O.as_float(O.global_average_pooling_forward(xh)) - mean_h).max() <= 1e-3
    ones = np.full((2, 4, 4, 8), 1.25, np.float32)  # 16 pixels: the reciprocal is exact
    assert np.array_equal(O.global_average_pooling_forward(ones), np.full((2, 8), 1.25, np.float32))


def test_batchnorm_inference_and_folding_agree():
    """Closed form in float64, and the identity that folding relies on: a linear layer followed by batch normalisation equals the layer
    with folded weights and bias. A dropped epsilon, a swapped mean / variance row or a wrong sign of the shift fails one of the two."""
    rng = np.random.default_rng(7)
    channels, features = 12, 20
    x = rng.standard_normal((30, features)).astype(np.float32)
    w = rng.standard_normal((channels, features)).astype(np.float32)
    b = rng.standard_normal(channels).astype(np.float32)
    gamma = (rng.standard_normal(channels) + 1.5).astype(np.float32)
    beta = rng.standard_normal(channels).astype(np.float32)
    stats = np.stack([rng.standard_normal(channels), rng.random(channels) * 1e-3]).astype(np.float32)  # tiny variances: epsilon matters
    z = O.gemm(x, w, bias=b)
    normed = O.batchnorm_inference(z, gamma, beta, stats)
    exact = (z.astype(np.float64) - stats[0]) * gamma / np.sqrt(stats[1].astype(np.float64) + 1e-6) + beta
    assert np.abs(normed - exact).max() / np.abs(exact).max() <= 1e-6
    fw, fb = O.fold_batchnorm(w, b, gamma, beta, stats)
    folded = O.gemm(x, fw, bias=fb)
    assert np.abs(folded - normed).max() / np.abs(normed).max() <= 1e-5
    relu = O.batchnorm_inference(z, gamma, beta, stats, act=O.RELU, alpha=0.5, beta=2.0, y=x[:, :channels].copy())
    assert np.abs(relu - (0.5 * np.maximum(exact, 0.0) + 2.0 * x[:, :channels])).max() / np.abs(exact).max() <= 1e-6
    none = O.batchnorm_inference(z, None, None, stats)
    assert np.abs(none - (z.astype(np.float64) - stats[0]) / np.sqrt(stats[1].astype(np.float64) + 1e-6)).max() / np.abs(none).max() <= 1e-6
    # depthwise weights: channels last
    dw = rng.standard_normal((3, 3, channels)).astype(np.float32)
    fdw, _ = O.fold_batchnorm(dw, b, gamma, beta, stats)
    scale = gamma / np.sqrt(stats[1].astype(np.float64) + 1e-6)
    assert np.abs(fdw - dw * scale).max() / np.abs(fdw).max() <= 1e-6


def attention_float64(x, heads, table=None, symmetric=False):
    """Textbook attention in float64 written from the definition: softmax(q k^T / sqrt(d) + bias) v per image and head."""
    b, h, w, c = x.shape
    parts = 2 if symmetric else 3
    e = c // parts
    d = e // heads
    xs = x.astype(np.float64).reshape(b, h * w, parts, heads, d)
    q, k, v = xs[:, :, 0], (xs[:, :, 0] if symmetric else xs[:, :, 1]), xs[:, :, parts - 1]
    s = np.einsum("bihd,bjhd->bhij", q, k) / np.sqrt(d)
    if table is not None:
        r = (table.shape[1] - 1) // 2
        rows, cols = np.divmod(np.arange(h * w), w)
        dh = np.clip(rows[None, :] - rows[:, None], -r, r) + r  # [query, key]
        dw = np.clip(cols[None, :] - cols[:, None], -r, r) + r
        s = s + table.astype(np.float64)[:, dh, dw][None]
    s = np.exp(s - s.max(axis=-1, keepdims=True))
    p = s / s.sum(axis=-1, keepdims=True)
    return np.einsum("bhij,bjhd->bihd", p, v).reshape(b, h, w, e)


def test_rmsnorm_closed_form_and_invariants():
    """Float64 closed form; rows leave with unit root-mean-square when gamma is absent; scaling a row by a positive constant changes
    nothing (up to the 1e-6 in the denominator); a dropped square root, a sum instead of a mean or gamma applied twice fails the first."""
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((13, 96)) * 3).astype(np.float32)
    g = (rng.standard_normal(96) + 1.0).astype(np.float32)
    rms = np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    assert np.abs(O.rmsnorm_forward(x, g) - g * x / (1e-6 + rms)).max() <= 2e-6 * np.abs(g).max() * 4
    plain = O.rmsnorm_forward(x)
    assert np.abs(np.sqrt((plain.astype(np.float64) ** 2).mean(axis=1)) - 1.0).max() <= 1e-5
    assert np.abs(O.rmsnorm_forward(x * np.float32(8.0)) - plain).max() <= 1e-5
    xh = O.to_half(x)
    rms_h = np.sqrt((O.from_half(xh).astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    assert np.abs(O.as_float(O.rmsnorm_forward(xh)) - O.from_half(xh) / rms_h).max() <= 4e-3
    assert np.array_equal(O.rmsnorm_forward(np.zeros((2, 8), np.float32)), np.zeros((2, 8), np.float32))  # 0 / (1e-6 + 0)


@pytest.mark.parametrize("symmetric", [False, True])
def test_attention_against_float64(symmetric):
    rng = np.random.default_rng(12)
    parts = 2 if symmetric else 3
    x = rng.standard_normal((2, 4, 6, parts * 48)).astype(np.float32)
    table = rng.standard_normal((3, 5, 8)).astype(np.float32)  # r = 3: offsets up to +-5 are clamped to +-2
    for t in (None, table):
        want = attention_float64(x, 3, t, symmetric)
        assert np.abs(O.multi_head_attention_forward(x, 3, t, symmetric) - want).max() <= 1e-5
    xh, th = O.to_half(x), O.to_half(table)
    want = attention_float64(O.from_half(xh), 3, O.from_half(th), symmetric)
    assert np.abs(O.as_float(O.multi_head_attention_forward(xh, 3, th, symmetric)) - want).max() <= 4e-3


def test_attention_special_cases():
    """(1) Equal keys give uniform attention: every output is the mean of the values. (2) A table that is hugely negative everywhere
    except at one offset makes every token copy the value of the neighbour at that offset (tokens whose neighbour is off the board see
    only clamped offsets and are skipped): pins the sign convention key - query, the row / column order of the table and the clamping."""
    rng = np.random.default_rng(13)
    b, h, w, heads, d = 2, 5, 6, 2, 8
    e = heads * d
    x = rng.standard_normal((b, h, w, 3, heads, d)).astype(np.float32)
    x[:, :, :, 1] = x[0, 0, 0, 1]  # all keys equal
    y = O.multi_head_attention_forward(x.reshape(b, h, w, 3 * e), heads)
    mean_v = x[:, :, :, 2].astype(np.float64).mean(axis=(1, 2), keepdims=True)
    assert np.abs(y.reshape(b, h, w, heads, d) - mean_v).max() <= 1e-6
    x = rng.standard_normal((b, h, w, 3 * e)).astype(np.float32)
    table = np.full((heads, 7, 8), -1.0e4, np.float32)  # r = 4 -> range 3
    table[:, 3 + 1, 3 - 2] = 0.0  # key one row below, two columns to the left of the query
    y = O.multi_head_attention_forward(x, heads, table).reshape(b, h, w, e)
    v = x.reshape(b, h, w, 3, e)[:, :, :, 2]
    assert np.abs(y[:, :h - 1, 2:] - v[:, 1:, :w - 2]).max() <= 1e-6
