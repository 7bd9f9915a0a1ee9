"""The CPU oracle against the reference itself: (1) the committed fixtures that the reference's compiled CPU backend produced
(tests/golden/make_fixtures.py) — runs everywhere; (2) the compiled reference library oracle/_ref where it has been built — bit for bit
on fresh random inputs, in fp32 and fp16, including the reference's split of K at 1024."""
import numpy as np
import pytest

import oracle as O
from util import mismatches, random_tensor

needs_ref = pytest.mark.skipif(O.reference() is None, reason="oracle/_ref (compiled reference CPU backend) is not built here")


@pytest.mark.parametrize("tag", ["f32", "f16"])
def test_fixtures_winograd(golden, tag):
    g = golden
    assert mismatches(O.winograd_weight_transform(g["wg_w_" + tag]), g["wg_wm_" + tag]) == 0
    assert mismatches(O.winograd_weight_transform(g["wg_w_" + tag], True), g["wg_wm_inverted_" + tag]) == 0
    assert mismatches(O.winograd_input_transform(g["wg_x_" + tag]), g["wg_v_" + tag]) == 0
    assert mismatches(O.gemm(g["wg_v_" + tag], g["wg_wm_" + tag]), g["wg_m_" + tag]) == 0
    y = O.winograd_output_transform(g["wg_m_" + tag], (2, 9, 11, 13), g["wg_bias_" + tag], g["wg_ext_" + tag], O.RELU)
    assert mismatches(y, g["wg_y_relu_" + tag]) == 0
    assert mismatches(O.winograd_output_transform(g["wg_m_" + tag], (2, 9, 11, 13), g["wg_bias_" + tag]), g["wg_y_linear_" + tag]) == 0


@pytest.mark.parametrize("tag", ["f32", "f16"])
def test_fixtures_gemm_and_conv(golden, tag):
    g = golden
    d = O.gemm(g["ge_a_" + tag], g["ge_b_" + tag], alpha=1.1, beta=0.1, C=g["ge_c_" + tag], bias=g["ge_bias_" + tag], act=O.RELU)
    assert mismatches(d, g["ge_d_" + tag]) == 0
    assert mismatches(O.gemm(g["gk_a_" + tag], g["gk_b_" + tag]), g["gk_d_" + tag]) == 0  # K = 1200 > 1024: two K tiles
    assert mismatches(O.im2row(g["cv_x_" + tag], 5), g["cv_rows_" + tag]) == 0
    y = O.conv2d_forward(g["cv_x_" + tag], g["cv_w_" + tag], g["cv_bias_" + tag], g["cv_add_" + tag], O.RELU)
    assert mismatches(y, g["cv_y_" + tag]) == 0
    got = O.add_bias_act(g["cv_x_" + tag], None, O.LINEAR)
    assert mismatches(got, g["cv_x_" + tag]) == 0


def test_fixtures_unpack_and_convert(golden):
    g = golden
    assert mismatches(O.unpack_input(g["up_packed"], (3, 5, 40), O.FLOAT32), g["up_f32"]) == 0
    assert mismatches(O.unpack_input(g["up_packed"], (3, 5, 40), O.FLOAT16), g["up_f16"]) == 0
    ours, theirs = O.to_half(g["cvt_src"]), g["cvt_f16"]
    # the reference's vector narrowing (vcvtps2ph, round toward zero) saturates to the largest finite half where the scalar table method
    # that the oracle restates (src/backend/cpu/fp16.hpp:61-68) gives infinity; everywhere else the two agree bit for bit
    finite = np.abs(g["cvt_src"]) < 65504.0
    assert mismatches(ours[finite], theirs[finite]) == 0


@needs_ref
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_reference_bit_exact(dtype):
    ref = O.reference()
    rng = np.random.default_rng(0)
    for shape, cout in (((3, 9, 11, 35), 21), ((3, 7, 11, 35), 35), ((1, 15, 15, 32), 16)):
        c = shape[3]
        w = random_tensor(rng, (cout, 3, 3, c), dtype)
        x = random_tensor(rng, shape, dtype)
        assert mismatches(O.winograd_weight_transform(w), ref.winograd_weight_transform(w)) == 0
        assert mismatches(O.winograd_weight_transform(w, True), ref.winograd_weight_transform(w, True)) == 0
        v = O.winograd_input_transform(x)
        assert mismatches(v, ref.winograd_input_transform(x)) == 0
        u = O.winograd_weight_transform(w)
        m = O.gemm(v, u)
        assert mismatches(m, ref.gemm_batched(v, u)) == 0
        out_shape = shape[:3] + (cout,)
        bias = random_tensor(rng, (cout,), dtype)
        ext = random_tensor(rng, out_shape, dtype)
        for act in (O.LINEAR, O.RELU, O.SIGMOID, O.TANH):
            assert mismatches(O.winograd_output_transform(m, out_shape, bias, ext, act), ref.winograd_output_transform(m, out_shape, bias, ext, act)) == 0
        if cout % 16 == 0:  # bias-less calls are only well defined in the reference for channel counts that skip its scalar tail loop
            assert mismatches(O.winograd_output_transform(m, out_shape), ref.winograd_output_transform(m, out_shape)) == 0


@needs_ref
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_reference_gemm_and_conv_bit_exact(dtype):
    ref = O.reference()
    rng = np.random.default_rng(1)
    for ops in ("nn", "nt", "tn", "tt"):
        A = random_tensor(rng, (30, 40) if ops[0] == "n" else (40, 30), dtype)
        Bm = random_tensor(rng, (40, 20) if ops[1] == "n" else (20, 40), dtype)
        assert mismatches(O.gemm(A, Bm, ops[0], ops[1], alpha=1.1), ref.gemm_ex(A, Bm, ops[0], ops[1], alpha=1.1)) == 0
    A = random_tensor(rng, (50, 2304), dtype, 0.1)
    Bm = random_tensor(rng, (20, 2304), dtype, 0.1)
    bias = random_tensor(rng, (20,), dtype)
    C = random_tensor(rng, (50, 20), dtype)
    got = O.gemm(A, Bm, alpha=0.7, beta=1.0, C=C, bias=bias, act=O.RELU)
    assert mismatches(got, ref.gemm_ex(A, Bm, alpha=0.7, beta=1.0, C=C, bias=bias, act=O.RELU)) == 0
    x = random_tensor(rng, (2, 7, 6, 128), dtype)
    w = random_tensor(rng, (24, 5, 5, 128), dtype, 0.1)
    b = random_tensor(rng, (24,), dtype)
    add = random_tensor(rng, (2, 7, 6, 24), dtype)
    assert mismatches(O.conv2d_forward(x, w, b, add, O.SIGMOID), ref.conv2d_forward(x, w, b, add, O.SIGMOID)) == 0
    assert mismatches(O.im2row(x, 5), ref.im2row(x, 5)) == 0
    bb = random_tensor(rng, (128,), dtype)
    assert mismatches(O.add_bias_act(x, bb, O.RELU), ref.add_bias_act(x, bb, O.RELU)) == 0


@needs_ref
def test_reference_network_bit_exact():
    """A 2-block network end to end: the oracle engine and the reference engine of oracle/cpu_net.py agree bit for bit."""
    from oracle.cpu_net import CpuResNet
    from minml_amd.resnet import make_input, make_parameters

    params = make_parameters(3, 32, 48, 2)
    x = make_input(3, 3, 15, 32)
    for conv in (lambda a: a, O.to_half):
        ps = [(conv(w), conv(b)) for (w, b) in params]
        a = CpuResNet(ps, 2, "oracle").forward(conv(x))
        b = CpuResNet(ps, 2, "reference").forward(conv(x))
        assert mismatches(a, b) == 0


@pytest.mark.parametrize("tag", ["f32", "f16"])
def test_fixtures_heads(golden, tag):
    g = golden
    assert mismatches(O.softmax_forward(g["sm_x_" + tag]), g["sm_y_" + tag]) == 0
    assert mismatches(O.softmax_forward(g["sm3_x_" + tag]), g["sm3_y_" + tag]) == 0
    assert mismatches(O.global_average_pooling_forward(g["gap_x_" + tag]), g["gap_y_" + tag]) == 0
    assert mismatches(O.global_average_pooling_forward(g["gap7_x_" + tag]), g["gap7_y_" + tag]) == 0  # scalar kernel only (fp16), 4 + 3 (fp32)


def test_fixtures_fold_batchnorm(golden):
    g = golden
    for key in ("fd", "fd3"):
        w, b = O.fold_batchnorm(g[key + "_w"], g[key + "_b"], g[key + "_gamma"], g[key + "_beta"], g[key + "_stats"])
        assert mismatches(w, g[key + "_w_out"]) == 0 and mismatches(b, g[key + "_b_out"]) == 0


@needs_ref
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_reference_heads_bit_exact(dtype):
    ref = O.reference()
    rng = np.random.default_rng(2)
    for shape in ((7, 225), (5, 3), (4, 1), (3, 1000), (2, 64)):
        x = random_tensor(rng, shape, dtype, 3.0)
        assert mismatches(O.softmax_forward(x), ref.softmax_forward(x)) == 0
    for shape in ((3, 13, 14, 136), (2, 15, 15, 256), (1, 1, 1, 8), (2, 5, 6, 7), (2, 3, 3, 37), (1, 4, 4, 3)):
        x = random_tensor(rng, shape, dtype)
        assert mismatches(O.global_average_pooling_forward(x), ref.global_average_pooling_forward(x)) == 0
    if dtype == "float32":
        for wshape in ((16, 3, 3, 8), (10, 33), (3, 3, 12)):
            channels = wshape[-1] if len(wshape) == 3 else wshape[0]
            w, b = random_tensor(rng, wshape, dtype), random_tensor(rng, (channels,), dtype)
            gamma, beta = random_tensor(rng, (channels,), dtype), random_tensor(rng, (channels,), dtype)
            stats = np.stack([rng.standard_normal(channels), rng.random(channels) + 0.05]).astype(np.float32)
            ours, theirs = O.fold_batchnorm(w, b, gamma, beta, stats), ref.fold_batchnorm(w, b, gamma, beta, stats)
            assert mismatches(ours[0], theirs[0]) == 0 and mismatches(ours[1], theirs[1]) == 0


def test_fixtures_transformer_pieces(golden):
    g = golden
    assert mismatches(O.rmsnorm_forward(g["rms_x"], g["rms_g"]), g["rms_y"]) == 0
    assert mismatches(O.rmsnorm_forward(g["rms_x"]), g["rms_y_plain"]) == 0
    assert mismatches(O.multi_head_attention_forward(g["mha_x"], 4, g["mha_table"]), g["mha_y"]) == 0
    assert mismatches(O.multi_head_attention_forward(g["mha_x"], 4), g["mha_y_plain"]) == 0
    assert mismatches(O.multi_head_attention_forward(g["mha_sym_x"], 2, None, True), g["mha_sym_y"]) == 0


@needs_ref
def test_reference_transformer_pieces_bit_exact():
    """fp32 only: the reference's RMS normalisation has no other branch and its attention reads the score matrix as fp32 whatever the type."""
    ref = O.reference()
    rng = np.random.default_rng(3)
    for shape in ((7, 256), (3, 15, 15, 64), (5, 33), (2, 1)):
        x, gamma = random_tensor(rng, shape, "float32", 2.0), random_tensor(rng, shape[-1:], "float32")
        assert mismatches(O.rmsnorm_forward(x, gamma), ref.rmsnorm_forward(x, gamma)) == 0
        assert mismatches(O.rmsnorm_forward(x), ref.rmsnorm_forward(x)) == 0
    for (b, h, w, heads, d, r) in ((2, 15, 15, 2, 32, 8), (1, 6, 5, 3, 24, 3), (2, 3, 3, 1, 7, 1)):
        x = random_tensor(rng, (b, h, w, 3 * heads * d), "float32")
        size = 2 * r - 1
        table = random_tensor(rng, (heads, size, (size + 3) // 4 * 4), "float32")
        assert mismatches(O.multi_head_attention_forward(x, heads, table), ref.multi_head_attention_forward(x, heads, table)) == 0
        assert mismatches(O.multi_head_attention_forward(x, heads), ref.multi_head_attention_forward(x, heads)) == 0
    x = random_tensor(rng, (2, 5, 5, 2 * 4 * 16), "float32")
    assert mismatches(O.multi_head_attention_forward(x, 4, None, True), ref.multi_head_attention_forward(x, 4)) == 0
