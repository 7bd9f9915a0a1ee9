"""GEMM entry points and fused convolution on the GPU against the CPU oracle, through the C-ABI.

Tolerances (max-abs relative error per result tensor, as stated for this path): fp32 1e-4, fp16 1e-2. The oracle accumulates like the
reference (sequential fused multiply-adds, K split at 1024 with a rounded intermediate store); the MFMA kernels accumulate the whole K
extent in fp32, so results agree to rounding, not bit for bit. im2row is byte movement and is compared exactly."""
import numpy as np
import pytest

import oracle as O
from minml_amd import core as ml
from util import TOL, max_abs_rel, mean_abs_diff, mismatches, random_tensor, init_for_test, storage

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("ops", ["nn", "nt", "tn", "tt"])
def test_gemm_all_ops(ctx, dtype, ops):
    """test/backend/test_gemms.cpp:178-374: 23 x 45 x 67, alpha = 1.1, beta = 0.1, mean-abs-diff <= 1e-4 (fp16: 1e-2)."""
    M, N, K = 23, 45, 67
    A = storage(init_for_test((M, K) if ops[0] == "n" else (K, M), 0.0), dtype)
    Bm = storage(init_for_test((K, N) if ops[1] == "n" else (N, K), 1.0), dtype)
    C = storage(init_for_test((M, N), 2.0), dtype)
    dC = ml.toDevice(ctx, C)
    ml.gemm(ctx, ops[0], ops[1], dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm), 1.1, 0.1)
    want = O.gemm(A, Bm, ops[0], ops[1], alpha=1.1, beta=0.1, C=C)
    assert mean_abs_diff(dC.copyToHost(ctx), want) <= (1e-4 if dtype == "float32" else 1e-2)
    assert max_abs_rel(dC.copyToHost(ctx), want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape", [(36, 48, 21, 35), (5, 77, 33, 40), (3, 300, 256, 256), (2, 130, 70, 264), (36, 16 * 8, 256, 32), (1, 1, 1, 8),
                                   (2, 129, 129, 1032)])
def test_gemm_batched_nt(ctx, dtype, shape):
    """The Winograd product M[i] = V[i] * U[i]^T: ragged M and N, K that is no multiple of the pipeline step, K > 1024."""
    bt, M, N, K = shape
    rng = np.random.default_rng(sum(shape))
    A = random_tensor(rng, (bt, M, K), dtype, 0.5)
    Bm = random_tensor(rng, (bt, N, K), dtype, 0.5)
    dC = ml.Tensor((bt, M, N), dtype)
    dC.setall(ctx, float("nan"))  # beta = 0 must not read C (the reference's workspace is uninitialised)
    ml.gemmBatched(ctx, "n", "t", dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm), 1.0, 0.0)
    got = dC.copyToHost(ctx)
    assert np.isfinite(O.as_float(got)).all()
    assert max_abs_rel(got, O.gemm(A, Bm)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape", [(36, 1000, 256), (36, 1027, 200), (300, 128, 64), (1, 33001, 128), (36, 900, 8), (7, 5000, 384), (257, 1, 256)])
def test_gemm_batched_nt_streaming_shapes(ctx, dtype, shape):
    """Rows of K of exactly 512 bytes (256 halfs / 128 floats) and at least 256 row blocks: the shapes of the Winograd product in the
    benchmark networks, which take the persistent streaming kernel. Ragged last row block, ragged and tiny N, more column slices than
    two, runs of row blocks that cross from one matrix into the next, one-row matrices."""
    bt, M, N = shape
    K = 256 if dtype == "float16" else 128
    rng = np.random.default_rng(sum(shape))
    A = random_tensor(rng, (bt, M, K), dtype, 0.5)
    Bm = random_tensor(rng, (bt, N, K), dtype, 0.5)
    dC = ml.Tensor((bt, M, N), dtype)
    dC.setall(ctx, float("nan"))
    ml.gemmBatched(ctx, "n", "t", dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm), 1.0, 0.0)
    got = dC.copyToHost(ctx)
    assert np.isfinite(O.as_float(got)).all()
    assert max_abs_rel(got, O.gemm(A, Bm)) <= TOL[dtype]
    # shared B operand (rank 2) through the same kernel
    dC.setall(ctx, float("nan"))
    ml.gemmBatched(ctx, "n", "t", dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm[0]), 1.0, 0.0)
    assert max_abs_rel(dC.copyToHost(ctx), O.gemm(A, Bm[0])) <= TOL[dtype]


@pytest.mark.parametrize("dtype,K", [("float16", 384), ("float16", 64), ("float16", 128), ("float32", 32), ("float32", 64)])
@pytest.mark.parametrize("shape", [(36, 1000, 384), (9, 4100, 72), (36, 950, 128)])
def test_gemm_batched_nt_streaming_other_row_lengths(ctx, dtype, K, shape):
    """The same kernel for K rows of 128, 256 and 768 bytes (Winograd products at 64, 128 and 384 channels)."""
    bt, M, N = shape
    rng = np.random.default_rng(sum(shape) + K)
    A = random_tensor(rng, (bt, M, K), dtype, 0.5)
    Bm = random_tensor(rng, (bt, N, K), dtype, 0.5)
    dC = ml.Tensor((bt, M, N), dtype)
    dC.setall(ctx, float("nan"))
    ml.gemmBatched(ctx, "n", "t", dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm), 1.0, 0.0)
    assert max_abs_rel(dC.copyToHost(ctx), O.gemm(A, Bm)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_gemm_batched_more_matrices_than_one_grid_dimension_holds(ctx, dtype):
    """65535 + 5 tiny products in one call (the reference's interface has no limit on the batch); with beta and a broadcast B operand."""
    rng = np.random.default_rng(11)
    bt, M, N, K = 65540, 3, 4, 8
    A = random_tensor(rng, (bt, M, K), dtype, 0.5)
    Bm = random_tensor(rng, (bt, N, K), dtype, 0.5)
    C = random_tensor(rng, (bt, M, N), dtype)
    dC = ml.toDevice(ctx, C)
    ml.gemmBatched(ctx, "n", "t", dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm), 1.0, 1.0)
    assert max_abs_rel(dC.copyToHost(ctx), O.gemm(A, Bm, beta=1.0, C=C)) <= TOL[dtype]
    dC.setall(ctx, float("nan"))
    ml.gemmBatched(ctx, "n", "t", dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm[7]), 1.0, 0.0)
    assert max_abs_rel(dC.copyToHost(ctx), O.gemm(A, Bm[7])) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_gemm_batched_broadcast_and_beta(ctx, dtype):
    rng = np.random.default_rng(5)
    A = random_tensor(rng, (4, 50, 24), dtype)
    Bm = random_tensor(rng, (30, 24), dtype)  # rank 2: broadcast (src/backend/cpu/gemm/gemm.cpp:18-29)
    C = random_tensor(rng, (4, 50, 30), dtype)
    dC = ml.toDevice(ctx, C)
    ml.gemmBatched(ctx, "n", "t", dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm), 0.5, 2.0)
    assert max_abs_rel(dC.copyToHost(ctx), O.gemm(A, Bm, alpha=0.5, beta=2.0, C=C)) <= TOL[dtype]
    # transposed batched forms (used by the reference's training path) run on the generic kernel
    At = random_tensor(rng, (3, 24, 50), dtype)
    Bn = random_tensor(rng, (3, 24, 30), dtype)
    dC = ml.Tensor((3, 50, 30), dtype)
    ml.gemmBatched(ctx, "t", "n", dC, ml.toDevice(ctx, At), ml.toDevice(ctx, Bn), 1.0, 0.0)
    assert max_abs_rel(dC.copyToHost(ctx), O.gemm(At, Bn, "t", "n")) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("act", ["linear", "relu", "sigmoid", "tanh"])
def test_gemm_ex_epilogue(ctx, dtype, act):
    """D = act(alpha A B^T + bias + beta C), C distinct from D (test/backend/test_gemms.cpp gemm_ex, src/backend/cpu/gemm/gemm.cpp:66-83)."""
    rng = np.random.default_rng(6)
    for (M, N, K) in ((123, 45, 72), (23, 45, 67), (500, 1, 256), (64, 128, 2304), (257, 136, 40)):
        A = random_tensor(rng, (M, K), dtype, 0.3)
        Bm = random_tensor(rng, (N, K), dtype, 0.3)
        C = random_tensor(rng, (M, N), dtype)
        bias = random_tensor(rng, (N,), dtype)
        dD = ml.Tensor((M, N), dtype)
        ml.gemm_ex(ctx, dD, 1.1, "n", ml.toDevice(ctx, A), "t", ml.toDevice(ctx, Bm), 0.1, ml.toDevice(ctx, C), ml.toDevice(ctx, bias), act)
        want = O.gemm(A, Bm, alpha=1.1, beta=0.1, C=C, bias=bias, act=ml.act_of(act))
        assert max_abs_rel(dD.copyToHost(ctx), want) <= TOL[dtype]
        # in place (C is D) and without bias
        dD = ml.toDevice(ctx, C)
        ml.gemm_ex(ctx, dD, 1.0, "n", ml.toDevice(ctx, A), "t", ml.toDevice(ctx, Bm), 1.0, dD, None, act)
        want = O.gemm(A, Bm, alpha=1.0, beta=1.0, C=C, act=ml.act_of(act))
        assert max_abs_rel(dD.copyToHost(ctx), want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("k_bytes", [128, 256, 512, 768])
@pytest.mark.parametrize("M,N", [(33001, 256), (32800, 100), (40000, 64), (33000, 28), (32769, 384)])
def test_gemm_ex_streaming_shapes(ctx, dtype, k_bytes, M, N):
    """gemm_ex with short K rows and many rows of A (1x1 convolutions, dense heads): the persistent streaming kernel with the fused
    epilogue. All three wavefront layouts (N > 128, > 64, <= 64), column counts that are no multiple of 32, a ragged last row block,
    more than 256 columns; bias + beta * C + ReLU, and a sigmoid in place. 768-byte rows take this kernel in fp16 (384 channels) and the
    tile engine in fp32."""
    K = k_bytes // (2 if dtype == "float16" else 4)
    rng = np.random.default_rng(M + N + k_bytes)
    A = random_tensor(rng, (M, K), dtype, 0.3)
    Bm = random_tensor(rng, (N, K), dtype, 0.3)
    C = random_tensor(rng, (M, N), dtype)
    bias = random_tensor(rng, (N,), dtype)
    dA, dB = ml.toDevice(ctx, A), ml.toDevice(ctx, Bm)
    dD = ml.Tensor((M, N), dtype)
    dD.setall(ctx, float("nan"))
    ml.gemm_ex(ctx, dD, 1.1, "n", dA, "t", dB, 0.5, ml.toDevice(ctx, C), ml.toDevice(ctx, bias), "relu")
    want = O.gemm(A, Bm, alpha=1.1, beta=0.5, C=C, bias=bias, act=O.RELU)
    assert max_abs_rel(dD.copyToHost(ctx), want) <= TOL[dtype]
    dD = ml.toDevice(ctx, C)
    ml.gemm_ex(ctx, dD, 1.0, "n", dA, "t", dB, 1.0, dD, None, "sigmoid")
    assert max_abs_rel(dD.copyToHost(ctx), O.gemm(A, Bm, alpha=1.0, beta=1.0, C=C, act=O.SIGMOID)) <= TOL[dtype]
    # epilogues that read nothing per element (no C): in fp16 they are finished in registers and stored 16 bytes per lane when the
    # width allows it (N = 100 and 28 do not: the functor's run-time form)
    dbias = ml.toDevice(ctx, bias)
    for alpha, use_bias, act in ((0.9, True, "relu"), (1.0, True, "linear"), (0.9, False, "linear")):
        dD = ml.Tensor((M, N), dtype)
        dD.setall(ctx, float("nan"))
        ml.gemm_ex(ctx, dD, alpha, "n", dA, "t", dB, 0.0, None, dbias if use_bias else None, act)
        want = O.gemm(A, Bm, alpha=alpha, bias=bias if use_bias else None, act=ml.act_of(act))
        assert max_abs_rel(dD.copyToHost(ctx), want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("N", [192, 320, 384, 448, 130, 576])
def test_gemm_ex_tile_engine_widths(ctx, dtype, N):
    """K rows of 1024 bytes take the direct-to-LDS tile engine. Its tile width follows N: 256 x 192 tiles for multiples of 192 that are no
    multiples of 256 (wavefront sub-tiles of 96 columns, whose epilogue walks the slab in two parts), 256 columns on wide tiles plus the
    rest on a narrower width for 320 / 448, a ragged width (130: the element-wise epilogue), and a ragged last row tile everywhere."""
    K = 1024 // (2 if dtype == "float16" else 4)
    M = 1000
    rng = np.random.default_rng(N)
    A = random_tensor(rng, (M, K), dtype, 0.3)
    Bm = random_tensor(rng, (N, K), dtype, 0.3)
    C = random_tensor(rng, (M, N), dtype)
    bias = random_tensor(rng, (N,), dtype)
    dA, dB = ml.toDevice(ctx, A), ml.toDevice(ctx, Bm)
    dD = ml.Tensor((M, N), dtype)
    dD.setall(ctx, float("nan"))
    ml.gemm_ex(ctx, dD, 1.1, "n", dA, "t", dB, 0.5, ml.toDevice(ctx, C), ml.toDevice(ctx, bias), "relu")
    assert max_abs_rel(dD.copyToHost(ctx), O.gemm(A, Bm, alpha=1.1, beta=0.5, C=C, bias=bias, act=O.RELU)) <= TOL[dtype]
    dD.setall(ctx, float("nan"))
    ml.gemm_ex(ctx, dD, 1.0, "n", dA, "t", dB, 0.0, None, None, "linear")
    assert max_abs_rel(dD.copyToHost(ctx), O.gemm(A, Bm)) <= TOL[dtype]


@pytest.mark.parametrize("tag,dtype", [("f32", "float32"), ("f16", "float16")])
def test_reference_fixtures(ctx, golden, tag, dtype):
    g = golden
    dD = ml.Tensor((23, 45), dtype)
    ml.gemm_ex(ctx, dD, 1.1, "n", ml.toDevice(ctx, g["ge_a_" + tag]), "t", ml.toDevice(ctx, g["ge_b_" + tag]), 0.1, ml.toDevice(ctx, g["ge_c_" + tag]),
               ml.toDevice(ctx, g["ge_bias_" + tag]), "relu")
    assert max_abs_rel(dD.copyToHost(ctx), g["ge_d_" + tag]) <= TOL[dtype]
    dD = ml.Tensor((9, 7), dtype)
    ml.gemm_ex(ctx, dD, 1.0, "n", ml.toDevice(ctx, g["gk_a_" + tag]), "t", ml.toDevice(ctx, g["gk_b_" + tag]), 0.0, None, None, "linear")
    assert max_abs_rel(dD.copyToHost(ctx), g["gk_d_" + tag]) <= TOL[dtype]
    rows = ml.Tensor((2 * 7 * 6, 25 * 8), dtype)
    ml.im2row(ctx, rows, ml.toDevice(ctx, g["cv_x_" + tag]), 5)
    assert mismatches(rows.copyToHost(ctx), g["cv_rows_" + tag]) == 0
    dy = ml.Tensor((2, 7, 6, 12), dtype)
    ml.convolutionImplicitGemmForward(ctx, ml.toDevice(ctx, g["cv_x_" + tag]), ml.toDevice(ctx, g["cv_w_" + tag]), dy, ml.toDevice(ctx, g["cv_bias_" + tag]),
                                      ml.toDevice(ctx, g["cv_add_" + tag]), "relu")
    assert max_abs_rel(dy.copyToHost(ctx), g["cv_y_" + tag]) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16", "int8"])
@pytest.mark.parametrize("shape,k", [((2, 7, 6, 16), 5), ((3, 5, 4, 3), 3), ((1, 19, 19, 8), 5), ((2, 6, 5, 7), 3), ((4, 12, 14, 32), 3)])
def test_im2row_exact(ctx, dtype, shape, k):
    """test/backend/test_gemm_conv.cpp:68-150: EXPECT_EQ(diff, 0)."""
    rng = np.random.default_rng(k + shape[3])
    x = rng.integers(-128, 128, shape).astype(np.int8) if dtype == "int8" else random_tensor(rng, shape, dtype)
    rows = ml.Tensor((shape[0] * shape[1] * shape[2], k * k * shape[3]), dtype)
    ml.im2row(ctx, rows, ml.toDevice(ctx, x), k)
    assert mismatches(rows.copyToHost(ctx), O.im2row(x, k)) == 0
    if dtype == "int8":  # padding with a zero point: same as shifting the data, gathering with zeros, shifting back
        ml.im2row(ctx, rows, ml.toDevice(ctx, x), k, False, -37)
        shifted = (x.astype(np.int16) + 37)
        want = O.im2row(shifted.astype(np.float32), k).astype(np.int16) - 37
        assert mismatches(rows.copyToHost(ctx), want.astype(np.int8)) == 0


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape,cout,k", [((2, 7, 6, 16), 24, 5), ((2, 9, 9, 32), 40, 3), ((3, 5, 7, 24), 8, 1), ((2, 6, 5, 7), 9, 3),
                                          ((1, 19, 19, 64), 64, 5), ((2, 19, 19, 64), 64, 1), ((1, 19, 19, 128), 128, 3), ((2, 15, 15, 256), 1, 1)])
def test_fused_convolution(ctx, dtype, shape, cout, k):
    """hip_convolution_implicit_gemm_forward and the reference's explicit sequence (im2row + gemm_ex) against explicit_gemm_forward of the
    oracle, with the fused bias + residual + ReLU epilogue (test/backend/test_conv2D.cpp:204-248,332-368,437-578)."""
    rng = np.random.default_rng(cout + k)
    b, h, w, cin = shape
    x = random_tensor(rng, shape, dtype)
    wt = random_tensor(rng, (cout, k, k, cin), dtype, (2.0 / (k * k * cin)) ** 0.5)
    bias = random_tensor(rng, (cout,), dtype)
    add = random_tensor(rng, (b, h, w, cout), dtype)
    dx, dw, db, da = ml.toDevice(ctx, x), ml.toDevice(ctx, wt), ml.toDevice(ctx, bias), ml.toDevice(ctx, add)
    want = O.conv2d_forward(x, wt, bias, add, O.RELU)
    dy = ml.Tensor((b, h, w, cout), dtype)
    ml.convolutionImplicitGemmForward(ctx, dx, dw, dy, db, da, "relu")
    assert max_abs_rel(dy.copyToHost(ctx), want) <= TOL[dtype]
    ws = ml.Tensor((max(1, b * h * w * k * k * cin),), dtype)
    dy2 = ml.Tensor((b, h, w, cout), dtype)
    ml.explicit_gemm_forward(ctx, dx, dy2, dw, db, ws, "relu", da)
    assert max_abs_rel(dy2.copyToHost(ctx), want) <= TOL[dtype]
    # no bias, no residual, linear
    ml.convolutionImplicitGemmForward(ctx, dx, dw, dy, None, None, "linear")
    assert max_abs_rel(dy.copyToHost(ctx), O.conv2d_forward(x, wt)) <= TOL[dtype]


def test_conv_sweep_config4_shapes(ctx):
    """19x19 boards, fp16, channel widths {64,128,256,384}, kernels 1 / 3 / 5 with bias + ReLU + residual, at a batch the oracle finishes."""
    rng = np.random.default_rng(44)
    for c in (64, 128, 256, 384):
        for k in (1, 3, 5):
            x = random_tensor(rng, (2, 19, 19, c), "float16")
            wt = random_tensor(rng, (c, k, k, c), "float16", (2.0 / (k * k * c)) ** 0.5)
            bias = random_tensor(rng, (c,), "float16", 0.01)
            add = random_tensor(rng, (2, 19, 19, c), "float16")
            dy = ml.Tensor((2, 19, 19, c), "float16")
            ml.convolutionImplicitGemmForward(ctx, ml.toDevice(ctx, x), ml.toDevice(ctx, wt), dy, ml.toDevice(ctx, bias), ml.toDevice(ctx, add), "relu")
            assert max_abs_rel(dy.copyToHost(ctx), O.conv2d_forward(x, wt, bias, add, O.RELU)) <= 1e-2


def test_convolution_linearity_at_full_size(ctx):
    """Size-independent property at config 4's full size (B = 512, 19x19, 128 channels, 5x5, fp32 so that sums are comparable):
    conv(x1 + x2) = conv(x1) + conv(x2) to rounding, and shifting the batch shifts the output."""
    rng = np.random.default_rng(45)
    shape = (512, 19, 19, 128)
    x1 = (rng.integers(-4, 5, shape)).astype(np.float32)  # small integers: products and sums are exact in fp32
    x2 = (rng.integers(-4, 5, shape)).astype(np.float32)
    wt = rng.integers(-2, 3, (128, 5, 5, 128)).astype(np.float32)
    dw = ml.toDevice(ctx, wt)
    outs = []
    for x in (x1, x2, x1 + x2):
        dy = ml.Tensor(shape[:3] + (128,), "float32")
        ml.convolutionImplicitGemmForward(ctx, ml.toDevice(ctx, x), dw, dy, None, None, "linear")
        outs.append(dy.copyToHost(ctx))
    assert np.array_equal(outs[0] + outs[1], outs[2])
    sample = O.conv2d_forward(x1[100:101], wt)
    assert np.array_equal(outs[0][100:101], sample)


@pytest.mark.parametrize("channels,k", [(64, 3), (64, 5), (128, 3)])
@pytest.mark.parametrize("shape", [(1, 19, 19), (2, 7, 5), (3, 30, 9), (64, 19, 19), (5, 1, 40), (2, 3, 100), (1, 2, 130)])
def test_narrow_convolution(ctx, shape, channels, k):
    """Convolutions of narrow fp16 layers (64 filters in and out, 3x3 and 5x5, 128 filters 3x3: the windowed kernels where the image is narrow enough for
    their pixel ring, the tile engine beyond that) against the oracle's explicit convolution, in every form the epilogue takes: bias +
    residual + ReLU, bias + ReLU, bias + residual, bias alone, and the bare product. Images of one row, of widths on both sides of what the
    ring allows, and batches whose pixel ranges span several units per workgroup."""
    rng = np.random.default_rng(sum(shape) + channels + k)
    b, h, w = shape
    x = random_tensor(rng, (b, h, w, channels), "float16")
    wt = random_tensor(rng, (channels, k, k, channels), "float16", (2.0 / (k * k * channels)) ** 0.5)
    bias = random_tensor(rng, (channels,), "float16")
    add = random_tensor(rng, (b, h, w, channels), "float16")
    dx, dw, db, da = (ml.toDevice(ctx, a) for a in (x, wt, bias, add))
    O.set_num_threads(8)
    for with_bias, with_add, act in ((True, True, "relu"), (True, False, "relu"), (True, True, "linear"), (True, False, "linear"), (False, False, "linear")):
        dy = ml.Tensor((b, h, w, channels), "float16")
        ml.convolutionImplicitGemmForward(ctx, dx, dw, dy, db if with_bias else None, da if with_add else None, act)
        want = O.conv2d_forward(x, wt, bias if with_bias else None, add if with_add else None, O.RELU if act == "relu" else O.LINEAR)
        assert max_abs_rel(dy.copyToHost(ctx), want) <= 1e-2, (with_bias, with_add, act)


@pytest.mark.parametrize("k", [3, 5])
def test_narrow_convolution_random_shapes(ctx, k):
    """The windowed kernels on 40 seeded random tensor shapes (1 to 24 images of 1 to 45 rows and columns): their pixel ranges, ring
    wrap-arounds, block-aligned and ragged range ends, images smaller than a unit and ranges that span many images all differ from shape
    to shape. Alternately bias + residual + ReLU and the bare product, against the oracle's explicit convolution."""
    rng = np.random.default_rng(9000 + k)
    O.set_num_threads(8)
    wt = random_tensor(rng, (64, k, k, 64), "float16", (2.0 / (k * k * 64)) ** 0.5)
    bias = random_tensor(rng, (64,), "float16")
    dw, db = ml.toDevice(ctx, wt), ml.toDevice(ctx, bias)
    for case in range(40):
        b, h, w = int(rng.integers(1, 25)), int(rng.integers(1, 46)), int(rng.integers(1, 46))
        x = random_tensor(rng, (b, h, w, 64), "float16")
        add = random_tensor(rng, (b, h, w, 64), "float16")
        dy = ml.Tensor((b, h, w, 64), "float16")
        if case % 2 == 0:
            ml.convolutionImplicitGemmForward(ctx, ml.toDevice(ctx, x), dw, dy, db, ml.toDevice(ctx, add), "relu")
            want = O.conv2d_forward(x, wt, bias, add, O.RELU)
        else:
            ml.convolutionImplicitGemmForward(ctx, ml.toDevice(ctx, x), dw, dy, None, None, "linear")
            want = O.conv2d_forward(x, wt)
        assert max_abs_rel(dy.copyToHost(ctx), want) <= 1e-2, (case, b, h, w)


@pytest.mark.parametrize("channels,k", [(64, 3), (64, 5), (128, 3)])
def test_narrow_convolution_at_full_size(ctx, channels, k):
    """Config 4's narrow rows at their full size (B = 512, 19x19, fp16, bias + residual + ReLU): positions are independent (a 2-position
    launch reproduces its slice of the full launch bit for bit), the first, the last and positions between match the oracle."""
    rng = np.random.default_rng(464 + channels + k)
    b = 512
    x = random_tensor(rng, (b, 19, 19, channels), "float16")
    wt = random_tensor(rng, (channels, k, k, channels), "float16", (2.0 / (k * k * channels)) ** 0.5)
    bias = random_tensor(rng, (channels,), "float16", 0.01)
    add = random_tensor(rng, (b, 19, 19, channels), "float16")
    dx, dw, db, da = (ml.toDevice(ctx, a) for a in (x, wt, bias, add))
    dy = ml.Tensor((b, 19, 19, channels), "float16")
    ml.convolutionImplicitGemmForward(ctx, dx, dw, dy, db, da, "relu")
    got = dy.copyToHost(ctx)
    per = 19 * 19 * channels
    for first in (0, 1, 255, 510):
        part = ml.Tensor((2, 19, 19, channels), "float16")
        ml.convolutionImplicitGemmForward(ctx, dx.view((2, 19, 19, channels), first * per), dw, part, db, da.view((2, 19, 19, channels), first * per), "relu")
        assert mismatches(part.copyToHost(ctx), got[first:first + 2]) == 0
    O.set_num_threads(8)
    sample = list(range(0, 512, 37)) + [511]
    want = O.conv2d_forward(x[sample], wt, bias, add[sample], O.RELU)
    assert max_abs_rel(got[sample], want) <= 1e-2


@pytest.mark.parametrize("cin,cout,k", [(64, 128, 3), (128, 128, 5), (192, 192, 3), (64, 384, 5), (128, 576, 3), (64, 128, 5)])
@pytest.mark.parametrize("shape", [(1, 19, 19), (3, 7, 5), (2, 30, 9), (4, 20, 21), (2, 12, 22), (1, 3, 43), (1, 2, 50), (5, 1, 40), (40, 19, 19)])
def test_windowed_tile_convolution(ctx, shape, cin, cout, k):
    """fp16 convolutions whose output width is 128 or a multiple of 192: the tile engine takes its A operand from a window of pixels held
    in LDS (walked slice by slice over the input channels) where the image is narrow enough for the window, and gathers tap by tap
    beyond that. Images on both sides of that width for 3x3 and 5x5, of one row, smaller than a tile, ragged last tiles, one to three
    128-byte slices per pixel; every form of the epilogue including one that is not fixed at compile time, against the oracle."""
    rng = np.random.default_rng(sum(shape) + cin + cout + k)
    b, h, w = shape
    x = random_tensor(rng, (b, h, w, cin), "float16")
    wt = random_tensor(rng, (cout, k, k, cin), "float16", (2.0 / (k * k * cin)) ** 0.5)
    bias = random_tensor(rng, (cout,), "float16")
    add = random_tensor(rng, (b, h, w, cout), "float16")
    dx, dw, db, da = (ml.toDevice(ctx, a) for a in (x, wt, bias, add))
    O.set_num_threads(8)
    forms = ((True, True, "relu"), (True, False, "relu"), (True, True, "linear"), (False, False, "linear"), (True, True, "sigmoid"))
    for with_bias, with_add, act in forms:
        dy = ml.Tensor((b, h, w, cout), "float16")
        ml.convolutionImplicitGemmForward(ctx, dx, dw, dy, db if with_bias else None, da if with_add else None, act)
        want = O.conv2d_forward(x, wt, bias if with_bias else None, add if with_add else None, ml.act_of(act))
        assert max_abs_rel(dy.copyToHost(ctx), want) <= 1e-2, (with_bias, with_add, act)


@pytest.mark.parametrize("cin,cout,k", [(64, 128, 5), (128, 192, 3)])
def test_windowed_tile_convolution_random_shapes(ctx, cin, cout, k):
    """The window form of the tile engine on 30 seeded random tensor shapes (1 to 12 images of 1 to 45 rows and columns): tile starts
    anywhere in an image, windows that begin before the tensor or end past it, images smaller than a tile and wider than the window
    allows all occur. Alternately bias + residual + ReLU and the bare product, against the oracle's explicit convolution."""
    rng = np.random.default_rng(9100 + cin + k)
    O.set_num_threads(8)
    wt = random_tensor(rng, (cout, k, k, cin), "float16", (2.0 / (k * k * cin)) ** 0.5)
    bias = random_tensor(rng, (cout,), "float16")
    dw, db = ml.toDevice(ctx, wt), ml.toDevice(ctx, bias)
    for case in range(30):
        b, h, w = int(rng.integers(1, 13)), int(rng.integers(1, 46)), int(rng.integers(1, 46))
        x = random_tensor(rng, (b, h, w, cin), "float16")
        add = random_tensor(rng, (b, h, w, cout), "float16")
        dy = ml.Tensor((b, h, w, cout), "float16")
        if case % 2 == 0:
            ml.convolutionImplicitGemmForward(ctx, ml.toDevice(ctx, x), dw, dy, db, ml.toDevice(ctx, add), "relu")
            want = O.conv2d_forward(x, wt, bias, add, O.RELU)
        else:
            ml.convolutionImplicitGemmForward(ctx, ml.toDevice(ctx, x), dw, dy, None, None, "linear")
            want = O.conv2d_forward(x, wt)
        assert max_abs_rel(dy.copyToHost(ctx), want) <= 1e-2, (case, b, h, w)


@pytest.mark.parametrize("channels,k", [(384, 3), (384, 5), (256, 5), (384, 1), (128, 5), (256, 3)])
def test_config4_full_size_fp16(ctx, channels, k):
    """Config 4 at its full size (B = 512, 19x19 boards, fp16, bias + residual + ReLU) at the widest channel counts: positions are
    independent (a 2-position launch reproduces its slice of the full launch bit for bit: every output's reduction runs over K in the
    same order whatever the number of rows), and a sample of positions matches the oracle's explicit convolution within 1e-2."""
    rng = np.random.default_rng(46 + channels + k)
    b = 512
    x = random_tensor(rng, (b, 19, 19, channels), "float16")
    wt = random_tensor(rng, (channels, k, k, channels), "float16", (2.0 / (k * k * channels)) ** 0.5)
    bias = random_tensor(rng, (channels,), "float16", 0.01)
    add = random_tensor(rng, (b, 19, 19, channels), "float16")
    dx, dw, db, da = (ml.toDevice(ctx, a) for a in (x, wt, bias, add))
    dy = ml.Tensor((b, 19, 19, channels), "float16")
    ml.convolutionImplicitGemmForward(ctx, dx, dw, dy, db, da, "relu")
    got = dy.copyToHost(ctx)
    per = 19 * 19 * channels
    for first in (0, 301, 510):
        part = ml.Tensor((2, 19, 19, channels), "float16")
        ml.convolutionImplicitGemmForward(ctx, dx.view((2, 19, 19, channels), first * per), dw, part, db, da.view((2, 19, 19, channels), first * per), "relu")
        assert mismatches(part.copyToHost(ctx), got[first:first + 2]) == 0
    O.set_num_threads(8)
    sample = [0, 255, 511]
    want = O.conv2d_forward(x[sample], wt, bias, add[sample], O.RELU)
    assert max_abs_rel(got[sample], want) <= 1e-2


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_elementwise_neighbours(ctx, dtype):
    rng = np.random.default_rng(7)
    x = random_tensor(rng, (6, 5, 7, 12), dtype)
    b = random_tensor(rng, (12,), dtype)
    y0 = random_tensor(rng, (6, 5, 7, 12), dtype)
    for act in ("linear", "relu", "sigmoid", "tanh", "leaky_relu", "exp"):
        dy = ml.Tensor(x.shape, dtype)
        ml.addBiasAct(ctx, 1.0, ml.toDevice(ctx, x), ml.toDevice(ctx, b), 0.0, dy, act)
        assert max_abs_rel(dy.copyToHost(ctx), O.add_bias_act(x, b, ml.act_of(act))) <= TOL[dtype]
        dy = ml.toDevice(ctx, y0)
        ml.activationForward(ctx, 1.0, ml.toDevice(ctx, x), 0.0, dy, act)
        assert max_abs_rel(dy.copyToHost(ctx), O.add_bias_act(x, None, ml.act_of(act))) <= TOL[dtype]
    # y = act(x + b) * alpha + beta * y
    dy = ml.toDevice(ctx, y0)
    ml.addBiasAct(ctx, 0.5, ml.toDevice(ctx, x), ml.toDevice(ctx, b), 2.0, dy, "relu")
    want = 0.5 * O.as_float(O.add_bias_act(x, b, O.RELU)).astype(np.float64) + 2.0 * O.as_float(y0)
    assert np.abs(O.as_float(dy.copyToHost(ctx)) - want).max() / np.abs(want).max() <= TOL[dtype]
    # odd last dimension (scalar path)
    xo = random_tensor(rng, (9, 7), dtype)
    bo = random_tensor(rng, (7,), dtype)
    dy = ml.Tensor((9, 7), dtype)
    ml.addBiasAct(ctx, 1.0, ml.toDevice(ctx, xo), ml.toDevice(ctx, bo), 0.0, dy, "relu")
    assert mismatches(dy.copyToHost(ctx), O.add_bias_act(xo, bo, O.RELU)) == 0
    # weighted sum and scaling
    dy = ml.toDevice(ctx, y0)
    ml.addTensors(ctx, 0.5, ml.toDevice(ctx, x), -2.0, ml.toDevice(ctx, x), 0.0, None, 0.25, dy)
    assert max_abs_rel(dy.copyToHost(ctx), O.add_tensors(y0, 0.5, x, -2.0, x, 0.0, None, 0.25)) <= TOL[dtype]


@pytest.mark.parametrize("dtype,limit", [("float32", 1e-6), ("float16", 1e-3)])
def test_reference_tests_of_the_elementwise_neighbours(ctx, dtype, limit):
    """The reference's own tests, at their shapes and limits (test/backend/test_tensor_op.cpp:293-350, 408-435): addBiasAct in place with a
    sigmoid on [123, 48] (mean absolute difference at most 1e-6 in fp32, 1e-3 in fp16), addTensors of two [123, 14] tensors (1e-6)."""
    rng = np.random.default_rng(48)
    x = random_tensor(rng, (123, 48), dtype)
    b = random_tensor(rng, (48,), dtype)
    dy = ml.toDevice(ctx, x)
    ml.addBiasAct(ctx, 1.0, dy, ml.toDevice(ctx, b), 0.0, dy, "sigmoid")
    xf, bf = O.as_float(x).astype(np.float64), O.as_float(b).astype(np.float64)
    baseline = 1.0 / (1.0 + np.exp(-(xf + bf[None, :])))
    assert np.abs(O.as_float(dy.copyToHost(ctx)) - baseline).mean() <= limit
    if dtype == "float32":
        s1, s2 = random_tensor(rng, (123, 14), dtype), random_tensor(rng, (123, 14), dtype)
        dst = ml.Tensor((123, 14), dtype)
        dst.zeroall(ctx)
        ml.addTensors(ctx, 1.0, ml.toDevice(ctx, s1), 1.0, ml.toDevice(ctx, s2), 0.0, None, 0.0, dst)
        assert np.abs(dst.copyToHost(ctx).astype(np.float64) - (s1.astype(np.float64) + s2)).mean() <= 1e-6


def test_convert_and_unpack(ctx, golden):
    g = golden
    src = g["cvt_src"]
    dst = ml.Tensor(src.shape, "float16")
    ml.convertType(ctx, dst, ml.toDevice(ctx, src))
    got = dst.copyToHost(ctx)
    assert mismatches(got, O.to_half(src)[...]) <= 1  # 65519.9: infinity by the reference's scalar rule, largest finite half by its vector rule
    finite = np.abs(src) < 65504.0
    assert mismatches(got[finite], g["cvt_f16"][finite]) == 0
    back = ml.Tensor(src.shape, "float32")
    ml.convertType(ctx, back, dst)
    assert np.array_equal(back.copyToHost(ctx)[finite], O.from_half(got)[finite])
    for code, key in ((O.FLOAT32, "up_f32"), (O.FLOAT16, "up_f16")):
        d = ml.Tensor((3, 5, 40), code)
        ml.unpackInput(ctx, d, ml.toDevice(ctx, g["up_packed"].view(np.int32), "int32"))
        assert mismatches(d.copyToHost(ctx), g[key]) == 0


@pytest.mark.parametrize("last", [32, 40, 48, 7, 100])
@pytest.mark.parametrize("dtype", ["float16", "float32"])
def test_unpack_input_vector_and_scalar_forms(ctx, last, dtype):
    """Row lengths that take the 16-byte-store form (multiples of 8 halfs / 4 floats) and ones that do not, bit for bit."""
    rng = np.random.default_rng(last)
    words = (last + 31) // 32
    packed = rng.integers(0, 2 ** 32, size=(6 * 15 * 15, words), dtype=np.uint64).astype(np.uint32)
    d = ml.Tensor((6, 15, 15, last), dtype)
    ml.unpackInput(ctx, d, ml.toDevice(ctx, packed.view(np.int32), "int32"))
    want = O.unpack_input(packed, (6, 15, 15, last), O.FLOAT16 if dtype == "float16" else O.FLOAT32)
    assert mismatches(d.copyToHost(ctx), want) == 0


@pytest.mark.parametrize("elements", [8, 4099, 1 << 20])
def test_convert_type_vector_body_and_tail(ctx, elements):
    """Lengths with and without a scalar tail after the 8-element vector body; both directions, bit for bit."""
    rng = np.random.default_rng(elements)
    src = (rng.standard_normal(elements) * 50.0).astype(np.float32)
    dst = ml.Tensor((elements,), "float16")
    ml.convertType(ctx, dst, ml.toDevice(ctx, src))
    got = dst.copyToHost(ctx)
    assert mismatches(got, O.to_half(src)) == 0
    back = ml.Tensor((elements,), "float32")
    ml.convertType(ctx, back, dst)
    assert np.array_equal(back.copyToHost(ctx), O.from_half(got))


# ---- grouped product (reference: src/core/math.cpp:1079-1093, device backend only; checked against its definition) ---------------
def _grouped_reference(opA, opB, A, Bm, C, alpha, beta, groups):
    """One plain product of the oracle per group, on the group's column ranges."""
    ta, tb = opA == "t", opB == "t"
    pa, pb, pc = A.shape[1] // groups, Bm.shape[1] // groups, C.shape[1] // groups
    out = C.copy()
    for g in range(groups):
        a = np.ascontiguousarray(A[:, g * pa:(g + 1) * pa])
        b = np.ascontiguousarray(Bm[:, g * pb:(g + 1) * pb])
        c = np.ascontiguousarray(C[:, g * pc:(g + 1) * pc])
        out[:, g * pc:(g + 1) * pc] = O.gemm(a, b, opA, opB, alpha, beta, c if beta != 0.0 else None)
    return out


@pytest.mark.parametrize("dtype", ["float16", "float32"])
@pytest.mark.parametrize("case", [("n", "t", 300, 32, 64, 4, 1.0, 0.0), ("n", "t", 1000, 64, 256, 2, 1.0, 0.0), ("n", "t", 77, 12, 20, 3, 0.5, 1.5),
                                  ("n", "t", 513, 36, 128, 8, 1.0, 1.0), ("n", "n", 45, 24, 16, 2, 1.0, 0.0), ("t", "n", 30, 28, 50, 4, 2.0, 0.0)])
def test_group_gemm(ctx, dtype, case):
    """K rows of whole 128-byte chunks take the tile engine with the groups as its batch (operand rows a whole matrix row apart);
    everything else, the transposed forms of the backward pass included, the one-thread-per-output kernel."""
    opA, opB, M, N, K, groups, alpha, beta = case
    rng = np.random.default_rng(M + N + K)
    a_shape = (K, M * groups) if opA == "t" else (M, K * groups)
    b_shape = (N, K * groups) if opB == "t" else (K, N * groups)
    A = random_tensor(rng, a_shape, dtype)
    Bm = random_tensor(rng, b_shape, dtype, (1.0 / K) ** 0.5)
    C0 = random_tensor(rng, (M, N * groups), dtype)
    dC = ml.toDevice(ctx, C0)
    ml.gemmGrouped(ctx, opA, opB, dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm), alpha, beta, groups)
    want = _grouped_reference(opA, opB, A, Bm, C0, alpha, beta, groups)
    assert max_abs_rel(dC.copyToHost(ctx), want) <= TOL[dtype]


def test_grouped_1x1_convolution_layer(ctx):
    """Conv2D with groups > 1 as the reference runs it (src/layers/Conv2D.cpp:339-349): grouped product, then bias and activation; against
    one dense 1x1 convolution of the oracle per group."""
    from minml_amd.conv2d import Conv2D

    rng = np.random.default_rng(5)
    batch, board, cin, cout, groups = 3, 9, 128, 96, 4
    x = random_tensor(rng, (batch, board, board, cin), "float16")
    w = random_tensor(rng, (cout // groups, 1, 1, cin), "float16", 0.2)
    b = random_tensor(rng, (cout,), "float16", 0.1)
    layer = Conv2D(ctx, x.shape, cout, 1, "relu", True, "float16", groups=groups)
    layer.setWeights(w, b)
    y = ml.Tensor((batch, board, board, cout), "float16")
    layer.forward([ml.toDevice(ctx, x)], y)
    want = np.zeros((batch, board, board, cout), np.uint16)
    ci, co = cin // groups, cout // groups
    for g in range(groups):
        wg = np.ascontiguousarray(w[:, :, :, g * ci:(g + 1) * ci])
        # the reference stores the product, then adds bias and applies the activation in a second call: two roundings to fp16
        product = O.conv2d_forward(np.ascontiguousarray(x[..., g * ci:(g + 1) * ci]), wg, None, None, O.LINEAR)
        want[..., g * co:(g + 1) * co] = O.add_bias_act(product, np.ascontiguousarray(b[g * co:(g + 1) * co]), O.RELU)
    assert max_abs_rel(y.copyToHost(ctx), want) <= 1e-2


@pytest.mark.parametrize("dtype", ["float16", "float32"])
@pytest.mark.parametrize("case", [(230400 // 8, 1, 256), (5000, 1, 128), (4100, 3, 64), (4097, 4, 32), (6000, 2, 8), (4096, 1, 24), (9001, 1, 512), (7, 1, 256), (225, 2, 128)])
def test_gemm_ex_tall_with_few_columns(ctx, dtype, case):
    """Policy-head shapes: 1 to 4 columns, few to many rows. K rows of 16 * 2^i bytes take the one-pass matrix-vector kernel (every
    row block size from 1 to 64 lanes per row, ragged last groups); 24 elements per row take the general route. Bias, beta and ReLU included."""
    M, N, K = case
    rng = np.random.default_rng(M + N + K)
    A = random_tensor(rng, (M, K), dtype)
    Bm = random_tensor(rng, (N, K), dtype, (1.0 / K) ** 0.5)
    bias = random_tensor(rng, (N,), dtype, 0.3)
    C = random_tensor(rng, (M, N), dtype)
    dA, dB = ml.toDevice(ctx, A), ml.toDevice(ctx, Bm)
    dD = ml.Tensor((M, N), dtype)
    ml.gemm_ex(ctx, dD, 1.0, "n", dA, "t", dB, 0.0, None, ml.toDevice(ctx, bias), "linear")
    assert max_abs_rel(dD.copyToHost(ctx), O.gemm(A, Bm, bias=bias, act=O.LINEAR)) <= TOL[dtype]
    ml.gemm_ex(ctx, dD, 1.25, "n", dA, "t", dB, 0.5, ml.toDevice(ctx, C), ml.toDevice(ctx, bias), "relu")
    assert max_abs_rel(dD.copyToHost(ctx), O.gemm(A, Bm, alpha=1.25, beta=0.5, C=C, bias=bias, act=O.RELU)) <= TOL[dtype]
