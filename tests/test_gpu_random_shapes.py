"""Seeded sweeps over irregular shapes: every dispatch decision of the GEMM and convolution entry points (streaming kernel, tile
engine, small-tile engine, element-wise fallbacks; vector and scalar epilogues; ragged tiles; odd channel counts) is a function of the
shape, the alignment and the epilogue's parts, so shapes drawn at random reach combinations that the hand-picked cases of the other
test files do not. Every case is compared with the CPU oracle at the tolerance of its type (int8: bit for bit); a failing case prints
its own parameters."""
import numpy as np
import pytest

import oracle as O
from minml_amd import core as ml
from util import TOL, max_abs_rel, mismatches, random_tensor

pytestmark = pytest.mark.gpu

# K extents that decide the engine: rows of 128 / 256 / 512 / 768 bytes (streaming kernel), multiples of 128 bytes beyond (tile
# engine), multiples of 16 bytes (small-tile engine), anything else (element-wise fallback)
K_BYTES = [128, 256, 512, 768, 1024, 1152, 2048, 16, 48, 80, 144, 272, 6, 26, 70]
ACTS = ["linear", "relu", "sigmoid", "tanh"]


def _draw_extent(rng, limit):
    """mostly small extents, sometimes one around a tile boundary"""
    choice = rng.integers(0, 4)
    if choice == 0:
        return int(rng.integers(1, 9))
    if choice == 1:
        return int(rng.choice([31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257]))
    return int(rng.integers(1, limit + 1))


@pytest.mark.parametrize("seed", range(160))
def test_gemm_ex_random(ctx, seed):
    rng = np.random.default_rng(1000 + seed)
    dtype = ["float32", "float16"][seed % 2]
    esize = 4 if dtype == "float32" else 2
    K = max(1, int(rng.choice(K_BYTES)) // esize)
    M, N = _draw_extent(rng, 700), _draw_extent(rng, 300)
    alpha = float(rng.choice([1.0, 1.1, -0.5]))
    beta = float(rng.choice([0.0, 0.0, 0.5, 1.0]))
    use_bias = bool(rng.integers(0, 2))
    act = ACTS[int(rng.integers(0, len(ACTS)))]
    case = "seed %d: %s M=%d N=%d K=%d alpha=%g beta=%g bias=%s act=%s" % (seed, dtype, M, N, K, alpha, beta, use_bias, act)
    A = random_tensor(rng, (M, K), dtype, 0.5)
    Bm = random_tensor(rng, (N, K), dtype, (1.0 / K) ** 0.5)
    C = random_tensor(rng, (M, N), dtype)
    bias = random_tensor(rng, (N,), dtype)
    dD = ml.Tensor((M, N), dtype)
    dD.setall(ctx, float("nan"))
    ml.gemm_ex(ctx, dD, alpha, "n", ml.toDevice(ctx, A), "t", ml.toDevice(ctx, Bm), beta, ml.toDevice(ctx, C) if beta != 0.0 else None,
               ml.toDevice(ctx, bias) if use_bias else None, act)
    want = O.gemm(A, Bm, alpha=alpha, beta=beta, C=C if beta != 0.0 else None, bias=bias if use_bias else None, act=ml.act_of(act))
    assert max_abs_rel(dD.copyToHost(ctx), want) <= TOL[dtype], case


@pytest.mark.parametrize("seed", range(80))
def test_gemm_batched_random(ctx, seed):
    rng = np.random.default_rng(2000 + seed)
    dtype = ["float32", "float16"][seed % 2]
    esize = 4 if dtype == "float32" else 2
    K = max(1, int(rng.choice(K_BYTES)) // esize)
    batch = int(rng.choice([1, 2, 3, 7, 36]))
    M, N = _draw_extent(rng, 400), _draw_extent(rng, 260)
    beta = float(rng.choice([0.0, 0.0, 0.25]))
    alpha = float(rng.choice([1.0, 1.0, 0.75]))
    shared_b = bool(rng.integers(0, 3) == 0)  # a rank-2 B operand is used by every matrix of the batch (src/backend/cpu/gemm/gemm.cpp:18-24)
    case = "seed %d: %s batch=%d M=%d N=%d K=%d alpha=%g beta=%g shared_b=%s" % (seed, dtype, batch, M, N, K, alpha, beta, shared_b)
    A = random_tensor(rng, (batch, M, K), dtype, 0.5)
    Bm = random_tensor(rng, (N, K) if shared_b else (batch, N, K), dtype, (1.0 / K) ** 0.5)
    C = random_tensor(rng, (batch, M, N), dtype)
    dC = ml.toDevice(ctx, C)
    ml.gemmBatched(ctx, "n", "t", dC, ml.toDevice(ctx, A), ml.toDevice(ctx, Bm), alpha, beta)
    got = dC.copyToHost(ctx)
    for i in range(batch):
        want = O.gemm(A[i], Bm if shared_b else Bm[i], alpha=alpha, beta=beta, C=C[i] if beta != 0.0 else None)
        assert max_abs_rel(got[i], want) <= TOL[dtype], case + " matrix %d" % i


@pytest.mark.parametrize("seed", range(120))
def test_convolution_random(ctx, seed):
    rng = np.random.default_rng(3000 + seed)
    dtype = ["float32", "float16"][seed % 2]
    k = int(rng.choice([1, 3, 5]))
    b, h, w = int(rng.integers(1, 4)), int(rng.integers(1, 21)), int(rng.integers(1, 21))
    cin = int(rng.choice([1, 3, 7, 8, 16, 24, 32, 40, 64, 128, 256]))
    cout = _draw_extent(rng, 150)
    use_bias, use_add = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    act = ACTS[int(rng.integers(0, len(ACTS)))]
    case = "seed %d: %s [%d,%d,%d,%d] -> %d k=%d bias=%s add=%s act=%s" % (seed, dtype, b, h, w, cin, cout, k, use_bias, use_add, act)
    x = random_tensor(rng, (b, h, w, cin), dtype)
    wt = random_tensor(rng, (cout, k, k, cin), dtype, (2.0 / (k * k * cin)) ** 0.5)
    bias = random_tensor(rng, (cout,), dtype)
    add = random_tensor(rng, (b, h, w, cout), dtype)
    dy = ml.Tensor((b, h, w, cout), dtype)
    dy.setall(ctx, float("nan"))
    ml.convolutionImplicitGemmForward(ctx, ml.toDevice(ctx, x), ml.toDevice(ctx, wt), dy, ml.toDevice(ctx, bias) if use_bias else None,
                                      ml.toDevice(ctx, add) if use_add else None, act)
    want = O.conv2d_forward(x, wt, bias if use_bias else None, add if use_add else None, ml.act_of(act))
    assert max_abs_rel(dy.copyToHost(ctx), want) <= TOL[dtype], case


@pytest.mark.parametrize("seed", range(100))
def test_int8_convolution_random(ctx, seed):
    rng = np.random.default_rng(4000 + seed)
    k = int(rng.choice([1, 3, 5]))
    b, h, w = int(rng.integers(1, 4)), int(rng.integers(1, 17)), int(rng.integers(1, 17))
    cin = int(rng.choice([4, 7, 16, 20, 32, 48, 64, 128, 256]))
    cout = _draw_extent(rng, 140)
    use_ext = bool(rng.integers(0, 2))
    act = ["linear", "relu"][int(rng.integers(0, 2))]
    code = [O.INT8, O.FLOAT32][int(rng.integers(0, 2))]
    in_qd = (float(rng.random() * 0.2 + 0.01), float(rng.choice([0.0, 4.56, -3.3])))
    out_qd = (float(rng.random() * 0.1 + 0.02), float(rng.choice([0.0, 0.9, -0.9])))
    ext_qd = (float(rng.random() * 0.1 + 0.02), float(rng.choice([0.0, 0.9, -0.9])))
    case = "seed %d: [%d,%d,%d,%d] -> %d k=%d ext=%s act=%s out=%s in_qd=%s out_qd=%s ext_qd=%s" % (seed, b, h, w, cin, cout, k, use_ext, act,
                                                                                                  code, in_qd, out_qd, ext_qd)
    x = rng.integers(-128, 128, (b, h, w, cin)).astype(np.int8)
    wt = rng.integers(-127, 128, (cout, k, k, cin)).astype(np.int8)
    scales = (rng.random(cout) * 0.002 + 0.0005).astype(np.float32)
    bias = rng.standard_normal(cout).astype(np.float32)
    ext = rng.integers(-128, 128, (b, h, w, cout)).astype(np.int8)
    dy = ml.Tensor((b, h, w, cout), code)
    ml.quantizedConvForward(ctx, ml.toDevice(ctx, x), in_qd, ml.toDevice(ctx, wt), ml.toDevice(ctx, scales), ml.toDevice(ctx, bias), dy, out_qd,
                            ml.toDevice(ctx, ext) if use_ext else None, ext_qd, act)
    want = O.int8_conv2d_forward(x, in_qd, wt, scales, bias, code, out_qd, ext if use_ext else None, ext_qd, ml.act_of(act))
    assert mismatches(dy.copyToHost(ctx), want) == 0, case


@pytest.mark.parametrize("seed", range(80))
def test_winograd_transforms_random(ctx, seed):
    """The three transforms and the fused output -> input transform at random board sizes and channel counts (vector widths, edge tiles,
    one-pixel boards), bit for bit against the oracle with ReLU / linear epilogues."""
    rng = np.random.default_rng(5000 + seed)
    dtype = ["float32", "float16"][seed % 2]
    b, h, w = int(rng.integers(1, 4)), int(rng.integers(1, 22)), int(rng.integers(1, 22))
    c = int(rng.choice([1, 2, 3, 5, 8, 12, 16, 35, 64, 72, 128, 192, 256]))
    cout = c if rng.integers(0, 2) else int(rng.choice([1, 4, 6, 13, 32, 64, 100, 128]))
    use_bias, use_ext = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    act = [O.LINEAR, O.RELU][int(rng.integers(0, 2))]
    case = "seed %d: %s [%d,%d,%d,%d] -> %d bias=%s ext=%s act=%d" % (seed, dtype, b, h, w, c, cout, use_bias, use_ext, act)
    tiles = b * ((h + 3) // 4) * ((w + 3) // 4)
    wt = random_tensor(rng, (cout, 3, 3, c), dtype)
    dm = ml.Tensor((36, cout, c), dtype)
    ml.winogradWeightTransform(ctx, ml.toDevice(ctx, wt), dm, False)
    assert mismatches(dm.copyToHost(ctx), O.winograd_weight_transform(wt, False)) == 0, case
    x = random_tensor(rng, (b, h, w, c), dtype)
    dv = ml.Tensor((36, tiles, c), dtype)
    dv.setall(ctx, float("nan"))
    ml.winogradInputTransform(ctx, (cout, 3, 3, c), ml.toDevice(ctx, x), dv)
    assert mismatches(dv.copyToHost(ctx), O.winograd_input_transform(x)) == 0, case
    m = random_tensor(rng, (36, tiles, cout), dtype)
    bias = random_tensor(rng, (cout,), dtype)
    ext = random_tensor(rng, (b, h, w, cout), dtype)
    dmm = ml.toDevice(ctx, m)
    db = ml.toDevice(ctx, bias) if use_bias else None
    de = ml.toDevice(ctx, ext) if use_ext else None
    want_y = O.winograd_output_transform(m, (b, h, w, cout), bias if use_bias else None, ext if use_ext else None, act)
    dy = ml.Tensor((b, h, w, cout), dtype)
    dy.setall(ctx, 7.0)
    ml.winogradOutputTransform(ctx, (cout, 3, 3, cout), dmm, dy, db, de, act)
    assert mismatches(dy.copyToHost(ctx), want_y) == 0, case
    # the fused form writes y and the next layer's input matrices
    dy2 = ml.Tensor((b, h, w, cout), dtype)
    dy2.setall(ctx, 7.0)
    dv2 = ml.Tensor((36, tiles, cout), dtype)
    dv2.setall(ctx, float("nan"))
    ml.winogradOutputInputTransform(ctx, (cout, 3, 3, cout), dmm, (b, h, w, cout), dy2, db, de, act, dv2)
    assert mismatches(dy2.copyToHost(ctx), want_y) == 0, case
    assert mismatches(dv2.copyToHost(ctx), O.winograd_input_transform(want_y)) == 0, case


@pytest.mark.parametrize("seed", range(60))
def test_attention_and_rmsnorm_random(ctx, seed):
    rng = np.random.default_rng(6000 + seed)
    dtype = ["float32", "float16"][seed % 2]
    b, h, w = int(rng.integers(1, 4)), int(rng.integers(1, 17)), int(rng.integers(1, 17))
    heads = int(rng.choice([1, 2, 3, 4, 8]))
    d = int(rng.choice([8, 14, 16, 24, 32, 32, 64, 128]))
    symmetric = bool(rng.integers(0, 4) == 0)
    r = int(rng.choice([0, 1, 2, max(h, w), max(h, w) + 3, (max(h, w) + 1) // 2]))
    case = "seed %d: %s [%d,%d,%d] heads=%d d=%d symmetric=%s r=%d" % (seed, dtype, b, h, w, heads, d, symmetric, r)
    parts = 2 if symmetric else 3
    x = random_tensor(rng, (b, h, w, parts * heads * d), dtype, 1.5)
    table = None
    if r > 0:
        size = 2 * r - 1
        table = random_tensor(rng, (heads, size, (size + 3) // 4 * 4), dtype, 2.0)
    y = ml.Tensor((b, h, w, heads * d), dtype)
    y.setall(ctx, float("nan"))
    ml.multiHeadAttentionForward(ctx, ml.toDevice(ctx, x), y, None if table is None else ml.toDevice(ctx, table), None, None, None, heads, symmetric)
    got = y.copyToHost(ctx)
    assert np.isfinite(O.as_float(got)).all(), case
    assert max_abs_rel(got, O.multi_head_attention_forward(x, heads, table, symmetric)) <= TOL[dtype], case
    # RMS normalisation of the same tensor, with and without weights
    gamma = random_tensor(rng, (x.shape[3],), dtype)
    for g in (gamma, None):
        z = ml.Tensor(x.shape, dtype)
        ml.rmsnormForward(ctx, ml.toDevice(ctx, x), z, None if g is None else ml.toDevice(ctx, g))
        assert max_abs_rel(z.copyToHost(ctx), O.rmsnorm_forward(x, g)) <= TOL[dtype], case


@pytest.mark.parametrize("seed", range(60))
def test_heads_random(ctx, seed):
    """softmax, global average pooling and batch normalisation in inference mode at random extents (vector and scalar forms, one-column
    and many-column rows)."""
    rng = np.random.default_rng(7000 + seed)
    dtype = ["float32", "float16"][seed % 2]
    b, h, w = int(rng.integers(1, 70)), int(rng.integers(1, 12)), int(rng.integers(1, 12))
    c = int(rng.choice([1, 2, 3, 4, 7, 8, 16, 36, 64, 225, 256, 520, 1100]))
    case = "seed %d: %s [%d,%d,%d,%d]" % (seed, dtype, b, h, w, c)
    x = random_tensor(rng, (b, h, w, c), dtype, 2.0)
    dx = ml.toDevice(ctx, x)
    rows = x.reshape(b * h * w, c)
    y = ml.Tensor(rows.shape, dtype)
    ml.softmaxForward(ctx, y, ml.toDevice(ctx, rows))
    assert max_abs_rel(y.copyToHost(ctx), O.softmax_forward(rows)) <= TOL[dtype], case
    p = ml.Tensor((b, c), dtype)
    ml.globalAveragePoolingForward(ctx, 1.0, dx, 0.0, p)
    scale = float(np.abs(O.as_float(x)).mean())
    assert np.abs(O.as_float(p.copyToHost(ctx)).astype(np.float64) - O.as_float(O.global_average_pooling_forward(x))).max() / scale <= TOL[dtype], case
    gamma, bias = random_tensor(rng, (c,), dtype), random_tensor(rng, (c,), dtype)
    gamma = O.to_half(O.as_float(gamma) + np.float32(1.5)) if dtype == "float16" else gamma + np.float32(1.5)
    stats = np.stack([rng.standard_normal(c), rng.random(c) + 0.05]).astype(np.float32)
    act_name, act = [("linear", O.LINEAR), ("relu", O.RELU), ("tanh", O.TANH)][int(rng.integers(0, 3))]
    z = ml.Tensor((b, h, w, c), dtype)
    ml.batchnormInference(ctx, 1.0, dx, ml.toDevice(ctx, gamma), ml.toDevice(ctx, bias), ml.toDevice(ctx, stats), 0.0, z, act_name)
    assert max_abs_rel(z.copyToHost(ctx), O.batchnorm_inference(x, gamma, bias, stats, act)) <= TOL[dtype], case


@pytest.mark.parametrize("seed", range(60))
def test_mixture_of_experts_random(ctx, seed):
    """Expert-choice routing on tie-free scores, gather, the expert layers and scatter at random token counts, expert counts, capacities
    and widths: routing tables, gathered rows bit for bit; expert layers and scatter within the tolerance."""
    from oracle import moe as M
    rng = np.random.default_rng(8000 + seed)
    dtype = ["float32", "float16"][seed % 2]
    b, h, w = int(rng.integers(1, 4)), int(rng.integers(1, 11)), int(rng.integers(1, 11))
    tokens = h * w
    experts = int(rng.choice([1, 2, 3, 8, 12]))
    capacity = int(rng.integers(1, tokens + 1))
    c = int(rng.choice([4, 7, 16, 64, 128, 256]))
    n = int(rng.choice([4, 12, 36, 64, 128, 256]))
    act_name = ["linear", "relu"][int(rng.integers(0, 2))]
    case = "seed %d: %s [%d,%d,%d] experts=%d capacity=%d C=%d N=%d act=%s" % (seed, dtype, b, h, w, experts, capacity, c, n, act_name)
    base = np.linspace(-4.0, 4.0, tokens * b).astype(np.float32)
    scores = np.stack([rng.permutation(base).reshape(b, tokens) + np.float32(0.001 * j) for j in range(experts)], axis=-1).reshape(b, h, w, experts)
    if dtype == "float16":
        scores = O.to_half(scores)
        f = O.from_half(scores).reshape(b, tokens, experts)
        if any(np.unique(f[i, :, j]).size != tokens for i in range(b) for j in range(experts)):
            pytest.skip("scores tie after narrowing to fp16")
    iv = ml.Tensor((b, 2, experts, capacity), dtype)
    ml.expertChoiceRoutingForward(ctx, ml.toDevice(ctx, scores), iv)
    want_iv = M.expert_choice_routing(scores, capacity)
    got_iv = iv.copyToHost(ctx)
    assert np.array_equal(O.as_float(got_iv)[:, 0], O.as_float(want_iv)[:, 0]), case
    assert np.abs(O.as_float(got_iv)[:, 1].astype(np.float64) - O.as_float(want_iv)[:, 1]).max() <= (1e-6 if dtype == "float32" else 1e-3), case
    x = random_tensor(rng, (b, h, w, c), dtype)
    d_iv = ml.toDevice(ctx, want_iv)
    g = ml.Tensor((b, capacity, experts, c), dtype)
    g.setall(ctx, float("nan"))
    ml.gatherTokensForward(ctx, ml.toDevice(ctx, x), d_iv, 0.0, g)
    gathered = M.gather_tokens(x, want_iv)
    assert mismatches(g.copyToHost(ctx), gathered) == 0, case
    wt = random_tensor(rng, (experts, n, c), dtype, (1.0 / c) ** 0.5)
    bias = random_tensor(rng, (experts, n), dtype, 0.1)
    hidden = ml.Tensor((b, capacity, experts, n), dtype)
    ml.moeForward(ctx, g, ml.toDevice(ctx, wt), ml.toDevice(ctx, bias), 0.0, hidden, act_name)
    want_hidden = M.moe_forward(gathered, wt, bias, ml.act_of(act_name))
    assert max_abs_rel(hidden.copyToHost(ctx), want_hidden) <= TOL[dtype], case
    y0 = random_tensor(rng, (b, h, w, n), dtype)
    dy = ml.toDevice(ctx, y0)
    ml.scatterTokensForward(ctx, ml.toDevice(ctx, want_hidden), d_iv, 1.0, dy)
    assert max_abs_rel(dy.copyToHost(ctx), M.scatter_tokens(want_hidden, want_iv, (b, h, w, n), beta=1.0, y=y0)) <= TOL[dtype], case


# ---- the same entry points on tensors that do not start at an aligned address --------------------------------------------------------
# The reference hands the backend views into larger allocations (Tensor::view: the layer workspace is cut into the three Winograd
# matrices at element offsets, src/layers/Conv2D.cpp:365-367), so a pointer may be aligned to its element size only. The vector forms of
# every kernel check the addresses they are given; these cases give each operand its own small element offset.

def _np_dtype_name(array):
    return {np.dtype(np.uint16): "float16", np.dtype(np.float32): "float32", np.dtype(np.int8): "int8", np.dtype(np.int32): "int32"}[array.dtype]


def _at(ctx, array, offset):
    """device copy of `array` that starts `offset` elements into its allocation"""
    base = ml.Tensor((array.size + offset,), _np_dtype_name(array))
    view = base.view(array.shape, offset)
    view.copyFromHost(ctx, array)
    return view


def _out_at(ctx, shape, dtype, offset):
    base = ml.Tensor((int(np.prod(shape)) + offset,), dtype)
    view = base.view(shape, offset)
    if dtype in ("float32", "float16"):
        view.setall(ctx, float("nan"))
    return view


def _offsets(rng, count):
    return [int(rng.choice([0, 1, 2, 3, 4, 5, 8])) for _ in range(count)]


@pytest.mark.parametrize("seed", range(60))
def test_gemm_ex_on_offset_views(ctx, seed):
    rng = np.random.default_rng(9000 + seed)
    dtype = ["float32", "float16"][seed % 2]
    esize = 4 if dtype == "float32" else 2
    K = max(1, int(rng.choice(K_BYTES)) // esize)
    M, N = _draw_extent(rng, 500), _draw_extent(rng, 280)
    beta = float(rng.choice([0.0, 0.5]))
    use_bias = bool(rng.integers(0, 2))
    act = ["linear", "relu"][int(rng.integers(0, 2))]
    oa, ob, oc, od, obias = _offsets(rng, 5)
    case = "seed %d: %s M=%d N=%d K=%d beta=%g bias=%s act=%s offsets A %d B %d C %d D %d bias %d" % (seed, dtype, M, N, K, beta, use_bias, act, oa, ob, oc,
                                                                                                 od, obias)
    A = random_tensor(rng, (M, K), dtype, 0.5)
    Bm = random_tensor(rng, (N, K), dtype, (1.0 / K) ** 0.5)
    C = random_tensor(rng, (M, N), dtype)
    bias = random_tensor(rng, (N,), dtype)
    dD = _out_at(ctx, (M, N), dtype, od)
    ml.gemm_ex(ctx, dD, 1.0, "n", _at(ctx, A, oa), "t", _at(ctx, Bm, ob), beta, _at(ctx, C, oc) if beta != 0.0 else None,
               _at(ctx, bias, obias) if use_bias else None, act)
    want = O.gemm(A, Bm, alpha=1.0, beta=beta, C=C if beta != 0.0 else None, bias=bias if use_bias else None, act=ml.act_of(act))
    assert max_abs_rel(dD.copyToHost(ctx), want) <= TOL[dtype], case


@pytest.mark.parametrize("seed", range(40))
def test_gemm_batched_on_offset_views(ctx, seed):
    rng = np.random.default_rng(9500 + seed)
    dtype = ["float32", "float16"][seed % 2]
    esize = 4 if dtype == "float32" else 2
    K = max(1, int(rng.choice(K_BYTES)) // esize)
    batch = int(rng.choice([1, 3, 36]))
    M, N = _draw_extent(rng, 300), _draw_extent(rng, 260)
    oa, ob, oc = _offsets(rng, 3)
    case = "seed %d: %s batch=%d M=%d N=%d K=%d offsets A %d B %d C %d" % (seed, dtype, batch, M, N, K, oa, ob, oc)
    A = random_tensor(rng, (batch, M, K), dtype, 0.5)
    Bm = random_tensor(rng, (batch, N, K), dtype, (1.0 / K) ** 0.5)
    dC = _out_at(ctx, (batch, M, N), dtype, oc)
    ml.gemmBatched(ctx, "n", "t", dC, _at(ctx, A, oa), _at(ctx, Bm, ob), 1.0, 0.0)
    got = dC.copyToHost(ctx)
    for i in range(batch):
        assert max_abs_rel(got[i], O.gemm(A[i], Bm[i])) <= TOL[dtype], case + " matrix %d" % i


@pytest.mark.parametrize("seed", range(60))
def test_convolutions_on_offset_views(ctx, seed):
    """the float convolution, the int8 convolution and the Winograd transforms with every operand at its own offset"""
    rng = np.random.default_rng(9800 + seed)
    dtype = ["float32", "float16"][seed % 2]
    k = int(rng.choice([1, 3, 5]))
    b, h, w = int(rng.integers(1, 3)), int(rng.integers(1, 17)), int(rng.integers(1, 17))
    cin = int(rng.choice([3, 8, 16, 32, 64, 128, 256]))
    cout = _draw_extent(rng, 130)
    ox, ow, ob, oe, oy = _offsets(rng, 5)
    case = "seed %d: %s [%d,%d,%d,%d] -> %d k=%d offsets x %d w %d bias %d ext %d y %d" % (seed, dtype, b, h, w, cin, cout, k, ox, ow, ob, oe, oy)
    x = random_tensor(rng, (b, h, w, cin), dtype)
    wt = random_tensor(rng, (cout, k, k, cin), dtype, (2.0 / (k * k * cin)) ** 0.5)
    bias = random_tensor(rng, (cout,), dtype)
    add = random_tensor(rng, (b, h, w, cout), dtype)
    dy = _out_at(ctx, (b, h, w, cout), dtype, oy)
    ml.convolutionImplicitGemmForward(ctx, _at(ctx, x, ox), _at(ctx, wt, ow), dy, _at(ctx, bias, ob), _at(ctx, add, oe), "relu")
    assert max_abs_rel(dy.copyToHost(ctx), O.conv2d_forward(x, wt, bias, add, O.RELU)) <= TOL[dtype], case
    # int8, bit for bit
    xq = rng.integers(-128, 128, (b, h, w, cin)).astype(np.int8)
    wq = rng.integers(-127, 128, (cout, k, k, cin)).astype(np.int8)
    scales = (rng.random(cout) * 0.002 + 0.0005).astype(np.float32)
    fbias = rng.standard_normal(cout).astype(np.float32)
    ext = rng.integers(-128, 128, (b, h, w, cout)).astype(np.int8)
    in_qd, out_qd, ext_qd = (0.123, 4.56), (0.078, 0.9), (0.078, -0.9)
    dq = _out_at(ctx, (b, h, w, cout), "int8", oy)
    ml.quantizedConvForward(ctx, _at(ctx, xq, ox), in_qd, _at(ctx, wq, ow), _at(ctx, scales, ob), _at(ctx, fbias, oe), dq, out_qd, _at(ctx, ext, oe),
                            ext_qd, "relu")
    want = O.int8_conv2d_forward(xq, in_qd, wq, scales, fbias, O.INT8, out_qd, ext, ext_qd, O.RELU)
    assert mismatches(dq.copyToHost(ctx), want) == 0, case
    # Winograd transforms of the same tensors, bit for bit
    tiles = b * ((h + 3) // 4) * ((w + 3) // 4)
    dv = _out_at(ctx, (36, tiles, cin), dtype, oy)
    ml.winogradInputTransform(ctx, (cout, 3, 3, cin), _at(ctx, x, ox), dv)
    assert mismatches(dv.copyToHost(ctx), O.winograd_input_transform(x)) == 0, case
    m = random_tensor(rng, (36, tiles, cout), dtype)
    want_y = O.winograd_output_transform(m, (b, h, w, cout), bias, add, O.RELU)
    dy = _out_at(ctx, (b, h, w, cout), dtype, oy)
    dm = _at(ctx, m, ow)
    ml.winogradOutputTransform(ctx, (cout, 3, 3, cout), dm, dy, _at(ctx, bias, ob), _at(ctx, add, oe), O.RELU)
    assert mismatches(dy.copyToHost(ctx), want_y) == 0, case
    dy2 = _out_at(ctx, (b, h, w, cout), dtype, oy)
    dv2 = _out_at(ctx, (36, tiles, cout), dtype, ox)
    ml.winogradOutputInputTransform(ctx, (cout, 3, 3, cout), dm, (b, h, w, cout), dy2, _at(ctx, bias, ob), _at(ctx, add, oe), O.RELU, dv2)
    assert mismatches(dy2.copyToHost(ctx), want_y) == 0, case
    assert mismatches(dv2.copyToHost(ctx), O.winograd_input_transform(want_y)) == 0, case
