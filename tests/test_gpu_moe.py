"""Mixture-of-experts steps on the GPU against their CPU statement (oracle/moe.py; the reference has no CPU implementation of these,
so that statement is pinned by tests/test_oracle_moe.py against the baselines of the reference's own tests instead), through the C-ABI: routing tables must agree in every index (scores
are drawn so that no two tokens tie) and in the gates to rounding; gather is an exact copy; expert layers and scatter within the GEMM
tolerances (fp32 1e-4, fp16 1e-2 max-abs relative)."""
import numpy as np
import pytest

import oracle as O
from oracle import moe as M
from minml_amd import core as ml
from util import TOL, max_abs_rel, mismatches, random_tensor

pytestmark = pytest.mark.gpu


def distinct_scores(rng, shape, dtype):
    """Router logits without ties, also after narrowing to fp16: a random permutation of an arithmetic progression per expert."""
    b, h, w, e = shape
    t = h * w
    base = np.linspace(-4.0, 4.0, t * b).astype(np.float32)
    s = np.stack([rng.permutation(base).reshape(b, t) + np.float32(0.001 * j) for j in range(e)], axis=-1).reshape(shape)
    if dtype == "float16":
        s = O.to_half(s)
        f = O.from_half(s).reshape(b, t, e)
        for n in range(b):
            for j in range(e):
                assert np.unique(f[n, :, j]).size == t  # the progression's step is far above fp16 resolution at |x| <= 4 for these sizes
    return s


def index_plane(iv):
    return O.as_float(iv)[:, 0].astype(np.int64)


def gate_plane(iv):
    return O.as_float(iv)[:, 1].astype(np.float64)


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape,capacity", [((3, 15, 15, 8), 56), ((2, 5, 7, 6), 9), ((2, 4, 4, 3), 20), ((1, 19, 19, 4), 128), ((2, 1, 1, 2), 1)])
def test_expert_choice_routing(ctx, dtype, shape, capacity):
    rng = np.random.default_rng(sum(shape) + capacity)
    s = distinct_scores(rng, shape, dtype)
    iv = ml.Tensor((shape[0], 2, shape[3], capacity), dtype)
    ml.expertChoiceRoutingForward(ctx, ml.toDevice(ctx, s), iv)
    got, want = iv.copyToHost(ctx), M.expert_choice_routing(s, capacity)
    assert np.array_equal(index_plane(got), index_plane(want))
    assert np.abs(gate_plane(got) - gate_plane(want)).max() <= (1e-6 if dtype == "float32" else 1e-3)


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape,capacity", [((3, 15, 15, 8), 57), ((2, 5, 7, 6), 35), ((2, 4, 4, 3), 3), ((1, 19, 19, 16), 30)])
def test_token_choice_routing(ctx, dtype, shape, capacity):
    rng = np.random.default_rng(sum(shape) + capacity + 1)
    s = random_tensor(rng, shape, dtype, 2.0)
    bias = random_tensor(rng, (shape[3],), dtype, 0.3)
    for use_bias in (True, False):
        iv = ml.Tensor((shape[0], 2, shape[3], capacity), dtype)
        ml.tokenChoiceRoutingForward(ctx, ml.toDevice(ctx, s), ml.toDevice(ctx, bias) if use_bias else None, iv)
        got, want = iv.copyToHost(ctx), M.token_choice_routing(s, bias if use_bias else None, capacity)
        gi, wi, gg, wg = index_plane(got), index_plane(want), gate_plane(got), gate_plane(want)
        # the device exponential differs from the host's in the last place: a gate may land on the neighbouring fp16 / fp32 value, which can
        # swap two tokens whose gates are that close; compare the routed SETS per expert and the gates token by token
        for n in range(shape[0]):
            for e in range(shape[3]):
                g_tokens, w_tokens = gi[n, e][gi[n, e] >= 0], wi[n, e][wi[n, e] >= 0]
                if capacity >= shape[1] * shape[2]:
                    assert sorted(g_tokens.tolist()) == sorted(w_tokens.tolist())
                lookup = dict(zip(w_tokens.tolist(), wg[n, e][:w_tokens.size].tolist()))
                for token, gate in zip(g_tokens.tolist(), gg[n, e][:g_tokens.size].tolist()):
                    if token in lookup:
                        assert abs(gate - lookup[token]) <= (2e-6 if dtype == "float32" else 2e-3)
                assert (np.diff(gg[n, e][:g_tokens.size]) <= 0).all()
                assert g_tokens.size == w_tokens.size


def test_hash_routing(ctx):
    x = ml.Tensor((3, 5, 5, 4), "float16")
    iv = ml.Tensor((3, 2, 4, 7), "float16")
    ml.hashRouting(ctx, x, iv)
    assert mismatches(iv.copyToHost(ctx), M.hash_routing(np.zeros((3, 5, 5, 4), np.uint16), 7)) == 0


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape,experts,capacity", [((2, 15, 15, 256), 8, 56), ((2, 5, 7, 12), 3, 40), ((1, 4, 4, 7), 2, 5),
                                                    ((2, 6, 6, 16), 12, 5),      # more experts than one group of eight
                                                    ((1, 19, 19, 8), 40, 12),    # inverted table too large for LDS: the scanning form
                                                    ((1, 6, 6, 600), 4, 20),     # rows longer than one wavefront's 256 elements, the last piece ragged
                                                    ((2, 3, 3, 16), 5, 9), ((2, 3, 3, 16), 6, 9), ((2, 3, 3, 16), 7, 9),
                                                    ((2, 3, 3, 16), 8, 9),       # every expert holds every token: 5 to 8 contributions per token
                                                    ((1, 3, 3, 5), 11, 9)])      # the same through the one-element form
def test_gather_and_scatter(ctx, dtype, shape, experts, capacity):
    rng = np.random.default_rng(sum(shape))
    b, h, w, c = shape
    x = random_tensor(rng, shape, dtype)
    iv = M.expert_choice_routing(distinct_scores(rng, (b, h, w, experts), dtype), capacity)
    d_iv, d_x = ml.toDevice(ctx, iv), ml.toDevice(ctx, x)
    g = ml.Tensor((b, capacity, experts, c), dtype)
    g.setall(ctx, float("nan"))
    ml.gatherTokensForward(ctx, d_x, d_iv, 0.0, g)
    want_g = M.gather_tokens(x, iv)
    assert mismatches(g.copyToHost(ctx), want_g) == 0
    experts_out = random_tensor(rng, (b, capacity, experts, c), dtype)
    y = ml.Tensor(shape, dtype)
    y.setall(ctx, float("nan"))
    ml.scatterTokensForward(ctx, ml.toDevice(ctx, experts_out), d_iv, 0.0, y)
    assert max_abs_rel(y.copyToHost(ctx), M.scatter_tokens(experts_out, iv, shape)) <= TOL[dtype]
    y0 = random_tensor(rng, shape, dtype)
    dy = ml.toDevice(ctx, y0)
    ml.scatterTokensForward(ctx, ml.toDevice(ctx, experts_out), d_iv, 0.5, dy)
    assert max_abs_rel(dy.copyToHost(ctx), M.scatter_tokens(experts_out, iv, shape, beta=0.5, y=y0)) <= TOL[dtype]
    g0 = random_tensor(rng, (b, capacity, experts, c), dtype)
    dg = ml.toDevice(ctx, g0)
    ml.gatherTokensForward(ctx, d_x, d_iv, 2.0, dg)
    assert max_abs_rel(dg.copyToHost(ctx), M.gather_tokens(x, iv, beta=2.0, y=g0)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("dims", [(2, 56, 8, 256, 1024), (2, 56, 8, 1024, 256), (3, 7, 3, 20, 12), (1, 5, 2, 64, 36), (4, 56, 8, 64, 128)])
def test_expert_layers(ctx, dtype, dims):
    b, k, e, c, n = dims
    rng = np.random.default_rng(sum(dims))
    O.set_num_threads(8)
    x = random_tensor(rng, (b, k, e, c), dtype)
    w = random_tensor(rng, (e, n, c), dtype, (1.0 / c) ** 0.5)
    bias = random_tensor(rng, (e, n), dtype, 0.1)
    dx, dw, db = ml.toDevice(ctx, x), ml.toDevice(ctx, w), ml.toDevice(ctx, bias)
    for act, use_bias in (("relu", True), ("linear", False), ("sigmoid", True)):
        y = ml.Tensor((b, k, e, n), dtype)
        ml.moeForward(ctx, dx, dw, db if use_bias else None, 0.0, y, act)
        want = M.moe_forward(x, w, bias if use_bias else None, ml.act_of(act))
        assert max_abs_rel(y.copyToHost(ctx), want) <= TOL[dtype]
    y0 = random_tensor(rng, (b, k, e, n), dtype)
    dy = ml.toDevice(ctx, y0)
    ml.moeForward(ctx, dx, dw, db, 0.5, dy, "linear")
    assert max_abs_rel(dy.copyToHost(ctx), M.moe_forward(x, w, bias, O.LINEAR, beta=0.5, y=y0)) <= TOL[dtype]


# ---- the reference's own tests, mirrored: its device layers against the CPU baselines of test/backend/test_moe.cpp, fp32, 1e-4 -----------

def _routing_table(rng, batch, tokens, experts, slots, empty=0.15):
    table = np.zeros((batch, 2, experts, slots), np.float32)
    for b in range(batch):
        for e in range(experts):
            table[b, 0, e] = rng.permutation(tokens)[:slots]
    table[:, 1] = rng.random((batch, experts, slots), dtype=np.float32)
    table[:, 0][rng.random((batch, experts, slots)) < empty] = -1.0
    return table


def test_reference_test_router_token_choice_and_hash(ctx):
    """TestRouter (test_moe.cpp:956-981): token choice with capacity factor 1.25 on [128, 15, 15, 2] in fp32 against the test's
    BaselineRouter, difference at most 1e-4; and the baseline's hash branch."""
    import reference_moe_baselines as R
    rng = np.random.default_rng(31)
    shape = (128, 15, 15, 2)
    scores = rng.standard_normal(shape, dtype=np.float32)
    cap = R.capacity(1.25, 225, 2)
    iv = ml.Tensor((128, 2, 2, cap), "float32")
    ml.tokenChoiceRoutingForward(ctx, ml.toDevice(ctx, scores), None, iv)
    got, want = iv.copyToHost(ctx), R.token_choice_router(scores, cap)
    assert np.array_equal(got[:, 0], want[:, 0])
    assert np.abs(got[:, 1] - want[:, 1]).max() <= 1e-4
    ml.hashRouting(ctx, ml.toDevice(ctx, scores), iv)
    assert np.array_equal(iv.copyToHost(ctx), R.hash_router(128, 225, 2, cap))


def test_reference_test_gather_and_scatter(ctx):
    """TestGatherTopK / TestScatterTopK (test_moe.cpp:989-1056): [3, 11, 12, 56], 8 experts, 12 and 16 slots, fp32, against the test's
    baselines; gather is a copy (exact), scatter within 1e-4."""
    import reference_moe_baselines as R
    rng = np.random.default_rng(32)
    x = rng.standard_normal((3, 11, 12, 56), dtype=np.float32)
    table = _routing_table(rng, 3, 132, 8, 12)
    y = ml.Tensor((3, 12, 8, 56), "float32")
    y.setall(ctx, float("nan"))
    ml.gatherTokensForward(ctx, ml.toDevice(ctx, x), ml.toDevice(ctx, table), 0.0, y)
    assert np.array_equal(y.copyToHost(ctx), R.gather_tokens(x, table))
    rows = rng.standard_normal((3, 16, 8, 56), dtype=np.float32)
    table = _routing_table(rng, 3, 132, 8, 16)
    out = ml.Tensor((3, 11, 12, 56), "float32")
    out.setall(ctx, float("nan"))
    ml.scatterTokensForward(ctx, ml.toDevice(ctx, rows), ml.toDevice(ctx, table), 0.0, out)
    want = R.scatter_tokens(rows, table, (3, 11, 12, 56))
    assert np.abs(out.copyToHost(ctx) - want).max() / np.abs(want).max() <= 1e-4


@pytest.mark.parametrize("act", ["relu", "linear"])
def test_reference_test_mixture_of_experts(ctx, act):
    """TestMixtureOfExperts (test_moe.cpp:1067-1093): [32, 16, 32, 128] -> 64 neurons per expert in fp32 against the test's baseline
    (a plain triple loop per expert, then bias and activation), difference at most 1e-4."""
    import reference_moe_baselines as R
    rng = np.random.default_rng(33)
    x = rng.standard_normal((32, 16, 32, 128), dtype=np.float32)
    w = rng.standard_normal((32, 64, 128), dtype=np.float32) * np.float32(0.1)
    b = rng.standard_normal((32, 64), dtype=np.float32) * np.float32(0.1)
    y = ml.Tensor((32, 16, 32, 64), "float32")
    ml.moeForward(ctx, ml.toDevice(ctx, x), ml.toDevice(ctx, w), ml.toDevice(ctx, b), 0.0, y, act)
    want = R.expert_layers(x, w, b, act == "relu")
    assert np.abs(y.copyToHost(ctx) - want).max() / np.abs(want).max() <= 1e-4
