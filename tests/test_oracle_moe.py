"""What pins the mixture-of-experts statements of oracle/moe.py, for which the reference has no CPU implementation to compare with
(src/core/math.cpp:1328-1491 dispatches to CUDA only): each function is checked against what the mathematics fixes, written
independently of the oracle's own loops — a brute-force top-k, permutation equivariance, float64 softmax / sigmoid / matrix products,
index arithmetic by numpy fancy indexing, and the identity scatter(gather(x)) = x * (sum of the gates that selected each token)."""
import numpy as np
import pytest

import oracle as O
from oracle import moe as M


def scores(rng, b, h, w, e, dtype="float32"):
    s = rng.standard_normal((b, h, w, e)).astype(np.float32) * 2.0
    return O.to_half(s) if dtype == "float16" else s


def planes(iv):
    f = O.as_float(iv).astype(np.float64)
    return f[:, 0].astype(np.int64), f[:, 1]


def test_capacity_follows_the_reference_formula():
    # src/layers/Router.cpp:62-66
    assert M.get_capacity(2.0, 225, 8) == 56 and M.get_capacity(1.0, 225, 8) == 29 and M.get_capacity(1.0, 64, 8) == 8


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_expert_choice_is_a_top_k_by_brute_force(dtype):
    rng = np.random.default_rng(1)
    b, h, w, e, k = 3, 5, 7, 6, 9
    s = scores(rng, b, h, w, e, dtype)
    idx, gate = planes(M.expert_choice_routing(s, k))
    sf = O.as_float(s).astype(np.float64).reshape(b, h * w, e)
    for n in range(b):
        for j in range(e):
            left = sf[n, :, j].copy()
            for slot in range(k):  # repeated argmax: the k largest, largest first, lowest index among equals
                best = int(np.argmax(left))
                assert idx[n, j, slot] == best
                want = 1.0 / (1.0 + np.exp(-sf[n, best, j]))
                assert abs(gate[n, j, slot] - want) <= (1e-6 if dtype == "float32" else 1e-3)
                left[best] = -np.inf


def test_expert_choice_permutation_equivariance_and_padding():
    rng = np.random.default_rng(2)
    b, h, w, e = 2, 4, 4, 3
    s = scores(rng, b, h, w, e)
    perm = rng.permutation(h * w)
    sp = s.reshape(b, h * w, e)[:, perm].reshape(b, h, w, e)
    idx, gate = planes(M.expert_choice_routing(s, 5))
    idx_p, gate_p = planes(M.expert_choice_routing(sp, 5))
    assert np.array_equal(perm[idx_p], idx) and np.array_equal(gate_p, gate)
    # more slots than tokens: the rest are empty
    idx_big, gate_big = planes(M.expert_choice_routing(s, 20))
    assert (idx_big[:, :, 16:] == -1).all() and (gate_big[:, :, 16:] == 0).all() and (idx_big[:, :, :16] >= 0).all()


def test_token_choice_routes_every_token_once_to_its_best_expert():
    rng = np.random.default_rng(3)
    b, h, w, e = 2, 5, 5, 4
    s = scores(rng, b, h, w, e)
    bias = rng.standard_normal(e).astype(np.float32) * 0.5
    idx, gate = planes(M.token_choice_routing(s, bias, h * w))  # capacity = all tokens: nothing is dropped
    sf = s.astype(np.float64).reshape(b, h * w, e)
    for n in range(b):
        seen = idx[n][idx[n] >= 0]
        assert sorted(seen.tolist()) == list(range(h * w))
        for j in range(e):
            filled = idx[n, j][idx[n, j] >= 0]
            assert (np.argmax(sf[n, filled] + bias[None, :], axis=1) == j).all()
            p = np.exp(sf[n, filled] - (sf[n, filled] + bias).max(axis=1, keepdims=True))
            want = p[:, j] / p.sum(axis=1)
            got = gate[n, j, :filled.size]
            assert np.abs(got - want).max() <= 1e-6
            assert (np.diff(got) <= 0).all()  # best first
    # a small capacity keeps the best of each expert's run
    idx_small, gate_small = planes(M.token_choice_routing(s, bias, 3))
    assert np.array_equal(idx_small, idx[:, :, :3]) and np.array_equal(gate_small, gate[:, :, :3])
    # zero bias: plain softmax probability of the arg-max, at least 1 / E
    _, gate0 = planes(M.token_choice_routing(s, None, h * w))
    assert (gate0[gate0 > 0] >= 1.0 / e - 1e-6).all() and (gate0 <= 1.0).all()


def test_hash_routing_closed_form():
    iv = M.hash_routing(np.zeros((2, 3, 3, 4), np.float32), 3)
    idx, gate = planes(iv)
    for e in range(4):
        for k in range(3):
            token = k * 4 + e
            assert (idx[:, e, k] == (token if token < 9 else -1)).all() and (gate[:, e, k] == (1.0 if token < 9 else 0.0)).all()


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_gather_and_scatter_against_index_arithmetic(dtype):
    rng = np.random.default_rng(4)
    b, h, w, c, e, k = 2, 4, 5, 6, 3, 7
    conv = O.to_half if dtype == "float16" else (lambda a: np.ascontiguousarray(a, np.float32))
    x = conv(rng.standard_normal((b, h, w, c)))
    iv = M.expert_choice_routing(scores(rng, b, h, w, e, dtype), k)
    idx, gate = planes(iv)
    g = M.gather_tokens(x, iv)
    xf = O.as_float(x).reshape(b, h * w, c)
    want = xf[np.arange(b)[:, None, None], idx]  # [b, e, k, c]
    assert np.array_equal(O.as_float(g), np.transpose(want, (0, 2, 1, 3)))  # a pure copy: exact in both types
    # scatter(gather(x)) = x * sum of the gates that selected the token
    y = M.scatter_tokens(g, iv, (b, h, w, c))
    weight = np.zeros((b, h * w), np.float64)
    for n in range(b):
        np.add.at(weight[n], idx[n].ravel(), gate[n].ravel())
    want_y = xf.astype(np.float64) * weight[:, :, None]
    tol = 1e-6 if dtype == "float32" else 2e-3
    assert np.abs(O.as_float(y).reshape(b, h * w, c) - want_y).max() <= tol * max(1.0, np.abs(want_y).max())
    # beta: y = beta * y0 + ...
    y0 = conv(rng.standard_normal((b, h, w, c)))
    y1 = M.scatter_tokens(g, iv, (b, h, w, c), beta=0.5, y=y0)
    want_y1 = want_y + 0.5 * O.as_float(y0).reshape(b, h * w, c)
    assert np.abs(O.as_float(y1).reshape(b, h * w, c) - want_y1).max() <= tol * max(1.0, np.abs(want_y1).max())


def test_gather_leaves_empty_slots_zero_and_honours_beta():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((1, 2, 2, 3)).astype(np.float32)
    iv = M.expert_choice_routing(scores(rng, 1, 2, 2, 2), 6)  # 6 slots, 4 tokens
    g = M.gather_tokens(x, iv)
    assert not g[:, 4:].any()
    y0 = rng.standard_normal((1, 6, 2, 3)).astype(np.float32)
    g2 = M.gather_tokens(x, iv, beta=2.0, y=y0)
    assert np.allclose(g2, g + 2.0 * y0, atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_expert_layers_are_one_dense_product_per_expert(dtype):
    rng = np.random.default_rng(6)
    b, k, e, c, n = 2, 5, 3, 16, 12
    conv = O.to_half if dtype == "float16" else (lambda a: np.ascontiguousarray(a, np.float32))
    x, w, bias = conv(rng.standard_normal((b, k, e, c))), conv(rng.standard_normal((e, n, c)) * 0.3), conv(rng.standard_normal((e, n)))
    y = O.as_float(M.moe_forward(x, w, bias, O.RELU)).astype(np.float64)
    xf, wf, bf = (O.as_float(a).astype(np.float64) for a in (x, w, bias))
    want = np.maximum(np.einsum("bkec,enc->bken", xf, wf) + bf[None, None], 0.0)
    assert np.abs(y - want).max() <= (1e-5 if dtype == "float32" else 1e-2) * np.abs(want).max()
    # an expert's rows do not depend on the other experts' weights
    w2 = np.array(w, copy=True)
    w2[1] = conv(rng.standard_normal((n, c)))
    y2 = M.moe_forward(x, w2, bias, O.RELU)
    assert np.array_equal(np.asarray(y2)[:, :, 0], np.asarray(M.moe_forward(x, w, bias, O.RELU))[:, :, 0])


# ---- the reference's own test baselines (test/backend/test_moe.cpp), at the shapes its tests use ---------------------------------------

def _table(rng, batch, tokens, experts, slots, empty=0.15):
    """A routing table with distinct tokens per expert row, random gates and some empty (-1) slots."""
    table = np.zeros((batch, 2, experts, slots), np.float32)
    for b in range(batch):
        for e in range(experts):
            table[b, 0, e] = rng.permutation(tokens)[:slots]
    table[:, 1] = rng.random((batch, experts, slots), dtype=np.float32)
    hole = rng.random((batch, experts, slots)) < empty
    table[:, 0][hole] = -1.0
    return table


def test_gather_equals_the_reference_tests_baseline():
    """TestGatherTopK: [3, 11, 12, 56], 8 experts, 12 slots (test_moe.cpp:989-1000)."""
    import reference_moe_baselines as R
    rng = np.random.default_rng(21)
    x = rng.standard_normal((3, 11, 12, 56), dtype=np.float32)
    table = _table(rng, 3, 11 * 12, 8, 12)
    assert np.array_equal(M.gather_tokens(x, table), R.gather_tokens(x, table))


def test_scatter_equals_the_reference_tests_baseline():
    """TestScatterTopK: [3, 16, 8, 56] back to [3, 11, 12, 56] (test_moe.cpp:1028-1039). Same additions in the same order: equal bits."""
    import reference_moe_baselines as R
    rng = np.random.default_rng(22)
    x = rng.standard_normal((3, 16, 8, 56), dtype=np.float32)
    table = _table(rng, 3, 11 * 12, 8, 16)
    assert np.array_equal(M.scatter_tokens(x, table, (3, 11, 12, 56)), R.scatter_tokens(x, table, (3, 11, 12, 56)))


def test_hash_and_token_choice_routing_equal_the_reference_tests_baseline():
    """TestRouter: token choice with capacity factor 1.25 on [128, 15, 15, 2] (test_moe.cpp:956-981; a smaller batch here), and the
    baseline's hash branch. Tokens and slots must agree exactly (random fp32 scores have no equal probabilities), gates to rounding:
    the baseline shifts the softmax by the row maximum, the device kernel that the oracle follows by the maximum of score + bias."""
    import reference_moe_baselines as R
    rng = np.random.default_rng(23)
    scores = rng.standard_normal((16, 15, 15, 2), dtype=np.float32)
    cap = R.capacity(1.25, 225, 2)
    assert cap == M.get_capacity(1.25, 225, 2) == 140
    want = R.token_choice_router(scores, cap)
    got = M.token_choice_routing(scores, None, cap)
    assert np.array_equal(got[:, 0], want[:, 0])
    assert np.abs(got[:, 1] - want[:, 1]).max() <= 1e-6
    for experts in (2, 8, 7):
        cap = R.capacity(1.25, 225, experts)
        assert np.array_equal(M.hash_routing(np.zeros((3, 15, 15, experts), np.float32), cap), R.hash_router(3, 225, experts, cap))


def test_expert_layers_equal_the_reference_tests_baseline():
    """TestMixtureOfExperts: [32, 16, 32, 128] -> 64 neurons (test_moe.cpp:1067-1093; a smaller batch here), within the reference
    test's own bound of 1e-4 (the baseline sums a row's products one by one, the oracle in the order of the reference's GEMM)."""
    import reference_moe_baselines as R
    rng = np.random.default_rng(24)
    x = rng.standard_normal((4, 16, 32, 128), dtype=np.float32)
    w = (rng.standard_normal((32, 64, 128), dtype=np.float32) * np.float32(0.1))
    b = rng.standard_normal((32, 64), dtype=np.float32) * np.float32(0.1)
    for relu in (True, False):
        got = M.moe_forward(x, w, b, O.RELU if relu else O.LINEAR)
        want = R.expert_layers(x, w, b, relu)
        assert np.abs(got - want).max() / np.abs(want).max() <= 1e-4
