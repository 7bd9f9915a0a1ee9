"""CPU statement of the mixture-of-experts steps (routing, gather, expert layers, scatter). TEST INFRASTRUCTURE ONLY.

The reference's core dispatches these operations to the CUDA backend only (src/core/math.cpp:1328-1491 does nothing on the CPU), so no
CPU result of the reference's library exists to compare with. What the reference does hold is its own test file,
test/backend/test_moe.cpp, whose CPU baselines its device layers are tested against (difference at most 1e-4 in fp32). The functions
below state what the reference's device kernels compute (src/backend/cuda/kernels/moe.cu; lines cited per function) in plain numpy, and
are pinned as follows (tests/test_oracle_moe.py; the baselines are restated in tests/reference_moe_baselines.py):
  * gather_tokens, scatter_tokens, hash_routing, token_choice_routing (without bias), moe_forward, get_capacity: against those
    baselines at the shapes of the reference's tests - gather and hash exactly, scatter bit for bit (same additions, same order),
    the routed tokens and slots exactly and the gates to 1e-6, the expert layers within the reference test's own 1e-4;
  * expert_choice_routing: PARITY UNPINNED against the reference. The baseline's branch for it (test_moe.cpp:547-566) is nested
    inside the token-choice branch and never runs, and it computes a softmax over the selected scores where the device kernel
    applies a sigmoid (moe.cu:438-479); the function follows the kernel and is pinned by what the mathematics fixes: the top-k
    against a brute-force search, permutation equivariance, gate = sigmoid of the selected score;
  * the bias of token_choice_routing (the baseline has none) and beta != 0 in gather / scatter: by the kernels' text and by
    identities (scatter(gather(x)) = x * (sum of gates per token), beta-linearity).
Two freedoms that the reference's kernels leave are fixed here: (1) ties - the reference's bitonic sorts (and its baseline's std::sort)
order equal scores arbitrarily, here equal scores are ordered by ascending token index; (2) accumulation - the reference scatters with
atomic additions in the storage type (arrival order, one rounding per addition), here contributions are summed in fp32 in ascending
expert order (the order of the reference test's baseline) and rounded once. fp16 results are stored by truncation like everything
else in this backend's CPU counterpart (src/backend/cpu/fp16.hpp:61-68).

Tensors: scores [B, H, W, E]; indices_and_values [B, 2, E, K] in the storage type (plane 0: token indices as numbers, -1 for an empty
slot; plane 1: gate values); gathered tokens [B, K, E, C]; expert weights [E, N, C], bias [E, N].
"""
import numpy as np

import oracle as O


def _f32(a):
    return O.as_float(np.asarray(a)).astype(np.float32)


def _store(values, like):
    """fp32 values -> the storage type of `like` (uint16 fp16 bit patterns by truncation, or float32)."""
    values = np.ascontiguousarray(values, np.float32)
    return O.to_half(values) if np.asarray(like).dtype == np.uint16 else values


def get_capacity(capacity_factor, tokens, experts):
    """src/layers/Router.cpp:62-66."""
    tmp = int(capacity_factor * tokens / experts)
    return tmp if tmp * experts >= tokens else tmp + 1


def expert_choice_routing(scores, capacity):
    """Every expert takes its `capacity` best tokens of each image; gate = sigmoid(score) (moe.cu:438-479). Slot k holds the k-th best."""
    s = _f32(scores)
    b, h, w, e = s.shape
    t = h * w
    s = s.reshape(b, t, e)
    out = np.zeros((b, 2, e, capacity), np.float32)
    out[:, 0] = -1.0
    for n in range(b):
        for j in range(e):
            col = s[n, :, j]
            order = np.lexsort((np.arange(t), -col))  # score descending, token index ascending among equals
            k = min(capacity, t)
            out[n, 0, j, :k] = order[:k]
            out[n, 1, j, :k] = np.float32(1.0) / (np.float32(1.0) + np.exp(-col[order[:k]], dtype=np.float32))
    return _store(out, scores)


def token_choice_routing(scores, bias, capacity):
    """Every token picks the expert with the largest score + bias; gate = softmax(scores)[that expert] with the maximum of score + bias
    as the softmax's shift (moe.cu:191-264); per image, each expert keeps its `capacity` best tokens, best first (moe.cu:266-350)."""
    s = _f32(scores)
    b, h, w, e = s.shape
    t = h * w
    s = s.reshape(b, t, e)
    bs = np.zeros(e, np.float32) if bias is None else _f32(bias)
    out = np.zeros((b, 2, e, capacity), np.float32)
    out[:, 0] = -1.0
    for n in range(b):
        plus = s[n] + bs[None, :]
        choice = np.argmax(plus, axis=1)  # lowest expert index among equals
        shift = plus.max(axis=1)
        ex = np.exp(s[n] - shift[:, None], dtype=np.float32)
        total = np.zeros(t, np.float32)
        for j in range(e):  # sequential fp32 sum over the experts
            total = total + ex[:, j]
        gate = _f32(_store(ex[np.arange(t), choice] / total, scores))  # the reference keeps the per-token gate in the storage type
        for j in range(e):
            mine = np.nonzero(choice == j)[0]
            order = mine[np.lexsort((mine, -gate[mine]))]
            k = min(capacity, order.size)
            out[n, 0, j, :k] = order[:k]
            out[n, 1, j, :k] = gate[order[:k]]
    return _store(out, scores)


def hash_routing(scores, capacity):
    """Token k * E + e goes to slot k of expert e with gate 1 (moe.cu:167-189)."""
    b, h, w, e = np.asarray(scores).shape
    t = h * w
    out = np.zeros((b, 2, e, capacity), np.float32)
    out[:, 0] = -1.0
    for j in range(e):
        for k in range(capacity):
            token = k * e + j
            if token < t:
                out[:, 0, j, k] = token
                out[:, 1, j, k] = 1.0
    return _store(out, scores)


def gather_tokens(x, indices_and_values, beta=0.0, y=None):
    """y[b, k, e, :] = x[b, token(b, e, k), :] + beta * y[b, k, e, :] for filled slots (moe.cu:505-532); empty slots become 0 when
    beta = 0 (the reference leaves them unwritten; nothing downstream reads them) and keep beta * y otherwise."""
    xf = _f32(x)
    iv = _f32(indices_and_values)
    b, h, w, c = xf.shape
    _, _, e, k = iv.shape
    xf = xf.reshape(b, h * w, c)
    out = np.zeros((b, k, e, c), np.float32)
    if beta != 0.0:
        out = np.float32(beta) * _f32(y)
    for n in range(b):
        for j in range(e):
            for s in range(k):
                token = int(iv[n, 0, j, s])
                if token >= 0:
                    out[n, s, j] = xf[n, token] + (out[n, s, j] if beta != 0.0 else 0.0)
    return _store(out, x)


def moe_forward(x, weights, bias=None, act=O.LINEAR, beta=0.0, y=None):
    """y[b, k, e, :] = act(x[b, k, e, :] . w[e]^T + bias[e] + beta * y[b, k, e, :]): one dense layer per expert (moe.cu:1395-1432), each
    evaluated as gemm_ex does (fp32 accumulation over the whole row, one rounding at the end)."""
    x = np.asarray(x)
    b, k, e, c = x.shape
    n = np.asarray(weights).shape[1]
    out = np.zeros((b, k, e, n), x.dtype)
    for j in range(e):
        a = np.ascontiguousarray(x[:, :, j, :]).reshape(b * k, c)
        prev = None if beta == 0.0 else np.ascontiguousarray(np.asarray(y)[:, :, j, :]).reshape(b * k, n)
        d = O.gemm(a, np.ascontiguousarray(np.asarray(weights)[j]), beta=beta, C=prev, bias=None if bias is None else np.ascontiguousarray(np.asarray(bias)[j]),
                   act=act)
        out[:, :, j, :] = d.reshape(b, k, n)
    return out


def scatter_tokens(x, indices_and_values, shape, beta=0.0, y=None):
    """y[b, token, :] = beta * y[b, token, :] + sum over the slots (e ascending, then k) that hold this token of gate * x[b, k, e, :]
    (moe.cu:559-582, with the sum taken in fp32 in that fixed order instead of by atomic additions)."""
    xf = _f32(x)
    iv = _f32(indices_and_values)
    b, k, e, c = xf.shape
    _, h, w, _ = shape
    out = np.zeros((b, h * w, c), np.float32)
    if beta != 0.0:
        out = (np.float32(beta) * _f32(y)).reshape(b, h * w, c)
    for n in range(b):
        for j in range(e):
            for s in range(k):
                token = int(iv[n, 0, j, s])
                if token >= 0:
                    out[n, token] = out[n, token] + iv[n, 1, j, s] * xf[n, s, j]
    return _store(out.reshape(b, h, w, c), x)
