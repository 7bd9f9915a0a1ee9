"""The CPU baselines that the reference's own mixture-of-experts tests compare its device kernels with (test/backend/test_moe.cpp),
restated in numpy for the parity tests. The reference's tests run these baselines on the CPU and its CUDA layers on the device and ask
for a difference of at most 1e-4 in fp32 (test_moe.cpp:956-1093); here they stand in for the missing CPU implementation of the
reference's core (src/core/math.cpp:1328-1491 dispatches these operations to CUDA only) as the closest thing to a reference result.

Not restated: the baseline's expert-choice branch (test_moe.cpp:547-566). It sits inside the token-choice branch, is never reached, and
computes something else than the device kernel (a softmax over each expert's selected scores where kernel_expert_choice_routing applies
a sigmoid to every selected score, src/backend/cuda/kernels/moe.cu:438-479).
"""
import numpy as np


def capacity(capacity_factor, tokens, experts):
    """test_moe.cpp:467-468 (the same expression as src/layers/Router.cpp:62-66)."""
    tmp = int(capacity_factor * tokens / experts)
    return tmp if tmp * experts >= tokens else tmp + 1


def hash_router(batch, tokens, experts, cap):
    """test_moe.cpp:470-487: slot k of expert e holds token k * E + e with gate 1, or -1 / 0 past the last token."""
    out = np.zeros((batch, 2, experts, cap), np.float32)
    for e in range(experts):
        for k in range(cap):
            token = k * experts + e
            out[:, 0, e, k] = token if token < tokens else -1
            out[:, 1, e, k] = 1.0 if token < tokens else 0.0
    return out


def softmax_rows(x):
    """test_moe.cpp:104-130 in fp32: running maximum, exponentials summed in column order, one division per element."""
    x = np.asarray(x, np.float32)
    shifted = np.exp(x - x.max(axis=1, keepdims=True), dtype=np.float32)
    total = np.zeros(x.shape[0], np.float32)
    for j in range(x.shape[1]):
        total = total + shifted[:, j]
    return shifted / total[:, None]


def token_choice_router(scores, cap):
    """test_moe.cpp:492-545: softmax over the experts, every token takes the expert with the largest probability (the first among
    equals), the tokens are ordered by expert and, within an expert, by falling probability, and each expert keeps the first `cap`.
    std::sort leaves the order of equal probabilities open; here they keep their token order."""
    b, h, w, e = scores.shape
    t = h * w
    out = np.zeros((b, 2, e, cap), np.float32)
    out[:, 0] = -1.0
    for n in range(b):
        p = softmax_rows(np.asarray(scores[n], np.float32).reshape(t, e))
        choice = np.argmax(p, axis=1)
        value = p[np.arange(t), choice]
        order = sorted(range(t), key=lambda i: (choice[i], -float(value[i]), i))
        counter = [0] * e
        for i in order:
            j = int(choice[i])
            if counter[j] < cap:
                out[n, 0, j, counter[j]] = i
                out[n, 1, j, counter[j]] = value[i]
                counter[j] += 1
    return out


def gather_tokens(x, table):
    """test_moe.cpp:239-266: zeros, then row (b, k, e) = token table[b, 0, e, k] of image b where that index is not negative."""
    b, h, w, c = x.shape
    _, _, e, k = table.shape
    flat = np.asarray(x, np.float32).reshape(b, h * w, c)
    out = np.zeros((b, k, e, c), np.float32)
    for n in range(b):
        for j in range(e):
            for s in range(k):
                token = int(table[n, 0, j, s])
                if token >= 0:
                    out[n, s, j] = flat[n, token]
    return out


def scatter_tokens(x, table, shape):
    """test_moe.cpp:301-335 with T = float: zeros, then for every expert, image and slot in that order the token's row gains
    row (b, k, e) times the slot's gate (one multiplication, one addition, fp32)."""
    b, k, e, c = x.shape
    out = np.zeros((b, shape[1] * shape[2], c), np.float32)
    x = np.asarray(x, np.float32)
    for j in range(e):
        for n in range(b):
            for s in range(k):
                token = int(table[n, 0, j, s])
                if token >= 0:
                    out[n, token] = out[n, token] + x[n, s, j] * np.float32(table[n, 1, j, s])
    return out.reshape(shape)


def expert_layers(x, weights, bias, relu):
    """BaselineMixtureOfExperts::forward (test_moe.cpp:843-870): per expert y = x w^T by a plain triple loop in fp32 (baseline_gemm,
    test_moe.cpp:61-102: products summed in k order), then bias and activation."""
    b, k, e, c = x.shape
    n = weights.shape[1]
    out = np.zeros((b, k, e, n), np.float32)
    for j in range(e):
        a = np.asarray(x[:, :, j, :], np.float32).reshape(b * k, c)
        acc = np.zeros((b * k, n), np.float32)
        wj = np.asarray(weights[j], np.float32)
        for i in range(c):  # sequential fp32 accumulation over k, as the baseline's inner loop
            acc = acc + a[:, i:i + 1] * wj[None, :, i]
        acc = acc + np.asarray(bias[j], np.float32)[None, :]
        if relu:
            acc = np.maximum(acc, np.float32(0.0))
        out[:, :, j, :] = acc.reshape(b, k, n)
    return out
