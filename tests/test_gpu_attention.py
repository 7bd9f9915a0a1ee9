"""RMS normalisation and multi-head attention with a relative-position table on the GPU against the CPU oracle and the reference's
fixtures, through the C-ABI.

Tolerances (max-abs relative error per result tensor): fp32 1e-4, fp16 1e-2. The attention kernel accumulates the softmax over blocks of
32 keys with a running maximum and runs both products on MFMA (fp16 probabilities in the fp16 form), the normalisation sums its squares
across a wavefront: results agree with the sequential CPU loops to rounding, not bit for bit."""
import numpy as np
import pytest

import oracle as O
from minml_amd import core as ml
from util import TOL, max_abs_rel, mismatches, random_tensor

pytestmark = pytest.mark.gpu


def attention(ctx, x, heads, table=None, symmetric=False):
    parts = 2 if symmetric else 3
    dtype = "float16" if x.dtype == np.uint16 else "float32"
    y = ml.Tensor(x.shape[:3] + (x.shape[3] // parts,), dtype)
    y.zeroall(ctx)
    ml.multiHeadAttentionForward(ctx, ml.toDevice(ctx, x), y, None if table is None else ml.toDevice(ctx, table), None, None, None, heads, symmetric)
    return y.copyToHost(ctx)


def rmsnorm(ctx, x, gamma=None):
    dtype = "float16" if x.dtype == np.uint16 else "float32"
    y = ml.Tensor(x.shape, dtype)
    ml.rmsnormForward(ctx, ml.toDevice(ctx, x), y, None if gamma is None else ml.toDevice(ctx, gamma))
    return y.copyToHost(ctx)


def test_against_reference_fixtures(ctx, golden):
    g = golden
    assert max_abs_rel(rmsnorm(ctx, g["rms_x"], g["rms_g"]), g["rms_y"]) <= 1e-4
    assert max_abs_rel(rmsnorm(ctx, g["rms_x"]), g["rms_y_plain"]) <= 1e-4
    assert max_abs_rel(attention(ctx, g["mha_x"], 4, g["mha_table"]), g["mha_y"]) <= 1e-4  # heads of 8: the plain kernel
    assert max_abs_rel(attention(ctx, g["mha_x"], 4), g["mha_y_plain"]) <= 1e-4
    assert max_abs_rel(attention(ctx, g["mha_sym_x"], 2, None, True), g["mha_sym_y"]) <= 1e-4  # heads of 16


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("shape", [(230, 256), (64, 15, 15, 64), (7, 100), (5, 33), (3, 1), (9, 1024), (4, 2056), (1000, 8),
                                   (123, 43)])  # the last: the reference's own test (test/backend/test_normalization.cpp:977-986)
def test_rmsnorm_shapes(ctx, dtype, shape):
    rng = np.random.default_rng(sum(shape))
    x, gamma = random_tensor(rng, shape, dtype, 2.0), random_tensor(rng, shape[-1:], dtype)
    assert max_abs_rel(rmsnorm(ctx, x, gamma), O.rmsnorm_forward(x, gamma)) <= TOL[dtype]
    assert max_abs_rel(rmsnorm(ctx, x), O.rmsnorm_forward(x)) <= TOL[dtype]


def test_rmsnorm_in_place_and_zero_rows(ctx):
    rng = np.random.default_rng(1)
    x = random_tensor(rng, (37, 256), "float16", 3.0)
    x[5] = 0  # a zero row stays zero: 0 / (1e-6 + 0)
    d = ml.toDevice(ctx, x)
    ml.rmsnormForward(ctx, d, d, None)
    got = d.copyToHost(ctx)
    assert mismatches(got, rmsnorm(ctx, x)) == 0
    assert not O.as_float(got)[5].any() and np.isfinite(O.as_float(got)).all()


@pytest.mark.parametrize("dtype", ["float32", "float16"])
@pytest.mark.parametrize("case", [
    # (batch, height, width, heads, head_dim, r or 0, symmetric)
    (3, 15, 15, 8, 32, 15, False),   # the hybrid network's block: 225 tokens, 8 heads of 32, full-range table
    (2, 15, 15, 2, 32, 4, False),    # clamped offsets
    (2, 15, 15, 4, 32, 0, False),    # no table
    (2, 8, 8, 2, 32, 8, False),      # 64 tokens: no padding rows
    (2, 5, 7, 2, 32, 3, False),      # 35 tokens: one full and one ragged block of keys
    (1, 1, 1, 1, 32, 1, False),      # a single token attends to itself
    (2, 19, 19, 2, 64, 10, False),   # 361 tokens, heads of 64
    (1, 9, 9, 1, 128, 5, False),     # heads of 128
    (2, 15, 15, 4, 32, 8, True),     # symmetric layout: k = q
    (2, 6, 5, 3, 24, 3, False),      # heads of 24: the plain kernel
    (1, 20, 20, 2, 16, 0, True),     # heads of 16, 400 tokens: the plain kernel
    (3, 13, 14, 4, 14, 14, False),   # the reference's own test: 56 channels in 4 heads, table range max(13, 14) (test/backend/test_attention.cpp:441-451)
])
def test_attention_shapes(ctx, dtype, case):
    b, h, w, heads, d, r, symmetric = case
    rng = np.random.default_rng(b * 1000 + h * 100 + heads * 10 + d)
    parts = 2 if symmetric else 3
    x = random_tensor(rng, (b, h, w, parts * heads * d), dtype, 1.5)
    table = None
    if r > 0:
        size = 2 * r - 1
        table = random_tensor(rng, (heads, size, (size + 3) // 4 * 4), dtype, 2.0)
    got = attention(ctx, x, heads, table, symmetric)
    want = O.multi_head_attention_forward(x, heads, table, symmetric)
    assert np.isfinite(O.as_float(got)).all()
    assert max_abs_rel(got, want) <= TOL[dtype]


def test_attention_special_cases(ctx):
    """Equal keys: every output is the mean of the values. A table that forbids every offset but one: each token copies the value of
    that neighbour. Sharp rows (large logits) stay finite through the running-maximum rescaling."""
    rng = np.random.default_rng(2)
    b, h, w, heads, d = 2, 15, 15, 2, 32
    e = heads * d
    x = rng.standard_normal((b, h, w, 3, heads, d)).astype(np.float32)
    x[:, :, :, 1] = x[0, 0, 0, 1]
    y = attention(ctx, x.reshape(b, h, w, 3 * e), heads).reshape(b, h, w, heads, d)
    assert np.abs(y - x[:, :, :, 2].astype(np.float64).mean(axis=(1, 2), keepdims=True)).max() <= 1e-5
    x = rng.standard_normal((b, h, w, 3 * e)).astype(np.float32)
    table = np.full((heads, 7, 8), -1.0e4, np.float32)
    table[:, 3 + 1, 3 - 2] = 0.0  # key one row below, two columns to the left of the query
    y = attention(ctx, x, heads, table)
    v = x.reshape(b, h, w, 3, e)[:, :, :, 2]
    assert np.abs(y[:, :h - 1, 2:] - v[:, 1:, :w - 2]).max() <= 1e-5
    sharp = (rng.standard_normal((1, 15, 15, 3 * e)) * 30).astype(np.float32)  # logits in the hundreds
    got = attention(ctx, sharp, heads)
    assert np.isfinite(got).all() and max_abs_rel(got, O.multi_head_attention_forward(sharp, heads)) <= 1e-4


def test_attention_full_size_properties(ctx):
    """The hybrid configuration's size (B = 256, 15x15, 8 heads of 32, fp16): images are independent (the first ones reproduce a small
    batch bit for bit, which is checked against the oracle), repeated launches give the same bits, and a permutation of the heads
    permutes the output."""
    rng = np.random.default_rng(3)
    x = random_tensor(rng, (256, 15, 15, 768), "float16")
    table = random_tensor(rng, (8, 29, 32), "float16")
    a = attention(ctx, x, 8, table)
    assert mismatches(a, attention(ctx, x, 8, table)) == 0
    small = attention(ctx, x[:2], 8, table)
    assert mismatches(a[:2], small) == 0
    assert max_abs_rel(small, O.multi_head_attention_forward(x[:2], 8, table)) <= 1e-2
    perm = np.array([3, 0, 7, 1, 6, 2, 5, 4])
    xp = np.ascontiguousarray(x[:8].reshape(8, 15, 15, 3, 8, 32)[:, :, :, :, perm]).reshape(8, 15, 15, 768)
    got = attention(ctx, xp, 8, np.ascontiguousarray(table[perm]))
    assert mismatches(got.reshape(8, 15, 15, 8, 32), a[:8].reshape(8, 15, 15, 8, 32)[:, :, :, perm]) == 0


def test_workspace_size_and_bad_arguments(ctx):
    assert ml.multiHeadAttentionGetWorkspaceSize(ctx, (256, 15, 15, 768), (8, 29, 32), 8, False) == 0
    assert ml.multiHeadAttentionGetWorkspaceSize(ctx, (2, 15, 15, 768), (8, 29, 32), 8, True) == 2 * 2 * 8 * 225 * 225
    x = ml.Tensor((2, 4, 4, 96), "float32")
    with pytest.raises(ValueError):
        ml.multiHeadAttentionForward(ctx, x, ml.Tensor((2, 4, 4, 48), "float32"), None, None, None, None, 4, False)  # 96 / 3 = 32 channels out
    with pytest.raises(ValueError):
        ml.multiHeadAttentionForward(ctx, x, ml.Tensor((2, 4, 4, 32), "float32"), None, None, None, None, 5, False)  # 32 % 5
    with pytest.raises(ValueError):
        ml.multiHeadAttentionForward(ctx, x, ml.Tensor((2, 4, 4, 32), "float32"), ml.Tensor((4, 5, 5), "float32"), None, None, None, 4, False)
    with pytest.raises(ValueError):
        ml.multiHeadAttentionForward(ctx, x, ml.Tensor((2, 4, 4, 32), "float32"), None, None, None, ml.Tensor((2 * 4 * 16 * 16,), "float32"), 4, False)
    with pytest.raises(ValueError):
        ml.rmsnormForward(ctx, x, ml.Tensor((2, 4, 4, 96), "float32"), ml.Tensor((95,), "float32"))


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_attention_block_after_a_trunk(ctx, dtype):
    """The attention half of a transformer block on a trunk output [B, 15, 15, 256], every step on the device against the same chain of
    oracle calls: RMS normalisation -> Dense 256 -> 768 (q, k, v) -> attention with 8 heads and a full-range table -> Dense 256 -> 256
    with the block's input as residual (Dense rides on gemm_ex with beta = 1, as the reference's fused Add does)."""
    rng = np.random.default_rng(31)
    batch, board, c, heads = 8, 15, 256, 8
    rows = batch * board * board
    trunk = random_tensor(rng, (batch, board, board, c), dtype)
    gamma = random_tensor(rng, (c,), dtype, 0.2)
    w_qkv, b_qkv = random_tensor(rng, (3 * c, c), dtype, 0.08), random_tensor(rng, (3 * c,), dtype, 0.1)
    w_out, b_out = random_tensor(rng, (c, c), dtype, 0.08), random_tensor(rng, (c,), dtype, 0.1)
    table = random_tensor(rng, (heads, 2 * board - 1, 32), dtype)
    dt = ml.toDevice(ctx, trunk)
    normed = ml.Tensor((batch, board, board, c), dtype)
    ml.rmsnormForward(ctx, dt, normed, ml.toDevice(ctx, gamma))
    qkv = ml.Tensor((batch, board, board, 3 * c), dtype)
    ml.gemm_ex(ctx, qkv.view((rows, 3 * c)), 1.0, "n", normed.view((rows, c)), "t", ml.toDevice(ctx, w_qkv), 0.0, None, ml.toDevice(ctx, b_qkv), "linear")
    mixed = ml.Tensor((batch, board, board, c), dtype)
    ml.multiHeadAttentionForward(ctx, qkv, mixed, ml.toDevice(ctx, table), None, None, None, heads, False)
    out = ml.Tensor((batch, board, board, c), dtype)
    ml.gemm_ex(ctx, out.view((rows, c)), 1.0, "n", mixed.view((rows, c)), "t", ml.toDevice(ctx, w_out), 1.0, dt.view((rows, c)), ml.toDevice(ctx, b_out), "linear")
    want = O.rmsnorm_forward(trunk, gamma)
    assert max_abs_rel(normed.copyToHost(ctx), want) <= TOL[dtype]
    want = O.gemm(want.reshape(rows, c), w_qkv, bias=b_qkv).reshape(batch, board, board, 3 * c)
    assert max_abs_rel(qkv.copyToHost(ctx), want) <= TOL[dtype] * 2
    want = O.multi_head_attention_forward(want, heads, table)
    assert max_abs_rel(mixed.copyToHost(ctx), want) <= TOL[dtype] * 3
    want = O.gemm(want.reshape(rows, c), w_out, beta=1.0, C=trunk.reshape(rows, c), bias=b_out).reshape(batch, board, board, c)
    assert max_abs_rel(out.copyToHost(ctx), want) <= TOL[dtype] * 4  # four chained steps


def test_rmsnorm_full_size_properties(ctx):
    """The hybrid configuration's tensor (256 x 15 x 15 tokens of 256 channels, fp16): without gamma every row leaves with unit
    root-mean-square, scaling the input by a power of two changes no bit (up to the 1e-6 in the denominator), and a sample of rows
    matches the oracle."""
    rng = np.random.default_rng(4)
    x = random_tensor(rng, (256, 15, 15, 256), "float16", 2.0)
    y = rmsnorm(ctx, x)
    values = O.as_float(y).astype(np.float64)
    assert np.abs(np.sqrt((values ** 2).mean(axis=-1)) - 1.0).max() <= 2e-3  # truncation of 256 outputs per row
    doubled = O.to_half(O.as_float(x) * np.float32(2.0))
    assert mismatches(rmsnorm(ctx, doubled), y) <= y.size // 2000  # the 1e-6 moves a few results by one truncation step
    assert max_abs_rel(y[7:9], O.rmsnorm_forward(x[7:9])) <= 1e-2
