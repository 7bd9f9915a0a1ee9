"""Kernels whose dynamic LDS grows with the board: a first launch on a small board must not pin the kernel's LDS limit, a later launch of
the SAME instantiation on a board that needs more than the 64 KB default has to raise it. This file is collected before the other GPU
tests on purpose, so that these instantiations meet their small shape first in the process (attention: fp32, heads of 32, no table —
20 KB at 9x9, 92 KB at 19x19; fused output/input transform: fp32, 64-channel slices, ReLU without residual — 21 KB at 9x9, 93 KB at 19x19)."""
import numpy as np
import pytest

import oracle as O
from minml_amd import core as ml
from util import max_abs_rel, mismatches, random_tensor

pytestmark = pytest.mark.gpu


def test_attention_small_board_then_large_board(ctx):
    rng = np.random.default_rng(5)
    for board in (9, 19, 9):
        x = random_tensor(rng, (2, board, board, 3 * 64), "float32")
        y = ml.Tensor((2, board, board, 64), "float32")
        ml.multiHeadAttentionForward(ctx, ml.toDevice(ctx, x), y, None, None, None, None, 2, False)
        assert max_abs_rel(y.copyToHost(ctx), O.multi_head_attention_forward(x, 2, None, False)) <= 1e-4


def test_fused_transform_small_board_then_large_board(ctx):
    rng = np.random.default_rng(6)
    c = 64
    for board in (9, 19, 9):
        shape = (2, board, board, c)
        tiles = 2 * ((board + 3) // 4) ** 2
        m = random_tensor(rng, (36, tiles, c), "float32")
        bias = random_tensor(rng, (c,), "float32")
        dv = ml.Tensor((36, tiles, c), "float32")
        ml.winogradOutputInputTransform(ctx, (c, 3, 3, c), ml.toDevice(ctx, m), shape, None, ml.toDevice(ctx, bias), None, O.RELU, dv)
        want = O.winograd_input_transform(O.winograd_output_transform(m, shape, bias, None, O.RELU))
        assert mismatches(dv.copyToHost(ctx), want) == 0
