"""The on-path part of the hybrid convolution + attention network of benchmark configuration 5, run through the C-ABI.

Topology: the residual trunk of minml_amd.resnet (stem 3x3 conv, `blocks` residual blocks of two Winograd 3x3 convolutions, no head),
then `attention_blocks` attention half-blocks over the board's H*W tokens, each

    h   = rmsnorm(x; gamma)                                   RMSNormalization (reference: src/layers/RMSNormalization.cpp)
    qkv = h W_qkv^T + b_qkv                                   Dense           (gemm_ex on the [B*H*W, C] view, src/layers/Dense.cpp)
    a   = multi-head attention(qkv; relative-position table)  MultiHeadAttention (src/layers/MultiHeadAttention.cpp:35-44 for the table shape)
    x   = a W_o^T + b_o + x                                   Dense with the residual as the product's C operand (beta = 1)

and a 1x1 policy head. The feed-forward half of the configuration's transformer blocks is a top-2-of-8 mixture of experts; the reference
has those kernels for its CUDA backend only (src/core/math.cpp:1328-1491 dispatches nothing on the CPU), so there is no CPU result to
compare with and that half is left out here: this network is every layer of configuration 5 that has a CPU reference.
"""
import numpy as np

from . import core as ml
from .conv2d import Conv2D
from .resnet import ResNet


def make_hybrid_parameters(seed, input_planes, channels, blocks, attention_blocks, heads, board, sigma=0.02, bias_sigma=0.01):
    """fp32 parameters: {"trunk": [(w, b)] for stem + 2 * blocks convolutions, "attention": [dict per half-block], "head": (w, b)}.
    All weight matrices and the position tables are N(0, sigma), biases N(0, bias_sigma), the normalisation's gamma 1 + N(0, sigma)."""
    rng = np.random.default_rng(seed)
    normal = lambda shape, s: (rng.standard_normal(shape) * s).astype(np.float32)
    trunk = [(normal((channels, 3, 3, input_planes), sigma), normal((channels,), bias_sigma))]
    for _ in range(2 * blocks):
        trunk.append((normal((channels, 3, 3, channels), sigma), normal((channels,), bias_sigma)))
    size = 2 * board - 1
    attention = []
    for _ in range(attention_blocks):
        attention.append({"gamma": (1.0 + normal((channels,), sigma)).astype(np.float32),
                          "w_qkv": normal((3 * channels, channels), sigma), "b_qkv": normal((3 * channels,), bias_sigma),
                          "table": normal((heads, size, (size + 3) // 4 * 4), sigma),
                          "w_out": normal((channels, channels), sigma), "b_out": normal((channels,), bias_sigma)})
    head = (normal((1, 1, 1, channels), sigma), normal((1,), bias_sigma))
    return {"trunk": trunk, "attention": attention, "head": head}


class HybridNet:
    def __init__(self, context, batch, board, input_planes, channels, blocks, heads, dtype, params, to_storage, fused=True):
        self.context = context
        self.dtype = ml.dtype_of(dtype)
        self.batch, self.board, self.channels, self.heads = batch, board, channels, heads
        self.trunk = ResNet(context, batch, board, input_planes, channels, blocks, dtype, params["trunk"], to_storage, fused=fused, with_head=False)
        dev = lambda a: ml.toDevice(context, to_storage(a), self.dtype)
        self.attention = [{k: dev(v) for k, v in blk.items()} for blk in params["attention"]]
        shape = (batch, board, board, channels)
        self.head = Conv2D(context, shape, 1, 1, "linear", True, self.dtype)
        self.head.setWeights(to_storage(params["head"][0]), to_storage(params["head"][1]))
        self.normed = ml.Tensor(shape, self.dtype)
        self.qkv = ml.Tensor((batch, board, board, 3 * channels), self.dtype)
        self.attended = ml.Tensor(shape, self.dtype)
        self.stream = [ml.Tensor(shape, self.dtype) for _ in range(2)]
        self.output = ml.Tensor((batch, board, board, 1), self.dtype)
        self.workspace = ml.Tensor((max(1, self.head.getWorkspaceSize()),), self.dtype)
        self.observer = None

    def setInput(self, x_storage):
        self.trunk.setInput(x_storage)

    def _observe(self, name, tensor):
        if self.observer is not None:
            self.observer(name, tensor)

    def forward(self):
        ctx, rows, c = self.context, self.batch * self.board * self.board, self.channels
        ml.set_timer_label("trunk")
        x = self.trunk.forward()
        self._observe("trunk", x)
        for index, p in enumerate(self.attention):
            ml.set_timer_label("attention")
            ml.rmsnormForward(ctx, x, self.normed, p["gamma"])
            self._observe("rmsnorm%d" % index, self.normed)
            ml.gemm_ex(ctx, self.qkv.view((rows, 3 * c)), 1.0, "n", self.normed.view((rows, c)), "t", p["w_qkv"], 0.0, None, p["b_qkv"], "linear")
            self._observe("qkv%d" % index, self.qkv)
            ml.multiHeadAttentionForward(ctx, self.qkv, self.attended, p["table"], None, None, None, self.heads, False)
            self._observe("attention%d" % index, self.attended)
            out = self.stream[index % 2]
            ml.gemm_ex(ctx, out.view((rows, c)), 1.0, "n", self.attended.view((rows, c)), "t", p["w_out"], 1.0, x.view((rows, c)), p["b_out"], "linear")
            self._observe("block%d" % index, out)
            x = out
        ml.set_timer_label("head")
        self.head.forward([x], self.output, self.workspace)
        ml.set_timer_label(None)
        self.last = x
        return self.output

    def flops_per_forward(self):
        rows, c = self.batch * self.board * self.board, self.channels
        tokens = self.board * self.board
        per_block = 2.0 * rows * c * 3 * c + 2.0 * rows * c * c + 4.0 * self.batch * self.heads * tokens * tokens * (c // self.heads)
        return self.trunk.flops_per_forward() + len(self.attention) * per_block + 2.0 * rows * c
