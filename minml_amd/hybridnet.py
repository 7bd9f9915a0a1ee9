"""The on-path part of the hybrid convolution + attention network of benchmark configuration 5, run through the C-ABI.

Topology: the residual trunk of minml_amd.resnet (stem 3x3 conv, `blocks` residual blocks of two Winograd 3x3 convolutions, no head),
then `attention_blocks` attention half-blocks over the board's H*W tokens, each

    h   = rmsnorm(x; gamma)                                   RMSNormalization (reference: src/layers/RMSNormalization.cpp)
    qkv = h W_qkv^T + b_qkv                                   Dense           (gemm_ex on the [B*H*W, C] view, src/layers/Dense.cpp)
    a   = multi-head attention(qkv; relative-position table)  MultiHeadAttention (src/layers/MultiHeadAttention.cpp:35-44 for the table shape)
    x   = a W_o^T + b_o + x                                   Dense with the residual as the product's C operand (beta = 1)

and, with `moe=True`, the feed-forward half of each transformer block as a mixture of experts in the reference's layer sequence
(src/layers/{Router,GatherTokens,MixtureOfExperts,ScatterTokens}.cpp):

    h      = rmsnorm(x; gamma_ffn)
    scores = h W_router^T + b_router                          Dense to one logit per expert
    table  = expert-choice routing(scores)                    Router with capacity factor 2: each of the 8 experts takes 56 of the 225 tokens,
                                                              i.e. two experts per token on average ("top-2-of-8"); gate = sigmoid(score)
    g      = gather(h, table)                                 [B, K, E, C]
    u      = relu(g W_1[e]^T + b_1[e])                        MixtureOfExperts, hidden width 1024
    v      = u W_2[e]^T + b_2[e]                              MixtureOfExperts back to C
    x      = x + scatter(v, table)                            ScatterTokens with beta = 1 (gated sum per token added to x, one rounding)

and a 1x1 policy head. The reference has the mixture-of-experts kernels for its CUDA backend only (src/core/math.cpp:1328-1491
dispatches nothing on the CPU): that half is checked against this repository's own CPU statement of those steps, not against the
reference; `moe=False` leaves it out and keeps exactly the layers that have a CPU reference.
"""
import numpy as np

from . import core as ml
from .conv2d import Conv2D
from .resnet import ResNet


EXPERTS, HIDDEN, CAPACITY_FACTOR = 8, 1024, 2.0


def get_capacity(capacity_factor, tokens, experts):
    """Slots per expert (reference: src/layers/Router.cpp:62-66)."""
    tmp = int(capacity_factor * tokens / experts)
    return tmp if tmp * experts >= tokens else tmp + 1


def make_hybrid_parameters(seed, input_planes, channels, blocks, attention_blocks, heads, board, sigma=0.02, bias_sigma=0.01, experts=EXPERTS,
                           hidden=HIDDEN):
    """fp32 parameters: {"trunk": [(w, b)] for stem + 2 * blocks convolutions, "attention": [dict per half-block], "ffn": [dict per
    mixture-of-experts half-block], "head": (w, b)}. All weight matrices and the position tables are N(0, sigma), biases N(0, bias_sigma),
    the normalisations' gamma 1 + N(0, sigma). The "ffn" entries are drawn after everything else, so that the other parameters do not
    depend on whether the mixture-of-experts halves are used."""
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
    ffn = []
    for _ in range(attention_blocks):
        ffn.append({"gamma": (1.0 + normal((channels,), sigma)).astype(np.float32),
                    "w_router": normal((experts, channels), sigma), "b_router": normal((experts,), bias_sigma),
                    "w_1": normal((experts, hidden, channels), sigma), "b_1": normal((experts, hidden), bias_sigma),
                    "w_2": normal((experts, channels, hidden), sigma), "b_2": normal((experts, channels), bias_sigma)})
    return {"trunk": trunk, "attention": attention, "ffn": ffn, "head": head}


class HybridNet:
    def __init__(self, context, batch, board, input_planes, channels, blocks, heads, dtype, params, to_storage, fused=True, moe=False):
        self.context = context
        self.moe = moe
        self.dtype = ml.dtype_of(dtype)
        self.batch, self.board, self.channels, self.heads = batch, board, channels, heads
        self.trunk = ResNet(context, batch, board, input_planes, channels, blocks, dtype, params["trunk"], to_storage, fused=fused, with_head=False)
        dev = lambda a: ml.toDevice(context, to_storage(a), self.dtype)
        self.attention = [{k: dev(v) for k, v in blk.items()} for blk in params["attention"]]
        self.ffn = [{k: dev(v) for k, v in blk.items()} for blk in params["ffn"]] if moe else []
        if moe:
            self.experts, self.hidden = params["ffn"][0]["w_1"].shape[0], params["ffn"][0]["w_1"].shape[1]
            self.capacity = get_capacity(CAPACITY_FACTOR, board * board, self.experts)
            self.scores = ml.Tensor((batch, board, board, self.experts), self.dtype)
            self.table = ml.Tensor((batch, 2, self.experts, self.capacity), self.dtype)
            self.gathered = ml.Tensor((batch, self.capacity, self.experts, channels), self.dtype)
            self.expert_hidden = ml.Tensor((batch, self.capacity, self.experts, self.hidden), self.dtype)
            self.expert_out = ml.Tensor((batch, self.capacity, self.experts, channels), self.dtype)
        shape = (batch, board, board, channels)
        self.head = Conv2D(context, shape, 1, 1, "linear", True, self.dtype)
        self.head.setWeights(to_storage(params["head"][0]), to_storage(params["head"][1]))
        self.normed = ml.Tensor(shape, self.dtype)
        self.qkv = ml.Tensor((batch, board, board, 3 * channels), self.dtype)
        self.attended = ml.Tensor(shape, self.dtype)
        self.stream = [ml.Tensor(shape, self.dtype) for _ in range(3)]
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
            out = next(t for t in self.stream if t is not x)
            ml.gemm_ex(ctx, out.view((rows, c)), 1.0, "n", self.attended.view((rows, c)), "t", p["w_out"], 1.0, x.view((rows, c)), p["b_out"], "linear")
            self._observe("block%d" % index, out)
            x = out
            if self.moe:
                f = self.ffn[index]
                ml.set_timer_label("ffn")
                ml.rmsnormForward(ctx, x, self.normed, f["gamma"])
                self._observe("ffn_rmsnorm%d" % index, self.normed)
                ml.gemm_ex(ctx, self.scores.view((rows, self.experts)), 1.0, "n", self.normed.view((rows, c)), "t", f["w_router"], 0.0, None, f["b_router"],
                           "linear")
                self._observe("scores%d" % index, self.scores)
                ml.expertChoiceRoutingForward(ctx, self.scores, self.table)
                self._observe("table%d" % index, self.table)
                ml.gatherTokensForward(ctx, self.normed, self.table, 0.0, self.gathered)
                ml.moeForward(ctx, self.gathered, f["w_1"], f["b_1"], 0.0, self.expert_hidden, "relu")
                self._observe("hidden%d" % index, self.expert_hidden)
                ml.moeForward(ctx, self.expert_hidden, f["w_2"], f["b_2"], 0.0, self.expert_out, "linear")
                self._observe("experts%d" % index, self.expert_out)
                # the residual addition rides on the scatter: x = 1 * x + gated sum, accumulated in fp32 and rounded once
                ml.scatterTokensForward(ctx, self.expert_out, self.table, 1.0, x)
                self._observe("ffn%d" % index, x)
        ml.set_timer_label("head")
        self.head.forward([x], self.output, self.workspace)
        ml.set_timer_label(None)
        self.last = x
        return self.output

    def flops_per_forward(self):
        rows, c = self.batch * self.board * self.board, self.channels
        tokens = self.board * self.board
        per_block = 2.0 * rows * c * 3 * c + 2.0 * rows * c * c + 4.0 * self.batch * self.heads * tokens * tokens * (c // self.heads)
        if self.moe:
            slots = self.batch * self.capacity * self.experts
            per_block += 2.0 * rows * c * self.experts + 2 * 2.0 * slots * c * self.hidden
        return self.trunk.flops_per_forward() + len(self.attention) * per_block + 2.0 * rows * c
