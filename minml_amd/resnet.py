"""The synthetic board-game residual network of the benchmark configurations, executed layer by layer through Conv2D.

Topology (after the reference's FoldAdd graph pass, src/graph/graph_optimizers.cpp:186-218, which turns Add(x, conv(y)) into a
two-input Conv2D): stem 3x3 conv (+bias, ReLU); `blocks` residual blocks of conv3x3(+bias, ReLU) -> conv3x3(+bias, +block input,
ReLU); policy head 1x1 conv to one channel (+bias, linear). Layers run in insertion order on one context and share one workspace sized
to the largest request, as the reference's Graph does (src/graph/Graph.cpp:241-248,578-587).

`chunk` splits the batch into sub-batches that are pushed through the whole network one after the other. The layer entry points are
batch-size agnostic, so this changes nothing in the results; it bounds the workspace (2 x 36 x 16 x chunk x C elements). Measured on
MI355X, sub-batches small enough for the Winograd matrices to stay in the 256 MB last-level cache between the transform and GEMM
kernels were not faster than streaming the whole batch through HBM, so the default is the whole batch.
"""
import numpy as np

from . import backend as B
from . import core as ml
from .conv2d import Conv2D


# positions per sub-batch pushed through the whole network at once, by storage type (measured choice: the whole benchmark batch)
DEFAULT_CHUNK = {"float16": 1024, "float32": 256}


def he_normal_weights(rng, shape):
    """He-normal: sigma = sqrt(2 / fan_in), fan_in = k*k*Cin."""
    fan_in = shape[1] * shape[2] * shape[3]
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)


def make_parameters(seed, input_planes, channels, blocks, bias_sigma=0.01):
    """fp32 parameters of the net as a list of (weights [Cout,k,k,Cin], bias [Cout]); stem, 2*blocks convs, head."""
    rng = np.random.default_rng(seed)
    params = [(he_normal_weights(rng, (channels, 3, 3, input_planes)), (rng.standard_normal(channels) * bias_sigma).astype(np.float32))]
    for _ in range(2 * blocks):
        params.append((he_normal_weights(rng, (channels, 3, 3, channels)), (rng.standard_normal(channels) * bias_sigma).astype(np.float32)))
    params.append((he_normal_weights(rng, (1, 1, 1, channels)), (rng.standard_normal(1) * bias_sigma).astype(np.float32)))
    return params


def make_input(seed, batch, board, planes, p=0.3):
    """Binary feature planes, Bernoulli(p), as fp32 0/1."""
    rng = np.random.default_rng(seed + 1000003)
    return (rng.random((batch, board, board, planes)) < p).astype(np.float32)


class ResNet:
    def __init__(self, context, batch, board, input_planes, channels, blocks, dtype, params_host, to_storage, chunk=None, fused=False):
        """params_host: list from make_parameters; to_storage: fp32 ndarray -> ndarray in the storage type (identity or fp16 bits)."""
        self.context = context
        self.fused = fused
        # True: also fuse across the residual blocks' boundaries (the block's result is written and transformed for the next block in one
        # launch). Identical results and less memory traffic, but measured 0.3 % to 1 % slower on MI355X than two launches there, whose
        # second one finds the block's result in the last-level cache
        self.fuse_block_boundary = False
        # True: whole layers (product + both transforms) as one launch that keeps the product in the L2 cache. Identical results, but
        # measured slower than the separate product and fused transform on MI355X (about 430 us against 290 us per layer at batch 1024),
        # so it is off unless asked for
        self.fuse_layers = False
        self.dtype = ml.dtype_of(dtype)
        self.batch, self.board, self.channels, self.blocks = batch, board, channels, blocks
        self.chunk = min(chunk or batch, batch)
        cb = self.chunk
        self.layers = []
        shape = (cb, board, board, input_planes)
        stem = Conv2D(context, shape, channels, 3, "relu", True, self.dtype)
        self.layers.append(stem)
        shape = (cb, board, board, channels)
        for _ in range(2 * blocks):
            self.layers.append(Conv2D(context, shape, channels, 3, "relu", True, self.dtype))
        self.layers.append(Conv2D(context, shape, 1, 1, "linear", True, self.dtype))
        for layer, (w, b) in zip(self.layers, params_host):
            layer.setWeights(to_storage(w), to_storage(b))

        ws_elems = max(1, max(l.getWorkspaceSize() for l in self.layers))
        self.workspace = ml.Tensor((ws_elems,), self.dtype, context.device_index)
        # three rotating activation buffers per chunk: block input, intermediate, block output
        self.act = [ml.Tensor((cb, board, board, channels), self.dtype, context.device_index) for _ in range(3)]
        self.input = ml.Tensor((batch, board, board, input_planes), self.dtype, context.device_index)
        self.output = ml.Tensor((batch, board, board, 1), self.dtype, context.device_index)

    def setInput(self, x_storage):
        self.input.copyFromHost(self.context, x_storage)

    def _view_batch(self, tensor, start, count):
        per = tensor.volume() // tensor.shape[0]
        return tensor.view((count,) + tensor.shape[1:], start * per)

    def forward(self, fused=None):
        """One pass over the whole batch; asynchronous on the context's stream. With `fused` (default: the constructor's choice) the
        output transform of every 3x3 layer is merged with the input transform of the next one; results are bit-identical."""
        if self.fused if fused is None else fused:
            return self._forward_fused()
        for start in range(0, self.batch, self.chunk):
            n = min(self.chunk, self.batch - start)
            x = self._view_batch(self.input, start, n)
            a, b, c = (self._view_batch(t, 0, n) for t in self.act)
            ml.set_timer_label("stem")
            self.layers[0].forward([x], a, self.workspace)
            for blk in range(self.blocks):
                ml.set_timer_label("block_conv1")
                self.layers[1 + 2 * blk].forward([a], b, self.workspace)
                ml.set_timer_label("block_conv2")
                self.layers[2 + 2 * blk].forward([b, a], c, self.workspace)
                a, c = c, a
            ml.set_timer_label("head")
            self.layers[-1].forward([a], self._view_batch(self.output, start, n), self.workspace)
            ml.set_timer_label(None)
        return self.output

    def _forward_fused(self):
        """Same network with cross-layer fusion inside each residual block: the result of the block's first convolution goes from its
        output transform to the second convolution's input transform through LDS and is never written to memory."""
        L = self.layers
        for start in range(0, self.batch, self.chunk):
            n = min(self.chunk, self.batch - start)
            x = self._view_batch(self.input, start, n)
            a, b, c = (self._view_batch(t, 0, n) for t in self.act)
            ws = self.workspace
            ml.set_timer_label("stem")
            # the stem has fewer input than output channels: its output matrices start below the end of the next layer's input
            # matrices in the shared workspace, so its two transforms stay separate calls
            L[0].forward([x], a, ws)
            if self.blocks > 0:
                ml.set_timer_label("block_conv1")
                L[1].winograd_input(a, ws)
            for blk in range(self.blocks):
                conv1, conv2 = L[1 + 2 * blk], L[2 + 2 * blk]
                ml.set_timer_label("block_conv1")
                if self.fuse_layers:
                    conv1.winograd_layer_into(conv2, n, None, None, ws)
                else:
                    conv1.winograd_gemm(n, ws)
                    conv1.winograd_output_into(conv2, n, None if self.channels % 64 == 0 else b, None, ws)  # only conv2 reads this result
                ml.set_timer_label("block_conv2")
                boundary = blk + 1 < self.blocks and self.channels % 64 == 0 and self.fuse_block_boundary
                if boundary and self.fuse_layers:
                    conv2.winograd_layer_into(L[3 + 2 * blk], n, c, a, ws)
                    a, c = c, a
                    continue
                conv2.winograd_gemm(n, ws)
                # c = next block's input and residual: written to memory and, inside the same launch, transformed for the next block
                if boundary:
                    conv2.winograd_output_into(L[3 + 2 * blk], n, c, a, ws)
                else:
                    conv2.winograd_output(c, a, ws)
                    if blk + 1 < self.blocks:
                        ml.set_timer_label("block_conv1")
                        L[3 + 2 * blk].winograd_input(c, ws)
                a, c = c, a
            ml.set_timer_label("head")
            L[-1].forward([a], self._view_batch(self.output, start, n), ws)
            ml.set_timer_label(None)
        return self.output

    def trunk_output(self):
        """Activation buffer holding the last block's output of the last chunk processed (for per-layer checks)."""
        return self.act[0] if self.blocks % 2 == 0 else self.act[2]

    def flops_per_forward(self):
        """Executed (Winograd-domain) floating-point operations of one forward pass over the whole batch."""
        tiles = self.batch * ((self.board + 3) // 4) ** 2
        total = 0
        for layer in self.layers:
            cout, k, _, cin = layer.weight_shape
            if k == 3:
                total += 2 * 36 * tiles * cin * cout
            else:
                total += 2 * self.batch * self.board * self.board * cin * cout * k * k
        return total
