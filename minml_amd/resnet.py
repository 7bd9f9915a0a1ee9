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
    def __init__(self, context, batch, board, input_planes, channels, blocks, dtype, params_host, to_storage, chunk=None, fused=False,
                 with_head=True):
        """params_host: list from make_parameters; to_storage: fp32 ndarray -> ndarray in the storage type (identity or fp16 bits).
        with_head=False leaves the 1x1 policy head out (params_host then ends with the last block convolution) and forward() returns
        the trunk's activations [batch, board, board, channels]: the convolutional trunk of a larger network."""
        self.context = context
        self.with_head = with_head
        self.fused = fused
        # True: also fuse across the residual blocks' boundaries (the block's result is written and transformed for the next block in one
        # launch). Identical results, less memory traffic and one launch less per block: measured on MI355X 3 % faster at 512 positions,
        # 3 % at 128, 6 % at 32, and level (0.1 % slower) at 1024, where the second of two launches finds the block's result in the
        # last-level cache. On by default up to 8192 tiles per launch (512 positions of 15x15)
        self.fuse_block_boundary = min(chunk or batch, batch) * ((board + 3) // 4) ** 2 <= 8192
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
        if with_head:
            self.layers.append(Conv2D(context, shape, 1, 1, "linear", True, self.dtype))
        if len(params_host) != len(self.layers):
            raise ValueError("expected parameters of %d layers, got %d" % (len(self.layers), len(params_host)))
        for layer, (w, b) in zip(self.layers, params_host):
            layer.setWeights(to_storage(w), to_storage(b))

        ws_elems = max(1, max(l.getWorkspaceSize() for l in self.layers))
        self.workspace = ml.Tensor((ws_elems,), self.dtype, context.device_index)
        # three rotating activation buffers per chunk: block input, intermediate, block output
        self.act = [ml.Tensor((cb, board, board, channels), self.dtype, context.device_index) for _ in range(3)]
        self.input = ml.Tensor((batch, board, board, input_planes), self.dtype, context.device_index)
        # without a head the trunk's activations of every sub-batch are collected here
        self.output = ml.Tensor((batch, board, board, 1 if with_head else channels), self.dtype, context.device_index)

    def _finish(self, a, start, n, ws):
        """Head (or, without one, the copy of the trunk's result) of one sub-batch into its slice of the output."""
        out = self._view_batch(self.output, start, n)
        if self.with_head:
            self.layers[-1].forward([a], out, ws)
        else:
            out.copyFrom(self.context, a)

    def setInput(self, x_storage):
        self.input.copyFromHost(self.context, x_storage)

    def _observe(self, layer_index, tensor):
        """Hands a layer's output to `self.observer(layer_index, tensor)` when one is set (layer-by-layer pass only); used for calibration
        and per-layer checks."""
        if getattr(self, "observer", None) is not None:
            self.observer(layer_index, tensor)

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
            self._observe(0, a)
            for blk in range(self.blocks):
                ml.set_timer_label("block_conv1")
                self.layers[1 + 2 * blk].forward([a], b, self.workspace)
                self._observe(1 + 2 * blk, b)
                ml.set_timer_label("block_conv2")
                self.layers[2 + 2 * blk].forward([b, a], c, self.workspace)
                self._observe(2 + 2 * blk, c)
                a, c = c, a
            ml.set_timer_label("head")
            self._finish(a, start, n, self.workspace)
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
            self._finish(a, start, n, ws)
            ml.set_timer_label(None)
        if self.fuse_layers:
            # the whole-layer launch hands out producer / consumer roles among workgroups that must all be resident at once (64 per XCD);
            # on a device shared with other work its bounded waits can give up, and the results are then invalid: ask, and say so
            gave_up = ml.winogradLayerErrors(self.context)
            if gave_up:
                raise RuntimeError("%d workgroups of whole-layer Winograd launches gave up waiting for one another: the pass is invalid "
                                   "(device shared with other work?); run with fuse_layers = False" % gave_up)
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


def calibrate_activations(context, params_host, board, input_planes, channels, blocks, batches=64, batch_size=4, seed=0):
    """Per-tensor activation ranges for the int8 network: max |x| of the input and of every 3x3 layer's output over `batches` random
    batches, measured with the fp32 network on the device (benchmark configuration 3: "calibrated as the max-abs over 64 random batches").
    Returns [input, stem, conv 1, ..., conv 2*blocks]."""
    net = ResNet(context, batch_size, board, input_planes, channels, blocks, "float32", params_host, lambda a: np.ascontiguousarray(a, np.float32))
    ranges = np.zeros(2 + 2 * blocks, np.float64)

    def observer(index, tensor):
        ranges[1 + index] = max(ranges[1 + index], float(np.abs(tensor.copyToHost(context)).max()))

    net.observer = observer
    for i in range(batches):
        x = make_input(seed * 7919 + i + 1, batch_size, board, input_planes)
        ranges[0] = max(ranges[0], float(np.abs(x).max()))
        net.setInput(x)
        net.forward(fused=False)
    context.synchronize()
    return [float(r) for r in ranges]


class QuantizedResNet:
    """The same network with int8 activations and weights (benchmark configuration 3): every 3x3 layer is one fused int8 convolution
    (zero-point padding, int32 accumulation, per-channel scale + bias, int8 residual, ReLU, requantisation: src/layers/Conv2D.cpp:240-308),
    the 1x1 head returns fp32 logits. Weights are quantised per output channel (scale = max|w| / 127), activations per tensor and
    symmetric (scale = max|x| / 127 from `activation_ranges`, as returned by calibrate_activations)."""

    def __init__(self, context, batch, board, input_planes, channels, blocks, params_host, activation_ranges, int8_mode="fused"):
        from . import quantization as Q

        self.context = context
        self.batch, self.board, self.channels, self.blocks = batch, board, channels, blocks
        self.transforms = [Q.symmetric_transform(r) for r in activation_ranges]  # input, stem, conv 1 ... conv 2*blocks
        self.layers, self.host_parameters = [], []
        shape = (batch, board, board, input_planes)
        for index, (w, b) in enumerate(params_host):
            head = index == len(params_host) - 1
            layer = Conv2D(context, shape, w.shape[0], w.shape[1], "linear" if head else "relu", True, "int8")
            in_qd = self.transforms[index]  # the tensor this layer reads was written by layer index - 1 (or is the input)
            out_qd = (1.0, 0.0) if head else self.transforms[index + 1]
            # the residual of a block's second convolution is the block's input: the output of the layer two steps back
            ext_qd = self.transforms[index - 1] if (not head and index >= 2 and index % 2 == 0) else (1.0, 0.0)
            q, scales, folded = Q.quantize_weights(w, b, in_qd)
            layer.setupQuantization(q, scales, folded, [in_qd, ext_qd], out_qd, int8_mode)
            self.layers.append(layer)
            self.host_parameters.append((q, scales, folded, in_qd, ext_qd, out_qd))
            shape = (batch, board, board, channels)
        ws = max(1, max(l.getWorkspaceSize() for l in self.layers))
        self.workspace = ml.Tensor((ws,), "float32", context.device_index)  # 4-byte elements, as Conv2D counts them in int8 mode
        self.act = [ml.Tensor((batch, board, board, channels), "int8", context.device_index) for _ in range(3)]
        self.input = ml.Tensor((batch, board, board, input_planes), "int8", context.device_index)
        self.output = ml.Tensor((batch, board, board, 1), "float32", context.device_index)
        self.observer = None

    def setInput(self, x_real):
        """Real-valued input planes -> int8 with the input's transform, uploaded."""
        from . import quantization as Q

        self.input.copyFromHost(self.context, Q.quantize_tensor(x_real, self.transforms[0]))

    def forward(self):
        L, ws = self.layers, self.workspace
        a, b, c = self.act
        ml.set_timer_label("stem")
        L[0].forward([self.input], a, ws)
        self._observe(0, a)
        for blk in range(self.blocks):
            ml.set_timer_label("block_conv1")
            L[1 + 2 * blk].forward([a], b, ws)
            self._observe(1 + 2 * blk, b)
            ml.set_timer_label("block_conv2")
            L[2 + 2 * blk].forward([b, a], c, ws)
            self._observe(2 + 2 * blk, c)
            a, c = c, a
        ml.set_timer_label("head")
        L[-1].forward([a], self.output, ws)
        ml.set_timer_label(None)
        return self.output

    def _observe(self, layer_index, tensor):
        if self.observer is not None:
            self.observer(layer_index, tensor)

    def ops_per_forward(self):
        """Integer multiply-adds x 2 of one forward pass over the whole batch."""
        pixels = self.batch * self.board * self.board
        return sum(2 * pixels * int(np.prod(l.weight_shape)) for l in self.layers)
