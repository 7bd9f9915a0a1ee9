"""Conv2D layer (inference) on the HIP backend, mirroring the reference's src/layers/Conv2D.cpp.

What is mirrored, with the reference lines it follows:
  * algorithm choice per kernel size                        Conv2D.cpp:450-530 (device branch)
  * workspace sizing in elements of the layer dtype         Conv2D.cpp:141-191, src/core/math.cpp:1588-1594
  * transformed-weight cache (built on first forward)       Conv2D.cpp:356-363
  * Winograd sequence: input transform into workspace[0 : 36*T*Cin], gemmBatched('n','t'), output transform from
    workspace[36*T*Cin : ...] with bias / residual / activation       Conv2D.cpp:365-378
  * explicit GEMM (1x1)                                     Conv2D.cpp:329-353 -> src/core/math.cpp:1595-1626
  * grouped convolution (groups > 1): grouped product on the flattened tensors, then bias + activation as a second call
                                                            Conv2D.cpp:71-101 (weights [Cout / groups, k, k, Cin]), :339-349
  * int8 path: im2row with zero-point padding -> int8 GEMM -> quantized_scale_shift_act      Conv2D.cpp:214-239
  * quantisation set-up                                     src/layers/Layer.cpp:147-160, src/layers/quantization.cpp:55-93

One difference by design: kernel sizes other than 1 and 3 use the fused implicit-GEMM convolution (the reference reaches that entry
point only on cuDNN builds, Conv2D.cpp:478-485) because on this backend it needs no im2row workspace; `algorithm=` overrides the choice.
The int8 path has the reference's three-call sequence ("reference") and the single fused launch ("fused").
"""
import numpy as np

from . import backend as B
from . import core as ml

EXPLICIT_GEMM, WINOGRAD_NON_FUSED, IMPLICIT_GEMM = "explicit_gemm", "winograd_non_fused", "implicit_gemm"


def get_matrices_shape(kernel_size, tile_size, shape):
    """[ (tile+k-1)^2, B * ceil(H/tile) * ceil(W/tile), C ] (reference: Conv2D.cpp get_matrices_shape)."""
    t = tile_size + kernel_size - 1
    tiles = shape[0] * ((shape[1] + tile_size - 1) // tile_size) * ((shape[2] + tile_size - 1) // tile_size)
    return (t * t, tiles, shape[3])


def get_weight_matrices_shape(weight_shape, tile_size):
    t = tile_size + weight_shape[1] - 1
    return (t * t, weight_shape[0], weight_shape[3])


class Conv2D:
    def __init__(self, context, input_shape, filters, kernel_size, activation="linear", use_bias=True, dtype="float16", algorithm=None, groups=1):
        self.context = context
        self.groups = groups
        if groups != 1 and (input_shape[3] % groups != 0 or filters % groups != 0 or kernel_size != 1):
            # the reference flattens input and weights to matrices (Conv2D.cpp:341-344), which is a convolution only for a 1x1 kernel
            raise ValueError("grouped convolution: 1x1 kernels, filters divisible by the number of groups")
        self.input_shape = tuple(input_shape)
        self.kernel_size = kernel_size
        self.activation = ml.act_of(activation)
        self.use_bias = use_bias
        self.dtype = ml.dtype_of(dtype)
        self.weight_shape = (filters // groups, kernel_size, kernel_size, input_shape[3])
        self.output_shape = (input_shape[0], input_shape[1], input_shape[2], filters)
        self.weights = None
        self.bias = None
        self.transformed_weights = None
        self.winograd_tile_size = 4
        self.forward_algorithm = algorithm or self._choose_algorithm()
        # int8 state (Layer::setupQuantization)
        self.channel_scales = None
        self.input_transforms = None
        self.output_transform = None
        self.int8_mode = "fused"

    def _choose_algorithm(self):
        if self.kernel_size == 1:
            return EXPLICIT_GEMM
        if self.kernel_size == 3:
            return WINOGRAD_NON_FUSED
        return IMPLICIT_GEMM

    # ---- parameters -----------------------------------------------------------------------------------------------------
    def setWeights(self, weights, bias=None):
        """weights [Cout,k,k,Cin], bias [Cout] as numpy arrays of the layer dtype (uint16 bit patterns for fp16)."""
        w = np.ascontiguousarray(weights)
        if w.shape != self.weight_shape:
            raise ValueError("weights must have shape %s" % (self.weight_shape,))
        self.weights = ml.toDevice(self.context, w, self.dtype)
        self.bias = ml.toDevice(self.context, np.ascontiguousarray(bias), self.dtype if self.dtype != B.DTYPE_INT8 else B.DTYPE_FLOAT32) \
            if (bias is not None and self.use_bias) else None
        self.transformed_weights = None  # invalidateWeightsCache

    def setupQuantization(self, q_weights, channel_scales, q_bias, input_transforms, output_transform, int8_mode="fused"):
        """int8 weights + per-channel scales + folded bias as produced by quantize_weights(..., "per_first_dim", 8)."""
        self.dtype = B.DTYPE_INT8
        self.weights = ml.toDevice(self.context, np.ascontiguousarray(q_weights, np.int8))
        self.channel_scales = ml.toDevice(self.context, np.ascontiguousarray(channel_scales, np.float32))
        self.bias = ml.toDevice(self.context, np.ascontiguousarray(q_bias, np.float32))
        self.input_transforms = list(input_transforms)
        self.output_transform = output_transform
        self.int8_mode = int8_mode

    # ---- workspace contract ---------------------------------------------------------------------------------------------
    def getWorkspaceSize(self):
        """In elements of the workspace tensor (4-byte elements in int8 mode), as the reference counts it."""
        out_volume = int(np.prod(self.output_shape))
        in_volume = int(np.prod(self.input_shape))
        if self.dtype == B.DTYPE_INT8:
            if self.int8_mode == "fused":
                return 0
            tmp_output = out_volume  # int32 accumulators, one 4-byte element each
            if self.kernel_size == 1:
                return tmp_output
            return tmp_output + (in_volume * self.kernel_size ** 2 + 3) // 4
        if self.kernel_size == 1:
            return 0
        if self.forward_algorithm == EXPLICIT_GEMM:
            return (in_volume // self.input_shape[3]) * self.kernel_size ** 2 * self.input_shape[3]
        if self.forward_algorithm == WINOGRAD_NON_FUSED:
            win1 = get_matrices_shape(self.kernel_size, self.winograd_tile_size, self.input_shape)
            win2 = get_matrices_shape(self.kernel_size, self.winograd_tile_size, self.output_shape)
            return int(np.prod(win1)) + int(np.prod(win2)) + 1024
        return 0

    # ---- forward --------------------------------------------------------------------------------------------------------
    def forward(self, inputs, output, workspace=None):
        """inputs = [x] or [x, residual]; tensors may carry a smaller batch than the layer was sized for."""
        x = inputs[0]
        add = inputs[1] if len(inputs) == 2 else None
        ctx = self.context
        if self.dtype == B.DTYPE_INT8:
            return self._forward_int8(x, add, output, workspace)

        if self.forward_algorithm == IMPLICIT_GEMM:
            ml.convolutionImplicitGemmForward(ctx, x, self.weights, output, self.bias, add, self.activation)
        elif self.forward_algorithm == EXPLICIT_GEMM and self.groups > 1:
            if add is not None:
                raise ValueError("a grouped convolution takes no second input")
            rows = x.volume() // x.lastDim()
            output_matrix = output.view((rows, output.lastDim()))
            ml.gemmGrouped(ctx, "n", "t", output_matrix, x.view((rows, x.lastDim())), self.weights.view((self.weights.firstDim(), self.weights.volume() // self.weights.firstDim())), 1.0, 0.0, self.groups)
            if self.bias is not None:
                ml.addBiasAct(ctx, 1.0, output, self.bias, 0.0, output, self.activation)
            else:
                ml.activationForward(ctx, 1.0, output, 0.0, output, self.activation)
        elif self.forward_algorithm == EXPLICIT_GEMM:
            ml.explicit_gemm_forward(ctx, x, output, self.weights, self.bias, workspace, self.activation, add)
        else:
            self.winograd_input(x, workspace)
            self.winograd_gemm(x.shape[0], workspace)
            self.winograd_output(output, add, workspace)
        return output

    # ---- the three stages of the Winograd path, separately callable so that a runner can fuse across layers -------------------
    def _winograd_views(self, batch, workspace):
        """(input matrices, output matrices): views at element 0 and 36*T*Cin of the workspace (Conv2D.cpp:365-367)."""
        in_shape = get_matrices_shape(self.kernel_size, self.winograd_tile_size, (batch,) + self.input_shape[1:])
        out_shape = get_matrices_shape(self.kernel_size, self.winograd_tile_size, (batch,) + self.output_shape[1:])
        return workspace.view(in_shape), workspace.view(out_shape, int(np.prod(in_shape)))

    def winograd_input(self, x, workspace):
        input_matrices, _ = self._winograd_views(x.shape[0], workspace)
        ml.winogradInputTransform(self.context, self.weight_shape, x, input_matrices)

    def winograd_gemm(self, batch, workspace):
        """36 batched products of the input matrices already in the workspace with the cached transformed weights."""
        ctx = self.context
        if self.transformed_weights is None:
            self.transformed_weights = ml.Tensor(get_weight_matrices_shape(self.weight_shape, self.winograd_tile_size), self.dtype, ctx.device_index)
            ml.winogradWeightTransform(ctx, self.weights, self.transformed_weights, False)
        input_matrices, output_matrices = self._winograd_views(batch, workspace)
        ml.gemmBatched(ctx, "n", "t", output_matrices, input_matrices, self.transformed_weights, 1.0, 0.0)

    def winograd_output(self, output, add, workspace):
        _, output_matrices = self._winograd_views(output.shape[0], workspace)
        ml.winogradOutputTransform(self.context, self.weight_shape, output_matrices, output, self.bias, add, self.activation)

    def winograd_output_into(self, next_layer, batch, output, add, workspace):
        """Output transform of this layer fused with the input transform of `next_layer` (a Winograd layer on this layer's output,
        sharing the workspace): the next layer's input matrices land at element 0, where this layer's are no longer needed.
        `output` may be None when nothing else reads this layer's result."""
        _, output_matrices = self._winograd_views(batch, workspace)
        next_input, _ = next_layer._winograd_views(batch, workspace)
        if next_input.volume() > self._winograd_views(batch, workspace)[0].volume():
            raise ValueError("the next layer's input matrices would overlap this layer's output matrices in the workspace")
        out_shape = (batch,) + self.output_shape[1:]
        ml.winogradOutputInputTransform(self.context, self.weight_shape, output_matrices, out_shape, output, self.bias, add, self.activation, next_input)

    def winograd_layer_into(self, next_layer, batch, output, add, workspace):
        """Product, output transform and `next_layer`'s input transform in one call, from this layer's input matrices already in the
        workspace. The next layer's input matrices replace this layer's at element 0: a tile's rows are rewritten only after every
        position of that tile has been multiplied."""
        ctx = self.context
        if self.transformed_weights is None:
            self.transformed_weights = ml.Tensor(get_weight_matrices_shape(self.weight_shape, self.winograd_tile_size), self.dtype, ctx.device_index)
            ml.winogradWeightTransform(ctx, self.weights, self.transformed_weights, False)
        input_matrices, output_matrices = self._winograd_views(batch, workspace)
        next_input, _ = next_layer._winograd_views(batch, workspace)
        if next_input.volume() > input_matrices.volume():
            raise ValueError("the next layer's input matrices would overlap this layer's output matrices in the workspace")
        out_shape = (batch,) + self.output_shape[1:]
        ml.winogradLayerForward(ctx, self.weight_shape, input_matrices, self.transformed_weights, output_matrices, out_shape, output, self.bias, add,
                                self.activation, next_input)

    def _forward_int8(self, x, add, output, workspace):
        ctx = self.context
        ext_transform = self.input_transforms[1] if add is not None else (1.0, 0.0)
        if self.int8_mode == "fused":
            ml.quantizedConvForward(ctx, x, self.input_transforms[0], self.weights, self.channel_scales, self.bias, output, self.output_transform, add,
                                    ext_transform, self.activation)
            return output
        # the reference's device sequence: [im2row] -> int8 GEMM into the workspace -> requantisation
        rows = x.volume() // x.lastDim()
        cols = self.weights.volume() // self.weights.firstDim()
        filters = output.lastDim()
        output_matrix = workspace.view((rows * filters,)).reinterpretAs("int32").view((rows, filters))
        weight_matrix = self.weights.view((self.weights.firstDim(), cols))
        if self.kernel_size == 1:
            input_matrix = x.view((rows, x.lastDim()))
        else:
            bytes_view = workspace.view(((rows * cols + 3) // 4,), rows * filters).reinterpretAs("int8")
            input_matrix = bytes_view.view((rows, cols))
            scale, shift = self.input_transforms[0]
            # the reference's device branch casts with truncation (Conv2D.cpp:227); the CPU branch, which defines the results, rounds (:245)
            padding = int(np.round(np.float32(0.0) * (np.float32(1.0) / np.float32(scale)) + (-np.float32(shift) / np.float32(scale))))
            ml.im2row(ctx, input_matrix, x, self.kernel_size, False, padding)
        ml.gemm(ctx, "n", "t", output_matrix, input_matrix, weight_matrix, 1.0, 0.0)
        ml.quantized_scale_shift_act(ctx, output, self.output_transform, output_matrix, self.channel_scales, self.bias, self.activation, add,
                                     ext_transform)
        return output
