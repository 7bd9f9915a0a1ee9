"""Host-side mirror of the part of minml's core that drives the convolution / GEMM path on a device backend.

`Context`, `Tensor` and the free functions below have the names, argument order and meaning of the reference's
include/minml/core/{Context,Tensor,math}.hpp (dispatch: src/core/math.cpp, DeviceType::CUDA branch), so that tests written against
them read like the reference's own tests (test/backend/test_winograd.cpp, test_conv2D.cpp, test_gemms.cpp, test_quantization.cpp).
Every function converts its tensors to the by-value descriptors of the C-ABI and calls libminml_hip.so; nothing is computed here.

Where the reference asserts (shape / dtype / device agreement) these functions raise ValueError *before* calling the library, because
the library reports errors the reference's way, by C++ exceptions across the C boundary, which cannot be caught from Python.
"""
import ctypes

import numpy as np

from . import backend as B

_NP_OF = {B.DTYPE_FLOAT16: np.uint16, B.DTYPE_FLOAT32: np.float32, B.DTYPE_INT8: np.int8, B.DTYPE_INT32: np.int32, B.DTYPE_UINT8: np.uint8}
_NAME_OF = {"float16": B.DTYPE_FLOAT16, "float32": B.DTYPE_FLOAT32, "int8": B.DTYPE_INT8, "int32": B.DTYPE_INT32, "uint8": B.DTYPE_UINT8}
ACTIVATIONS = {"linear": B.ACTIVATION_LINEAR, "sigmoid": B.ACTIVATION_SIGMOID, "tanh": B.ACTIVATION_TANH, "relu": B.ACTIVATION_RELU,
               "leaky_relu": B.ACTIVATION_LEAKY_RELU, "exp": B.ACTIVATION_EXP, "gelu": B.ACTIVATION_EXP}


def dtype_of(x):
    if isinstance(x, str):
        return _NAME_OF[x]
    return int(x)


def act_of(a):
    if isinstance(a, str):
        return ACTIVATIONS[a]
    return int(a)


def number_of_devices():
    return B.fn("get_number_of_devices")()


class Context:
    """One stream on one device (reference: include/minml/core/Context.hpp; backend object src/backend/cuda/utils.hpp:28-66)."""

    def __init__(self, device_index=0):
        n = number_of_devices()
        if not (0 <= device_index < n):
            raise RuntimeError("no HIP device %d (devices found: %d)" % (device_index, n))
        self.device_index = device_index
        self.handle = B.fn("create_context")(device_index)

    def synchronize(self):
        B.fn("synchronize_with_context")(self.handle)

    def isReady(self):
        return bool(B.fn("is_context_ready")(self.handle))

    def stream(self):
        return B.fn("get_stream")(self.handle)

    def destroy(self):
        if self.handle:
            B.fn("destroy_context")(self.handle)
            self.handle = None


class Graph:
    """A pass recorded once on a context and replayed as one HIP graph (the library's hip_graph_* calls; no counterpart in the reference).

        graph = Graph.record(context, lambda: net.forward())    # after one ordinary pass
        graph.launch()                                          # replays the recorded launches on the context's stream
    """

    def __init__(self, context, handle):
        self.context = context
        self.handle = handle

    @staticmethod
    def record(context, function):
        if _TIMER is not None:
            raise RuntimeError("a kernel timer records events around every call: remove it before recording a graph")
        B.fn("graph_begin_capture")(context.handle)
        try:
            function()
        except BaseException:
            # the recording must be closed whatever happened; what it produced is dropped, and the caller sees the original failure
            try:
                handle = B.fn("graph_end_capture")(context.handle)
                if handle:
                    B.fn("graph_destroy")(handle)
            except Exception:
                pass
            raise
        return Graph(context, B.fn("graph_end_capture")(context.handle))

    def launch(self):
        if not self.handle:
            raise RuntimeError("the graph was destroyed")
        B.fn("graph_launch")(self.context.handle, self.handle)

    def destroy(self):
        if self.handle:
            handle, self.handle = self.handle, None
            B.fn("graph_destroy")(handle)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.destroy()
        return False

    def __del__(self):
        try:
            self.destroy()
        except Exception:  # interpreter shutdown: the library may be gone already
            pass


class Event:
    """Recorded on creation (reference: include/minml/core/Event.hpp, src/backend/cuda/cuda_event.cpp)."""

    def __init__(self, context):
        self.handle = B.fn("create_event")(context.handle)

    def synchronize(self):
        B.fn("wait_for_event")(self.handle)

    def isReady(self):
        return bool(B.fn("is_event_ready")(self.handle))

    @staticmethod
    def getElapsedTime(start, end):
        return B.fn("get_time_between_events")(start.handle, end.handle)

    def destroy(self):
        if self.handle:
            B.fn("destroy_event")(self.handle)
            self.handle = None


class Tensor:
    """Dense row-major device tensor: pointer + shape + dtype + ownership flag (reference: src/core/Tensor.cpp, ml_memory.cpp:135-177).

    fp16 data crosses the host boundary as numpy uint16 bit patterns.
    """

    def __init__(self, shape, dtype, device_index=0, _ptr=None, _owner=None):
        self.shape = tuple(int(d) for d in shape)
        self.dtype = dtype_of(dtype)
        self.device_index = device_index
        self._owner = _owner
        if _ptr is None:
            self.ptr = B.fn("malloc")(device_index, max(self.sizeInBytes(), 1))
            self._owning = True
        else:
            self.ptr = _ptr
            self._owning = False

    # ---- shape helpers named as in the reference's Shape / Tensor
    def rank(self):
        return len(self.shape)

    def dim(self, i):
        return self.shape[i]

    def volume(self):
        v = 1
        for d in self.shape:
            v *= d
        return v if self.shape else 0

    def firstDim(self):
        return self.shape[0]

    def lastDim(self):
        return self.shape[-1]

    def sizeInBytes(self):
        return self.volume() * B.DTYPE_SIZE[self.dtype]

    def isEmpty(self):
        return self.volume() == 0

    def view(self, shape, offset=0):
        """Non-owning tensor over the same memory, `offset` in elements (reference: Tensor::view)."""
        shape = tuple(int(d) for d in shape)
        vol = int(np.prod(shape)) if shape else 0
        if offset + vol > self.volume():
            raise ValueError("view exceeds the tensor")
        p = B.fn("create_view")(self.ptr, offset * B.DTYPE_SIZE[self.dtype], vol * B.DTYPE_SIZE[self.dtype])
        return Tensor(shape, self.dtype, self.device_index, _ptr=p, _owner=self)

    def reinterpretAs(self, dtype):
        """Same bytes, other element type; the last dimension is rescaled (used for the int32 view of the workspace)."""
        new = dtype_of(dtype)
        nbytes = self.sizeInBytes()
        if nbytes % B.DTYPE_SIZE[new] != 0:
            raise ValueError("size is not a multiple of the new element size")
        return Tensor((nbytes // B.DTYPE_SIZE[new],), new, self.device_index, _ptr=self.ptr, _owner=self)

    # ---- host <-> device
    def copyFromHost(self, context, array):
        arr = np.ascontiguousarray(array)
        if arr.dtype != _NP_OF[self.dtype] or arr.size != self.volume():
            raise ValueError("host array does not match tensor (dtype %s size %d vs %s %d)" % (arr.dtype, arr.size, _NP_OF[self.dtype], self.volume()))
        if arr.size:
            B.fn("memcpy_from_host")(context.handle if context else None, self.ptr, 0, arr.ctypes.data_as(ctypes.c_void_p), arr.nbytes)
            if context is not None:
                context.synchronize()  # the host array may go away
        return self

    def copyFrom(self, context, other):
        """Device-to-device copy of `other` into this tensor, asynchronous on the context's stream (reference: Tensor::copyFrom,
        src/core/Tensor.cpp -> ml::memcpy -> cuda_memcpy_within_device)."""
        if other.sizeInBytes() != self.sizeInBytes():
            raise ValueError("copyFrom: sizes differ")
        if self.sizeInBytes():
            B.fn("memcpy_within_device")(context.handle if context else None, self.ptr, 0, other.ptr, 0, self.sizeInBytes())
        return self

    def copyToHost(self, context=None):
        out = np.empty(self.shape, _NP_OF[self.dtype])
        if out.size:
            if context is not None:
                context.synchronize()
            B.fn("memcpy_to_host")(None, out.ctypes.data_as(ctypes.c_void_p), self.ptr, 0, out.nbytes)
        return out

    def zeroall(self, context=None):
        if self.sizeInBytes():
            B.fn("memset")(context.handle if context else None, self.ptr, 0, self.sizeInBytes(), None, 0)

    def setall(self, context, value):
        pattern = np.array([value], _NP_OF[self.dtype]) if self.dtype != B.DTYPE_FLOAT16 else np.array([value], np.float16).view(np.uint16)
        if self.sizeInBytes():
            B.fn("memset")(context.handle if context else None, self.ptr, 0, self.sizeInBytes(), pattern.ctypes.data_as(ctypes.c_void_p),
                           pattern.nbytes)

    def free(self):
        if self._owning and self.ptr:
            B.fn("free")(self.ptr)
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    # ---- descriptors
    def desc(self):
        return B.make_tensor(self.ptr, self.dtype, self.shape)

    def shape_desc(self):
        return B.make_shape(self.shape)


def toDevice(context, array, dtype=None):
    """numpy array -> new device tensor (uint16 arrays are fp16 bit patterns)."""
    arr = np.ascontiguousarray(array)
    if dtype is None:
        dtype = {np.dtype(np.uint16): B.DTYPE_FLOAT16, np.dtype(np.float32): B.DTYPE_FLOAT32, np.dtype(np.int8): B.DTYPE_INT8,
                 np.dtype(np.int32): B.DTYPE_INT32, np.dtype(np.uint8): B.DTYPE_UINT8}[arr.dtype]
    t = Tensor(arr.shape, dtype, context.device_index)
    t.copyFromHost(context, arr)
    return t


_EMPTY = B.make_tensor(None, B.DTYPE_UNKNOWN, ())


def _desc(t):
    return _EMPTY if (t is None or t.isEmpty()) else t.desc()


def _ptr(t):
    return None if (t is None or t.isEmpty()) else t.ptr


def _require(cond, msg):
    if not cond:
        raise ValueError(msg)


class KernelTimer:
    """Brackets every call of the named entry points with two events on the context's stream, so that the duration of each kernel is
    measured where it runs; `summary()` returns {name: (launches, average seconds)}. Installed with set_kernel_timer()."""

    def __init__(self, context):
        self.context = context
        self.records = {}

    def call(self, name, function, *args):
        start = Event(self.context)
        function(*args)
        end = Event(self.context)
        self.records.setdefault(name, []).append((start, end))
        if _TIMER_LABEL is not None:
            self.records.setdefault(name + "@" + _TIMER_LABEL, []).append((start, end))

    def summary(self):
        self.context.synchronize()
        result = {}
        for name, pairs in self.records.items():
            total = sum(Event.getElapsedTime(s, e) for s, e in pairs)
            result[name] = (len(pairs), total / len(pairs))
        for name, pairs in self.records.items():
            if "@" not in name:  # labelled entries share their events with the unlabelled ones
                for s, e in pairs:
                    s.destroy()
                    e.destroy()
        self.records = {}
        return result


_TIMER = None
_TIMER_LABEL = None


def set_kernel_timer(timer):
    global _TIMER
    _TIMER = timer


def set_timer_label(label):
    """While a kernel timer is installed, launches are also recorded under "<entry point>@<label>" (None switches this off)."""
    global _TIMER_LABEL
    _TIMER_LABEL = label


def _launch(name, *args):
    if _TIMER is None:
        B.fn(name)(*args)
    else:
        _TIMER.call(name, B.fn(name), *args)


def _same_dtype(*tensors):
    ts = [t for t in tensors if t is not None and not t.isEmpty()]
    return all(t.dtype == ts[0].dtype for t in ts)


def get_winograd_tile(weight_shape, matrices_shape):
    """reference: src/core/math.cpp:107-118 — the tile size is derived from the number of matrices."""
    _require(weight_shape[1] == weight_shape[2], "only square filters")
    root = int(round(matrices_shape[0] ** 0.5))
    _require(root * root == matrices_shape[0], "number of Winograd matrices is not a square")
    return root - (weight_shape[1] - 1)


def _require_winograd_supported(tile, kernel, dtype):
    if not (tile == 4 and kernel == 3 and dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32)):
        raise RuntimeError("No suitable Winograd transform runtime")  # reference: src/backend/cpu/winograd/winograd_runtime.cpp:516


def winogradWeightTransform(context, weights, matrices, invert=False):
    tile = get_winograd_tile(weights.shape, matrices.shape)
    _require_winograd_supported(tile, weights.shape[1], weights.dtype)
    _require(_same_dtype(weights, matrices), "dtype mismatch")
    _require(matrices.shape == (36, weights.shape[0], weights.shape[3]), "matrices must be [36, Cout, Cin]")
    _launch("winograd_weight_transform", context.handle, tile, weights.desc(), matrices.desc(), bool(invert))


def winogradInputTransform(context, weight_shape, input, matrices):
    tile = get_winograd_tile(weight_shape, matrices.shape)
    _require_winograd_supported(tile, weight_shape[1], input.dtype)
    _require(_same_dtype(input, matrices), "dtype mismatch")
    b, h, w, c = input.shape
    _require(matrices.shape == (36, b * ((h + 3) // 4) * ((w + 3) // 4), c), "matrices must be [36, tiles, C]")
    _launch("winograd_input_transform", context.handle, tile, input.desc(), matrices.desc())


def winogradOutputTransform(context, weight_shape, matrices, output, bias, add, act):
    tile = get_winograd_tile(weight_shape, matrices.shape)
    _require_winograd_supported(tile, weight_shape[1], output.dtype)
    _require(_same_dtype(matrices, output, bias, add), "dtype mismatch")
    b, h, w, c = output.shape
    _require(matrices.shape == (36, b * ((h + 3) // 4) * ((w + 3) // 4), c), "matrices must be [36, tiles, C]")
    _require(bias is None or bias.isEmpty() or bias.volume() == c, "bias must be [C]")
    _require(add is None or add.isEmpty() or add.shape == output.shape, "add must have the output's shape")
    _launch("winograd_output_transform", context.handle, tile, matrices.desc(), _desc(bias), _desc(add), output.desc(), act_of(act))


def winogradOutputInputTransform(context, weight_shape, matrices, output_shape, output, bias, add, act, next_matrices):
    """Output transform of one layer fused with the input transform of the next 3x3 layer (no counterpart in the reference's math.hpp).
    `output` may be None when y itself is not needed in memory."""
    tile = get_winograd_tile(weight_shape, matrices.shape)
    _require_winograd_supported(tile, weight_shape[1], matrices.dtype)
    _require(_same_dtype(matrices, next_matrices, output, bias, add), "dtype mismatch")
    b, h, w, c = output_shape
    expected = (36, b * ((h + 3) // 4) * ((w + 3) // 4), c)
    _require(matrices.shape == expected and next_matrices.shape == expected, "matrices must be [36, tiles, C]")
    _require(output is None or output.shape == tuple(output_shape), "output must have the given shape")
    _require(bias is None or bias.isEmpty() or bias.volume() == c, "bias must be [C]")
    _require(add is None or add.isEmpty() or add.shape == tuple(output_shape), "add must have the output's shape")
    _require(output is not None or c % 64 == 0, "without an output tensor the channel count must be a multiple of 64")
    _launch("winograd_output_input_transform", context.handle, tile, matrices.desc(), _desc(bias), _desc(add), B.make_shape(output_shape), _ptr(output),
            act_of(act), next_matrices.desc())


def winogradLayerForward(context, weight_shape, input_matrices, weight_matrices, output_matrices, output_shape, output, bias, add, act, next_matrices,
                         static_memory=False):
    """Batched product, output transform and the next 3x3 layer's input transform in one call (no counterpart in the reference's
    math.hpp): identical to gemmBatched into `output_matrices` followed by winogradOutputInputTransform. For fp16, 256 channels and 16
    tiles per image the product stays in the L2 cache and `output_matrices` is not touched. static_memory=True calls the entry point
    that allocates nothing (counters and scratch in the library's static device array; at most 4096 images per call)."""
    tile = get_winograd_tile(weight_shape, input_matrices.shape)
    _require_winograd_supported(tile, weight_shape[1], input_matrices.dtype)
    _require(_same_dtype(input_matrices, weight_matrices, output_matrices, next_matrices, output, bias, add), "dtype mismatch")
    b, h, w, c = output_shape
    tiles = b * ((h + 3) // 4) * ((w + 3) // 4)
    _require(input_matrices.shape == (36, tiles, weight_shape[3]) and weight_matrices.shape == (36, c, weight_shape[3]), "input / weight matrices shape")
    _require(output_matrices.shape == (36, tiles, c) and next_matrices.shape == (36, tiles, c), "output / next matrices must be [36, tiles, C]")
    _require(output is None or output.shape == tuple(output_shape), "output must have the given shape")
    _require(bias is None or bias.isEmpty() or bias.volume() == c, "bias must be [C]")
    _require(add is None or add.isEmpty() or add.shape == tuple(output_shape), "add must have the output's shape")
    _require(output is not None or c % 64 == 0, "without an output tensor the channel count must be a multiple of 64")
    _require(not static_memory or b <= 4096, "the static-memory form takes at most 4096 images per call")
    _launch("winograd_layer_forward_static" if static_memory else "winograd_layer_forward", context.handle, tile, input_matrices.desc(), weight_matrices.desc(), output_matrices.desc(), _desc(bias), _desc(add),
            B.make_shape(output_shape), _ptr(output), act_of(act), next_matrices.desc())


def winogradLayerErrors(context):
    """Waits for the context and returns how many workgroups of whole-layer launches gave up waiting since the last call (0 = all good)."""
    return int(B.fn("winograd_layer_errors")(context.handle))


def _gemm_dims(opA, A, opB, Bm):
    ta, tb = opA in "tT", opB in "tT"
    _require(opA in "ntNT" and opB in "ntNT", "op must be n or t")
    M = A.shape[-1] if ta else A.shape[-2]
    K = A.shape[-2] if ta else A.shape[-1]
    N = Bm.shape[-2] if tb else Bm.shape[-1]
    Kb = Bm.shape[-1] if tb else Bm.shape[-2]
    _require(K == Kb, "inner dimensions differ")
    return M, N, K


def gemm(context, opA, opB, C, A, Bm, alpha=1.0, beta=0.0):
    """C = alpha op(A) op(B) + beta C; an int32 C selects the int8 product (reference: src/core/math.cpp:643-660)."""
    _require(A.rank() == 2 and Bm.rank() == 2 and C.rank() == 2, "gemm takes matrices")
    M, N, K = _gemm_dims(opA, A, opB, Bm)
    _require(C.shape == (M, N), "shape of C")
    if C.dtype == B.DTYPE_INT32:
        _require(A.dtype == B.DTYPE_INT8 and Bm.dtype == B.DTYPE_INT8 and alpha == 1.0 and beta == 0.0, "int8 product: int8 operands, alpha 1, beta 0")
    else:
        _require(_same_dtype(A, Bm, C) and C.dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), "dtype mismatch")
    _launch("gemm_v2", context.handle, opA.encode(), opB.encode(), alpha, A.desc(), Bm.desc(), beta, C.desc())


def gemmGrouped(context, opA, opB, C, A, Bm, alpha=1.0, beta=0.0, groups=1):
    """The last dimension of A, B and C is cut into `groups` equal column ranges; range i of C = alpha op(A range i) op(B range i) + beta C
    (reference: src/core/math.cpp:1079-1093, device only; shapes as src/backend/cuda/kernels/group_conv.cu:120-139 derives them)."""
    _require(A.rank() == 2 and Bm.rank() == 2 and C.rank() == 2, "gemmGrouped takes matrices")
    _require(groups >= 1 and A.shape[1] % groups == 0 and Bm.shape[1] % groups == 0 and C.shape[1] % groups == 0, "last dimensions must be multiples of groups")
    _require(opA in "ntNT" and opB in "ntNT", "op must be n or t")
    ta, tb = opA in "tT", opB in "tT"
    M = A.shape[1] // groups if ta else A.shape[0]
    K = A.shape[0] if ta else A.shape[1] // groups
    N = Bm.shape[0] if tb else Bm.shape[1] // groups
    _require((Bm.shape[1] // groups if tb else Bm.shape[0]) == K and C.shape == (M, N * groups), "shapes do not agree")
    _require(_same_dtype(A, Bm, C) and C.dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), "dtype mismatch")
    _launch("group_gemm", context.handle, opA.encode(), opB.encode(), alpha, A.desc(), Bm.desc(), beta, C.desc(), groups)


def gemmBatched(context, opA, opB, C, A, Bm, alpha=1.0, beta=0.0):
    """reference: src/core/math.cpp:662-680; rank-2 operands are broadcast over the batch."""
    _require(C.rank() == 3 and (A.rank() == 3 or Bm.rank() == 3), "gemmBatched takes rank-3 tensors")
    M, N, K = _gemm_dims(opA, A, opB, Bm)
    _require(C.shape[1:] == (M, N), "shape of C")
    _require(A.rank() == 2 or A.shape[0] == C.shape[0], "batch of A")
    _require(Bm.rank() == 2 or Bm.shape[0] == C.shape[0], "batch of B")
    _require(_same_dtype(A, Bm, C) and C.dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), "dtype mismatch")
    _launch("gemm_batched_v2", context.handle, opA.encode(), opB.encode(), alpha, A.desc(), Bm.desc(), beta, C.desc())


def gemm_ex(context, D, alpha, opA, A, opB, Bm, beta, C, bias, act):
    """D = act(alpha op(A) op(B) + beta C + bias) (reference: src/core/math.cpp:682-702)."""
    M, N, K = _gemm_dims(opA, A, opB, Bm)
    _require(D.shape == (M, N), "shape of D")
    _require(beta == 0.0 or (C is not None and C.shape == (M, N)), "shape of C")
    _require(_same_dtype(A, Bm, C, D, bias) and D.dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), "dtype mismatch")
    _require(bias is None or bias.isEmpty() or bias.volume() == N, "bias must be [N]")
    c = C if (C is not None and not C.isEmpty()) else D
    _launch("gemm_ex", context.handle, D.dtype, D.shape_desc(), D.ptr, alpha, opA.encode(), A.shape_desc(), A.ptr, opB.encode(), Bm.shape_desc(), Bm.ptr,
                    beta, c.shape_desc(), c.ptr, _ptr(bias), act_of(act))


def im2row(context, output, input, kernel_size, invert=False, padding=None):
    """reference: src/core/math.cpp (im2row) -> cuda_im2row; `padding` is one host value or None for zeros."""
    b, h, w, c = input.shape
    _require(output.volume() == b * h * w * kernel_size * kernel_size * c, "im2row output size")
    pad = None
    if padding is not None:
        pad = np.array([padding], _NP_OF[input.dtype])
    _launch("im2row", context.handle, input.dtype, input.shape_desc(), output.ptr, input.ptr, kernel_size, bool(invert),
                   None if pad is None else pad.ctypes.data_as(ctypes.c_void_p))


def convolutionImplicitGemmForward(context, input, weights, output, bias, add, act):
    """y = act(conv(x, w) + bias + add) (reference: src/core/math.cpp:399-416)."""
    _require(input.rank() == 4 and weights.rank() == 4 and output.rank() == 4, "NHWC tensors")
    _require(input.shape[3] == weights.shape[3] and output.shape[3] == weights.shape[0], "filters mismatch")
    _require(output.shape[:3] == input.shape[:3], "stride 1, same padding")
    _require(_same_dtype(input, weights, output, bias, add) and input.dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), "dtype mismatch")
    _require(add is None or add.isEmpty() or add.shape == output.shape, "add must have the output's shape")
    _launch("convolution_implicit_gemm_forward", context.handle, weights.dtype, input.shape_desc(), weights.shape_desc(), input.ptr, weights.ptr,
                                              output.ptr, _ptr(bias), _ptr(add), act_of(act))


def explicit_gemm_forward(context, input, output, weights, bias, workspace, activation, add=None):
    """im2row + gemm_ex('n','t'), exactly the reference's sequence (src/core/math.cpp:1595-1626)."""
    k = weights.shape[1]
    _require(weights.shape[1] == weights.shape[2], "square kernel")
    rows = input.volume() // input.lastDim()
    cols = weights.volume() // weights.firstDim()
    if k == 1:
        input_matrix = input.view((rows, input.lastDim()))
    else:
        input_matrix = workspace.view((rows, cols))
        im2row(context, input_matrix, input, k, False, None)
    output_matrix = output.view((rows, output.lastDim()))
    weight_matrix = weights.view((weights.firstDim(), cols))
    if add is None or add.isEmpty():
        gemm_ex(context, output_matrix, 1.0, "n", input_matrix, "t", weight_matrix, 0.0, output_matrix, bias, activation)
    else:
        gemm_ex(context, output_matrix, 1.0, "n", input_matrix, "t", weight_matrix, 1.0, add.view(output_matrix.shape), bias, activation)


def quantized_scale_shift_act(context, output, output_transform, input, scales, bias, act, ext=None, ext_transform=(1.0, 0.0)):
    """reference: src/core/math.cpp (quantized_scale_shift_act) -> cuda_quantized_scale_shift_act; transforms are (scale, shift)."""
    _require(input.dtype == B.DTYPE_INT32 and scales.dtype == B.DTYPE_FLOAT32 and bias.dtype == B.DTYPE_FLOAT32, "int32 input, fp32 scales / bias")
    _require(output.dtype in (B.DTYPE_INT8, B.DTYPE_FLOAT32, B.DTYPE_FLOAT16), "output must be int8, fp16 or fp32")
    _require(input.volume() == output.volume() and scales.volume() == output.lastDim() and bias.volume() == output.lastDim(), "shape mismatch")
    _require(ext is None or ext.isEmpty() or (ext.dtype == B.DTYPE_INT8 and ext.volume() == output.volume()), "ext must be int8 of the output's shape")
    _launch("quantized_scale_shift_act", context.handle, output.dtype, output.shape_desc(), output.ptr, B.mlQuantizationData_t(*output_transform), input.ptr,
                                      scales.ptr, bias.ptr, act_of(act), _ptr(ext), B.mlQuantizationData_t(*ext_transform))


def quantizedConvForward(context, input, input_transform, weights, scales, bias, output, output_transform, ext=None, ext_transform=(1.0, 0.0),
                         act="linear"):
    """Whole int8 convolution of reference src/layers/Conv2D.cpp:240-308 in one call (no counterpart in the reference's math.hpp)."""
    _require(input.dtype == B.DTYPE_INT8 and weights.dtype == B.DTYPE_INT8, "int8 input and weights")
    _require(input.shape[3] == weights.shape[3] and output.shape[3] == weights.shape[0] and output.shape[:3] == input.shape[:3], "shape mismatch")
    _require(output.dtype in (B.DTYPE_INT8, B.DTYPE_FLOAT32), "output must be int8 or fp32")
    _require(scales.volume() == weights.shape[0] and bias.volume() == weights.shape[0], "scales / bias must be [Cout]")
    _require(ext is None or ext.isEmpty() or (ext.dtype == B.DTYPE_INT8 and ext.shape == output.shape), "ext must be int8 of the output's shape")
    _launch("quantized_conv_forward", context.handle, input.shape_desc(), weights.shape_desc(), input.ptr, B.mlQuantizationData_t(*input_transform),
                                   weights.ptr, scales.ptr, bias.ptr, output.dtype, output.ptr, B.mlQuantizationData_t(*output_transform), _ptr(ext),
                                   B.mlQuantizationData_t(*ext_transform), act_of(act))


def addBiasAct(context, alpha, input, bias, beta, output, act):
    _require(_same_dtype(input, bias, output) and input.volume() == output.volume(), "shape / dtype mismatch")
    _require(bias is None or bias.isEmpty() or bias.volume() == input.lastDim(), "bias must be [last dim]")
    B.fn("add_bias_act")(context.handle, alpha, input.desc(), _desc(bias), beta, output.desc(), act_of(act))


def activationForward(context, alpha, input, beta, output, act):
    _require(_same_dtype(input, output) and input.volume() == output.volume(), "shape / dtype mismatch")
    B.fn("activation_forward")(context.handle, alpha, input.desc(), beta, output.desc(), act_of(act))


def addTensors(context, alpha1, x1, alpha2, x2, alpha3, x3, beta, y):
    for x in (x1, x2, x3):
        _require(x is None or x.isEmpty() or (x.volume() == y.volume() and x.dtype == y.dtype), "shape / dtype mismatch")
    B.fn("add_tensors")(context.handle, alpha1, _desc(x1), alpha2, _desc(x2), alpha3, _desc(x3), beta, y.desc())


def convertType(context, dst, src):
    _require(dst.volume() == src.volume(), "size mismatch")
    pair = (src.dtype, dst.dtype)
    ok = src.dtype == dst.dtype or pair in ((B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), (B.DTYPE_FLOAT32, B.DTYPE_FLOAT16))
    if not ok:
        raise ValueError("unsupported conversion")  # reference: std::logic_error("unsupported conversion"), src/backend/cpu/dispatcher.cpp:61
    B.fn("convert_type")(context.handle, dst.ptr, dst.dtype, src.ptr, src.dtype, src.volume())


def unpackInput(context, dst, src):
    """dst [..., C] <- bit planes packed 32 per uint32 word (reference: src/backend/cpu/dispatcher.cpp:112-123,143-174)."""
    words = (dst.lastDim() + 31) // 32
    _require(src.sizeInBytes() >= (dst.volume() // dst.lastDim()) * words * 4, "packed input too small")
    B.fn("unpack_input")(context.handle, dst.shape_desc(), dst.dtype, dst.ptr, src.ptr)


def softmaxForward(context, output, input):
    """Row-wise softmax over the last dimension; output may be the input (reference: src/core/math.cpp:1013-1029)."""
    _require(_same_dtype(input, output) and input.volume() == output.volume(), "shape / dtype mismatch")
    _launch("softmax_forward", context.handle, input.dtype, input.shape_desc(), output.ptr, input.ptr)


def globalAveragePoolingForward(context, alpha, input, beta, output):
    """[B, H, W, C] -> [B, C]: alpha * mean over the pixels + beta * output (reference: src/core/math.cpp:515-531)."""
    _require(len(input.shape) == 4 and len(output.shape) == 2, "input must be [B, H, W, C] and output [B, C]")
    _require(input.shape[0] == output.shape[0] and input.shape[3] == output.shape[1] and _same_dtype(input, output), "shape / dtype mismatch")
    _launch("global_average_pooling_forward", context.handle, alpha, input.desc(), beta, output.desc())


def batchnormInference(context, alpha, input, weights, bias, avg_var, beta, output, act="linear"):
    """alpha * act((x - mean) * gamma / sqrt(var + 1e-6) + bias) + beta * output; avg_var fp32 [2, C] (reference: src/core/math.cpp:722-737)."""
    _require(_same_dtype(input, weights, bias, output) and input.volume() == output.volume(), "shape / dtype mismatch")
    _require(avg_var.dtype == B.DTYPE_FLOAT32 and avg_var.volume() == 2 * input.lastDim(), "statistics must be fp32 [2, C]")
    for t in (weights, bias):
        _require(t is None or t.isEmpty() or t.volume() == input.lastDim(), "gamma / bias must be [C]")
    _launch("batchnorm_inference", context.handle, alpha, input.desc(), _desc(weights), _desc(bias), avg_var.desc(), beta, output.desc(), act_of(act))


def rmsnormForward(context, input, output, weights=None):
    """y = (gamma * x) / (1e-6 + sqrt(mean x^2)) over the last dimension; weights (gamma) may be None (reference: src/core/math.cpp:844-860)."""
    _require(_same_dtype(input, output, weights) and input.volume() == output.volume(), "shape / dtype mismatch")
    _require(weights is None or weights.isEmpty() or weights.volume() == input.shape[-1], "weights must have one element per column")
    _launch("rmsnorm_forward", context.handle, input.shape_desc(), input.dtype, input.ptr, output.ptr,
            None if weights is None or weights.isEmpty() else weights.ptr)


def multiHeadAttentionGetWorkspaceSize(context, input_shape, weights_shape, num_heads, training=False):
    """Elements of workspace that multiHeadAttentionForward needs (reference: src/core/math.cpp:881-895)."""
    return B.fn("multi_head_attention_get_workspace_size")(B.make_shape(input_shape), B.make_shape(weights_shape), num_heads, training)


def multiHeadAttentionForward(context, input, output, weights, bias, workspace, backward_data, num_heads, symmetric):
    """Self-attention over the H*W tokens of every image: input [B, H, W, (3 - symmetric) * E] holds q, k, v per token (k = q when
    symmetric), weights is the relative-position table [heads, 2r-1, round_up(2r-1, 4)] or None, output [B, H, W, E]; bias and workspace
    are accepted and unused, backward_data must be None or empty (reference: src/core/math.cpp:896-915)."""
    parts = 2 if symmetric else 3
    _require(len(input.shape) == 4 and input.shape[3] % parts == 0, "input must be [B, H, W, (3 - symmetric) * E]")
    _require(tuple(output.shape) == tuple(input.shape[:3]) + (input.shape[3] // parts,) and _same_dtype(input, output, weights), "shape / dtype mismatch")
    empty = lambda t: t is None or t.isEmpty()
    _require((input.shape[3] // parts) % num_heads == 0, "embedding must be divisible by the number of heads")
    _require(empty(backward_data), "keeping the attention matrix for a backward pass is not implemented (inference only)")
    if not empty(weights):
        size = weights.shape[1] if len(weights.shape) == 3 else 0
        _require(len(weights.shape) == 3 and weights.shape[0] == num_heads and size % 2 == 1 and weights.shape[2] == (size + 3) // 4 * 4,
                 "the position table must be [heads, 2r-1, round_up(2r-1, 4)]")
    _launch("multi_head_attention_forward", context.handle, input.shape_desc(), B.make_shape(() if empty(weights) else weights.shape),
            B.make_shape(() if empty(bias) else bias.shape), input.dtype, input.ptr, output.ptr, None if empty(weights) else weights.ptr,
            None if empty(bias) else bias.ptr, None if empty(workspace) else workspace.ptr, None if empty(backward_data) else backward_data.ptr,
            num_heads, bool(symmetric))


def _require_routing(input, indices_and_values):
    _require(len(input.shape) == 4 and len(indices_and_values.shape) == 4 and indices_and_values.shape[1] == 2, "scores [B, H, W, E], routing table [B, 2, E, K]")
    _require(input.shape[0] == indices_and_values.shape[0] and input.shape[3] == indices_and_values.shape[2], "batch size or number of experts differ")
    _require(_same_dtype(input, indices_and_values) and input.dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), "fp16 or fp32 tensors of one type")
    _require(input.shape[1] * input.shape[2] <= 2048 and input.shape[3] <= 4096 and input.shape[0] <= 65535, "at most 2048 tokens per image, 4096 experts")


def expertChoiceRoutingForward(context, input, indicesAndValues):
    """Every expert takes its K best tokens of each image (reference: src/core/math.cpp:1371-1383)."""
    _require_routing(input, indicesAndValues)
    _launch("expert_choice_routing_forward", context.handle, input.desc(), indicesAndValues.desc())


def tokenChoiceRoutingForward(context, input, bias, indicesAndValues):
    """Every token takes the expert with the largest score + bias (reference: src/core/math.cpp:1343-1355)."""
    _require_routing(input, indicesAndValues)
    _require(bias is None or bias.isEmpty() or (bias.volume() == input.shape[3] and bias.dtype == input.dtype), "bias must be [E] of the scores' type")
    _launch("token_choice_routing_forward", context.handle, input.desc(), _desc(bias), indicesAndValues.desc())


def hashRouting(context, input, indicesAndValues):
    """reference: src/core/math.cpp:1329-1341."""
    _require_routing(input, indicesAndValues)
    _launch("hash_routing", context.handle, input.desc(), indicesAndValues.desc())


def gatherTokensForward(context, input, indicesAndValues, beta, output):
    """[B, H, W, C] -> [B, K, E, C] (reference: src/core/math.cpp:1410-1422)."""
    _require(len(input.shape) == 4 and len(output.shape) == 4 and len(indicesAndValues.shape) == 4 and indicesAndValues.shape[1] == 2, "rank-4 tensors")
    b, k, e, c = output.shape
    _require(input.shape[0] == b and input.shape[3] == c and indicesAndValues.shape == (b, 2, e, k), "shapes do not agree")
    _require(_same_dtype(input, output, indicesAndValues) and input.dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), "fp16 or fp32 tensors of one type")
    _launch("gather_tokens_forward", context.handle, input.desc(), indicesAndValues.desc(), beta, output.desc())


def moeForward(context, input, weights, bias, beta, output, act):
    """One dense layer per expert on [B, K, E, C] (reference: src/core/math.cpp:1462-1475)."""
    _require(len(input.shape) == 4 and len(output.shape) == 4 and len(weights.shape) == 3, "x [B, K, E, C], weights [E, N, C], y [B, K, E, N]")
    b, k, e, c = input.shape
    n = weights.shape[1]
    _require(weights.shape == (e, n, c) and output.shape == (b, k, e, n), "shapes do not agree")
    _require(bias is None or bias.isEmpty() or bias.volume() == e * n, "bias must be [E, N]")
    _require(_same_dtype(input, output, weights, bias) and input.dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), "fp16 or fp32 tensors of one type")
    _require(b * k <= 0x7fffffff and e <= 65535, "too large")
    _launch("moe_forward", context.handle, input.desc(), weights.desc(), _desc(bias), beta, output.desc(), act_of(act))


def scatterTokensForward(context, input, indicesAndValues, beta, output):
    """[B, K, E, C] -> [B, H, W, C], every token the gated sum of its slots (reference: src/core/math.cpp:1436-1448)."""
    _require(len(input.shape) == 4 and len(output.shape) == 4 and len(indicesAndValues.shape) == 4 and indicesAndValues.shape[1] == 2, "rank-4 tensors")
    b, k, e, c = input.shape
    _require(output.shape[0] == b and output.shape[3] == c and indicesAndValues.shape == (b, 2, e, k), "shapes do not agree")
    _require(_same_dtype(input, output, indicesAndValues) and input.dtype in (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32), "fp16 or fp32 tensors of one type")
    _launch("scatter_tokens_forward", context.handle, input.desc(), indicesAndValues.desc(), beta, output.desc())


def foldBatchnorm(context, layer_weights, layer_bias, bn_weights, bn_bias, bn_avg_var):
    """Folds a batch normalisation into the preceding layer's weights and bias, in place (reference: src/core/math.cpp:786-802, which
    also synchronises with the context afterwards)."""
    channels = layer_weights.shape[-1] if len(layer_weights.shape) == 3 else layer_weights.shape[0]
    _require(_same_dtype(layer_weights, layer_bias, bn_weights, bn_bias) and layer_bias.volume() == channels, "shape / dtype mismatch")
    _require(bn_avg_var.dtype == B.DTYPE_FLOAT32 and bn_avg_var.volume() == 2 * channels, "statistics must be fp32 [2, channels]")
    B.fn("fold_batchnorm")(context.handle, layer_weights.desc(), layer_bias.desc(), _desc(bn_weights), _desc(bn_bias), bn_avg_var.desc())
    context.synchronize()
