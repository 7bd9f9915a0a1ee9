"""numpy front-end of the CPU oracle (liboracle.so) and of the compiled reference CPU backend (oracle/_ref).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the CPU-baseline leg of bench.py. The HIP backend
package (minml_amd) never imports this module.

fp16 tensors are numpy uint16 arrays holding raw bit patterns (so that no converter sits on a comparison path);
`to_half` / `from_half` convert with the reference's truncating rule.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libminml_cpu_ref.so")

FLOAT16, FLOAT32, INT8, INT32 = 2, 3, 6, 8
LINEAR, SIGMOID, TANH, RELU, LEAKY_RELU, EXP = range(6)

_c_void_p = ctypes.c_void_p
_sz = ctypes.c_size_t
_i = ctypes.c_int
_f = ctypes.c_float


def build(reference="/root/reference"):
    """Compiles liboracle.so and, when a reference checkout is present, oracle/_ref: the reference's CPU backend as a library, the
    generator of the int8 layer fixtures, and (when the HIP library has been built) the reference's dispatcher, layers and graph linked
    on top of the HIP library (`dropin_graph`, the link-time swap of the device backend)."""
    subprocess.run(["make", "-s", "-C", HERE, "oracle"], check=True)
    if os.path.isdir(os.path.join(reference, "src", "backend", "cpu")):
        targets = ["ref", "fixtures"]
        if os.path.exists(os.path.join(HERE, "..", "minml_amd", "libminml_hip.so")):
            targets.append("dropin")
        subprocess.run(["make", "-s", "-j8", "-C", HERE] + targets + ["REF=" + reference], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.oracle_fp32_to_fp16.restype = ctypes.c_uint16
        _lib.oracle_fp32_to_fp16.argtypes = [_f]
        _lib.oracle_fp16_to_fp32.restype = _f
        _lib.oracle_fp16_to_fp32.argtypes = [ctypes.c_uint16]
        _lib.oracle_quantize.restype = ctypes.c_int32
        _lib.oracle_quantize.argtypes = [_f, _i]
        _lib.oracle_set_num_threads.argtypes = [_i]
        _lib.oracle_convert_fp32_to_fp16.argtypes = [_c_void_p, _c_void_p, _sz]
        _lib.oracle_convert_fp16_to_fp32.argtypes = [_c_void_p, _c_void_p, _sz]
        _lib.oracle_winograd_weight_transform.argtypes = [_i, _i, _i, _c_void_p, _c_void_p, _i]
        _lib.oracle_winograd_input_transform.argtypes = [_i, _i, _i, _i, _i, _c_void_p, _c_void_p]
        _lib.oracle_winograd_output_transform.argtypes = [_i, _i, _i, _i, _i, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i]
        _lib.oracle_gemm.argtypes = [_i, ctypes.c_char, ctypes.c_char, _i, _i, _i, _i, _f, _c_void_p, _sz, _c_void_p, _sz, _f, _c_void_p,
                                     _c_void_p, _sz, _c_void_p, _i, _i]
        _lib.oracle_int8_gemm_nt.argtypes = [_i, _i, _i, _c_void_p, _c_void_p, _c_void_p]
        _lib.oracle_im2row.argtypes = [_i, _i, _i, _i, _i, _i, _c_void_p, _c_void_p]
        _lib.oracle_conv2d_forward.argtypes = [_i, _i, _i, _i, _i, _i, _i, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i, _i]
        _lib.oracle_int8_conv2d_forward.argtypes = [_i, _i, _i, _i, _i, _i, _c_void_p, _f, _f, _c_void_p, _c_void_p, _c_void_p, _i, _c_void_p,
                                                    _f, _f, _c_void_p, _f, _f, _i]
        _lib.oracle_quantized_scale_shift_act.argtypes = [_i, _sz, _i, _c_void_p, _f, _f, _c_void_p, _c_void_p, _c_void_p, _i, _c_void_p, _f, _f]
        _lib.oracle_quantize_weights.argtypes = [_i, _i, _c_void_p, _c_void_p, _f, _f, _c_void_p, _c_void_p, _c_void_p]
        _lib.oracle_add_bias_act.argtypes = [_i, _sz, _i, _c_void_p, _c_void_p, _c_void_p, _i]
        _lib.oracle_add_tensors.argtypes = [_i, _sz, _f, _c_void_p, _f, _c_void_p, _f, _c_void_p, _f, _c_void_p]
        _lib.oracle_unpack_input.argtypes = [_i, _sz, _i, _c_void_p, _c_void_p]
        _lib.oracle_softmax_forward.argtypes = [_i, _sz, _i, _c_void_p, _c_void_p]
        _lib.oracle_global_average_pooling_forward.argtypes = [_i, _i, _i, _i, _f, _c_void_p, _f, _c_void_p]
        _lib.oracle_batchnorm_inference.argtypes = [_i, _sz, _i, _f, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _f, _c_void_p, _i]
        _lib.oracle_fold_batchnorm.argtypes = [_i, _i, _i, _i, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p]
        _lib.oracle_rmsnorm_forward.argtypes = [_i, _sz, _i, _c_void_p, _c_void_p, _c_void_p]
        _lib.oracle_multi_head_attention_forward.argtypes = [_i, _i, _i, _i, _i, _i, _i, _c_void_p, _c_void_p, _c_void_p, _i]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(_c_void_p)


def _c(a, dtype=None):
    if a is None:
        return None
    return np.ascontiguousarray(a, dtype=dtype)


def dtype_code(a):
    return {np.dtype(np.uint16): FLOAT16, np.dtype(np.float32): FLOAT32, np.dtype(np.int8): INT8, np.dtype(np.int32): INT32}[a.dtype]


def np_dtype(code):
    return {FLOAT16: np.uint16, FLOAT32: np.float32, INT8: np.int8, INT32: np.int32}[code]


def set_num_threads(n):
    lib().oracle_set_num_threads(int(n))


def to_half(x):
    """float32 array -> uint16 bit patterns, truncating toward zero like the reference."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_convert_fp32_to_fp16(_p(x), _p(out), x.size)
    return out


def from_half(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().oracle_convert_fp16_to_fp32(_p(h), _p(out), h.size)
    return out


def as_float(a):
    """Any oracle tensor as float32 / float64-comparable values."""
    return from_half(a) if a.dtype == np.uint16 else a


def winograd_weight_transform(w, invert=False):
    w = _c(w)
    cout, _, _, cin = w.shape
    out = np.empty((36, cout, cin), w.dtype)
    lib().oracle_winograd_weight_transform(dtype_code(w), cout, cin, _p(w), _p(out), int(invert))
    return out


def winograd_input_transform(x):
    x = _c(x)
    b, h, w, c = x.shape
    tiles = b * ((h + 3) // 4) * ((w + 3) // 4)
    out = np.empty((36, tiles, c), x.dtype)
    lib().oracle_winograd_input_transform(dtype_code(x), b, h, w, c, _p(x), _p(out))
    return out


def winograd_output_transform(matrices, shape, bias=None, ext=None, act=LINEAR):
    matrices = _c(matrices)
    b, h, w, c = shape
    out = np.zeros(shape, matrices.dtype)
    bias, ext = _c(bias), _c(ext)
    lib().oracle_winograd_output_transform(dtype_code(matrices), b, h, w, c, _p(matrices), _p(out), _p(bias), _p(ext), act)
    return out


def gemm(A, B, opA="n", opB="t", alpha=1.0, beta=0.0, C=None, bias=None, act=LINEAR, k_tile=1024):
    """D = act(alpha * op(A) op(B) + bias + beta * C); rank-3 operands are batched, rank-2 ones broadcast."""
    A, B, C, bias = _c(A), _c(B), _c(C), _c(bias)
    ta, tb = opA in "tT", opB in "tT"
    M = A.shape[-1] if ta else A.shape[-2]
    K = A.shape[-2] if ta else A.shape[-1]
    N = B.shape[-2] if tb else B.shape[-1]
    batched = A.ndim == 3 or B.ndim == 3
    batch = (A.shape[0] if A.ndim == 3 else B.shape[0]) if batched else 1
    D = np.zeros((batch, M, N) if batched else (M, N), A.dtype)
    sa = A.shape[-1] * A.shape[-2] if A.ndim == 3 else 0
    sb = B.shape[-1] * B.shape[-2] if B.ndim == 3 else 0
    lib().oracle_gemm(dtype_code(A), opA.encode(), opB.encode(), M, N, K, batch, alpha, _p(A), sa, _p(B), sb, beta, _p(C), _p(D), M * N, _p(bias), act,
                      k_tile)
    return D


def int8_gemm_nt(A, B):
    A, B = _c(A, np.int8), _c(B, np.int8)
    C = np.empty((A.shape[0], B.shape[0]), np.int32)
    lib().oracle_int8_gemm_nt(A.shape[0], B.shape[0], A.shape[1], _p(A), _p(B), _p(C))
    return C


def im2row(x, kernel_size):
    x = _c(x)
    b, h, w, c = x.shape
    out = np.empty((b * h * w, kernel_size * kernel_size * c), x.dtype)
    lib().oracle_im2row(x.dtype.itemsize, b, h, w, c, kernel_size, _p(x), _p(out))
    return out


def conv2d_forward(x, w, bias=None, add=None, act=LINEAR, k_tile=1024):
    x, w, bias, add = _c(x), _c(w), _c(bias), _c(add)
    b, h, wd, cin = x.shape
    cout, k = w.shape[0], w.shape[1]
    out = np.zeros((b, h, wd, cout), x.dtype)
    lib().oracle_conv2d_forward(dtype_code(x), b, h, wd, cin, cout, k, _p(x), _p(w), _p(out), _p(bias), _p(add), act, k_tile)
    return out


def quantize(x, bits=8):
    return lib().oracle_quantize(float(x), bits)


def int8_conv2d_forward(x, in_qd, w, scales, bias, out_dtype, out_qd, ext=None, ext_qd=(1.0, 0.0), act=LINEAR):
    x, w, ext = _c(x, np.int8), _c(w, np.int8), _c(ext, np.int8)
    scales, bias = _c(scales, np.float32), _c(bias, np.float32)
    b, h, wd, cin = x.shape
    cout, k = w.shape[0], w.shape[1]
    out = np.zeros((b, h, wd, cout), np_dtype(out_dtype))
    lib().oracle_int8_conv2d_forward(b, h, wd, cin, cout, k, _p(x), in_qd[0], in_qd[1], _p(w), _p(scales), _p(bias), out_dtype, _p(out), out_qd[0],
                                     out_qd[1], _p(ext), ext_qd[0], ext_qd[1], act)
    return out


def quantized_scale_shift_act(acc, scales, bias, out_dtype, out_qd, ext=None, ext_qd=(1.0, 0.0), act=LINEAR):
    acc, ext = _c(acc, np.int32), _c(ext, np.int8)
    scales, bias = _c(scales, np.float32), _c(bias, np.float32)
    last = acc.shape[-1]
    out = np.zeros(acc.shape, np_dtype(out_dtype))
    lib().oracle_quantized_scale_shift_act(out_dtype, acc.size // last, last, _p(out), out_qd[0], out_qd[1], _p(acc), _p(scales), _p(bias), act, _p(ext),
                                           ext_qd[0], ext_qd[1])
    return out


def quantized_scale_shift_act_device_form(acc, scales, bias, out_qd, ext=None, ext_qd=(1.0, 0.0), act=LINEAR):
    """The int8 requantisation as the reference's DEVICE kernel writes it (src/backend/cuda/kernels/quantized.cu:44-47, 232-254):
    x = acc * scale + bias (+ ext * ext_scale + ext_shift), activation, then clamp(round((x - shift) / scale)) — where the CPU layer,
    which quantized_scale_shift_act above and the HIP library follow, evaluates clamp(round(x * (1 / scale) + (-shift / scale))).
    PARITY UNPINNED: that kernel cannot run here, and whether its compiler contracts `acc * scale + bias` into one fused operation is
    unknown (evaluated unfused here). Used only to count how often the two formulas disagree. int8 output, linear or ReLU."""
    f = np.float32
    acc = np.asarray(acc, np.int32).astype(f)
    x = acc * np.asarray(scales, f) + np.asarray(bias, f)
    if ext is not None:
        x = x + (np.asarray(ext, np.int8).astype(f) * f(ext_qd[0]) + f(ext_qd[1]))
    if act == RELU:
        x = np.maximum(x, f(0.0))
    elif act != LINEAR:
        raise ValueError("linear or ReLU only")
    q = (x - f(out_qd[1])) / f(out_qd[0])
    q = np.sign(q) * np.floor(np.abs(q) + f(0.5))  # round(): halves away from zero
    return np.clip(q, -128.0, 127.0).astype(np.int8)


def quantize_weights(w, bias, in_qd):
    w = _c(w, np.float32)
    rows, cols = w.shape[0], w.size // w.shape[0]
    bias = _c(bias, np.float32)
    q = np.empty(w.shape, np.int8)
    scales = np.empty(rows, np.float32)
    qb = np.empty(rows, np.float32)
    lib().oracle_quantize_weights(rows, cols, _p(w), _p(bias), in_qd[0], in_qd[1], _p(q), _p(scales), _p(qb))
    return q, scales, qb


def add_bias_act(x, bias=None, act=LINEAR):
    x, bias = _c(x), _c(bias)
    out = np.empty_like(x)
    lib().oracle_add_bias_act(dtype_code(x), x.size // x.shape[-1], x.shape[-1], _p(out), _p(x), _p(bias), act)
    return out


def add_tensors(y, a1=0.0, x1=None, a2=0.0, x2=None, a3=0.0, x3=None, beta=0.0):
    y = np.array(y, copy=True, order="C")
    x1, x2, x3 = _c(x1), _c(x2), _c(x3)
    lib().oracle_add_tensors(dtype_code(y), y.size, a1, _p(x1), a2, _p(x2), a3, _p(x3), beta, _p(y))
    return y


def unpack_input(packed, shape, dtype):
    packed = _c(packed, np.uint32)
    out = np.empty(shape, np_dtype(dtype))
    lib().oracle_unpack_input(dtype, out.size // shape[-1], shape[-1], _p(out), _p(packed))
    return out


def softmax_forward(x):
    """Row-wise softmax over the last dimension."""
    x = _c(x)
    out = np.empty_like(x)
    lib().oracle_softmax_forward(dtype_code(x), x.size // x.shape[-1], x.shape[-1], _p(out), _p(x))
    return out


def global_average_pooling_forward(x, alpha=1.0, beta=0.0, y=None):
    """[B, H, W, C] -> [B, C]: alpha * mean over the pixels + beta * y."""
    x = _c(x)
    b, h, w, c = x.shape
    out = np.zeros((b, c), x.dtype) if y is None else np.array(y, copy=True, order="C")
    lib().oracle_global_average_pooling_forward(dtype_code(x), b, h * w, c, alpha, _p(x), beta, _p(out))
    return out


def batchnorm_inference(x, gamma, bias, avg_var, act=LINEAR, alpha=1.0, beta=0.0, y=None):
    """alpha * act((x - mean) * gamma / sqrt(var + 1e-6) + bias) + beta * y; avg_var fp32 [2, C]."""
    x, gamma, bias = _c(x), _c(gamma), _c(bias)
    avg_var = _c(avg_var, np.float32)
    out = np.zeros_like(x) if y is None else np.array(y, copy=True, order="C")
    lib().oracle_batchnorm_inference(dtype_code(x), x.size // x.shape[-1], x.shape[-1], alpha, _p(x), _p(gamma), _p(bias), _p(avg_var), beta,
                                     _p(out), act)
    return out


def fold_batchnorm(layer_weights, layer_bias, bn_weights, bn_bias, bn_avg_var):
    """Returns (weights, bias) with the batch normalisation folded in. Rank-3 weights are depthwise (channels last)."""
    w = np.array(layer_weights, copy=True, order="C")
    b = np.array(layer_bias, copy=True, order="C")
    last = w.ndim == 3
    channels = w.shape[-1] if last else w.shape[0]
    lib().oracle_fold_batchnorm(dtype_code(w), channels, w.size // channels, int(last), _p(w), _p(b), _p(_c(bn_weights)), _p(_c(bn_bias)),
                                _p(_c(bn_avg_var, np.float32)))
    return w, b


# ---------------------------------------------------------------------------------------------------------------------------
# the reference's own CPU backend, compiled from its sources by `make -C oracle ref` (present only where that was built)
# ---------------------------------------------------------------------------------------------------------------------------
def rmsnorm_forward(x, weights=None):
    """y = (gamma * x) / (1e-6 + sqrt(mean x^2)) over the last dimension; `weights` (gamma, [last_dim]) may be None."""
    x = _c(x)
    w = None if weights is None else _c(weights)
    out = np.empty_like(x)
    lib().oracle_rmsnorm_forward(dtype_code(x), x.size // x.shape[-1], x.shape[-1], _p(x), _p(out), _p(w))
    return out


def multi_head_attention_forward(x, num_heads, table=None, symmetric=False):
    """x [B, H, W, (3 - symmetric) * E] -> [B, H, W, E]; table [heads, 2r-1, round_up(2r-1, 4)] (relative-position bias) or None."""
    x = _c(x)
    t = None if table is None else _c(table)
    b, h, w, c = x.shape
    e = c // (2 if symmetric else 3)
    out = np.empty((b, h, w, e), x.dtype)
    lib().oracle_multi_head_attention_forward(dtype_code(x), b, h, w, e, num_heads, int(bool(symmetric)), _p(x), _p(out), _p(t),
                                              0 if t is None else t.shape[1])
    return out


class _Shape(ctypes.Structure):
    _fields_ = [("rank", _i), ("dim", _i * 6)]


class _Tensor(ctypes.Structure):
    _fields_ = [("data", _c_void_p), ("dtype", _i), ("rank", _i), ("dim", _i * 6)]


def _tensor(a):
    t = _Tensor()
    if a is None:
        return t
    t.data = a.ctypes.data
    t.dtype = dtype_code(a)
    t.rank = a.ndim
    for k, d in enumerate(a.shape):
        t.dim[k] = int(d)
    return t


def _shape(*dims):
    s = _Shape()
    s.rank = len(dims)
    for k, d in enumerate(dims):
        s.dim[k] = int(d)
    return s


class Reference:
    """Thin caller of the reference's cpu_* C-ABI (include/minml/backend/cpu_backend.h). One thread, like the reference."""

    def __init__(self, path=REF_PATH):
        self.lib = ctypes.CDLL(path)
        L = self.lib
        L.cpu_create_context.restype = _c_void_p
        L.cpu_destroy_context.argtypes = [_c_void_p]
        L.cpu_winograd_weight_transform.argtypes = [_c_void_p, _i, _i, _Shape, _c_void_p, _c_void_p, ctypes.c_bool]
        L.cpu_winograd_input_transform.argtypes = [_c_void_p, _i, _i, _Shape, _Shape, _c_void_p, _c_void_p]
        L.cpu_winograd_output_transform.argtypes = [_c_void_p, _i, _i, _Shape, _Shape, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i]
        L.cpu_gemm_batched.argtypes = [_c_void_p, _i, _Shape, _c_void_p, _Shape, _c_void_p, _Shape, _c_void_p, ctypes.c_char, ctypes.c_char, _f, _f]
        L.cpu_gemm_ex.argtypes = [_c_void_p, _i, _Shape, _c_void_p, _f, ctypes.c_char, _Shape, _c_void_p, ctypes.c_char, _Shape, _c_void_p, _f, _Shape,
                                  _c_void_p, _c_void_p, _i]
        L.cpu_im2row.argtypes = [_c_void_p, _i, _Shape, _c_void_p, _c_void_p, _i, ctypes.c_bool, _c_void_p]
        L.cpu_add_bias_act.argtypes = [_c_void_p, _i, _Shape, _c_void_p, _c_void_p, _c_void_p, _i]
        L.cpu_unpack_input.argtypes = [_c_void_p, _Shape, _i, _c_void_p, _c_void_p]
        L.cpu_convert_type.argtypes = [_c_void_p, _c_void_p, _i, _c_void_p, _i, _i]
        L.cpu_softmax_forward.argtypes = [_c_void_p, _i, _Shape, _c_void_p, _c_void_p]
        L.cpu_global_average_pooling_forward.argtypes = [_c_void_p, _f, _Tensor, _f, _Tensor]
        L.cpu_fold_batchnorm.argtypes = [_c_void_p, _Tensor, _Tensor, _Tensor, _Tensor, _Tensor]
        L.cpu_rmsnorm_forward.argtypes = [_c_void_p, _Shape, _i, _c_void_p, _c_void_p, _c_void_p]
        L.cpu_multi_head_attention_forward.argtypes = [_c_void_p, _Tensor, _Tensor, _Tensor, _Tensor, _Tensor, _i]
        self.ctx = L.cpu_create_context()

    @staticmethod
    def available(path=REF_PATH):
        return os.path.exists(path)

    def winograd_weight_transform(self, w, invert=False):
        w = _c(w)
        cout, k, _, cin = w.shape
        out = np.zeros((36, cout, cin), w.dtype)
        self.lib.cpu_winograd_weight_transform(self.ctx, 4, dtype_code(w), _shape(*w.shape), _p(w), _p(out), bool(invert))
        return out

    def winograd_input_transform(self, x):
        x = _c(x)
        b, h, w, c = x.shape
        out = np.zeros((36, b * ((h + 3) // 4) * ((w + 3) // 4), c), x.dtype)
        self.lib.cpu_winograd_input_transform(self.ctx, 4, dtype_code(x), _shape(c, 3, 3, c), _shape(*x.shape), _p(x), _p(out))
        return out

    def winograd_output_transform(self, matrices, shape, bias=None, ext=None, act=LINEAR):
        matrices, bias, ext = _c(matrices), _c(bias), _c(ext)
        out = np.zeros(shape, matrices.dtype)
        c = shape[-1]
        self.lib.cpu_winograd_output_transform(self.ctx, 4, dtype_code(matrices), _shape(c, 3, 3, c), _shape(*shape), _p(matrices), _p(out), _p(bias),
                                               _p(ext), act)
        return out

    def gemm_batched(self, A, B, opA="n", opB="t", alpha=1.0, beta=0.0, C=None):
        A, B = _c(A), _c(B)
        ta, tb = opA in "tT", opB in "tT"
        M = A.shape[-1] if ta else A.shape[-2]
        N = B.shape[-2] if tb else B.shape[-1]
        batch = A.shape[0] if A.ndim == 3 else B.shape[0]
        D = np.zeros((batch, M, N), A.dtype) if C is None else np.array(C, copy=True, order="C")
        self.lib.cpu_gemm_batched(self.ctx, dtype_code(A), _shape(*D.shape), _p(D), _shape(*A.shape), _p(A), _shape(*B.shape), _p(B), opA.encode(),
                                  opB.encode(), alpha, beta)
        return D

    def gemm_ex(self, A, B, opA="n", opB="t", alpha=1.0, beta=0.0, C=None, bias=None, act=LINEAR):
        A, B, C, bias = _c(A), _c(B), _c(C), _c(bias)
        ta, tb = opA in "tT", opB in "tT"
        M = A.shape[1] if ta else A.shape[0]
        N = B.shape[0] if tb else B.shape[1]
        D = np.zeros((M, N), A.dtype)
        c = C if C is not None else D
        self.lib.cpu_gemm_ex(self.ctx, dtype_code(A), _shape(M, N), _p(D), alpha, opA.encode(), _shape(*A.shape), _p(A), opB.encode(), _shape(*B.shape),
                             _p(B), beta, _shape(M, N), _p(c), _p(bias), act)
        return D

    def im2row(self, x, kernel_size):
        x = _c(x)
        b, h, w, c = x.shape
        out = np.zeros((b * h * w, kernel_size * kernel_size * c), x.dtype)
        code = {1: INT8, 2: FLOAT16, 4: FLOAT32}[x.dtype.itemsize]
        self.lib.cpu_im2row(self.ctx, code, _shape(*x.shape), _p(out), _p(x), kernel_size, False, None)
        return out

    def conv2d_forward(self, x, w, bias=None, add=None, act=LINEAR):
        """explicit_gemm_forward of the reference core (src/core/math.cpp:1595-1626) spelled with its backend calls."""
        x, w = _c(x), _c(w)
        b, h, wd, cin = x.shape
        cout, k = w.shape[0], w.shape[1]
        matrix = x.reshape(b * h * wd, cin) if k == 1 else self.im2row(x, k)
        wm = w.reshape(cout, -1)
        if add is None:
            out = self.gemm_ex(matrix, wm, bias=bias, act=act)
        else:
            out = self.gemm_ex(matrix, wm, beta=1.0, C=_c(add).reshape(-1, cout), bias=bias, act=act)
        return out.reshape(b, h, wd, cout)

    def add_bias_act(self, x, bias, act):
        x, bias = _c(x), _c(bias)
        out = np.zeros_like(x)
        self.lib.cpu_add_bias_act(self.ctx, dtype_code(x), _shape(*x.shape), _p(out), _p(x), _p(bias), act)
        return out

    def unpack_input(self, packed, shape, dtype):
        packed = _c(packed, np.uint32)
        out = np.zeros(shape, np_dtype(dtype))
        self.lib.cpu_unpack_input(self.ctx, _shape(*shape), dtype, _p(out), _p(packed))
        return out

    def convert(self, x, dst_dtype):
        x = _c(x)
        out = np.zeros(x.shape, np_dtype(dst_dtype))
        self.lib.cpu_convert_type(self.ctx, _p(out), dst_dtype, _p(x), dtype_code(x), x.size)
        return out

    def softmax_forward(self, x):
        x = _c(x)
        out = np.zeros_like(x)
        self.lib.cpu_softmax_forward(self.ctx, dtype_code(x), _shape(x.size // x.shape[-1], x.shape[-1]), _p(out), _p(x))
        return out

    def global_average_pooling_forward(self, x):
        x = _c(x)
        out = np.zeros((x.shape[0], x.shape[3]), x.dtype)
        self.lib.cpu_global_average_pooling_forward(self.ctx, 1.0, _tensor(x), 0.0, _tensor(out))
        return out

    def fold_batchnorm(self, layer_weights, layer_bias, bn_weights, bn_bias, bn_avg_var):
        """fp32 only (the reference reads every argument as float)."""
        w = np.array(layer_weights, dtype=np.float32, copy=True, order="C")
        b = np.array(layer_bias, dtype=np.float32, copy=True, order="C")
        g, bb, st = _c(bn_weights, np.float32), _c(bn_bias, np.float32), _c(bn_avg_var, np.float32)
        self.lib.cpu_fold_batchnorm(self.ctx, _tensor(w), _tensor(b), _tensor(g), _tensor(bb), _tensor(st))
        return w, b


    def rmsnorm_forward(self, x, weights=None):
        """fp32 only (the reference has no other branch: normalization.cpp:460)."""
        x = _c(x, np.float32)
        w = None if weights is None else _c(weights, np.float32)
        out = np.zeros_like(x)
        self.lib.cpu_rmsnorm_forward(self.ctx, _shape(*x.shape), dtype_code(x), _p(x), _p(out), _p(w))
        return out

    def multi_head_attention_forward(self, x, num_heads, table=None):
        """fp32 only; the layout (symmetric or not) follows from the channel count as in attention.cpp:408."""
        x = _c(x, np.float32)
        t = None if table is None else _c(table, np.float32)
        b, h, w, c = x.shape
        e = c // 3 if c % 3 == 0 else c // 2
        out = np.zeros((b, h, w, e), np.float32)
        workspace = np.zeros((b * num_heads * h * w * h * w,), np.float32)
        self.lib.cpu_multi_head_attention_forward(self.ctx, _tensor(x), _tensor(out), _tensor(t), _tensor(workspace), _tensor(None), num_heads)
        return out


_ref = None


def reference():
    """The compiled reference CPU backend, or None where oracle/_ref was not built."""
    global _ref
    if _ref is None and Reference.available():
        _ref = Reference()
    return _ref
