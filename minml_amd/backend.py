"""ctypes binding of libminml_hip.so — the C-ABI declared in include/minml_hip_backend.h.

This is the only place that touches the shared library. The library is hand-written HIP for gfx950 and there is no fallback:
if it has not been built, loading fails with an error that says how to build it.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libminml_hip.so")

# mlDataType_t / mlActivationType_t (reference: include/minml/backend/backend_types.h:40-63)
DTYPE_UNKNOWN, DTYPE_FLOAT8, DTYPE_FLOAT16, DTYPE_FLOAT32, DTYPE_FLOAT64, DTYPE_UINT8, DTYPE_INT8, DTYPE_INT16, DTYPE_INT32 = range(9)
ACTIVATION_LINEAR, ACTIVATION_SIGMOID, ACTIVATION_TANH, ACTIVATION_RELU, ACTIVATION_LEAKY_RELU, ACTIVATION_EXP = range(6)

DTYPE_SIZE = {DTYPE_FLOAT16: 2, DTYPE_FLOAT32: 4, DTYPE_INT8: 1, DTYPE_UINT8: 1, DTYPE_INT16: 2, DTYPE_INT32: 4, DTYPE_FLOAT64: 8}


class mlShape_t(ctypes.Structure):
    _fields_ = [("rank", ctypes.c_int), ("dim", ctypes.c_int * 6)]


class mlQuantizationData_t(ctypes.Structure):
    _fields_ = [("scale", ctypes.c_float), ("shift", ctypes.c_float)]


class mlTensor_t(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int), ("rank", ctypes.c_int), ("dim", ctypes.c_int * 6)]


def make_shape(dims):
    s = mlShape_t()
    s.rank = len(dims)
    for i, d in enumerate(dims):
        s.dim[i] = int(d)
    return s


def make_tensor(ptr, dtype, dims):
    t = mlTensor_t()
    t.data = ptr
    t.dtype = dtype
    t.rank = len(dims) if ptr else 0
    if ptr:
        for i, d in enumerate(dims):
            t.dim[i] = int(d)
    return t


_vp, _sz, _i, _f, _b, _c = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_float, ctypes.c_bool, ctypes.c_char
_T, _S, _Q = mlTensor_t, mlShape_t, mlQuantizationData_t

# name -> (restype, argtypes); must list every function declared in include/minml_hip_backend.h
SIGNATURES = {
    "get_number_of_devices": (_i, []),
    "get_memory": (_i, [_i]),
    "supports_type": (_b, [_i, _i]),
    "get_device_info": (ctypes.c_char_p, [_i]),
    "get_device_features": (ctypes.c_char_p, [_i]),
    "enable_tf32": (None, [_vp, _b]),
    "create_context": (_vp, [_i]),
    "synchronize_with_context": (None, [_vp]),
    "is_context_ready": (_b, [_vp]),
    "destroy_context": (None, [_vp]),
    "create_event": (_vp, [_vp]),
    "get_time_between_events": (ctypes.c_double, [_vp, _vp]),
    "wait_for_event": (None, [_vp]),
    "is_event_ready": (_b, [_vp]),
    "destroy_event": (None, [_vp]),
    "malloc": (_vp, [_i, _sz]),
    "page_lock": (None, [_vp, _sz]),
    "page_unlock": (None, [_vp]),
    "free": (None, [_vp]),
    "create_view": (_vp, [_vp, _sz, _sz]),
    "destroy_view": (None, [_vp]),
    "memset": (None, [_vp, _vp, _sz, _sz, _vp, _sz]),
    "memcpy_within_device": (None, [_vp, _vp, _sz, _vp, _sz, _sz]),
    "memcpy_from_host": (None, [_vp, _vp, _sz, _vp, _sz]),
    "memcpy_to_host": (None, [_vp, _vp, _vp, _sz, _sz]),
    "unpack_input": (None, [_vp, _S, _i, _vp, _vp]),
    "convert_type": (None, [_vp, _vp, _i, _vp, _i, _i]),
    "winograd_weight_transform": (None, [_vp, _i, _T, _T, _b]),
    "winograd_input_transform": (None, [_vp, _i, _T, _T]),
    "winograd_output_transform": (None, [_vp, _i, _T, _T, _T, _T, _i]),
    "winograd_output_input_transform": (None, [_vp, _i, _T, _T, _T, _S, _vp, _i, _T]),
    "winograd_layer_forward": (None, [_vp, _i, _T, _T, _T, _T, _T, _S, _vp, _i, _T]),
    "winograd_layer_forward_static": (None, [_vp, _i, _T, _T, _T, _T, _T, _S, _vp, _i, _T]),
    "winograd_layer_errors": (_i, [_vp]),
    "gemm_v2": (None, [_vp, _c, _c, _f, _T, _T, _f, _T]),
    "gemm_batched_v2": (None, [_vp, _c, _c, _f, _T, _T, _f, _T]),
    "gemm": (None, [_vp, _i, _S, _vp, _S, _vp, _S, _vp, _c, _c, _f, _f]),
    "gemm_batched": (None, [_vp, _i, _S, _vp, _S, _vp, _S, _vp, _c, _c, _f, _f]),
    "gemm_ex": (None, [_vp, _i, _S, _vp, _f, _c, _S, _vp, _c, _S, _vp, _f, _S, _vp, _vp, _i]),
    "convolution_implicit_gemm_forward": (None, [_vp, _i, _S, _S, _vp, _vp, _vp, _vp, _vp, _i]),
    "im2row": (None, [_vp, _i, _S, _vp, _vp, _i, _b, _vp]),
    "quantized_scale_shift_act": (None, [_vp, _i, _S, _vp, _Q, _vp, _vp, _vp, _i, _vp, _Q]),
    "add_bias_act": (None, [_vp, _f, _T, _T, _f, _T, _i]),
    "activation_forward": (None, [_vp, _f, _T, _f, _T, _i]),
    "add_tensors": (None, [_vp, _f, _T, _f, _T, _f, _T, _f, _T]),
    "scale_tensor": (None, [_vp, _f, _T]),
    "group_gemm": (None, [_vp, _c, _c, _f, _T, _T, _f, _T, _i]),
    "softmax_forward": (None, [_vp, _i, _S, _vp, _vp]),
    "global_average_pooling_forward": (None, [_vp, _f, _T, _f, _T]),
    "batchnorm_inference": (None, [_vp, _f, _T, _T, _T, _T, _f, _T, _i]),
    "fold_batchnorm": (None, [_vp, _T, _T, _T, _T, _T]),
    "rmsnorm_forward": (None, [_vp, _S, _i, _vp, _vp, _vp]),
    "multi_head_attention_get_workspace_size": (_i, [_S, _S, _i, _b]),
    "multi_head_attention_forward": (None, [_vp, _S, _S, _S, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _b]),
    "expert_choice_routing_forward": (None, [_vp, _T, _T]),
    "token_choice_routing_forward": (None, [_vp, _T, _T, _T]),
    "hash_routing": (None, [_vp, _T, _T]),
    "gather_tokens_forward": (None, [_vp, _T, _T, _f, _T]),
    "moe_forward": (None, [_vp, _T, _T, _T, _f, _T, _i]),
    "scatter_tokens_forward": (None, [_vp, _T, _T, _f, _T]),
    "quantized_conv_forward": (None, [_vp, _S, _S, _vp, _Q, _vp, _vp, _vp, _i, _vp, _Q, _vp, _Q, _i]),
    "get_stream": (_vp, [_vp]),
    "graph_begin_capture": (None, [_vp]),
    "graph_end_capture": (_vp, [_vp]),
    "graph_launch": (None, [_vp, _vp]),
    "graph_destroy": (None, [_vp]),
    "set_error_capture": (None, [_i]),
    "take_last_error": (_i, [ctypes.c_char_p, _i]),
    "error_flag_address": (_vp, []),
}

_lib = None


def load():
    """Loads libminml_hip.so and declares the prototypes. Raises if the library has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python -m minml_amd.build` (hipcc, --offload-arch=gfx950); "
                               "the HIP backend has no CPU fallback" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, "hip_" + name)
            fn.restype = restype
            fn.argtypes = argtypes
        # exceptions cannot unwind through ctypes: the library records failures instead and fn()'s wrappers raise them
        lib.hip_set_error_capture(1)
        global _error_flag
        _error_flag = ctypes.c_int.from_address(lib.hip_error_flag_address())
        _lib = lib
    return _lib


_error_flag = None
_error_buffer = ctypes.create_string_buffer(2048)
_checked = {}


def check_error():
    """Raises what a library call recorded: ValueError for a std::logic_error (a bad argument), RuntimeError otherwise."""
    kind = _lib.hip_take_last_error(_error_buffer, 2048)
    if kind != 0:
        message = _error_buffer.value.decode("utf-8", "replace")
        raise (ValueError if kind == 1 else RuntimeError)(message)


def fn(name):
    """The entry point hip_<name>, wrapped so that a failure inside the library surfaces as a Python exception."""
    wrapped = _checked.get(name)
    if wrapped is None:
        raw = getattr(load(), "hip_" + name)
        flag = _error_flag

        def wrapped(*args):
            if flag.value != 0:  # left behind by a raw call that went round this wrapper: report it as what it is, not as this call's failure
                _lib.hip_take_last_error(_error_buffer, 2048)
                raise RuntimeError("an earlier call into the library failed and its error was never collected: %s"
                                   % _error_buffer.value.decode("utf-8", "replace"))
            result = raw(*args)
            if flag.value != 0:
                check_error()
            return result

        _checked[name] = wrapped
    return wrapped
