"""No-GPU checks of the boundary and of the host logic: the shared library loads and exports every declared symbol and every symbol of
the reference's device ABI; error behaviour of the C-ABI (C++ exceptions, checked before any device call); Conv2D's algorithm choice and
workspace contract; argument validation of the Python mirror."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from minml_amd import backend as B
from minml_amd import core as ml
from minml_amd.conv2d import EXPLICIT_GEMM, IMPLICIT_GEMM, WINOGRAD_NON_FUSED, Conv2D, get_matrices_shape, get_weight_matrices_shape
from minml_amd.resnet import ResNet

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "minml_hip_backend.h")).read()
    return sorted(set(re.findall(r"\b(hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = B.load()
    names = declared_functions()
    assert len(names) >= 44
    for name in names:
        assert hasattr(lib, name), name
    # the ctypes prototypes cover the header, and nothing else
    assert sorted("hip_" + n for n in B.SIGNATURES) == names


def test_library_exports_the_reference_device_abi():
    """Every cuda_* / cudnn_* symbol of the reference's include/minml/backend/cuda_backend.h must link (tests/golden/cuda_backend_symbols.txt)."""
    lib = B.load()
    names = open(os.path.join(ROOT, "tests", "golden", "cuda_backend_symbols.txt")).read().split()
    assert len(names) == 113
    for name in names:
        assert hasattr(lib, name), name
    # the path's entry points are one function under two names
    for name in ("winograd_input_transform", "gemm_batched_v2", "gemm_ex", "convolution_implicit_gemm_forward", "quantized_scale_shift_act",
                 "malloc", "create_context"):
        a = ctypes.cast(getattr(lib, "hip_" + name), ctypes.c_void_p).value
        b = ctypes.cast(getattr(lib, "cuda_" + name), ctypes.c_void_p).value
        assert a == b, name


def test_descriptor_layout_matches_the_reference():
    """mlShape_t {int rank; int dim[6]}, mlTensor_t {void*; enum; int; int[6]} (include/minml/backend/backend_types.h:28-73)."""
    assert ctypes.sizeof(B.mlShape_t) == 28
    assert ctypes.sizeof(B.mlTensor_t) == 40
    assert B.mlTensor_t.dtype.offset == 8 and B.mlTensor_t.rank.offset == 12 and B.mlTensor_t.dim.offset == 16
    assert ctypes.sizeof(B.mlQuantizationData_t) == 8
    assert (B.DTYPE_FLOAT16, B.DTYPE_FLOAT32, B.DTYPE_INT8, B.DTYPE_INT32) == (2, 3, 6, 8)
    assert (B.ACTIVATION_LINEAR, B.ACTIVATION_RELU, B.ACTIVATION_EXP) == (0, 3, 5)


def test_cabi_error_behaviour(tmp_path):
    exe = str(tmp_path / "cabi_errors")
    libdir = os.path.join(ROOT, "minml_amd")
    subprocess.run(["g++", "-std=c++17", "-O1", "-o", exe, os.path.join(ROOT, "tests", "cabi_errors.cpp"), "-L" + libdir, "-lminml_hip",
                    "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"], check=True)
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode == 0, res.stdout
    assert "ALL OK" in res.stdout and "FAIL" not in res.stdout
    assert res.stdout.count("OK ") >= 15


def test_no_device_is_reported_not_hidden():
    if ml.number_of_devices() == 0:
        with pytest.raises(RuntimeError):
            ml.Context(0)


def test_conv2d_algorithm_choice_and_workspace_contract():
    """src/layers/Conv2D.cpp:141-191,450-530; sizes of benchmark configuration 2: 36 * 16384 * 256 elements per matrices tensor."""
    c3 = Conv2D(None, (1024, 15, 15, 256), 256, 3, "relu", True, "float16")
    assert c3.forward_algorithm == WINOGRAD_NON_FUSED and c3.winograd_tile_size == 4
    assert get_matrices_shape(3, 4, (1024, 15, 15, 256)) == (36, 16384, 256)
    assert get_weight_matrices_shape((256, 3, 3, 256), 4) == (36, 256, 256)
    assert c3.getWorkspaceSize() == 2 * 36 * 16384 * 256 + 1024
    stem = Conv2D(None, (1024, 15, 15, 32), 256, 3, "relu", True, "float16")
    assert stem.getWorkspaceSize() == 36 * 16384 * 32 + 36 * 16384 * 256 + 1024
    c1 = Conv2D(None, (1024, 15, 15, 256), 1, 1, "linear", True, "float16")
    assert c1.forward_algorithm == EXPLICIT_GEMM and c1.getWorkspaceSize() == 0
    c5 = Conv2D(None, (512, 19, 19, 64), 64, 5, "relu", True, "float16")
    assert c5.forward_algorithm == IMPLICIT_GEMM and c5.getWorkspaceSize() == 0
    c5e = Conv2D(None, (2, 19, 19, 64), 64, 5, "relu", True, "float16", algorithm=EXPLICIT_GEMM)
    assert c5e.getWorkspaceSize() == 2 * 19 * 19 * 25 * 64  # src/core/math.cpp:1588-1594
    q = Conv2D(None, (2, 15, 15, 64), 32, 3, "relu", True, "int8")
    q.dtype = B.DTYPE_INT8
    q.int8_mode = "reference"
    assert q.getWorkspaceSize() == 2 * 15 * 15 * 32 + (2 * 15 * 15 * 64 * 9 + 3) // 4  # Conv2D.cpp:143-153
    q.int8_mode = "fused"
    assert q.getWorkspaceSize() == 0
    # edge tiles: 19 = 4*4 + 3
    assert get_matrices_shape(3, 4, (2, 19, 19, 8)) == (36, 2 * 25, 8)


def test_winograd_tile_is_derived_from_the_matrices():
    """src/core/math.cpp:107-118."""
    assert ml.get_winograd_tile((8, 3, 3, 8), (36, 10, 8)) == 4
    assert ml.get_winograd_tile((8, 3, 3, 8), (49, 10, 8)) == 5
    assert ml.get_winograd_tile((8, 5, 5, 8), (36, 10, 8)) == 2
    with pytest.raises(ValueError):
        ml.get_winograd_tile((8, 3, 3, 8), (35, 10, 8))


class FakeTensor:
    """Shape / dtype carrier for validation tests that must not touch a device."""

    def __init__(self, shape, dtype):
        self.shape, self.dtype, self.ptr = tuple(shape), ml.dtype_of(dtype), 1

    rank = ml.Tensor.rank
    volume = ml.Tensor.volume
    lastDim = ml.Tensor.lastDim
    firstDim = ml.Tensor.firstDim
    isEmpty = ml.Tensor.isEmpty
    sizeInBytes = ml.Tensor.sizeInBytes


def test_python_mirror_validates_before_calling_the_library():
    ctx = None
    f16, f32 = "float16", "float32"
    with pytest.raises(RuntimeError, match="No suitable Winograd transform runtime"):
        ml.winogradInputTransform(ctx, (8, 3, 3, 8), FakeTensor((1, 5, 5, 8), f32), FakeTensor((49, 1, 8), f32))
    with pytest.raises(RuntimeError, match="No suitable Winograd transform runtime"):
        ml.winogradWeightTransform(ctx, FakeTensor((8, 5, 5, 8), f32), FakeTensor((36, 8, 8), f32))
    with pytest.raises(ValueError):
        ml.winogradInputTransform(ctx, (8, 3, 3, 8), FakeTensor((1, 5, 5, 8), f32), FakeTensor((36, 3, 8), f32))  # 4 tiles expected
    with pytest.raises(ValueError):
        ml.winogradOutputTransform(ctx, (8, 3, 3, 8), FakeTensor((36, 4, 8), f32), FakeTensor((1, 5, 5, 8), f32), FakeTensor((7,), f32), None, "relu")
    with pytest.raises(ValueError):
        ml.gemm(ctx, "n", "t", FakeTensor((4, 4), f32), FakeTensor((4, 5), f32), FakeTensor((4, 6), f32))
    with pytest.raises(ValueError):
        ml.gemm(ctx, "n", "t", FakeTensor((4, 4), f16), FakeTensor((4, 5), f32), FakeTensor((4, 5), f32))
    with pytest.raises(ValueError):
        ml.gemmBatched(ctx, "n", "t", FakeTensor((3, 4, 4), f32), FakeTensor((2, 4, 5), f32), FakeTensor((3, 4, 5), f32))
    with pytest.raises(ValueError):
        ml.convolutionImplicitGemmForward(ctx, FakeTensor((1, 5, 5, 8), f16), FakeTensor((4, 3, 3, 16), f16), FakeTensor((1, 5, 5, 4), f16), None, None, "relu")
    with pytest.raises(ValueError, match="unsupported conversion"):
        ml.convertType(ctx, FakeTensor((4,), "int32"), FakeTensor((4,), f32))
    with pytest.raises(ValueError):
        ml.quantized_scale_shift_act(ctx, FakeTensor((4, 8), "int8"), (1.0, 0.0), FakeTensor((4, 8), f32), FakeTensor((8,), f32), FakeTensor((8,), f32), "relu")


def test_flop_count_of_the_benchmark_network():
    """40 * 7.73e10 + 9.66e9 + 1.18e8 = 3.10e12 executed flops per batch of 1024 (benchmark configuration 2)."""
    net = ResNet.__new__(ResNet)
    net.batch, net.board, net.channels, net.blocks = 1024, 15, 256, 20

    class L:
        def __init__(self, ws):
            self.weight_shape = ws

    net.layers = [L((256, 3, 3, 32))] + [L((256, 3, 3, 256))] * 40 + [L((1, 1, 1, 256))]
    assert abs(net.flops_per_forward() - (40 * 2 * 36 * 16384 * 256 * 256 + 2 * 36 * 16384 * 32 * 256 + 2 * 230400 * 256)) < 1
    assert abs(net.flops_per_forward() / 3.10e12 - 1) < 0.01


def test_host_side_quantisation_matches_the_oracle():
    """minml_amd/quantization.py (what the product uses to prepare an int8 layer) against the oracle's restatement of the reference's
    quantize / quantize_weights (src/layers/quantization.cpp:39-93), bit for bit, including halves (rounded away from zero) and clamping."""
    import oracle as O
    from minml_amd import quantization as Q

    rng = np.random.default_rng(17)
    x = np.concatenate([(rng.standard_normal(2000) * 60).astype(np.float32), np.array([0.5, -0.5, 1.5, 2.5, -2.5, 126.5, 127.5, -128.5, 1e9, -1e9], np.float32)])
    assert np.array_equal(Q.quantize(x), np.array([O.quantize(float(v)) for v in x], np.int32))
    for shape in ((44, 3, 3, 36), (64, 3, 3, 64), (7, 1, 1, 5)):
        w = (rng.standard_normal(shape) * 0.1).astype(np.float32)
        b = (rng.standard_normal(shape[0]) * 0.01).astype(np.float32)
        for transform in ((0.031, 0.0), (0.02, -1.3)):
            ours, theirs = Q.quantize_weights(w, b, transform), O.quantize_weights(w, b, transform)
            for got, want in zip(ours, theirs):
                assert np.array_equal(np.asarray(got).reshape(-1), np.asarray(want).reshape(-1))
    values = (rng.standard_normal(500) * 3).astype(np.float32)
    transform = Q.symmetric_transform(np.abs(values).max())
    q = Q.quantize_tensor(values, transform)
    assert q.dtype == np.int8 and np.abs(q.astype(np.int32)).max() == 127 and np.abs(q * np.float32(transform[0]) - values).max() <= transform[0] * 0.5001


def test_library_errors_surface_as_python_exceptions():
    """Exceptions cannot unwind through ctypes: the binding switches the library's error capture on, and a failed entry point raises
    ValueError (std::logic_error: a bad argument) or RuntimeError (std::runtime_error) in Python instead of ending the process. Only
    argument checks are exercised here: they run before the context or the device is touched."""
    from minml_amd import backend as B

    desc = B.make_tensor(1, B.DTYPE_FLOAT32, (1, 4, 4, 4))  # never dereferenced: both calls fail on their arguments
    with pytest.raises(RuntimeError, match="No suitable Winograd transform runtime"):
        B.fn("winograd_input_transform")(None, 3, desc, B.make_tensor(1, B.DTYPE_FLOAT32, (36, 1, 4)))
    with pytest.raises(ValueError, match="matrix op"):
        B.fn("gemm_v2")(None, b"x", b"n", 1.0, desc, desc, 0.0, desc)
    # entry points written in terms of others (gemm_v2 above; scale_tensor -> add_tensors here): the inner failure unwinds to the outermost
    # call and is reported once, as that call's failure
    with pytest.raises(ValueError, match="add_tensors: unsupported data type"):
        B.fn("scale_tensor")(None, 2.0, B.make_tensor(1, B.DTYPE_INT32, (8,)))
    # the failure was taken: the next call starts clean, and one that succeeds raises nothing
    assert B.fn("take_last_error")(None, 0) == 0
    assert B.fn("get_number_of_devices")() >= 0
    # with capture off the library throws as the reference's backends do (tests/cabi_errors.cpp covers that side from C++)
