"""MI355X-native (gfx950, hand-written HIP) backend for minml's convolution / GEMM inference path.

  include/minml_hip_backend.h   the C-ABI (drop-in for the reference's cuda_* device backend entry points)
  minml_amd/csrc/               HIP kernels and the C-ABI implementation -> minml_amd/libminml_hip.so
  minml_amd/backend.py          ctypes binding of that library
  minml_amd/core.py             Context / Tensor / math functions named as in the reference's core
  minml_amd/conv2d.py           Conv2D layer mirror (algorithm choice, workspace contract, int8 path)
  minml_amd/resnet.py           the synthetic residual network of the benchmark configurations
"""
from . import backend  # noqa: F401
from . import core  # noqa: F401
from .conv2d import Conv2D  # noqa: F401
from .resnet import ResNet  # noqa: F401
