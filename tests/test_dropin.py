"""The link-time swap of the device backend, performed for real: the reference's own dispatcher, layers and graph (compiled from the
reference's sources by oracle/Makefile, target `dropin`) linked against libminml_hip.so in place of src/backend/cuda_dummy_backend.cpp
(the reference swaps backends the same way: CMakeLists.txt:60-65; dispatcher: src/core/math.cpp, DeviceType::CUDA branches).

CPU part: the executable links with --no-undefined, defines no cuda_* symbol itself, takes them all from the HIP library and starts.
GPU part: it builds benchmark configuration 1 as a reference Graph (with the reference's FoldAdd pass), runs Graph::predict on
Device::cuda(0) — the HIP backend — and on Device::cpu(), in fp32 and after Graph::convertTo(FLOAT16), and compares the heads.
The executable is built where the reference checkout is mounted and travels to the GPU machine like the other built libraries."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "oracle", "_ref", "dropin_graph")
REFERENCE = "/root/reference"

needs_binary = pytest.mark.skipif(not os.path.exists(BINARY) and not os.path.isdir(os.path.join(REFERENCE, "src", "core")),
                                  reason="oracle/_ref/dropin_graph is not built and no reference checkout is mounted to build it from")


def _binary():
    if os.path.isdir(os.path.join(REFERENCE, "src", "core")) and os.path.exists(os.path.join(ROOT, "minml_amd", "libminml_hip.so")):
        subprocess.run(["make", "-s", "-j8", "-C", os.path.join(ROOT, "oracle"), "dropin", "REF=" + REFERENCE], check=True)
    assert os.path.exists(BINARY)
    return BINARY


def _symbols(path, flag):
    out = subprocess.run(["nm", "-D", flag, path], check=True, stdout=subprocess.PIPE, text=True).stdout
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


@needs_binary
def test_reference_dispatcher_links_against_the_hip_library():
    binary = _binary()
    undefined = {s for s in _symbols(binary, "--undefined-only") if s.startswith(("cuda_", "cudnn_"))}
    defined = {s for s in _symbols(binary, "--defined-only") if s.startswith(("cuda_", "cudnn_"))}
    assert not defined, "a dummy device backend was linked in: %s" % sorted(defined)[:5]
    assert len(undefined) >= 90  # every device entry point the dispatcher names
    exported = _symbols(os.path.join(ROOT, "minml_amd", "libminml_hip.so"), "--defined-only")
    assert undefined <= exported, "not provided by the HIP library: %s" % sorted(undefined - exported)
    # the hot-path entry points are among them, so Graph::predict on Device::cuda() reaches this library
    for name in ("cuda_winograd_input_transform", "cuda_winograd_output_transform", "cuda_winograd_weight_transform", "cuda_gemm_batched_v2",
                 "cuda_gemm_ex", "cuda_create_context", "cuda_malloc", "cuda_memcpy_from_host"):
        assert name in undefined, name
    run = subprocess.run([binary, "link"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert run.returncode == 0, run.stdout
    assert "linked" in run.stdout


@pytest.mark.gpu
@pytest.mark.skipif(not os.path.exists(BINARY), reason="oracle/_ref/dropin_graph is not built")
def test_reference_graph_predicts_on_the_hip_backend():
    """Configuration 1's topology (10 blocks x 128 channels, 15x15, 32 input planes) at batch 16 through the reference's Graph."""
    run = subprocess.run([BINARY, "run", "16", "128", "10"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    print(run.stdout, flush=True)
    assert run.returncode == 0, run.stdout
    assert "dropin ok" in run.stdout
