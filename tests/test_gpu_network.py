"""Whole-network parity and runtime behaviour on the GPU.

The network is the synthetic residual net of the benchmark configurations run layer by layer through the C-ABI (minml_amd.resnet),
checked against the CPU execution of the same call sequence (oracle/cpu_net.py) "per layer and at the network head": fp32 within 1e-4,
fp16 within 1e-2 max-abs relative error."""
import time

import numpy as np
import pytest

import oracle as O
from oracle.cpu_net import CpuResNet
from minml_amd import backend as B
from minml_amd import core as ml
from minml_amd.resnet import ResNet, make_input, make_parameters
from util import TOL, max_abs_rel, mismatches

pytestmark = pytest.mark.gpu


def run_both(ctx, batch, channels, blocks, dtype, seed, chunk=None):
    conv = O.to_half if dtype == "float16" else (lambda a: np.ascontiguousarray(a, np.float32))
    params = make_parameters(seed, 32, channels, blocks)
    x = make_input(seed, batch, 15, 32)
    net = ResNet(ctx, batch, 15, 32, channels, blocks, dtype, params, conv, chunk=chunk)
    net.setInput(conv(x))
    head = net.forward().copyToHost(ctx)
    trunk = net.trunk_output().copyToHost(ctx)
    cpu = CpuResNet([(conv(w), conv(b)) for (w, b) in params], blocks, "oracle")
    want_head, want_trunk = cpu.forward(conv(x), return_trunk=True)
    return head, trunk, want_head, want_trunk


def test_config1_topology_fp32(ctx):
    """Config 1's topology (stem 32 -> 128, 10 residual blocks x 128, 1x1 policy head, fp32, seed 0) at a batch the oracle finishes."""
    O.set_num_threads(8)
    head, trunk, want_head, want_trunk = run_both(ctx, 4, 128, 10, "float32", 0)
    assert max_abs_rel(trunk, want_trunk) <= 1e-4
    assert max_abs_rel(head, want_head) <= 1e-4


def test_config2_topology_fp16(ctx):
    """Config 2's topology (20 blocks x 256 channels, fp16 storage, fp32 accumulation, seed 1) at batch 2."""
    O.set_num_threads(8)
    head, trunk, want_head, want_trunk = run_both(ctx, 2, 256, 20, "float16", 1)
    assert max_abs_rel(trunk, want_trunk) <= 1e-2
    assert max_abs_rel(head, want_head) <= 1e-2


@pytest.mark.parametrize("config", [("config 1", 4, 128, 10, "float32", 0), ("config 2", 2, 256, 20, "float16", 1)])
def test_error_per_layer_along_the_network(ctx, config):
    """The benchmark networks at a batch the oracle finishes: the output of EVERY 3x3 layer (errors accumulated along the network, as a
    user sees them) and the head against the CPU execution, and the figures printed so that the margin to the tolerance is on record."""
    name, batch, channels, blocks, dtype, seed = config
    O.set_num_threads(8)
    conv = O.to_half if dtype == "float16" else (lambda a: np.ascontiguousarray(a, np.float32))
    params = make_parameters(seed, 32, channels, blocks)
    x = conv(make_input(seed, batch, 15, 32))
    net = ResNet(ctx, batch, 15, 32, channels, blocks, dtype, params, conv)
    seen = {}
    net.observer = lambda index, tensor: seen.__setitem__(index, tensor.copyToHost(ctx))
    net.setInput(x)
    head = net.forward(fused=False).copyToHost(ctx)
    want_layers = []
    want_head = CpuResNet([(conv(w), conv(b)) for (w, b) in params], blocks, "oracle").forward(x, per_layer=want_layers)
    errors = [max_abs_rel(seen[i], want_layers[i]) for i in range(len(want_layers))]
    head_error = max_abs_rel(head, want_head)
    print("%s topology, batch %d, %s: max-abs relative error per 3x3 layer: first %.2e, worst %.2e (layer %d), last %.2e; head %.2e; tolerance %.0e"
          % (name, batch, dtype, errors[0], max(errors), int(np.argmax(errors)), errors[-1], head_error, TOL[dtype]), flush=True)
    assert len(errors) == 1 + 2 * blocks
    assert max(errors) <= TOL[dtype] and head_error <= TOL[dtype]
    # the fused pass (output transform + next input transform in one launch) is bit-identical to the layer-by-layer pass
    assert mismatches(net.forward(fused=True).copyToHost(ctx), head) == 0


def test_per_layer_fp16(ctx):
    """Every layer of a 3-block fp16 network against the oracle run on the GPU's own input of that layer (no error accumulation)."""
    rng = np.random.default_rng(2)
    params = make_parameters(2, 32, 64, 3)
    x = O.to_half(make_input(2, 3, 15, 32))
    from minml_amd.conv2d import Conv2D

    cur = x
    residual = None
    for idx, (w, b) in enumerate(params[:-1]):
        wq, bq = O.to_half(w), O.to_half(b)
        layer = Conv2D(ctx, cur.shape, w.shape[0], 3, "relu", True, "float16")
        layer.setWeights(wq, bq)
        ws = ml.Tensor((layer.getWorkspaceSize(),), "float16")
        out = ml.Tensor(cur.shape[:3] + (w.shape[0],), "float16")
        use_res = idx > 0 and idx % 2 == 0
        inputs = [ml.toDevice(ctx, cur)] + ([ml.toDevice(ctx, residual)] if use_res else [])
        layer.forward(inputs, out, ws)
        got = out.copyToHost(ctx)
        v = O.winograd_input_transform(cur)
        m = O.gemm(v, O.winograd_weight_transform(wq))
        want = O.winograd_output_transform(m, out.shape, bq, residual if use_res else None, O.RELU)
        assert max_abs_rel(got, want) <= 1e-2
        if idx % 2 == 0:
            residual = got
        cur = got


def test_chunked_execution_is_bit_identical(ctx):
    """Splitting the batch into cache-resident sub-batches must not change a single bit (positions are independent)."""
    params = make_parameters(5, 32, 64, 2)
    x = O.to_half(make_input(5, 12, 15, 32))
    outs = []
    for chunk in (12, 4, 5):
        net = ResNet(ctx, 12, 15, 32, 64, 2, "float16", params, O.to_half, chunk=chunk)
        net.setInput(x)
        outs.append(net.forward().copyToHost(ctx))
    assert mismatches(outs[0], outs[1]) == 0
    assert mismatches(outs[0], outs[2]) == 0


@pytest.mark.parametrize("dtype,channels,blocks", [("float16", 64, 3), ("float32", 128, 2), ("float16", 40, 2)])
def test_cross_layer_fusion_is_bit_identical(ctx, dtype, channels, blocks):
    """Merging each output transform with the next layer's input transform (activations stay in LDS between them) must not change a
    single bit of the head output or of the last block's output; 40 channels exercise the entry point's two-kernel route."""
    conv = O.to_half if dtype == "float16" else (lambda a: np.ascontiguousarray(a, np.float32))
    params = make_parameters(9, 32, channels, blocks)
    x = conv(make_input(9, 6, 15, 32))
    net = ResNet(ctx, 6, 15, 32, channels, blocks, dtype, params, conv)
    net.setInput(x)
    plain = net.forward(fused=False).copyToHost(ctx)
    trunk_plain = net.trunk_output().copyToHost(ctx)
    for across_blocks in (False, True):  # fusion inside the residual blocks only, then also across their boundaries
        net.fuse_block_boundary = across_blocks
        fused = net.forward(fused=True).copyToHost(ctx)
        trunk_fused = net.trunk_output().copyToHost(ctx)
        assert mismatches(plain, fused) == 0
        assert mismatches(trunk_plain, trunk_fused) == 0


def test_full_size_batch_1024_properties(ctx):
    """The benchmark workload itself (config 2: B = 1024): repeated passes are bit-identical (no races, no stale workspace), and the
    first positions reproduce a batch-4 run of the same network bit for bit, which in turn is checked against the oracle."""
    params = make_parameters(1, 32, 256, 20)
    x = O.to_half(make_input(1, 1024, 15, 32))
    net = ResNet(ctx, 1024, 15, 32, 256, 20, "float16", params, O.to_half)
    net.setInput(x)
    a = net.forward().copyToHost(ctx)
    b = net.forward().copyToHost(ctx)
    assert mismatches(a, b) == 0
    assert mismatches(a, net.forward(fused=True).copyToHost(ctx)) == 0  # the benchmark's fused pass computes the same bits
    net.fuse_block_boundary = True
    assert mismatches(a, net.forward(fused=True).copyToHost(ctx)) == 0  # and so does fusion across the blocks' boundaries
    net.fuse_layers = True  # whole layers as single launches (product kept in the L2 cache): the same bits again
    assert mismatches(a, net.forward(fused=True).copyToHost(ctx)) == 0
    assert ml.winogradLayerErrors(ctx) == 0
    net.fuse_layers = False
    small = ResNet(ctx, 4, 15, 32, 256, 20, "float16", params, O.to_half)
    small.setInput(x[:4])
    c = small.forward().copyToHost(ctx)
    assert mismatches(a[:4], c) == 0
    assert np.isfinite(O.from_half(a)).all()
    O.set_num_threads(8)
    cpu = CpuResNet([(O.to_half(w), O.to_half(bb)) for (w, bb) in params], 20, "oracle")
    assert max_abs_rel(c[:1], cpu.forward(x[:1])) <= 1e-2


# ---- runtime: context, events, memory ---------------------------------------------------------------------------------------------
def test_device_identity():
    assert ml.number_of_devices() >= 1
    info = B.fn("get_device_info")(0).decode()
    assert "gfx950" in info
    assert B.fn("get_memory")(0) > 100000  # MB
    for dtype, ok in ((B.DTYPE_FLOAT16, True), (B.DTYPE_FLOAT32, True), (B.DTYPE_INT8, True), (B.DTYPE_INT32, True), (B.DTYPE_FLOAT64, False)):
        assert bool(B.fn("supports_type")(0, dtype)) == ok
    assert B.fn("get_device_features")(0)


def test_memory_calls(ctx):
    t = ml.Tensor((1000,), "float32")
    t.setall(ctx, 1.5)
    assert np.array_equal(t.copyToHost(ctx), np.full(1000, 1.5, np.float32))
    t.zeroall(ctx)
    assert not t.copyToHost(ctx).any()
    h = ml.Tensor((7,), "float16")
    h.setall(None, 2.0)  # context-less calls are synchronous
    assert np.array_equal(h.copyToHost(), np.full(7, 0x4000, np.uint16))
    src = ml.toDevice(ctx, np.arange(100, dtype=np.int32))
    dst = ml.Tensor((100,), "int32")
    dst.zeroall(ctx)
    B.fn("memcpy_within_device")(ctx.handle, dst.ptr, 40, src.ptr, 80, 120)  # 30 ints from src[20:] to dst[10:]
    got = dst.copyToHost(ctx)
    assert np.array_equal(got[10:40], np.arange(20, 50)) and not got[:10].any() and not got[40:].any()
    view = src.view((10,), 90)
    assert np.array_equal(view.copyToHost(ctx), np.arange(90, 100))
    with pytest.raises(ValueError):
        src.view((20,), 90)


def test_events_and_context(ctx):
    x = ml.Tensor((1 << 24,), "float32")
    start = ml.Event(ctx)
    for _ in range(10):
        x.setall(ctx, 1.0)
    end = ml.Event(ctx)
    end.synchronize()
    assert start.isReady() and end.isReady()
    dt = ml.Event.getElapsedTime(start, end)
    assert 0.0 < dt < 1.0
    ctx.synchronize()
    assert ctx.isReady()
    other = ml.Context(0)  # a second context = a second stream on the same device
    y = ml.Tensor((16,), "int32")
    y.setall(other, 3)
    other.synchronize()
    assert np.array_equal(y.copyToHost(other), np.full(16, 3, np.int32))
    other.destroy()
    start.destroy()
    end.destroy()


@pytest.mark.parametrize("mode", [0, 1])
def test_network_driven_from_cpp_through_the_cabi(ctx, tmp_path, mode):
    """The same network driven by a C++ program that includes only include/minml_hip_backend.h and links the library (tests/cabi_network.cpp:
    descriptors by value from real C++, the reference's workspace layout, its call sequence per layer): the head output must equal the
    Python mirror's bit for bit, in the three-call form and with the fused transform inside the residual blocks."""
    import os
    import subprocess

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    libdir = os.path.join(root, "minml_amd")
    exe = str(tmp_path / "cabi_network")
    subprocess.run(["g++", "-std=c++17", "-O2", "-o", exe, os.path.join(root, "tests", "cabi_network.cpp"), "-L" + libdir, "-lminml_hip",
                    "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"], check=True)
    batch, board, planes, channels, blocks = 6, 15, 32, 64, 3
    params = make_parameters(12, planes, channels, blocks)
    x = O.to_half(make_input(12, batch, board, planes))
    with open(tmp_path / "parameters.bin", "wb") as f:
        for w, b in params:
            f.write(O.to_half(w).tobytes())
            f.write(O.to_half(b).tobytes())
    x.tofile(tmp_path / "input.bin")
    res = subprocess.run([exe, str(tmp_path / "parameters.bin"), str(tmp_path / "input.bin"), str(tmp_path / "output.bin"), str(batch), str(board),
                          str(planes), str(channels), str(blocks), str(mode), "3"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode == 0 and "ALL OK" in res.stdout, res.stdout
    got = np.fromfile(tmp_path / "output.bin", dtype=np.uint16).reshape(batch, board, board, 1)
    net = ResNet(ctx, batch, board, planes, channels, blocks, "float16", params, O.to_half)
    net.setInput(x)
    want = net.forward(fused=bool(mode)).copyToHost(ctx)
    assert mismatches(got, want) == 0


def test_recorded_pass_replays_bit_identically(ctx):
    """A forward pass recorded as a HIP graph (hip_graph_begin_capture / end_capture / launch): every replay must equal the eager pass
    bit for bit, also after other work and synchronisations on the same context between replays, and after the input changed in place."""
    params = make_parameters(9, 32, 64, 3)
    conv = O.to_half
    net = ResNet(ctx, 8, 15, 32, 64, 3, "float16", params, conv, fused=True)
    x1, x2 = conv(make_input(9, 8, 15, 32)), conv(make_input(10, 8, 15, 32))
    net.setInput(x1)
    want1 = net.forward().copyToHost(ctx)  # the ordinary pass also does the first-use work (weight transforms) outside the recording
    graph = ml.Graph.record(ctx, lambda: net.forward())
    for replay in range(3):
        net.output.zeroall(ctx)
        graph.launch()
        assert mismatches(net.output.copyToHost(ctx), want1) == 0
        # unrelated eager work and a synchronisation between replays
        scratch = ml.Tensor((1024,), "float32")
        scratch.zeroall(ctx)
        ctx.synchronize()
        scratch.free()
    net.setInput(x2)
    want2 = net.forward().copyToHost(ctx)
    assert mismatches(want2, want1) > 0
    net.output.zeroall(ctx)
    graph.launch()  # same buffers, new contents
    assert mismatches(net.output.copyToHost(ctx), want2) == 0
    graph.destroy()
