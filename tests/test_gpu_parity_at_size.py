"""Parity at the benchmark configurations' own sizes, on samples large enough to mean something.

The tolerance statements ("fp32 within 1e-4, fp16 within 1e-2 max-abs relative error per layer and at the network head") are maxima over
a tensor, so they grow with the number of positions looked at. These tests run every configuration at its full batch on the device and
compare EVERY 3x3 layer's output and the head — of the whole batch for the residual networks in fp16 and fp32, of a spread sample of
positions (the first, the last and a stride between) for the int8 and the hybrid networks — with the CPU execution of the same positions: the reference's own CPU backend compiled into oracle/_ref where that library is present (one thread,
as the reference runs), this repository's C restatement on 16 threads otherwise (the two are bit-identical, tests/test_oracle_vs_reference.py).
The worst error per configuration is printed so that the margin to the tolerance is on record.
"""
import numpy as np
import pytest

import oracle as O
from oracle.cpu_net import CpuHybridNet, CpuResNet
from minml_amd import core as ml
from minml_amd.hybridnet import HybridNet, get_capacity, make_hybrid_parameters
from minml_amd.resnet import ResNet, make_input, make_parameters
from util import TOL, max_abs_rel, mismatches

pytestmark = pytest.mark.gpu


def cpu_engine():
    if O.reference() is not None:
        return "reference"
    O.set_num_threads(16)
    return "oracle"


def spread(batch, count):
    """`count` positions at a constant stride from the first one, plus the last one."""
    step = max(1, batch // count)
    return np.unique(np.concatenate([np.arange(0, batch, step), [batch - 1]]))


def residual_network_at_size(ctx, name, batch, channels, blocks, dtype, seed, sample):
    conv = O.to_half if dtype == "float16" else (lambda a: np.ascontiguousarray(a, np.float32))
    params = make_parameters(seed, 32, channels, blocks)
    x = conv(make_input(seed, batch, 15, 32))
    net = ResNet(ctx, batch, 15, 32, channels, blocks, dtype, params, conv)
    seen = {}
    net.observer = lambda index, tensor: seen.__setitem__(index, tensor.copyToHost(ctx)[sample])
    net.setInput(x)
    head_all = net.forward(fused=False).copyToHost(ctx)
    net.observer = None
    engine = cpu_engine()
    want_layers = []
    want_head = CpuResNet([(conv(w), conv(b)) for (w, b) in params], blocks, engine).forward(x[sample], per_layer=want_layers)
    assert len(want_layers) == 1 + 2 * blocks == len(seen)
    errors = [max_abs_rel(seen[i], want_layers[i]) for i in range(len(want_layers))]
    head_error = max_abs_rel(head_all[sample], want_head)
    print("%s, batch %d, %s, %d positions (%d ... %d) against the CPU engine '%s': max-abs relative error per 3x3 layer: first %.2e, worst %.2e "
          "(layer %d), last %.2e; head %.2e; tolerance %.0e" % (name, batch, dtype, len(sample), sample[0], sample[-1], engine, errors[0], max(errors),
                                                             int(np.argmax(errors)), errors[-1], head_error, TOL[dtype]), flush=True)
    # the benchmark's pass (transforms fused across layers) computes the same bits as the layer-by-layer pass just checked
    assert mismatches(net.forward(fused=True).copyToHost(ctx), head_all) == 0
    assert max(errors) <= TOL[dtype], "layer %d: %.3e" % (int(np.argmax(errors)), max(errors))
    assert head_error <= TOL[dtype]


def test_config2_every_layer_of_all_1024_positions(ctx):
    """Config 2 as benchmarked (20 blocks x 256 channels, fp16 storage, fp32 accumulation, B = 1024, seed 1): all 41 3x3 layers and the
    head of every position of the batch (about 17 s of the reference's CPU backend on one core)."""
    residual_network_at_size(ctx, "config 2", 1024, 256, 20, "float16", 1, np.arange(1024))


def test_config1_every_layer_of_all_256_positions(ctx):
    """Config 1 (10 blocks x 128 channels, fp32, B = 256, seed 0): all 21 3x3 layers and the head of every position."""
    residual_network_at_size(ctx, "config 1", 256, 128, 10, "float32", 0, np.arange(256))


SEED5, BOARD, PLANES, CHANNELS, BLOCKS5, ATTENTION_BLOCKS, HEADS = 4, 15, 32, 256, 10, 4, 8


def storage_params5(params, moe):
    conv = O.to_half
    ps = {"trunk": [(conv(w), conv(b)) for (w, b) in params["trunk"]],
          "attention": [{k: conv(v) for k, v in blk.items()} for blk in params["attention"]],
          "head": (conv(params["head"][0]), conv(params["head"][1]))}
    if moe:
        ps["ffn"] = [{k: conv(v) for k, v in blk.items()} for blk in params["ffn"]]
    return ps


@pytest.mark.parametrize("moe", [False, True])
def test_config5_33_positions_at_batch_256(ctx, moe):
    """Config 5 at B = 256 in both forms (attention half-blocks only: every layer has a CPU implementation in the reference; and with
    the mixture-of-experts halves): the trunk's result, every half-block's result and the head of positions 0, 8, ..., 248 and 255. With
    experts the CPU pass follows the device's routing tables (two summation orders may rank two nearly equal scores differently; the
    tables themselves are held to the CPU statement on identical scores in tests/test_gpu_config5.py and tests/test_gpu_moe.py)."""
    O.set_num_threads(16)
    batch = 256
    sample = spread(batch, 32)
    params = make_hybrid_parameters(SEED5, PLANES, CHANNELS, BLOCKS5, ATTENTION_BLOCKS, HEADS, BOARD)
    x = O.to_half(make_input(SEED5, batch, BOARD, PLANES))
    net = HybridNet(ctx, batch, BOARD, PLANES, CHANNELS, BLOCKS5, HEADS, "float16", params, O.to_half, moe=moe)
    watched = ("trunk", "block", "ffn", "table")
    seen = {}

    def observer(name, tensor):
        if name.startswith(watched) and not name.startswith("ffn_"):
            seen[name] = tensor.copyToHost(ctx)[sample]

    net.observer = observer
    net.setInput(x)
    head = net.forward().copyToHost(ctx)
    cpu = CpuHybridNet(storage_params5(params, moe), BLOCKS5, HEADS)
    want = {}
    if moe:
        want_head = cpu.forward(x[sample], want, moe_capacity=get_capacity(2.0, BOARD * BOARD, 8),
                                tables=[seen["table%d" % i] for i in range(ATTENTION_BLOCKS)])
    else:
        want_head = cpu.forward(x[sample], want)
    worst = {name: max_abs_rel(seen[name], want[name]) for name in seen if not name.startswith("table")}
    assert "trunk" in worst and "block3" in worst and (("ffn3" in worst) == moe)
    worst["head"] = max_abs_rel(head[sample], want_head)
    print("config 5 %s, batch 256, %d positions (%d ... %d): max-abs relative error: %s; tolerance 1e-02"
          % ("with experts" if moe else "attention halves only", len(sample), sample[0], sample[-1], {k: "%.2e" % v for k, v in sorted(worst.items())}),
          flush=True)
    assert max(worst.values()) <= 1e-2, worst


def test_config3_every_layer_of_33_positions_at_batch_1024_bit_exact(ctx):
    """Config 3 as benchmarked (the int8 form of config 2, activation ranges calibrated on 64 batches, B = 1024): the int8 output of all
    41 3x3 layers and the fp32 head of positions 0, 32, ..., 992 and 1023, bit for bit against the oracle's restatement of the
    reference's integer branch (src/layers/Conv2D.cpp:240-308; itself held to vectors recorded from the reference's own layer,
    tests/test_oracle_int8_reference.py)."""
    from minml_amd import quantization as Q
    from minml_amd.resnet import QuantizedResNet, calibrate_activations
    from oracle.cpu_net import CpuQuantizedResNet

    O.set_num_threads(16)
    board, planes, channels, blocks, batch = 15, 32, 256, 20, 1024
    sample = spread(batch, 32)
    params = make_parameters(1, planes, channels, blocks)
    ranges = calibrate_activations(ctx, params, board, planes, channels, blocks, batches=64, batch_size=4, seed=1)
    x = make_input(1, batch, board, planes)
    net = QuantizedResNet(ctx, batch, board, planes, channels, blocks, params, ranges)
    seen = {}
    net.observer = lambda index, tensor: seen.__setitem__(index, tensor.copyToHost(ctx)[sample])
    net.setInput(x)
    head = net.forward().copyToHost(ctx)
    want_layers = []
    want_head = CpuQuantizedResNet(net.host_parameters, blocks).forward(Q.quantize_tensor(x[sample], net.transforms[0]), want_layers)
    assert len(want_layers) == 1 + 2 * blocks == len(seen)
    wrong = [mismatches(seen[i], want_layers[i]) for i in range(len(want_layers))]
    print("config 3, batch 1024, int8, %d positions (%d ... %d): mismatching int8 outputs per 3x3 layer: %s; mismatching fp32 logits: %d"
          % (len(sample), sample[0], sample[-1], wrong, mismatches(head[sample], want_head)), flush=True)
    assert not any(wrong)
    assert np.array_equal(head[sample], want_head)
    assert max(int(np.abs(seen[i].astype(np.int32)).max()) for i in seen) > 20  # the calibrated ranges are in use
