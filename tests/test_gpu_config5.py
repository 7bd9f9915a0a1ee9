"""Benchmark configuration 5 on the GPU, the part of it that has a CPU reference: residual trunk of 10 blocks x 256 channels on 15x15
boards (fp16 storage, fp32 accumulation, weights N(0, 0.02), seed 4), then four attention half-blocks (RMS normalisation, dense qkv,
multi-head attention with 8 heads of 32 and the 2-D relative-position table, dense output + residual), then the 1x1 policy head —
against the CPU execution of the same layers (oracle/cpu_net.py:CpuHybridNet), fp16 within 1e-2 max-abs relative error per layer and at
the head. The feed-forward (mixture-of-experts) halves of the transformer blocks have no CPU implementation in the reference
(src/core/math.cpp:1328-1491) and are not part of this network."""
import numpy as np
import pytest

import oracle as O
from oracle.cpu_net import CpuHybridNet
from minml_amd import core as ml
from minml_amd.hybridnet import HybridNet, make_hybrid_parameters
from minml_amd.resnet import make_input
from util import max_abs_rel, mismatches

pytestmark = pytest.mark.gpu

SEED, BOARD, PLANES, CHANNELS, BLOCKS, ATTENTION_BLOCKS, HEADS = 4, 15, 32, 256, 10, 4, 8


def storage_params(params):
    conv = O.to_half
    return {"trunk": [(conv(w), conv(b)) for (w, b) in params["trunk"]],
            "attention": [{k: conv(v) for k, v in blk.items()} for blk in params["attention"]],
            "head": (conv(params["head"][0]), conv(params["head"][1]))}


def test_config5_per_layer_small_batch(ctx):
    """Batch 2: every intermediate tensor of the attention half-blocks, the trunk's result and the head against the CPU execution; and
    each attention-block layer once more against the oracle applied to the GPU's own input of that layer (no accumulated error)."""
    O.set_num_threads(8)
    params = make_hybrid_parameters(SEED, PLANES, CHANNELS, BLOCKS, ATTENTION_BLOCKS, HEADS, BOARD)
    x = O.to_half(make_input(SEED, 2, BOARD, PLANES))
    net = HybridNet(ctx, 2, BOARD, PLANES, CHANNELS, BLOCKS, HEADS, "float16", params, O.to_half)
    seen = {}
    net.observer = lambda name, tensor: seen.__setitem__(name, tensor.copyToHost(ctx))
    net.setInput(x)
    head = net.forward().copyToHost(ctx)
    ps = storage_params(params)
    cpu = CpuHybridNet(ps, BLOCKS, HEADS)
    want = {}
    want_head = cpu.forward(x, want)
    worst = {}
    for name, tensor in want.items():
        worst[name] = max_abs_rel(seen[name], tensor)
    worst["head"] = max_abs_rel(head, want_head)
    print("config 5, batch 2, max-abs relative error per layer:", {k: "%.2e" % v for k, v in worst.items()}, flush=True)
    assert max(worst.values()) <= 1e-2, worst
    # layer by layer on the GPU's own inputs
    rows = 2 * BOARD * BOARD
    for index, p in enumerate(ps["attention"]):
        x_in = seen["trunk"] if index == 0 else seen["block%d" % (index - 1)]
        assert max_abs_rel(seen["rmsnorm%d" % index], O.rmsnorm_forward(x_in, p["gamma"])) <= 1e-2
        qkv = O.gemm(seen["rmsnorm%d" % index].reshape(rows, CHANNELS), p["w_qkv"], bias=p["b_qkv"], act=O.LINEAR)
        assert max_abs_rel(seen["qkv%d" % index].reshape(rows, -1), qkv) <= 1e-2
        att = O.multi_head_attention_forward(seen["qkv%d" % index], HEADS, p["table"], False)
        assert max_abs_rel(seen["attention%d" % index], att) <= 1e-2
        out = O.gemm(seen["attention%d" % index].reshape(rows, CHANNELS), p["w_out"], beta=1.0, C=x_in.reshape(rows, CHANNELS), bias=p["b_out"],
                     act=O.LINEAR)
        assert max_abs_rel(seen["block%d" % index].reshape(rows, -1), out) <= 1e-2


def test_config5_full_size(ctx):
    """Batch 256 (the configuration's size): the head of a sample of positions against the CPU execution, repeatability bit for bit, and
    batch independence (a 4-position network reproduces those positions' logits within the tolerance; bitwise equality is not required
    because the dense layers pick their tiling by the number of rows)."""
    O.set_num_threads(8)
    batch = 256
    params = make_hybrid_parameters(SEED, PLANES, CHANNELS, BLOCKS, ATTENTION_BLOCKS, HEADS, BOARD)
    x = O.to_half(make_input(SEED, batch, BOARD, PLANES))
    net = HybridNet(ctx, batch, BOARD, PLANES, CHANNELS, BLOCKS, HEADS, "float16", params, O.to_half)
    net.setInput(x)
    head = net.forward().copyToHost(ctx)
    again = net.forward().copyToHost(ctx)
    assert mismatches(head, again) == 0
    assert np.isfinite(O.from_half(head)).all()
    sample = [0, 1, 254, 255]
    cpu = CpuHybridNet(storage_params(params), BLOCKS, HEADS)
    want = cpu.forward(x[sample])
    err = max_abs_rel(head[sample], want)
    print("config 5, batch 256: head of positions %s vs CPU: %.2e" % (sample, err), flush=True)
    assert err <= 1e-2
    small = HybridNet(ctx, 4, BOARD, PLANES, CHANNELS, BLOCKS, HEADS, "float16", params, O.to_half)
    small.setInput(x[sample])
    assert max_abs_rel(small.forward().copyToHost(ctx), head[sample]) <= 1e-2


# ---- the whole configuration: the mixture-of-experts halves included -------------------------------------------------------------

def test_config5_with_experts_per_layer_small_batch(ctx):
    """Batch 2 with the feed-forward halves (expert-choice routing with capacity factor 2 = 56 of 225 tokens per expert, 8 experts of
    hidden width 1024). Every mixture-of-experts layer is checked against the CPU statement (oracle/moe.py) applied to the device's own
    input of that layer, the routing table exactly; then the head against a CPU pass that follows the device's routing tables (two
    summation orders may order two nearly equal scores differently; the tables themselves were just checked on identical scores)."""
    from oracle import moe as M
    from minml_amd.hybridnet import get_capacity

    O.set_num_threads(8)
    params = make_hybrid_parameters(SEED, PLANES, CHANNELS, BLOCKS, ATTENTION_BLOCKS, HEADS, BOARD)
    x = O.to_half(make_input(SEED, 2, BOARD, PLANES))
    net = HybridNet(ctx, 2, BOARD, PLANES, CHANNELS, BLOCKS, HEADS, "float16", params, O.to_half, moe=True)
    seen = {}
    net.observer = lambda name, tensor: seen.__setitem__(name, tensor.copyToHost(ctx))
    net.setInput(x)
    head = net.forward().copyToHost(ctx)
    ps = storage_params(params)
    ps["ffn"] = [{k: O.to_half(v) for k, v in blk.items()} for blk in params["ffn"]]
    capacity = get_capacity(2.0, BOARD * BOARD, 8)
    assert capacity == 56 and net.capacity == 56
    rows = 2 * BOARD * BOARD
    worst = {}
    for index, p in enumerate(ps["ffn"]):
        x_in = seen["block%d" % index]
        worst["ffn_rmsnorm"] = max(worst.get("ffn_rmsnorm", 0.0), max_abs_rel(seen["ffn_rmsnorm%d" % index], O.rmsnorm_forward(x_in, p["gamma"])))
        normed = seen["ffn_rmsnorm%d" % index]
        scores = O.gemm(normed.reshape(rows, CHANNELS), p["w_router"], bias=p["b_router"], act=O.LINEAR)
        worst["scores"] = max(worst.get("scores", 0.0), max_abs_rel(seen["scores%d" % index].reshape(rows, -1), scores))
        table = seen["table%d" % index]
        want_table = M.expert_choice_routing(seen["scores%d" % index], capacity)
        assert np.array_equal(O.from_half(table)[:, 0], O.from_half(want_table)[:, 0])  # the same tokens in the same slots
        assert np.abs(O.from_half(table)[:, 1] - O.from_half(want_table)[:, 1]).max() <= 1e-3
        gathered = M.gather_tokens(normed, table)
        worst["hidden"] = max(worst.get("hidden", 0.0), max_abs_rel(seen["hidden%d" % index], M.moe_forward(gathered, p["w_1"], p["b_1"], O.RELU)))
        worst["experts"] = max(worst.get("experts", 0.0), max_abs_rel(seen["experts%d" % index], M.moe_forward(seen["hidden%d" % index], p["w_2"], p["b_2"], O.LINEAR)))
        want = M.scatter_tokens(seen["experts%d" % index], table, x_in.shape, beta=1.0, y=x_in)
        worst["ffn"] = max(worst.get("ffn", 0.0), max_abs_rel(seen["ffn%d" % index], want))
    cpu = CpuHybridNet(ps, BLOCKS, HEADS)
    want_head = cpu.forward(x, moe_capacity=capacity, tables=[seen["table%d" % i] for i in range(ATTENTION_BLOCKS)])
    worst["head"] = max_abs_rel(head, want_head)
    print("config 5 with experts, batch 2, max-abs relative error per layer type:", {k: "%.2e" % v for k, v in worst.items()}, flush=True)
    assert max(worst.values()) <= 1e-2, worst
    # every token that an expert selected moved: the feed-forward half is not a no-op
    assert max_abs_rel(seen["ffn0"], seen["block0"]) > 1e-3


def test_config5_with_experts_full_size(ctx):
    """Batch 256, the complete configuration: repeatable bit for bit, finite, and the head of a sample of positions within 1e-2 of a CPU
    pass over those positions that follows the device's routing tables."""
    from minml_amd.hybridnet import get_capacity

    O.set_num_threads(8)
    batch = 256
    params = make_hybrid_parameters(SEED, PLANES, CHANNELS, BLOCKS, ATTENTION_BLOCKS, HEADS, BOARD)
    x = O.to_half(make_input(SEED, batch, BOARD, PLANES))
    net = HybridNet(ctx, batch, BOARD, PLANES, CHANNELS, BLOCKS, HEADS, "float16", params, O.to_half, moe=True)
    tables = {}
    net.observer = lambda name, tensor: tables.__setitem__(name, tensor.copyToHost(ctx)) if name.startswith("table") else None
    net.setInput(x)
    head = net.forward().copyToHost(ctx)
    net.observer = None
    assert mismatches(net.forward().copyToHost(ctx), head) == 0
    assert np.isfinite(O.from_half(head)).all()
    sample = [0, 255]
    ps = storage_params(params)
    ps["ffn"] = [{k: O.to_half(v) for k, v in blk.items()} for blk in params["ffn"]]
    cpu = CpuHybridNet(ps, BLOCKS, HEADS)
    want = cpu.forward(x[sample], moe_capacity=get_capacity(2.0, BOARD * BOARD, 8), tables=[tables["table%d" % i][sample] for i in range(ATTENTION_BLOCKS)])
    err = max_abs_rel(head[sample], want)
    print("config 5 with experts, batch 256: head of positions %s vs CPU: %.2e" % (sample, err), flush=True)
    assert err <= 1e-2
