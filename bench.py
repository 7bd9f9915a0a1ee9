#!/usr/bin/env python3
"""Benchmark of the convolution / GEMM inference path on one MI355X.

A step is one forward pass of the synthetic 20-block x 256-channel 15x15 residual network (fp16 storage, fp32 accumulation) over one
batch of 1024 positions already resident in HBM: stem 3x3 conv 32->256, 40 3x3 convs 256->256 as Winograd F(4x4,3x3) (input transform,
36 batched GEMMs on MFMA, output transform with bias + residual + ReLU), 1x1 policy head. By default the output transform of each 3x3
layer and the input transform of the next run as one launch (bit-identical results; --unfused runs the reference's three calls per
layer). Prints ONE JSON line:

  value        positions / second over the timed steps (wall clock between two stream synchronisations)
               the better of two ways of issuing the same pass: the whole batch on one stream, or its two halves on two streams of the
               device (`config.execution` says which; `single_stream` and `two_streams` hold both); every per-kernel figure below comes from
               the single-stream pass, where launches do not overlap
  roofline     the dominant kernel, the 36-way batched Winograd GEMM of the 40 block convolutions. With N = K = 256 it has 127 flop per
               byte, below the chip's ridge of ~312 flop/byte, so HBM bounds it: `achieved` = algorithmic bytes of one launch
               (s * 36 * (T*K + N*K + T*N)) / average launch duration, against 8 TB/s. Durations come from HIP events recorded on the
               context's stream around every launch in a second, instrumented run of the same steps. `traffic` = HBM bytes of one
               launch from rocprofv3 counters (FETCH_SIZE + WRITE_SIZE, each scaled by what it reads for a copy kernel of known size);
               the figure and the commands that produced it are in profiles/.
  gemm_mfma    the same launches against the dense fp16 MFMA peak (executed flops 2 * 36 * T * K * N per launch)
  transforms   the transform launches of the block convolutions: algorithmic bytes / average duration against 8 TB/s
  cpu_baseline the same network on a bounded number of positions on the host's cores: the reference's own CPU backend compiled from
               its sources (kind "reference", one thread, as the reference runs) when that library is present, otherwise this
               repository's C restatement (kind "port")

  reference_call_sequence   the same batch through the reference's own call sequence (three calls per 3x3 layer: input transform, batched GEMM,
               output transform; src/layers/Conv2D.cpp:365-378) — what the timed `value` gains over it is the cross-layer transform fusion,
               an entry point that no unchanged minml caller uses
  dropin_graph_predict      the reference's own Graph / Conv2D / dispatcher code (compiled from its sources into oracle/_ref/dropin_graph and linked
               against this backend in place of its CUDA backend) timed the way its launcher times a network (launcher/minml.cpp:3924-3936:
               predict + synchronize in a loop): the throughput an unchanged minml gets. Run as a child process before this process touches the GPU.

--config cfg4_conv_sweep_fp16_b512 runs the implicit-GEMM convolution sweep (19x19 boards, batch 512, 64 / 128 / 256 / 384 channels, kernels
1 / 3 / 5, bias + residual + ReLU fused): a step is the 12 layers one after the other; `rows` prices each against its own roofline.

--config cfg3_resnet20x256_int8_b1024 runs the int8 form of the same network instead (per-channel int8 weights, per-tensor int8
activations calibrated on 64 random batches, every 3x3 layer one fused int8 implicit-GEMM convolution with int32 accumulation and
requantisation); its roofline object prices that convolution against the dense int8 MFMA peak (5 POP/s).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

PEAK_MFMA_TFLOPS = {"float16": 2500.0, "float32": 157.3}  # MI355X dense matrix peaks
PEAK_HBM_GBS = 8000.0

CONFIGS = {
    # name: (batch, board, input planes, channels, blocks, dtype, seed)
    "cfg2_resnet20x256_fp16_b1024": (1024, 15, 32, 256, 20, "float16", 1),
    "cfg1_resnet10x128_fp32_b256": (256, 15, 32, 128, 10, "float32", 0),
    # the int8 form of configuration 2: same parameters (seed 1), per-channel int8 weights, per-tensor int8 activations calibrated on 64 batches
    "cfg3_resnet20x256_int8_b1024": (1024, 15, 32, 256, 20, "int8", 1),
    # the part of configuration 5 that has a CPU reference: 10-block x 256 trunk, then 4 attention half-blocks (8 heads), N(0, 0.02) weights
    "cfg5_hybrid10x256_attention4_fp16_b256": (256, 15, 32, 256, 10, "hybrid", 4),
    # the whole of configuration 5: the same plus the feed-forward halves as mixtures of 8 experts (hidden 1024, expert-choice routing
    # with capacity factor 2 = two experts per token on average); that half has no CPU reference (checked against this repository's own CPU statement)
    "cfg5_hybrid10x256_attention4_moe8_fp16_b256": (256, 15, 32, 256, 10, "hybrid_moe", 4),
}
PEAK_INT8_TOPS = 5000.0
CONV_SWEEP = "cfg4_conv_sweep_fp16_b512"


def run_dropin_graph(batch, channels, blocks, dtype, seconds):
    """Spawns oracle/_ref/dropin_graph (the reference's Graph on this backend) in its timing mode and parses its launcher-style line.
    Must run before this process initialises the GPU. Returns the dropin_graph_predict object (value None with a reason when unavailable)."""
    import re
    import subprocess

    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle", "_ref", "dropin_graph")
    what = "Graph::predict + Context::synchronize of the reference's own graph code on Device::cuda(0) = this backend (three calls per 3x3 layer)"
    if not os.path.exists(exe):
        return {"value": None, "unit": "positions/sec", "what": what, "skipped": "oracle/_ref/dropin_graph is not built (make -C oracle dropin)"}
    cmd = [exe, "time", str(batch), str(channels), str(blocks), "fp16" if dtype == "float16" else "fp32", "%g" % seconds, "3"]
    try:
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60 + 4 * seconds)
    except subprocess.TimeoutExpired:
        return {"value": None, "unit": "positions/sec", "what": what, "skipped": "timed out"}
    m = re.search(r"time = ([0-9.]+)s, repeats = (\d+), n/s = ([0-9.]+), ms per predict = ([0-9.]+)", res.stdout)
    if res.returncode != 0 or m is None:
        return {"value": None, "unit": "positions/sec", "what": what, "skipped": "exit code %d: %s" % (res.returncode, res.stdout[-300:])}
    return {"value": float(m.group(3)), "unit": "positions/sec", "ms_per_step": float(m.group(4)), "repeats": int(m.group(2)),
            "seconds": float(m.group(1)), "what": what}


def timed_passes(ctx, forward, steps, warmup):
    """Seconds per pass: `warmup` untimed passes, then `steps` passes between two synchronisations of the context's stream."""
    for _ in range(warmup):
        forward()
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        forward()
    ctx.synchronize()
    return (time.perf_counter() - t0) / steps

def measured_gemm_traffic_bytes(config):
    """HBM bytes of one launch of the block-convolution GEMM kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs, each counter
    scaled by its reading for a 256 MiB copy kernel in the same run), as recorded in profiles/hbm_traffic_<config>.md together with the
    hash of the kernel's source file. None when there is no such record or the kernel has changed since it was measured."""
    import hashlib
    import re

    root = os.path.dirname(os.path.abspath(__file__))
    try:
        text = open(os.path.join(root, "profiles", "hbm_traffic_%s.md" % config)).read()
        m = re.search(r"kernel_gemm_stream_wide_nt traffic_bytes=(\d+) source=(\S+) sha256=([0-9a-f]{64})", text)
        if m is None:
            return None
        current = hashlib.sha256(open(os.path.join(root, m.group(2)), "rb").read()).hexdigest()
        return float(m.group(1)) if current == m.group(3) else None
    except OSError:
        return None



def to_storage_factory(dtype):
    if dtype == "float16":
        # input preparation on the host: IEEE round-to-nearest narrowing of the synthetic fp32 parameters; both sides get these bits
        return lambda a: np.ascontiguousarray(a, np.float32).astype(np.float16).view(np.uint16)
    return lambda a: np.ascontiguousarray(a, np.float32)


def run_cpu_baseline(params_storage, x_storage, blocks, budget_seconds):
    """Times the CPU engine on as many positions as fit the budget (at least 4); returns the cpu_baseline object."""
    import oracle as O
    from oracle.cpu_net import CpuResNet

    if O.reference() is not None:
        kind, engine, cores = "reference", "reference", 1
    else:
        kind, engine, cores = "port", "oracle", min(16, os.cpu_count() or 1)
        O.set_num_threads(cores)
    net = CpuResNet(params_storage, blocks, engine)
    positions = 4
    t = net.timed_forward(x_storage[:positions])
    per_position = t / positions
    target = int(max(4, min(x_storage.shape[0], budget_seconds / max(per_position, 1e-9))))
    if target > positions:
        positions = target
        t = net.timed_forward(x_storage[:positions])
    return {"value": positions / t, "unit": "positions/sec", "cores": cores, "kind": kind,
            "sample": "%d positions of the same network and inputs, one forward pass, %.1f s" % (positions, t)}


def run_int8_cpu_baseline(layers, blocks, x_int8, budget_seconds):
    """The oracle's restatement of the reference's integer branch (the reference has no backend entry point for it: the arithmetic lives in
    src/layers/Conv2D.cpp:240-308 and walks tensors element by element), multi-threaded, on as many positions as fit the budget."""
    import oracle as O
    from oracle.cpu_net import CpuQuantizedResNet

    cores = min(16, os.cpu_count() or 1)
    O.set_num_threads(cores)
    net = CpuQuantizedResNet(layers, blocks)
    positions = 1
    t0 = time.perf_counter()
    net.forward(x_int8[:positions])
    t = time.perf_counter() - t0
    target = int(max(1, min(x_int8.shape[0], budget_seconds / max(t, 1e-9))))
    if target > positions:
        positions = target
        t0 = time.perf_counter()
        net.forward(x_int8[:positions])
        t = time.perf_counter() - t0
    return {"value": positions / t, "unit": "positions/sec", "cores": cores, "kind": "port",
            "sample": "%d positions of the same int8 network and inputs, one forward pass, %.1f s" % (positions, t)}


def run_int8(args, ml):
    """Configuration 3: the int8 network, every 3x3 layer one fused int8 implicit-GEMM convolution (--unfused: the reference's three calls)."""
    from minml_amd import quantization as Q
    from minml_amd.resnet import QuantizedResNet, calibrate_activations, make_input, make_parameters

    batch, board, planes, channels, blocks, _, seed = CONFIGS[args.config]
    params = make_parameters(seed, planes, channels, blocks)
    x = make_input(seed, batch, board, planes)
    ctx = ml.Context(0)
    ranges = calibrate_activations(ctx, params, board, planes, channels, blocks, batches=64, batch_size=4, seed=seed)
    net = QuantizedResNet(ctx, batch, board, planes, channels, blocks, params, ranges, "reference" if args.unfused else "fused")
    net.setInput(x)
    for _ in range(args.warmup):
        net.forward()
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        net.forward()
    ctx.synchronize()
    elapsed = time.perf_counter() - t0
    timer = ml.KernelTimer(ctx)
    ml.set_kernel_timer(timer)
    for _ in range(max(1, min(args.steps, 5))):
        net.forward()
    kernels = timer.summary()
    ml.set_kernel_timer(None)
    entry = "gemm_v2" if args.unfused else "quantized_conv_forward"
    count = sum(kernels.get(entry + "@" + l, (0, 0.0))[0] for l in ("block_conv1", "block_conv2"))
    total = sum(kernels.get(entry + "@" + l, (0, 0.0))[0] * kernels.get(entry + "@" + l, (0, 0.0))[1] for l in ("block_conv1", "block_conv2"))
    t_conv = total / count if count else float("nan")
    pix = batch * board * board
    conv_ops = 2.0 * pix * 9 * channels * channels
    conv_bytes = pix * channels * 2.5 + 9 * channels * channels + 8 * channels  # int8 in, int8 out, the residual on every second layer
    tops = conv_ops / t_conv / 1e12
    result = {
        "metric": "positions/sec (%s)" % args.config, "value": batch / (elapsed / args.steps), "unit": "positions/sec", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": 1e3 * elapsed / args.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "i8",
        "data": "synthetic (Bernoulli(0.3) input planes, He-normal weights quantised per output channel, activation ranges from 64 random "
                "batches of 4 through the fp32 network, seed %d)" % seed,
        "config": {"workload": args.config, "batch": batch, "board": board, "channels": channels, "blocks": blocks,
                   "single_launch_int8_convolution": not args.unfused},
        "tops_executed": net.ops_per_forward() / (elapsed / args.steps) / 1e12,
        "roofline": {"bound": "mfma", "achieved": tops, "peak": PEAK_INT8_TOPS, "unit": "TOP/s", "frac": tops / PEAK_INT8_TOPS, "traffic": None,
                     "kernel": ("int8 GEMM of the three-call form" if args.unfused else "kernel_gemm_dma<int8, im2row, requantisation>")
                     + " (3x3 convolution as implicit GEMM, M=%d N=%d K=%d)" % (pix, channels, 9 * channels),
                     "algorithmic_ops": conv_ops, "algorithmic_bytes": conv_bytes, "launches_timed": count, "avg_launch_us": t_conv * 1e6},
    }
    if not args.unfused and not args.skip_three_call:
        # the reference's route for an int8 layer on a device: im2row -> int8 GEMM into int32 -> requantisation (src/layers/Conv2D.cpp:214-239)
        three = QuantizedResNet(ctx, batch, board, planes, channels, blocks, params, ranges, "reference")
        three.setInput(x)
        t3 = timed_passes(ctx, three.forward, args.steps, args.warmup)
        result["reference_call_sequence"] = {"value": batch / t3, "unit": "positions/sec", "ms_per_step": 1e3 * t3,
                                             "what": "im2row, int8 GEMM (gemm_v2 into int32) and quantized_scale_shift_act as three calls per layer"}
    if args.cpu_seconds > 0:
        result["cpu_baseline"] = run_int8_cpu_baseline(net.host_parameters, blocks, Q.quantize_tensor(x, net.transforms[0]), args.cpu_seconds)
    print(json.dumps(result))


def run_hybrid(args, ml):
    """Configuration 5 without its mixture-of-experts halves (those have no CPU implementation in the reference): residual trunk, four
    attention half-blocks (RMS normalisation, dense qkv, attention with the relative-position table, dense output + residual), 1x1 head."""
    import oracle as O
    from oracle.cpu_net import CpuHybridNet
    from minml_amd.hybridnet import HybridNet, make_hybrid_parameters
    from minml_amd.resnet import make_input

    batch, board, planes, channels, blocks, kind, seed = CONFIGS[args.config]
    moe = kind == "hybrid_moe"
    attention_blocks, heads = 4, 8
    to_storage = to_storage_factory("float16")
    params = make_hybrid_parameters(seed, planes, channels, blocks, attention_blocks, heads, board)
    x = make_input(seed, batch, board, planes)
    ctx = ml.Context(0)
    net = HybridNet(ctx, batch, board, planes, channels, blocks, heads, "float16", params, to_storage, moe=moe)
    net.setInput(to_storage(x))
    for _ in range(args.warmup):
        net.forward()
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        net.forward()
    ctx.synchronize()
    elapsed = time.perf_counter() - t0
    timer = ml.KernelTimer(ctx)
    ml.set_kernel_timer(timer)
    for _ in range(max(1, min(args.steps, 5))):
        net.forward()
    kernels = timer.summary()
    ml.set_kernel_timer(None)
    per_pass = max(1, min(args.steps, 5))
    breakdown = {name: {"launches_per_pass": n / per_pass, "avg_launch_us": t * 1e6, "ms_per_pass": n * t * 1e3 / per_pass}
                 for name, (n, t) in sorted(kernels.items()) if "@" not in name}
    tiles = batch * ((board + 3) // 4) ** 2
    n_gemm, t_gemm = kernels.get("gemm_batched_v2", (0, float("nan")))
    gemm_bytes = 2 * 36 * (2 * tiles * channels + channels * channels)
    gemm_flops = 2.0 * 36 * tiles * channels * channels
    n_att, t_att = kernels.get("multi_head_attention_forward", (0, float("nan")))
    tokens = board * board
    result = {
        "metric": "positions/sec (%s)" % args.config, "value": batch / (elapsed / args.steps), "unit": "positions/sec", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": 1e3 * elapsed / args.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16",
        "data": "synthetic (Bernoulli(0.3) input planes, N(0, 0.02) weights and position tables, N(0, 0.01) biases, seed %d)" % seed,
        "config": {"workload": args.config, "batch": batch, "board": board, "channels": channels, "blocks": blocks,
                   "attention_blocks": attention_blocks, "heads": heads,
                   "mixture_of_experts_halves": "8 experts, hidden 1024, expert-choice routing, capacity factor 2" if moe else "not included (no CPU reference)"},
        "tflops_executed": net.flops_per_forward() / (elapsed / args.steps) / 1e12,
        "roofline": {"bound": "hbm", "achieved": gemm_bytes / t_gemm / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": gemm_bytes / t_gemm / 1e9 / PEAK_HBM_GBS, "traffic": None,
                     "kernel": "kernel_gemm_stream_wide_nt (36 batched Winograd GEMMs of the trunk, M=%d N=K=%d)" % (tiles, channels),
                     "algorithmic_bytes": gemm_bytes, "launches_timed": n_gemm, "avg_launch_us": t_gemm * 1e6},
        "gemm_mfma": {"achieved": gemm_flops / t_gemm / 1e12, "peak": PEAK_MFMA_TFLOPS["float16"], "unit": "TFLOP/s",
                      "frac": gemm_flops / t_gemm / 1e12 / PEAK_MFMA_TFLOPS["float16"]},
        "attention": {"avg_launch_us": t_att * 1e6, "launches_timed": n_att,
                      "tflops": 4.0 * batch * heads * tokens * tokens * (channels // heads) / t_att / 1e12},
        "entry_points": breakdown,
    }
    if args.cpu_seconds > 0:
        cores = min(16, os.cpu_count() or 1)
        O.set_num_threads(cores)
        conv = to_storage
        ps = {"trunk": [(conv(w), conv(b)) for (w, b) in params["trunk"]], "attention": [{k: conv(v) for k, v in blk.items()} for blk in params["attention"]],
              "head": (conv(params["head"][0]), conv(params["head"][1]))}
        capacity = None
        if moe:
            from minml_amd.hybridnet import get_capacity

            ps["ffn"] = [{k: conv(v) for k, v in blk.items()} for blk in params["ffn"]]
            capacity = get_capacity(2.0, board * board, 8)
        cpu = CpuHybridNet(ps, blocks, heads)
        xs = conv(x)
        positions = 2
        t0 = time.perf_counter()
        cpu.forward(xs[:positions], moe_capacity=capacity)
        t = time.perf_counter() - t0
        target = int(max(2, min(batch, args.cpu_seconds / max(t / positions, 1e-9))))
        if target > positions:
            positions = target
            t0 = time.perf_counter()
            cpu.forward(xs[:positions], moe_capacity=capacity)
            t = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": positions / t, "unit": "positions/sec", "cores": cores, "kind": "port",
                                  "sample": "%d positions of the same network and inputs, one forward pass, %.1f s" % (positions, t)}
    print(json.dumps(result))


def run_conv_sweep(args, ml):
    """Configuration 4: hip_convolution_implicit_gemm_forward on 19x19 boards, batch 512, fp16, N(0,1) inputs, He-normal weights, with bias,
    residual and ReLU in the kernel's epilogue, for 64 / 128 / 256 / 384 channels and kernels 1 / 3 / 5. A step is the 12 layers one after
    the other. Every row is priced with its algorithmic work (2 * M * C * C * k * k flops; input, residual and output once, weights and bias
    once) against whichever of HBM and the fp16 MFMA peak bounds it; the top-level roofline object is the row that takes longest."""
    batch, board = args.batch or 512, 19
    pix = batch * board * board
    rng = np.random.default_rng(3)
    half = lambda a: np.ascontiguousarray(a, np.float32).astype(np.float16).view(np.uint16)
    ctx = ml.Context(0)
    layers = []
    host = {}
    for chans in (64, 128, 256, 384):
        xh = half(rng.standard_normal((batch, board, board, chans), dtype=np.float32))
        rh = half(rng.standard_normal((batch, board, board, chans), dtype=np.float32))
        bh = half(rng.standard_normal(chans, dtype=np.float32) * 0.1)
        x, res, bias = ml.toDevice(ctx, xh, "float16"), ml.toDevice(ctx, rh, "float16"), ml.toDevice(ctx, bh, "float16")
        y = ml.Tensor((batch, board, board, chans), "float16")
        for k in (1, 3, 5):
            wh = half(rng.standard_normal((chans, k, k, chans), dtype=np.float32) * np.sqrt(2.0 / (k * k * chans)))
            layers.append((chans, k, x, ml.toDevice(ctx, wh, "float16"), y, bias, res))
            host[(chans, k)] = (xh, wh, bh, rh)

    def step():
        for chans, k, x, w, y, bias, res in layers:
            ml.set_timer_label("C%d_k%d" % (chans, k))
            ml.convolutionImplicitGemmForward(ctx, x, w, y, bias, res, "relu")
        ml.set_timer_label(None)

    t_step = timed_passes(ctx, step, args.steps, args.warmup)
    timer = ml.KernelTimer(ctx)
    ml.set_kernel_timer(timer)
    for _ in range(max(1, min(args.steps, 5))):
        step()
    kernels = timer.summary()
    ml.set_kernel_timer(None)
    rows = []
    for chans, k, *_ in layers:
        n, t = kernels["convolution_implicit_gemm_forward@C%d_k%d" % (chans, k)]
        flops = 2.0 * pix * chans * chans * k * k
        nbytes = 2.0 * (3 * pix * chans + k * k * chans * chans + chans)
        hbm = nbytes / (PEAK_HBM_GBS * 1e9) >= flops / (PEAK_MFMA_TFLOPS["float16"] * 1e12)
        achieved = nbytes / t / 1e9 if hbm else flops / t / 1e12
        peak = PEAK_HBM_GBS if hbm else PEAK_MFMA_TFLOPS["float16"]
        rows.append({"channels": chans, "kernel_size": k, "avg_launch_us": t * 1e6, "launches_timed": n, "bound": "hbm" if hbm else "mfma",
                     "achieved": achieved, "peak": peak, "unit": "GB/s" if hbm else "TFLOP/s", "frac": achieved / peak,
                     "algorithmic_bytes": nbytes, "algorithmic_flops": flops})
    def kernel_of(chans, k):
        """which kernel conv.hip runs for a layer of the sweep (19x19 boards, fp16, C -> C filters, bias + residual + ReLU)"""
        if k == 1:
            return "kernel_gemm_stream_wide_nt<fp16> (1x1: the pixels are the GEMM's rows)"
        if chans == 64:
            return "kernel_conv_window<fp16>" if k == 3 else "kernel_conv_window_split<fp16>"
        if chans % 256 != 0 and (chans % 192 == 0 or chans == 128):
            return "kernel_conv_dma_window<fp16> (tile engine, A operand from a window of pixels in LDS)"
        return "kernel_gemm_dma<fp16, im2row> (tile engine, gathered A operand)"

    for r in rows:
        r["kernel"] = kernel_of(r["channels"], r["kernel_size"])
    slowest = max(rows, key=lambda r: r["avg_launch_us"])
    total_flops = sum(r["algorithmic_flops"] for r in rows)
    result = {
        "metric": "positions/sec (%s)" % CONV_SWEEP, "value": batch / t_step, "unit": "positions/sec", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": 1e3 * t_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic (N(0,1) inputs and residuals, He-normal weights, N(0,0.1) biases, seed 3)",
        "config": {"workload": CONV_SWEEP, "batch": batch, "board": board, "channels": [64, 128, 256, 384], "kernel_sizes": [1, 3, 5],
                   "epilogue": "bias + residual + ReLU inside the convolution kernel", "step": "the 12 layers one after the other"},
        "tflops_executed": total_flops / t_step / 1e12,
        "roofline": {"bound": slowest["bound"], "achieved": slowest["achieved"], "peak": slowest["peak"], "unit": slowest["unit"], "frac": slowest["frac"],
                     "traffic": None, "kernel": "%s, bias + residual + ReLU (C=%d, k=%d: M=%d N=%d K=%d)"
                     % (slowest["kernel"], slowest["channels"], slowest["kernel_size"], pix, slowest["channels"], slowest["kernel_size"] ** 2 * slowest["channels"]),
                     "algorithmic_flops": slowest["algorithmic_flops"], "algorithmic_bytes": slowest["algorithmic_bytes"],
                     "launches_timed": slowest["launches_timed"], "avg_launch_us": slowest["avg_launch_us"]},
        "rows": rows,
    }
    if args.cpu_seconds > 0:
        import oracle as O

        ref = O.reference()
        if ref is not None:
            kind, cores, conv = "reference", 1, ref.conv2d_forward
        else:
            cores = min(16, os.cpu_count() or 1)
            O.set_num_threads(cores)
            kind, conv = "port", O.conv2d_forward

        def cpu_step(positions):
            t0 = time.perf_counter()
            for (chans, k), (xh, wh, bh, rh) in host.items():
                conv(xh[:positions], wh, bh, rh[:positions], O.RELU)
            return time.perf_counter() - t0

        positions = 1
        t = cpu_step(positions)
        # at most 192 positions: the reference counts the bytes of the im2row matrix (positions x 361 x 25 x 384 halfs) in 32-bit integers
        target = int(max(1, min(batch, 192, args.cpu_seconds / max(t, 1e-9))))
        if target > positions:
            positions = target
            t = cpu_step(positions)
        result["cpu_baseline"] = {"value": positions / t, "unit": "positions/sec", "cores": cores, "kind": kind,
                                  "sample": "%d positions through the same 12 layers (im2row + gemm_ex with the fused epilogue, the reference's "
                                            "explicit-GEMM convolution), %.1f s" % (positions, t)}
    print(json.dumps(result))


def copy_calibration(ml, ctx):
    """One copy kernel of known size (256 MiB read, 256 MiB written) so that a counter run can be scaled against it."""
    n = 128 * 1024 * 1024
    src = ml.Tensor((n,), "float16")
    dst = ml.Tensor((n,), "float16")
    src.zeroall(ctx)
    dst.zeroall(ctx)
    ml.addTensors(ctx, 1.0, src, 0.0, None, 0.0, None, 0.0, dst)  # y = 1 * x: one read and one write of every byte
    ctx.synchronize()
    src.free()
    dst.free()


def main():
    import faulthandler

    faulthandler.enable()
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="cfg2_resnet20x256_fp16_b1024", choices=sorted(CONFIGS) + [CONV_SWEEP])
    ap.add_argument("--dropin-seconds", type=float, default=3.0,
                    help="seconds the reference's own Graph is timed on this backend in a child process (0 disables; residual-network configurations)")
    ap.add_argument("--chunk", type=int, default=0, help="positions per sub-batch (0 = library default: the whole batch)")
    ap.add_argument("--batch", type=int, default=0, help="override the configuration's batch size (experiments only; the metric is quoted at the default)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the CPU baseline leg (0 disables it)")
    ap.add_argument("--streams", type=int, default=2, choices=[1, 2],
                    help="2: also time the batch as two halves on two streams and report the faster way as `value` (the roofline figures always "
                         "come from the single-stream pass, where launches do not overlap)")
    ap.add_argument("--skip-three-call", action="store_true",
                    help="leave the second timed leg (the reference's call sequence per layer) out, e.g. under a profiler")
    ap.add_argument("--unfused", action="store_true", help="run every layer as the reference's three calls (no cross-layer transform fusion)")
    ap.add_argument("--layer-launch", action="store_true", help="experimental: product and both transforms of a layer as one launch (slower)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one 256 MiB copy kernel (kernel_axpy3) for scaling hardware counters")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this path runs on one GPU (positions are independent; it shards by batch with no communication) — use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    dropin = None
    if args.config != CONV_SWEEP and CONFIGS[args.config][5] in ("float16", "float32") and args.dropin_seconds > 0 and not args.chunk:
        # first of all: the child process has the device to itself, and this process has not touched the GPU yet
        b, _, _, c, n, d, _ = CONFIGS[args.config]
        dropin = run_dropin_graph(args.batch or b, c, n, d, args.dropin_seconds)

    from minml_amd import core as ml
    from minml_amd.resnet import ResNet, make_input, make_parameters, DEFAULT_CHUNK

    if args.config == CONV_SWEEP:
        return run_conv_sweep(args, ml)
    if CONFIGS[args.config][5] == "int8":
        return run_int8(args, ml)
    if CONFIGS[args.config][5] in ("hybrid", "hybrid_moe"):
        return run_hybrid(args, ml)
    batch, board, planes, channels, blocks, dtype, seed = CONFIGS[args.config]
    batch = args.batch or batch
    chunk = args.chunk or DEFAULT_CHUNK.get(dtype, batch)
    to_storage = to_storage_factory(dtype)
    params = make_parameters(seed, planes, channels, blocks)
    x = make_input(seed, batch, board, planes)

    ctx = ml.Context(0)
    if args.copy_calibration:
        copy_calibration(ml, ctx)
    net = ResNet(ctx, batch, board, planes, channels, blocks, dtype, params, to_storage, chunk=chunk, fused=not args.unfused)
    net.fuse_layers = bool(args.layer_launch) and not args.unfused
    net.setInput(to_storage(x))

    for _ in range(args.warmup):
        net.forward()
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        net.forward()
    ctx.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / args.steps
    value = batch / (elapsed / args.steps)
    execution = "the whole batch on one stream"
    single_stream = {"value": value, "ms_per_step": ms_per_step}

    # the same batch as two halves on two contexts (two streams of the one device): one half's launch starts up and drains while the
    # other's is in its steady state. Same results bit for bit; whichever of the two ways is faster is the throughput of the step.
    two_streams = None
    if args.streams == 2 and batch % 2 == 0 and not args.unfused and net.chunk == batch:
        half = batch // 2
        contexts = [ml.Context(0), ml.Context(0)]
        halves = [ResNet(c, half, board, planes, channels, blocks, dtype, params, to_storage, fused=True) for c in contexts]
        for i, part in enumerate(halves):
            part.setInput(to_storage(x[i * half:(i + 1) * half]))

        def both():
            for part in halves:
                part.forward()

        for _ in range(args.warmup):
            both()
        for c in contexts:
            c.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            both()
        for c in contexts:
            c.synchronize()
        t2 = (time.perf_counter() - t0) / args.steps
        two_streams = {"value": batch / t2, "ms_per_step": 1e3 * t2}
        if two_streams["value"] > value:
            value, ms_per_step, execution = two_streams["value"], two_streams["ms_per_step"], "two halves of the batch on two streams"
        del halves

    # instrumented run: HIP events around every launch, on the stream the kernels run on
    timer = ml.KernelTimer(ctx)
    ml.set_kernel_timer(timer)
    for _ in range(max(1, min(args.steps, 5))):
        net.forward()
    kernels = timer.summary()
    ml.set_kernel_timer(None)

    def timed(entry, labels):
        count = sum(kernels.get(entry + "@" + l, (0, 0.0))[0] for l in labels)
        total = sum(kernels.get(entry + "@" + l, (0, 0.0))[0] * kernels.get(entry + "@" + l, (0, 0.0))[1] for l in labels)
        return count, (total / count if count else float("nan"))

    esize = 2 if dtype == "float16" else 4
    tiles = net.chunk * ((board + 3) // 4) ** 2  # T of one launch
    pix = net.chunk * board * board
    block_labels = ("block_conv1", "block_conv2")
    # 36 batched GEMMs of the block convolutions (Cin = Cout = channels)
    n_gemm, t_gemm = timed("gemm_batched_v2", block_labels)
    gemm_flops = 2.0 * 36 * tiles * channels * channels
    gemm_bytes = esize * 36 * (tiles * channels + channels * channels + tiles * channels)
    gemm_gbs = gemm_bytes / t_gemm / 1e9
    gemm_tflops = gemm_flops / t_gemm / 1e12
    # transforms of the block convolutions. Fused mode: inside a residual block one launch does the first convolution's output transform
    # and the second one's input transform (nothing else read or written); block boundaries use the two stand-alone transforms.
    mat_bytes = esize * 36 * tiles * channels
    act_bytes = esize * pix * channels
    transforms = {}
    for entry, kernel, label, nbytes in (
            ("winograd_output_input_transform", "kernel_output_input_transform_4x4_3x3", "block_conv1", 2 * mat_bytes),
            ("winograd_output_input_transform", "kernel_output_input_transform_4x4_3x3 (+residual, y written)", "block_conv2", 2 * mat_bytes + 2 * act_bytes),
            ("winograd_input_transform", "kernel_input_transform_4x4_3x3", "block_conv1", mat_bytes + act_bytes),
            ("winograd_input_transform", "kernel_input_transform_4x4_3x3", "block_conv2", mat_bytes + act_bytes),
            ("winograd_output_transform", "kernel_output_transform_4x4_3x3", "block_conv1", mat_bytes + act_bytes),
            ("winograd_output_transform", "kernel_output_transform_4x4_3x3 (+residual)", "block_conv2", mat_bytes + 2 * act_bytes)):
        n_t, t_t = timed(entry, (label,))
        if n_t:
            transforms["%s@%s" % (entry, label)] = {"kernel": kernel, "launches_timed": n_t, "avg_launch_us": t_t * 1e6, "algorithmic_bytes": nbytes,
                                                   "gbs": nbytes / t_t / 1e9, "frac_hbm": nbytes / t_t / 1e9 / PEAK_HBM_GBS}
    kernel_name = "kernel_gemm_stream_wide_nt" if channels * esize in (128, 256, 512) else "kernel_gemm_dma"
    # the roofline that bounds the dominant kernel: whichever of its algorithmic bytes and flops takes longer at the chip's peaks
    hbm_bound = gemm_bytes / (PEAK_HBM_GBS * 1e9) >= gemm_flops / (PEAK_MFMA_TFLOPS[dtype] * 1e12)
    if hbm_bound:
        roofline = {"bound": "hbm", "achieved": gemm_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gemm_gbs / PEAK_HBM_GBS}
    else:
        roofline = {"bound": "mfma", "achieved": gemm_tflops, "peak": PEAK_MFMA_TFLOPS[dtype], "unit": "TFLOP/s",
                    "frac": gemm_tflops / PEAK_MFMA_TFLOPS[dtype]}
    roofline.update({"traffic": measured_gemm_traffic_bytes(args.config) if net.chunk == batch else None,
                     "kernel": "%s (36 batched Winograd GEMMs, M=%d N=K=%d)" % (kernel_name, tiles, channels),
                     "algorithmic_bytes": gemm_bytes, "launches_timed": n_gemm, "avg_launch_us": t_gemm * 1e6})
    result = {
        "metric": "positions/sec at batch 1024 (20x256 res-net fp16); % MFMA peak in conv GEMMs" if args.config.startswith("cfg2")
        else "positions/sec (%s)" % args.config,
        "value": value, "unit": "positions/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16" if dtype == "float16" else "f32",
        "data": "synthetic (Bernoulli(0.3) input planes, He-normal weights, N(0,0.01) biases, seed %d)" % seed,
        "config": {"workload": args.config, "batch": batch, "board": board, "channels": channels, "blocks": blocks,
                   "positions_per_launch": net.chunk, "cross_layer_transform_fusion": not args.unfused, "execution": execution},
        "single_stream": single_stream, "two_streams": two_streams,
        "tflops_executed": net.flops_per_forward() / (ms_per_step * 1e-3) / 1e12,
        "roofline": roofline,
        "gemm_mfma": {"achieved": gemm_tflops, "peak": PEAK_MFMA_TFLOPS[dtype], "unit": "TFLOP/s", "frac": gemm_tflops / PEAK_MFMA_TFLOPS[dtype],
                      "flops_per_launch": gemm_flops,
                      "hbm_limited_ceiling_frac": min(1.0, gemm_flops / gemm_bytes * PEAK_HBM_GBS * 1e9 / (PEAK_MFMA_TFLOPS[dtype] * 1e12))},
        "transforms": transforms,
    }
    if not args.unfused and not args.skip_three_call:
        t3 = timed_passes(ctx, lambda: net.forward(fused=False), args.steps, args.warmup)
        result["reference_call_sequence"] = {"value": batch / t3, "unit": "positions/sec", "ms_per_step": 1e3 * t3,
                                             "what": "winograd_input_transform, gemm_batched_v2 and winograd_output_transform as three calls per 3x3 layer, "
                                                     "as src/layers/Conv2D.cpp:365-378 issues them; same results bit for bit"}
    if dropin is not None:
        result["dropin_graph_predict"] = dropin
    if args.cpu_seconds > 0:
        params_storage = [(to_storage(w), to_storage(b)) for (w, b) in params]
        result["cpu_baseline"] = run_cpu_baseline(params_storage, to_storage(x), blocks, args.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
