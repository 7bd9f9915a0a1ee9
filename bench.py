#!/usr/bin/env python3
"""Benchmark of the convolution / GEMM inference path on one MI355X.

A step is one forward pass of the synthetic 20-block x 256-channel 15x15 residual network (fp16 storage, fp32 accumulation) over one
batch of 1024 positions already resident in HBM: stem 3x3 conv 32->256, 40 3x3 convs 256->256 as Winograd F(4x4,3x3) (input transform,
36 batched GEMMs on MFMA, output transform with bias + residual + ReLU), 1x1 policy head. Prints ONE JSON line:

  value        positions / second over the timed steps (wall clock between two stream synchronisations)
  roofline     the 36-way batched Winograd GEMM kernel against the dense fp16 MFMA peak: executed flops of one launch
               (2 * 36 * tiles * Cin * Cout) divided by the kernel's average duration, taken with HIP events recorded on the context's
               stream around every launch in a second, instrumented run of the same steps
  cpu_baseline the same network on a bounded number of positions on the host's cores: the reference's own CPU backend compiled from
               its sources (kind "reference", one thread, as the reference runs) when that library is present, otherwise this
               repository's C restatement (kind "port")
"""
import argparse
import json
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

PEAK_FP16_MFMA_TFLOPS = 2500.0  # MI355X dense fp16 matrix peak
PEAK_HBM_GBS = 8000.0

CONFIGS = {
    # name: (batch, board, input planes, channels, blocks, dtype, seed)
    "cfg2_resnet20x256_fp16_b1024": (1024, 15, 32, 256, 20, "float16", 1),
    "cfg1_resnet10x128_fp32_b256": (256, 15, 32, 128, 10, "float32", 0),
}


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="cfg2_resnet20x256_fp16_b1024", choices=sorted(CONFIGS))
    ap.add_argument("--chunk", type=int, default=0, help="positions per cache-resident sub-batch (0 = library default)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the CPU baseline leg (0 disables it)")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this path runs on one GPU (positions are independent; it shards by batch with no communication) — use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    from minml_amd import core as ml
    from minml_amd.resnet import ResNet, make_input, make_parameters, DEFAULT_CHUNK

    batch, board, planes, channels, blocks, dtype, seed = CONFIGS[args.config]
    chunk = args.chunk or DEFAULT_CHUNK.get(dtype, batch)
    to_storage = to_storage_factory(dtype)
    params = make_parameters(seed, planes, channels, blocks)
    x = make_input(seed, batch, board, planes)

    ctx = ml.Context(0)
    net = ResNet(ctx, batch, board, planes, channels, blocks, dtype, params, to_storage, chunk=chunk)
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

    # instrumented run: HIP events around every launch, on the stream the kernels run on
    timer = ml.KernelTimer(ctx)
    ml.set_kernel_timer(timer)
    for _ in range(max(1, min(args.steps, 5))):
        net.forward()
    kernels = timer.summary()
    ml.set_kernel_timer(None)

    tiles_per_launch = net.chunk * ((board + 3) // 4) ** 2
    gemm_flops = 2.0 * 36 * tiles_per_launch * channels * channels  # the 40 block convolutions (Cin = Cout = channels)
    # the stem launch has Cin = planes: average flops per launch over the launches actually timed
    launches_per_pass = (batch + net.chunk - 1) // net.chunk
    flops_per_launch = (2 * blocks * gemm_flops + 2.0 * 36 * tiles_per_launch * planes * channels) / (2 * blocks + 1)
    n_gemm, t_gemm = kernels.get("gemm_batched_v2", (0, float("nan")))
    achieved = flops_per_launch / t_gemm / 1e12
    esize = 2 if dtype == "float16" else 4
    n_in, t_in = kernels.get("winograd_input_transform", (0, float("nan")))
    n_out, t_out = kernels.get("winograd_output_transform", (0, float("nan")))
    pix = net.chunk * board * board
    in_bytes = esize * (pix * channels + 36 * tiles_per_launch * channels)
    out_bytes = esize * (36 * tiles_per_launch * channels + 2 * pix * channels)  # matrices + y, + residual on every second layer
    result = {
        "metric": "positions/sec at batch 1024 (20x256 res-net fp16); % MFMA peak in conv GEMMs" if args.config.startswith("cfg2")
        else "positions/sec (%s)" % args.config,
        "value": value, "unit": "positions/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16" if dtype == "float16" else "f32",
        "data": "synthetic (Bernoulli(0.3) input planes, He-normal weights, N(0,0.01) biases, seed %d)" % seed,
        "config": {"workload": args.config, "batch": batch, "board": board, "channels": channels, "blocks": blocks,
                   "cache_resident_chunk": net.chunk, "launches_per_pass_per_layer": launches_per_pass},
        "tflops_executed": net.flops_per_forward() / (elapsed / args.steps) / 1e12,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP16_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_FP16_MFMA_TFLOPS, "traffic": None, "kernel": "kernel_gemm_nt (36 batched Winograd GEMMs)",
                     "launches_timed": n_gemm, "avg_launch_us": t_gemm * 1e6},
        "transforms": {"input": {"avg_launch_us": t_in * 1e6, "gbs": in_bytes / t_in / 1e9, "frac_hbm": in_bytes / t_in / 1e9 / PEAK_HBM_GBS},
                       "output": {"avg_launch_us": t_out * 1e6, "gbs": out_bytes / t_out / 1e9, "frac_hbm": out_bytes / t_out / 1e9 / PEAK_HBM_GBS}},
    }
    if args.cpu_seconds > 0:
        params_storage = [(to_storage(w), to_storage(b)) for (w, b) in params]
        result["cpu_baseline"] = run_cpu_baseline(params_storage, to_storage(x), blocks, args.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
