"""Child process of tests/test_zz_no_alloc.py: in a process that has made no other library call, the FIRST call of
hip_winograd_layer_forward_static is recorded under hip_graph_begin_capture / hip_graph_end_capture. The capture is thread-local, so any
device allocation inside the call would fail it: a completed recording shows that the entry point allocates nothing, also on its first
call. The graph is replayed twice with eager work between the replays and compared bit for bit with an eager call of the same entry point
and of the allocating one. Prints "static entry under capture: ok" on success."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from minml_amd import core as ml  # noqa: E402
from util import mismatches, random_tensor  # noqa: E402


def main():
    batch, channels, board = int(sys.argv[1]), int(sys.argv[2]), 15
    ctx = ml.Context(0)
    rng = np.random.default_rng(batch + channels)
    tiles = batch * 16
    shape = (batch, board, board, channels)
    dv = ml.toDevice(ctx, random_tensor(rng, (36, tiles, channels), "float16"))
    du = ml.toDevice(ctx, random_tensor(rng, (36, channels, channels), "float16", (1.0 / channels) ** 0.5))
    db = ml.toDevice(ctx, random_tensor(rng, (channels,), "float16", 0.1))
    de = ml.toDevice(ctx, random_tensor(rng, shape, "float16"))
    m = ml.Tensor((36, tiles, channels), "float16")
    nxt = ml.Tensor((36, tiles, channels), "float16")
    y = ml.Tensor(shape, "float16")
    scratch = ml.Tensor((1024,), "float32")
    ctx.synchronize()

    def call(static):
        ml.winogradLayerForward(ctx, (channels, 3, 3, channels), dv, du, m, shape, y, db, de, "relu", nxt, static_memory=static)

    graph = ml.Graph.record(ctx, lambda: call(True))  # the process's first call of the entry point happens inside the recording
    replays = []
    for _ in range(2):
        nxt.setall(ctx, float("nan"))
        y.setall(ctx, float("nan"))
        graph.launch()
        replays.append((nxt.copyToHost(ctx), y.copyToHost(ctx)))
        scratch.zeroall(ctx)  # unrelated eager work and a synchronisation between the replays
        ctx.synchronize()
    assert ml.winogradLayerErrors(ctx) == 0
    graph.destroy()
    results = []
    for static in (True, False):
        nxt.setall(ctx, float("nan"))
        y.setall(ctx, float("nan"))
        call(static)
        results.append((nxt.copyToHost(ctx), y.copyToHost(ctx)))
        assert ml.winogradLayerErrors(ctx) == 0
    assert np.isfinite(results[1][0].view(np.float16).astype(np.float32)).all()
    for got_next, got_y in replays + results[:1]:
        assert mismatches(got_next, results[1][0]) == 0
        assert mismatches(got_y, results[1][1]) == 0
    print("static entry under capture: ok", flush=True)


if __name__ == "__main__":
    main()
