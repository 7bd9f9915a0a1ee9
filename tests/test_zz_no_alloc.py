"""hip_winograd_layer_forward_static — the entry point that allocates nothing (counters and scratch of the whole-layer launch live in a
static device array of the library) — against hip_winograd_layer_forward, whose kernels it shares and which keeps the same memory in the
context's growable workspace: bit-identical next-layer matrices and outputs, on two calls in a row through the C-ABI, the second with a
smaller batch (the static array keeps the first call's contents: counters must be cleared, stale scratch must not leak), for the shape
the one-launch form takes (fp16, 256 -> 256 channels, 15x15 boards) and for one it hands to the two-call route. And, in a process of
its own, the entry point's first call recorded under a thread-local graph capture (which refuses allocations) and replayed."""
import os
import subprocess
import sys

import numpy as np
import pytest

import oracle as O
from minml_amd import core as ml
from util import mismatches, random_tensor

pytestmark = pytest.mark.gpu


def run_layer(ctx, rng, batch, channels, board, static_memory, with_ext, keep_output):
    tiles = batch * ((board + 3) // 4) ** 2
    shape = (batch, board, board, channels)
    v = random_tensor(rng, (36, tiles, channels), "float16")
    u = random_tensor(rng, (36, channels, channels), "float16", (1.0 / channels) ** 0.5)
    bias = random_tensor(rng, (channels,), "float16", 0.1)
    ext = random_tensor(rng, shape, "float16")
    dv, du, db = ml.toDevice(ctx, v), ml.toDevice(ctx, u), ml.toDevice(ctx, bias)
    de = ml.toDevice(ctx, ext) if with_ext else None
    results = []
    for static in (False, static_memory):
        m = ml.Tensor((36, tiles, channels), "float16")
        nxt = ml.Tensor((36, tiles, channels), "float16")
        nxt.setall(ctx, float("nan"))
        y = ml.Tensor(shape, "float16") if keep_output else None
        ml.winogradLayerForward(ctx, (channels, 3, 3, channels), dv, du, m, shape, y, db, de, "relu", nxt, static_memory=static)
        results.append((nxt.copyToHost(ctx), None if y is None else y.copyToHost(ctx)))
        assert ml.winogradLayerErrors(ctx) == 0
    return results


@pytest.mark.parametrize("channels,board", [(256, 15), (128, 15)])
def test_static_memory_entry_point_matches_the_allocating_one(ctx, channels, board):
    rng = np.random.default_rng(channels + board)
    for batch, with_ext, keep_output in ((64, True, True), (32, False, False), (96, True, False), (32, True, True)):
        (want_next, want_y), (got_next, got_y) = run_layer(ctx, rng, batch, channels, board, True, with_ext, keep_output)
        assert np.isfinite(O.from_half(want_next)).all()
        assert mismatches(got_next, want_next) == 0
        if keep_output:
            assert mismatches(got_y, want_y) == 0


@pytest.mark.parametrize("batch,channels", [(64, 256), (8, 128)])
def test_first_call_allocates_nothing_recorded_under_capture(batch, channels):
    """tests/static_entry_under_capture.py in a fresh process: the first call ever of the static entry point, inside a recording."""
    here = os.path.dirname(os.path.abspath(__file__))
    run = subprocess.run([sys.executable, os.path.join(here, "static_entry_under_capture.py"), str(batch), str(channels)], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True, timeout=110)
    print(run.stdout, flush=True)
    assert run.returncode == 0, run.stdout
    assert "static entry under capture: ok" in run.stdout


def test_static_entry_refuses_only_what_would_use_its_memory(ctx):
    """More images than the static counters cover: refused at the shape whose launch uses them, accepted at a shape that runs as the
    batched product plus the fused transform (no library-side memory)."""
    from minml_amd import backend as B

    def call(batch, channels, static):
        tiles = batch * 16
        shape = (batch, 15, 15, channels)
        v = ml.Tensor((36, tiles, channels), "float16")
        v.zeroall(ctx)
        u = ml.Tensor((36, channels, channels), "float16")
        u.zeroall(ctx)
        m = ml.Tensor((36, tiles, channels), "float16")
        nxt = ml.Tensor((36, tiles, channels), "float16")
        y = ml.Tensor(shape, "float16")
        try:
            B.fn("winograd_layer_forward_static" if static else "winograd_layer_forward")(
                ctx.handle, 4, v.desc(), u.desc(), m.desc(), ml._desc(None), ml._desc(None), B.make_shape(shape), y.ptr, ml.act_of("relu"), nxt.desc())
            ctx.synchronize()
            return nxt.copyToHost(ctx)
        finally:
            for t in (v, u, m, nxt, y):
                t.free()

    with pytest.raises(ValueError, match="4096"):
        call(4100, 256, True)
    assert not call(4100, 64, True).any()  # zero matrices in, zero matrices out
