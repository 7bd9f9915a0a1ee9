"""Per-kernel roofline table of the convolution / GEMM path on one MI355X:  python3 kernel_bench.py [--group NAME] [--json]

Every row launches one entry point of the library on synthetic tensors of a benchmark configuration's shape (resident in HBM), times
`--reps` launches with two events on the context's stream, and prices the launch with its ALGORITHMIC work: the bytes every
implementation must move (inputs once, outputs once) and the flops / integer ops of the algorithm. The bound of a row is whichever of
the two takes longer at the chip's peaks (HBM 8 TB/s; dense MFMA fp16 2.5 PFLOP/s, int8 5.0 POP/s, fp32 157.3 TFLOP/s); `frac` is the
achieved fraction of that peak.

Groups: winograd (transforms and batched GEMM at the residual-network shapes), small (the same launches at 1 to 128 positions), conv (implicit-GEMM sweep: 19x19 boards, batch 512,
channels 64..384, kernels 1 / 3 / 5, bias + residual + ReLU), int8 (quantised 3x3 convolution at 256 channels and its three-call form),
misc (im2row, element-wise neighbours), heads (softmax, global average pooling, batch normalisation in inference mode), transformer
(RMS normalisation and multi-head attention at the hybrid configuration's shape), moe (routing, gather, the two expert layers and
scatter of that configuration's mixture-of-experts half-block), ceilings (what the chip sustains independent of the
backend's kernels: read / write / copy streams over buffers that fit the L2s, the 256 MB last-level cache or neither, and a pure MFMA
loop on constant and on random operands with the shader clock it ran at; its probe kernels are ceilings.hip beside this file, compiled into libminml_ceilings.so by
`python3 kernel_bench.py --build-ceilings`, which __graft_entry__.build() also runs),
library (only on request, needs PyTorch: the vendor GEMM library on plain dense products of the convolutions' shapes, as a yardstick).
"""
import argparse
import ctypes
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from minml_amd import core as ml  # noqa: E402

PEAK = {"hbm": 8000.0e9, "float16": 2500.0e12, "float32": 157.3e12, "int8": 5000.0e12}
ESIZE = {"float16": 2, "float32": 4, "int8": 1, "int32": 4}


def _random(ctx, shape, dtype, rng, scale=1.0):
    n = int(np.prod(shape))
    if dtype == "int8":
        host = rng.integers(-127, 128, n, dtype=np.int8)
    elif dtype == "float16":
        host = (rng.standard_normal(n, dtype=np.float32) * scale).astype(np.float16).view(np.uint16)
    else:
        host = rng.standard_normal(n, dtype=np.float32) * np.float32(scale)
    return ml.toDevice(ctx, host.reshape(shape), dtype)


class Bench:
    def __init__(self, reps):
        self.ctx = ml.Context(0)
        self.reps = reps
        self.rng = np.random.default_rng(7)
        self.rows = []

    def time(self, fn):
        fn()
        self.ctx.synchronize()
        start = ml.Event(self.ctx)
        for _ in range(self.reps):
            fn()
        end = ml.Event(self.ctx)
        self.ctx.synchronize()
        t = ml.Event.getElapsedTime(start, end) / self.reps
        start.destroy()
        end.destroy()
        return t

    def row(self, group, name, shape, fn, nbytes, ops=0.0, op_type="float16"):
        t = self.time(fn)
        t_hbm = nbytes / PEAK["hbm"]
        t_mfma = ops / PEAK[op_type]
        bound = "hbm" if t_hbm >= t_mfma else "mfma"
        achieved = nbytes / t / 1e9 if bound == "hbm" else ops / t / 1e12
        peak = PEAK["hbm"] / 1e9 if bound == "hbm" else PEAK[op_type] / 1e12
        r = {"group": group, "kernel": name, "shape": shape, "us": t * 1e6, "bound": bound, "achieved": achieved,
             "unit": "GB/s" if bound == "hbm" else ("TOP/s" if op_type == "int8" else "TFLOP/s"), "peak": peak, "frac": achieved / peak,
             "algorithmic_MB": nbytes / 1e6, "algorithmic_Gop": ops / 1e9}
        self.rows.append(r)
        print("%-9s %-34s %-34s %9.1f us  %-4s %9.1f %-7s  %5.1f %%" % (group, name, shape, r["us"], bound, achieved, r["unit"], 100 * r["frac"]),
              flush=True)

    # ---- groups ---------------------------------------------------------------------------------------------------------
    def winograd(self):
        ctx, rng = self.ctx, self.rng
        for tag, batch, board, chans, dtype in (("cfg2", 1024, 15, 256, "float16"), ("cfg1", 256, 15, 128, "float32"),
                                                ("cfg4", 512, 19, 64, "float16"), ("cfg4", 512, 19, 128, "float16"),
                                                ("cfg4", 512, 19, 256, "float16"), ("cfg4", 512, 19, 384, "float16")):
            s = ESIZE[dtype]
            tiles = batch * ((board + 3) // 4) ** 2
            pix = batch * board * board
            x = _random(ctx, (batch, board, board, chans), dtype, rng)
            y = ml.Tensor((batch, board, board, chans), dtype)
            w = _random(ctx, (chans, 3, 3, chans), dtype, rng, 0.05)
            bias = _random(ctx, (chans,), dtype, rng, 0.1)
            U = ml.Tensor((36, chans, chans), dtype)
            V = ml.Tensor((36, tiles, chans), dtype)
            M = ml.Tensor((36, tiles, chans), dtype)
            M.zeroall(ctx)
            wshape = (chans, 3, 3, chans)
            shape = "%s B=%d %dx%d C=%d %s" % (tag, batch, board, board, chans, "f16" if s == 2 else "f32")
            self.row("winograd", "winograd_weight_transform", shape, lambda: ml.winogradWeightTransform(ctx, w, U), s * 45 * chans * chans)
            self.row("winograd", "winograd_input_transform", shape, lambda: ml.winogradInputTransform(ctx, wshape, x, V),
                     s * (pix * chans + 36 * tiles * chans))
            self.row("winograd", "gemm_batched (36 x T x C x C)", shape, lambda: ml.gemmBatched(ctx, "n", "t", M, V, U, 1.0, 0.0),
                     s * 36 * (2 * tiles * chans + chans * chans), 2.0 * 36 * tiles * chans * chans, dtype)
            self.row("winograd", "winograd_output_transform", shape, lambda: ml.winogradOutputTransform(ctx, wshape, M, y, bias, None, "relu"),
                     s * (36 * tiles * chans + pix * chans + chans))
            self.row("winograd", "winograd_output_transform +res", shape, lambda: ml.winogradOutputTransform(ctx, wshape, M, y, bias, x, "relu"),
                     s * (36 * tiles * chans + 2 * pix * chans + chans))
            if chans % 64 == 0:
                V2 = ml.Tensor((36, tiles, chans), dtype)
                oshape = (batch, board, board, chans)
                self.row("winograd", "winograd_output_input_transform", shape,
                         lambda: ml.winogradOutputInputTransform(ctx, wshape, M, oshape, None, bias, None, "relu", V2), s * 2 * 36 * tiles * chans)
                self.row("winograd", "winograd_output_input_transform +res, y", shape,
                         lambda: ml.winogradOutputInputTransform(ctx, wshape, M, oshape, y, bias, x, "relu", V2),
                         s * (2 * 36 * tiles * chans + 2 * pix * chans))
                if tag == "cfg2":  # product and both transforms as one launch (experimental): priced with the bytes that must move
                    self.row("winograd", "winograd_layer_forward (one launch)", shape,
                             lambda: ml.winogradLayerForward(ctx, wshape, V, U, M, oshape, None, bias, None, "relu", V2),
                             s * (2 * 36 * tiles * chans + 36 * chans * chans), 2.0 * 36 * tiles * chans * chans, dtype)
                V2.free()
            for t in (x, y, w, bias, U, V, M):
                t.free()

    def small(self):
        """The launches of one residual block of the 20 x 256 network at small batches (1, 8, 32, 128 positions): there the time of a launch is
        its start-up and one pass through its pipeline, not bandwidth or arithmetic; 'of peak' is shown for completeness only."""
        ctx, rng = self.ctx, self.rng
        board, chans, dtype, s = 15, 256, "float16", 2
        wshape = (chans, 3, 3, chans)
        w = _random(ctx, wshape, dtype, rng, 0.05)
        bias = _random(ctx, (chans,), dtype, rng, 0.1)
        U = ml.Tensor((36, chans, chans), dtype)
        ml.winogradWeightTransform(ctx, w, U)
        for batch in (1, 8, 32, 128):
            tiles, pix = batch * 16, batch * board * board
            x = _random(ctx, (batch, board, board, chans), dtype, rng)
            y = ml.Tensor((batch, board, board, chans), dtype)
            V = ml.Tensor((36, tiles, chans), dtype)
            M = ml.Tensor((36, tiles, chans), dtype)
            V2 = ml.Tensor((36, tiles, chans), dtype)
            M.zeroall(ctx)
            shape = "cfg2 layer at B=%d 15x15 C=256 f16" % batch
            oshape = (batch, board, board, chans)
            self.row("small", "winograd_input_transform", shape, lambda: ml.winogradInputTransform(ctx, wshape, x, V), s * (pix * chans + 36 * tiles * chans))
            self.row("small", "gemm_batched (36 x T x C x C)", shape, lambda: ml.gemmBatched(ctx, "n", "t", M, V, U, 1.0, 0.0),
                     s * 36 * (2 * tiles * chans + chans * chans), 2.0 * 36 * tiles * chans * chans, dtype)
            self.row("small", "winograd_output_input_transform", shape,
                     lambda: ml.winogradOutputInputTransform(ctx, wshape, M, oshape, None, bias, None, "relu", V2), s * 2 * 36 * tiles * chans)
            self.row("small", "winograd_output_transform +res", shape, lambda: ml.winogradOutputTransform(ctx, wshape, M, y, bias, x, "relu"),
                     s * (36 * tiles * chans + 2 * pix * chans + chans))
            for t in (x, y, V, M, V2):
                t.free()
        for t in (w, bias, U):
            t.free()

    def conv(self):
        ctx, rng = self.ctx, self.rng
        batch, board, dtype, s = 512, 19, "float16", 2
        pix = batch * board * board
        for chans in (64, 128, 256, 384):
            x = _random(ctx, (batch, board, board, chans), dtype, rng)
            res = _random(ctx, (batch, board, board, chans), dtype, rng)
            y = ml.Tensor((batch, board, board, chans), dtype)
            bias = _random(ctx, (chans,), dtype, rng, 0.1)
            for k in (1, 3, 5):
                w = _random(ctx, (chans, k, k, chans), dtype, rng, (2.0 / (k * k * chans)) ** 0.5)
                shape = "cfg4 B=512 19x19 C=%d k=%d f16" % (chans, k)
                self.row("conv", "convolution_implicit_gemm_forward", shape,
                         lambda: ml.convolutionImplicitGemmForward(ctx, x, w, y, bias, res, "relu"),
                         s * (3 * pix * chans + k * k * chans * chans + chans), 2.0 * pix * chans * chans * k * k, dtype)
                w.free()
            for t in (x, res, y, bias):
                t.free()
        # the policy head of the residual networks: 1x1 convolution to one channel (a matrix-vector product)
        x = _random(ctx, (1024 * 225, 256), dtype, rng)
        w = _random(ctx, (1, 256), dtype, rng, 0.1)
        b1 = _random(ctx, (1,), dtype, rng, 0.1)
        out = ml.Tensor((1024 * 225, 1), dtype)
        self.row("conv", "gemm_ex (1x1 head, N=1)", "cfg2 M=230400 K=256 f16", lambda: ml.gemm_ex(ctx, out, 1.0, "n", x, "t", w, 0.0, out, b1, "linear"),
                 s * (1024 * 225 * 257 + 256), 2.0 * 1024 * 225 * 256, dtype)
        for t in (x, w, b1, out):
            t.free()

    def int8(self):
        ctx, rng = self.ctx, self.rng
        batch, board, chans = 1024, 15, 256
        pix = batch * board * board
        x = _random(ctx, (batch, board, board, chans), "int8", rng)
        ext = _random(ctx, (batch, board, board, chans), "int8", rng)
        y = ml.Tensor((batch, board, board, chans), "int8")
        scales = ml.toDevice(ctx, (rng.random(chans, dtype=np.float32) * 1e-4 + 1e-5), "float32")
        bias = _random(ctx, (chans,), "float32", rng, 0.1)
        for k in (3, 1):
            w = _random(ctx, (chans, k, k, chans), "int8", rng)
            shape = "cfg3 B=1024 15x15 C=256 k=%d i8" % k
            ops = 2.0 * pix * chans * chans * k * k
            self.row("int8", "quantized_conv_forward", shape,
                     lambda: ml.quantizedConvForward(ctx, x, (0.02, 0.0), w, scales, bias, y, (0.03, 0.0), None, (1.0, 0.0), "relu"),
                     2 * pix * chans + k * k * chans * chans + 8 * chans, ops, "int8")
            self.row("int8", "quantized_conv_forward +res", shape,
                     lambda: ml.quantizedConvForward(ctx, x, (0.02, 0.0), w, scales, bias, y, (0.03, 0.0), ext, (0.05, 0.0), "relu"),
                     3 * pix * chans + k * k * chans * chans + 8 * chans, ops, "int8")
            w.free()
        # the reference's three-call form: im2row (int8), int8 GEMM to int32, requantisation
        acc = ml.Tensor((pix, chans), "int32")
        rows = ml.Tensor((pix, 9 * chans), "int8")
        w = _random(ctx, (chans, 9 * chans), "int8", rng)
        self.row("int8", "im2row (int8, k=3)", "cfg3 B=1024 15x15 C=256", lambda: ml.im2row(ctx, rows, x, 3, False, 0), pix * chans * 10)
        self.row("int8", "gemm (int8 -> int32)", "cfg3 M=230400 N=256 K=2304", lambda: ml.gemm(ctx, "n", "t", acc, rows, w, 1.0, 0.0),
                 pix * 9 * chans + 9 * chans * chans + 4 * pix * chans, 2.0 * pix * chans * 9 * chans, "int8")
        self.row("int8", "quantized_scale_shift_act", "cfg3 [230400, 256] i32 -> i8",
                 lambda: ml.quantized_scale_shift_act(ctx, y.view((pix, chans)), (0.03, 0.0), acc, scales, bias, "relu", ext.view((pix, chans)), (0.05, 0.0)),
                 pix * chans * 6 + 8 * chans)
        for t in (x, ext, y, scales, bias, acc, rows, w):
            t.free()

    def misc(self):
        ctx, rng = self.ctx, self.rng
        batch, board, chans, dtype, s = 1024, 15, 256, "float16", 2
        pix = batch * board * board
        x = _random(ctx, (batch, board, board, chans), dtype, rng)
        z = _random(ctx, (batch, board, board, chans), dtype, rng)
        y = ml.Tensor((batch, board, board, chans), dtype)
        bias = _random(ctx, (chans,), dtype, rng, 0.1)
        shape = "cfg2 [1024,15,15,256] f16"
        self.row("misc", "add_bias_act (relu)", shape, lambda: ml.addBiasAct(ctx, 1.0, x, bias, 0.0, y, "relu"), s * 2 * pix * chans)
        self.row("misc", "activation_forward (sigmoid)", shape, lambda: ml.activationForward(ctx, 1.0, x, 0.0, y, "sigmoid"), s * 2 * pix * chans)
        self.row("misc", "add_tensors (x1 + x2)", shape, lambda: ml.addTensors(ctx, 1.0, x, 1.0, z, 0.0, None, 0.0, y), s * 3 * pix * chans)
        x32 = ml.Tensor((batch, board, board, chans), "float32")
        self.row("misc", "convert_type (f16 -> f32)", shape, lambda: ml.convertType(ctx, x32, x), 6 * pix * chans)
        packed = ml.toDevice(ctx, rng.integers(0, 2 ** 32, (batch, board, board), dtype=np.uint32).view(np.int32), "int32")
        planes = ml.Tensor((batch, board, board, 32), dtype)
        self.row("misc", "unpack_input (32 planes)", "cfg2 [1024,15,15] u32 -> f16", lambda: ml.unpackInput(ctx, planes, packed), pix * (4 + 64))
        small = _random(ctx, (128, 19, 19, 64), dtype, rng)
        rows = ml.Tensor((128 * 361, 25 * 64), dtype)
        self.row("misc", "im2row (k=5)", "B=128 19x19 C=64 f16", lambda: ml.im2row(ctx, rows, small, 5, False, None), s * 128 * 361 * 64 * 26)
        for t in (x, z, y, bias, x32, packed, planes, small, rows):
            t.free()


    def heads(self):
        ctx, rng = self.ctx, self.rng
        batch, board, chans, dtype, s = 1024, 15, 256, "float16", 2
        pix = batch * board * board
        x = _random(ctx, (batch, board, board, chans), dtype, rng)
        y = ml.Tensor((batch, board, board, chans), dtype)
        pooled = ml.Tensor((batch, chans), dtype)
        gamma = _random(ctx, (chans,), dtype, rng, 0.1)
        bias = _random(ctx, (chans,), dtype, rng, 0.1)
        stats = ml.toDevice(ctx, np.stack([rng.standard_normal(chans), rng.random(chans) + 0.5]).astype(np.float32), "float32")
        shape = "cfg2 [1024,15,15,256] f16"
        self.row("heads", "global_average_pooling_forward", shape, lambda: ml.globalAveragePoolingForward(ctx, 1.0, x, 0.0, pooled),
                 s * (pix * chans + batch * chans))
        self.row("heads", "batchnorm_inference (relu)", shape, lambda: ml.batchnormInference(ctx, 1.0, x, gamma, bias, stats, 0.0, y, "relu"),
                 s * 2 * pix * chans)
        logits = _random(ctx, (batch, board * board), dtype, rng, 3.0)
        policy = ml.Tensor((batch, board * board), dtype)
        self.row("heads", "softmax_forward (policy)", "cfg2 [1024,225] f16", lambda: ml.softmaxForward(ctx, policy, logits), s * 2 * batch * board * board)
        many = _random(ctx, (pix, chans), dtype, rng, 3.0)
        self.row("heads", "softmax_forward (256 columns)", "[230400,256] f16", lambda: ml.softmaxForward(ctx, y, many), s * 2 * pix * chans)
        for t in (x, y, pooled, gamma, bias, stats, logits, policy, many):
            t.free()

    def transformer(self):
        """The hybrid configuration's transformer block pieces: 256 images of 225 tokens, 8 heads of 32, fp16 (and the same in fp32)."""
        ctx, rng = self.ctx, self.rng
        batch, board, heads, head_dim = 256, 15, 8, 32
        tokens, emb = board * board, heads * head_dim
        for dtype, s in (("float16", 2), ("float32", 4)):
            tag = "cfg5 B=256 15x15 8x32 " + ("f16" if s == 2 else "f32")
            x = _random(ctx, (batch, board, board, emb), dtype, rng)
            y = ml.Tensor((batch, board, board, emb), dtype)
            gamma = _random(ctx, (emb,), dtype, rng)
            self.row("transf.", "rmsnorm_forward", tag, lambda: ml.rmsnormForward(ctx, x, y, gamma), s * 2 * batch * tokens * emb)
            qkv = _random(ctx, (batch, board, board, 3 * emb), dtype, rng)
            table = _random(ctx, (heads, 2 * board - 1, 32), dtype, rng)
            flops = 4.0 * batch * heads * tokens * tokens * head_dim  # q k^T and p v
            self.row("transf.", "multi_head_attention_forward", tag, lambda: ml.multiHeadAttentionForward(ctx, qkv, y, table, None, None, None, heads, False),
                     s * 4 * batch * tokens * emb, flops, dtype)
            for t in (x, y, gamma, qkv, table):
                t.free()

    def moe(self):
        """The hybrid configuration's mixture-of-experts half-block: 256 images of 225 tokens, 256 channels, 8 experts of hidden width
        1024, capacity factor 2 (56 slots per expert and image), fp16."""
        ctx, rng = self.ctx, self.rng
        batch, board, emb, experts, hidden, dtype, s = 256, 15, 256, 8, 1024, "float16", 2
        tokens = board * board
        tmp = int(2.0 * tokens / experts)
        capacity = tmp if tmp * experts >= tokens else tmp + 1
        tag = "cfg5 B=256 225 tokens C=256 E=8 K=%d f16" % capacity
        x = _random(ctx, (batch, board, board, emb), dtype, rng)
        scores = _random(ctx, (batch, board, board, experts), dtype, rng)
        table = ml.Tensor((batch, 2, experts, capacity), dtype)
        gathered = ml.Tensor((batch, capacity, experts, emb), dtype)
        mid = ml.Tensor((batch, capacity, experts, hidden), dtype)
        out = ml.Tensor((batch, capacity, experts, emb), dtype)
        y = ml.Tensor((batch, board, board, emb), dtype)
        w1 = _random(ctx, (experts, hidden, emb), dtype, rng, 0.02)
        b1 = _random(ctx, (experts, hidden), dtype, rng, 0.01)
        w2 = _random(ctx, (experts, emb, hidden), dtype, rng, 0.02)
        b2 = _random(ctx, (experts, emb), dtype, rng, 0.01)
        rows = batch * capacity * experts
        self.row("moe", "expert_choice_routing_forward", tag, lambda: ml.expertChoiceRoutingForward(ctx, scores, table),
                 s * (batch * tokens * experts + 2 * batch * experts * capacity))
        self.row("moe", "gather_tokens_forward", tag, lambda: ml.gatherTokensForward(ctx, x, table, 0.0, gathered), s * (batch * tokens * emb + rows * emb))
        self.row("moe", "moe_forward (256 -> 1024, relu)", tag, lambda: ml.moeForward(ctx, gathered, w1, b1, 0.0, mid, "relu"),
                 s * (rows * emb + rows * hidden + experts * hidden * emb), 2.0 * rows * emb * hidden, dtype)
        self.row("moe", "moe_forward (1024 -> 256, linear)", tag, lambda: ml.moeForward(ctx, mid, w2, b2, 0.0, out, "linear"),
                 s * (rows * emb + rows * hidden + experts * hidden * emb), 2.0 * rows * emb * hidden, dtype)
        self.row("moe", "scatter_tokens_forward", tag, lambda: ml.scatterTokensForward(ctx, out, table, 0.0, y), s * (rows * emb + batch * tokens * emb))
        self.row("moe", "scatter_tokens_forward (beta = 1)", tag, lambda: ml.scatterTokensForward(ctx, out, table, 1.0, y),
                 s * (rows * emb + 2 * batch * tokens * emb))
        for t in (x, scores, table, gathered, mid, out, y, w1, b1, w2, b2):
            t.free()

    def ceilings(self):
        """Plain streams and a pure MFMA loop: the ceilings the other groups' rows can be read against."""
        ctx = self.ctx
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libminml_ceilings.so")
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: build it with `python3 kernel_bench.py --build-ceilings`" % path)
        raw = ctypes.CDLL(path)
        vp = ctypes.c_void_p
        raw.ceil_last_error.restype = ctypes.c_char_p

        class Checked:
            """The probe library's entry points return 0 or -1 (message from ceil_last_error): a failure raises here."""

            def __init__(self, **argtypes):
                for name, types in argtypes.items():
                    fn = getattr(raw, name)
                    fn.argtypes, fn.restype = types, ctypes.c_int
                    setattr(self, name, self._wrap(name, fn))

            @staticmethod
            def _wrap(name, fn):
                def call(*args):
                    if fn(*args) != 0:
                        raise RuntimeError("%s: %s" % (name, raw.ceil_last_error().decode()))
                return call

        lib = Checked(ceil_stream=[vp, vp, vp, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int],
                      ceil_mfma=[vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int],
                      ceil_fused_layer_operand_stream=[vp, vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                       ctypes.c_int, ctypes.POINTER(ctypes.c_size_t)])
        stream = ctx.stream()
        mib = 1 << 20

        def report(name, shape, t, nbytes):
            gbs = nbytes / t / 1e9
            r = {"group": "ceilings", "kernel": name, "shape": shape, "us": t * 1e6, "bound": "hbm", "achieved": gbs, "unit": "GB/s",
                 "peak": PEAK["hbm"] / 1e9, "frac": gbs / (PEAK["hbm"] / 1e9), "algorithmic_MB": nbytes / 1e6, "algorithmic_Gop": 0.0}
            self.rows.append(r)
            print("%-9s %-34s %-34s %9.1f us  %-4s %9.1f %-7s  %5.1f %%" % ("ceilings", name, shape, r["us"], "hbm", gbs, "GB/s", 100 * r["frac"]),
                  flush=True)

        for size_mib, where in ((16, "fits the L2s"), (64, "fits the last-level cache"), (128, "fits the last-level cache"), (1024, "HBM")):
            nbytes = size_mib * mib
            a = ml.Tensor((nbytes,), "uint8")
            b = ml.Tensor((nbytes,), "uint8")
            a.zeroall(ctx)
            b.zeroall(ctx)
            wgs = 2048
            shape = "%d MiB, %s" % (size_mib, where)
            for nt in (0, 1):
                tag = " (non-temporal)" if nt else ""
                report("read stream" + tag, shape, self.time(lambda: lib.ceil_stream(stream, None, a.ptr, nbytes, 0, nt, wgs)), nbytes)
                report("write stream" + tag, shape, self.time(lambda: lib.ceil_stream(stream, b.ptr, None, nbytes, 1, nt, wgs)), nbytes)
                report("copy stream (read + write)" + tag, shape, self.time(lambda: lib.ceil_stream(stream, b.ptr, a.ptr, nbytes, 2, nt, wgs)), 2 * nbytes)
            if size_mib == 1024:
                # the same streams cut into 16 KiB pieces, one per workgroup, handed out in address order: at any moment the resident
                # workgroups cover one dense window of memory instead of 2048 separate positions
                fine = nbytes // (16 * 1024)
                for nt in (0, 1):
                    tag = " (non-temporal)" if nt else ""
                    shape = "%d MiB, HBM, 16 KiB per workgroup" % size_mib
                    report("read stream" + tag, shape, self.time(lambda: lib.ceil_stream(stream, None, a.ptr, nbytes, 0, nt, fine)), nbytes)
                    report("write stream" + tag, shape, self.time(lambda: lib.ceil_stream(stream, b.ptr, None, nbytes, 1, nt, fine)), nbytes)
                    report("copy stream (read + write)" + tag, shape, self.time(lambda: lib.ceil_stream(stream, b.ptr, a.ptr, nbytes, 2, nt, fine)),
                           2 * nbytes)
            a.free()
            b.free()
        # producer -> consumer chains: launch i reads what launch i-1 wrote; three buffers in rotation
        for size_mib in (32, 64, 512):
            nbytes = size_mib * mib
            bufs = [ml.Tensor((nbytes,), "uint8") for _ in range(3)]
            for t in bufs:
                t.zeroall(ctx)
            state = {"i": 0}

            def step():
                i = state["i"]
                lib.ceil_stream(stream, bufs[(i + 1) % 3].ptr, bufs[i % 3].ptr, nbytes, 2, 0, 2048)
                state["i"] = i + 1

            report("copy chain over 3 buffers", "3 x %d MiB" % size_mib, self.time(step), 2 * nbytes)
            for t in bufs:
                t.free()
        # operand delivery of a one-kernel Winograd layer at the 20 x 256 network's shape (16384 tiles, 256 -> 256 channels, fp16)
        tiles, columns = 16384, 256
        v = ml.Tensor((36 * tiles * 512,), "uint8")
        u = ml.Tensor((36 * columns * 512,), "uint8")
        v.zeroall(ctx)
        u.zeroall(ctx)
        for from_x in (0, 1):  # A operand fetched as transformed rows, or as the pixels a workgroup would transform itself
            for group, width in ((32, 64), (64, 32)):
                moved = ctypes.c_size_t(0)
                t = self.time(lambda: lib.ceil_fused_layer_operand_stream(stream, v.ptr, u.ptr, tiles, columns, group, width, 256, from_x, ctypes.byref(moved)))
                report("one-kernel Winograd layer: operands" + (", A from pixels" if from_x else ""),
                       "%d tiles x %d columns x 36 per task" % (group, width), t, moved.value)
        v.free()
        u.free()
        out8 = ml.Tensor((4096,), "uint8")
        iters, wgs = 20000, 256
        for int8, name, peak, ops_per_mfma in ((0, "v_mfma_f32_32x32x16_f16", PEAK["float16"], 2.0 * 32 * 32 * 16),
                                                (1, "v_mfma_i32_32x32x32_i8", PEAK["int8"], 2.0 * 32 * 32 * 32),
                                                (2, "v_mfma_f32_32x32x2_f32", PEAK["float32"], 2.0 * 32 * 32 * 2)):
            for random in (0, 1):
                t = self.time(lambda: lib.ceil_mfma(stream, out8.ptr, iters, random, int8, wgs))
                ticks = out8.copyToHost(ctx).view(np.uint64)
                clock_ghz = float(ticks[0]) / max(1.0, float(ticks[1])) * 0.1
                ops = ops_per_mfma * 16 * iters * 4 * wgs
                rate = ops / t
                r = {"group": "ceilings", "kernel": name + " loop", "shape": "%s operands, %d CUs x 4 wavefronts" % ("random" if random else "constant", wgs),
                     "us": t * 1e6, "bound": "mfma", "achieved": rate / 1e12, "unit": "TOP/s" if int8 == 1 else "TFLOP/s", "peak": peak / 1e12,
                     "frac": rate / peak, "algorithmic_MB": 0.0, "algorithmic_Gop": ops / 1e9, "shader_clock_GHz": clock_ghz}
                self.rows.append(r)
                print("%-9s %-34s %-34s %9.1f us  %-4s %9.1f %-7s  %5.1f %%  shader clock %.2f GHz" % (
                    "ceilings", r["kernel"], r["shape"], r["us"], "mfma", r["achieved"], r["unit"], 100 * r["frac"], clock_ghz), flush=True)
        out8.free()


def library(reps):
    """Yardstick, not part of the backend: what the vendor's GEMM library (hipBLASLt / rocBLAS as PyTorch calls them) reaches on PLAIN dense
    products of the shapes that the implicit-GEMM convolutions and expert layers reduce to, random operands, no gather, no epilogue.
    Needs PyTorch; prints a note and returns when it is not importable. Runs in a process that has not loaded the backend library (PyTorch
    brings a HIP runtime of its own)."""
    try:
        import torch
    except ImportError:
        print("library   (PyTorch is not importable: no library yardstick)", flush=True)
        return
    dev = "cuda"
    torch.manual_seed(0)

    def row(name, M, N, K, dtype):
        if dtype == "int8":
            a = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=dev)
            b = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=dev)
            fn = lambda: torch._int_mm(a, b)
        else:
            a = torch.randn(M, K, dtype=torch.float16, device=dev)
            b = torch.randn(N, K, dtype=torch.float16, device=dev) * 0.05
            fn = lambda: torch.matmul(a, b.t())
        fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            fn()
        end.record()
        torch.cuda.synchronize()
        t = start.elapsed_time(end) / reps * 1e-3
        ops = 2.0 * M * N * K
        peak = PEAK[dtype]
        r = {"group": "library", "kernel": name, "shape": "M=%d N=%d K=%d %s" % (M, N, K, "i8" if dtype == "int8" else "f16"), "us": t * 1e6,
             "bound": "mfma", "achieved": ops / t / 1e12, "unit": "TOP/s" if dtype == "int8" else "TFLOP/s", "peak": peak / 1e12,
             "frac": ops / t / peak, "algorithmic_MB": 0.0, "algorithmic_Gop": ops / 1e9}
        print("%-9s %-34s %-34s %9.1f us  %-4s %9.1f %-7s  %5.1f %%" % ("library", name, r["shape"], r["us"], "mfma", r["achieved"], r["unit"],
                                                                        100 * r["frac"]), flush=True)

    row("torch.matmul (cfg4 3x3 C=256 as GEMM)", 184832, 256, 2304, "float16")
    row("torch.matmul (cfg4 5x5 C=256 as GEMM)", 184832, 256, 6400, "float16")
    row("torch.matmul (cfg4 3x3 C=384 as GEMM)", 184832, 384, 3456, "float16")
    row("torch.matmul (cfg5 expert layer 1)", 114688, 1024, 256, "float16")
    row("torch.matmul (cfg5 expert layer 2)", 114688, 256, 1024, "float16")
    row("torch.matmul (square)", 8192, 8192, 8192, "float16")
    row("torch._int_mm (cfg3 3x3 C=256 as GEMM)", 230400, 256, 2304, "int8")
    row("torch._int_mm (square)", 8192, 8192, 8192, "int8")

    # the same for memory streams: PyTorch's own copy and element-wise kernels on tensors beyond the last-level cache
    def stream_row(name, fn, nbytes):
        fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            fn()
        end.record()
        torch.cuda.synchronize()
        t = start.elapsed_time(end) / reps * 1e-3
        print("%-9s %-34s %-34s %9.1f us  %-4s %9.1f %-7s  %5.1f %%" % ("library", name, "%d MiB moved per call" % (nbytes >> 20), t * 1e6, "hbm",
                                                                        nbytes / t / 1e9, "GB/s", 100 * nbytes / t / PEAK["hbm"]), flush=True)
    n = 1 << 29  # halfs: 1 GiB per tensor
    x = torch.randn(n, dtype=torch.float16, device=dev)
    y = torch.empty_like(x)
    z = torch.randn(n, dtype=torch.float16, device=dev)
    stream_row("torch copy_ (1 GiB -> 1 GiB)", lambda: y.copy_(x), 2 * n * 2)
    stream_row("torch add (2 x 1 GiB -> 1 GiB)", lambda: torch.add(x, z, out=y), 3 * n * 2)
    stream_row("torch relu_ in place (1 GiB)", lambda: torch.relu_(y), 2 * n * 2)
    stream_row("torch sum (1 GiB read)", lambda: x.sum(), n * 2)
    stream_row("torch fill_ (1 GiB written)", lambda: y.fill_(1.0), n * 2)



def streams(steps=10):
    """The 20 x 256 fp16 network on several contexts (HIP streams) of the one device, every stream with its own network object and
    workspace: a batch of 1024 positions split into 2 or 4 equal parts, or two whole batches of 1024 in flight at once. While one stream's
    launch starts up or drains, another's is in its steady state. Prints wall-clock positions per second (repeated rows show drift)."""
    import time
    from minml_amd.resnet import ResNet, make_input, make_parameters
    to_storage = lambda a: np.ascontiguousarray(a, np.float32).astype(np.float16).view(np.uint16)
    params = make_parameters(1, 32, 256, 20)
    x = to_storage(make_input(1, 1024, 15, 32))
    for parts, per in ((1, 1024), (2, 512), (4, 256), (2, 1024), (2, 512), (1, 1024), (2, 1024)):
        contexts = [ml.Context(0) for _ in range(parts)]
        nets = [ResNet(c, per, 15, 32, 256, 20, "float16", params, to_storage, fused=True) for c in contexts]
        for i, net in enumerate(nets):
            net.setInput(x[(i * per) % 1024:(i * per) % 1024 + per])
        def one_pass():
            for net in nets:
                net.forward()
        for _ in range(3):
            one_pass()
        for c in contexts:
            c.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            one_pass()
        for c in contexts:
            c.synchronize()
        dt = (time.perf_counter() - t0) / steps
        print("streams   cfg2 network, %d x %4d positions on %d stream(s): %7.3f ms per round of passes, %7.0f positions/s"
              % (parts, per, parts, dt * 1e3, parts * per / dt), flush=True)
        del nets, contexts


def latency(reps=50):
    """The 20 x 256 fp16 network at small batches (1 ... 512 positions per pass): wall-clock time of a pass issued call by call from
    this Python mirror, and of the same pass recorded once and replayed as one HIP graph (hip_graph_*). Below about 128 positions a
    pass is a chain of dependent launches of a few microseconds each; the replay removes the host's share of it."""
    import time
    from minml_amd.resnet import ResNet, make_input, make_parameters
    to_storage = lambda a: np.ascontiguousarray(a, np.float32).astype(np.float16).view(np.uint16)
    params = make_parameters(1, 32, 256, 20)
    ctx = ml.Context(0)
    for batch in (1, 8, 32, 64, 128, 256, 512):
        net = ResNet(ctx, batch, 15, 32, 256, 20, "float16", params, to_storage, fused=True)
        net.setInput(to_storage(make_input(1, batch, 15, 32)))
        n = reps if batch <= 128 else max(1, reps // 5)

        def timed(fn):
            for _ in range(3):
                fn()
            ctx.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                fn()
            ctx.synchronize()
            return (time.perf_counter() - t0) / n
        eager = timed(net.forward)
        graph = ml.Graph.record(ctx, net.forward)
        replayed = timed(graph.launch)
        graph.destroy()
        print("latency   cfg2 network, %4d positions per pass: call by call %7.3f ms, recorded and replayed %7.3f ms (%7.0f -> %7.0f positions/s)"
              % (batch, eager * 1e3, replayed * 1e3, batch / eager, batch / replayed), flush=True)
        del net


def build_ceilings(verbose=False):
    """Compiles ceilings.hip (beside this file) into libminml_ceilings.so (beside this file) for gfx950, with the backend's flags."""
    import subprocess
    from minml_amd.build import COMMON, hipcc

    here = os.path.dirname(os.path.abspath(__file__))
    out = os.path.join(here, "libminml_ceilings.so")
    cmd = [hipcc()] + COMMON + ["-shared", os.path.join(here, "ceilings.hip"), "-o", out]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), res.stdout))
    if verbose:
        print("built", out)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--build-ceilings", action="store_true", help="compile the probe kernels of the ceilings group and exit")
    ap.add_argument("--group", default="all", choices=["all", "winograd", "small", "conv", "int8", "misc", "heads", "transformer", "moe", "ceilings", "library", "streams", "latency"])
    ap.add_argument("--reps", type=int, default=10)
    ap.add_argument("--json", action="store_true", help="print one JSON object per row after the table")
    args = ap.parse_args()
    if args.build_ceilings:
        build_ceilings(verbose=True)
        return 0
    if args.group == "latency":  # only on request: whole passes at small batches, wall-clock
        latency()
        return 0
    if args.group == "streams":  # only on request: whole passes on several streams, wall-clock
        streams()
        return 0
    if args.group == "library":  # only on request: a yardstick that needs PyTorch
        print("%-9s %-34s %-34s %12s  %-4s %9s %-7s  %7s" % ("group", "entry point", "shape", "time", "bnd", "achieved", "", "of peak"))
        library(args.reps)
        return 0
    bench = Bench(args.reps)
    print("%-9s %-34s %-34s %12s  %-4s %9s %-7s  %7s" % ("group", "entry point", "shape", "time", "bnd", "achieved", "", "of peak"))
    for group in ("winograd", "small", "conv", "int8", "misc", "heads", "transformer", "moe", "ceilings"):
        if args.group in ("all", group):
            getattr(bench, group)()
    if args.json:
        for r in bench.rows:
            print(json.dumps(r))
    return 0


if __name__ == "__main__":
    sys.exit(main())
