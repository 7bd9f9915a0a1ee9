"""Per-kernel roofline table of the convolution / GEMM path on one MI355X:  python3 -m minml_amd.kernel_bench [--group NAME] [--json]

Every row launches one entry point of the library on synthetic tensors of a benchmark configuration's shape (resident in HBM), times
`--reps` launches with two events on the context's stream, and prices the launch with its ALGORITHMIC work: the bytes every
implementation must move (inputs once, outputs once) and the flops / integer ops of the algorithm. The bound of a row is whichever of
the two takes longer at the chip's peaks (HBM 8 TB/s; dense MFMA fp16 2.5 PFLOP/s, int8 5.0 POP/s, fp32 157.3 TFLOP/s); `frac` is the
achieved fraction of that peak.

Groups: winograd (transforms and batched GEMM at the residual-network shapes), conv (implicit-GEMM sweep: 19x19 boards, batch 512,
channels 64..384, kernels 1 / 3 / 5, bias + residual + ReLU), int8 (quantised 3x3 convolution at 256 channels and its three-call form),
misc (im2row, element-wise neighbours), heads (softmax, global average pooling, batch normalisation in inference mode), transformer
(RMS normalisation and multi-head attention at the hybrid configuration's shape).
"""
import argparse
import json
import sys

import numpy as np

from . import core as ml

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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--group", default="all", choices=["all", "winograd", "conv", "int8", "misc", "heads", "transformer"])
    ap.add_argument("--reps", type=int, default=10)
    ap.add_argument("--json", action="store_true", help="print one JSON object per row after the table")
    args = ap.parse_args()
    bench = Bench(args.reps)
    print("%-9s %-34s %-34s %12s  %-4s %9s %-7s  %7s" % ("group", "entry point", "shape", "time", "bnd", "achieved", "", "of peak"))
    for group in ("winograd", "conv", "int8", "misc", "heads", "transformer"):
        if args.group in ("all", group):
            getattr(bench, group)()
    if args.json:
        for r in bench.rows:
            print(json.dumps(r))
    return 0


if __name__ == "__main__":
    sys.exit(main())
