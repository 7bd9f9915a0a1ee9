"""CPU execution of the synthetic residual network, layer by layer, for checking and for the CPU-baseline timing.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py). Two engines with one interface:
  * engine="oracle":     this repository's C restatement (oracle.c), optionally multi-threaded;
  * engine="reference":  the reference's own CPU backend compiled into oracle/_ref (single-threaded, as the reference runs it:
                         its GEMM has no threading and the OpenMP pragmas of its input / output transforms are commented out,
                         src/backend/cpu/winograd/winograd_runtime.cpp:121,133,180,198).
Both run every 3x3 convolution as Winograd F(4x4,3x3): weight transform (cached) -> input transform -> 36 batched GEMMs ('n','t')
-> output transform with bias, residual and ReLU; the 1x1 head is gemm_ex on the [B*H*W, C] view — the call sequence of
src/layers/Conv2D.cpp:329-378.
"""
import time

import numpy as np

import oracle as O


class CpuResNet:
    def __init__(self, params_storage, blocks, engine="oracle"):
        """params_storage: list of (weights, bias) already in the storage type (float32 arrays or uint16 fp16 bit patterns)."""
        self.blocks = blocks
        self.params = params_storage
        self.engine = engine
        self.ref = O.reference() if engine == "reference" else None
        if engine == "reference" and self.ref is None:
            raise RuntimeError("oracle/_ref is not built")
        e = self.ref if self.ref is not None else O
        self.transformed = [e.winograd_weight_transform(w) if w.shape[1] == 3 else None for (w, _) in params_storage]

    def _conv3x3(self, idx, x, add, act):
        w, b = self.params[idx]
        e = self.ref if self.ref is not None else O
        v = e.winograd_input_transform(x)
        if self.ref is not None:
            m = self.ref.gemm_batched(v, self.transformed[idx])
        else:
            m = O.gemm(v, self.transformed[idx])
        shape = x.shape[:3] + (w.shape[0],)
        return e.winograd_output_transform(m, shape, b, add, act)

    def forward(self, x, return_trunk=False, per_layer=None):
        """per_layer (a list) receives the output of every 3x3 layer in order (stem, then two per block)."""
        a = self._conv3x3(0, x, None, O.RELU)
        if per_layer is not None:
            per_layer.append(a)
        for blk in range(self.blocks):
            t = self._conv3x3(1 + 2 * blk, a, None, O.RELU)
            a = self._conv3x3(2 + 2 * blk, t, a, O.RELU)
            if per_layer is not None:
                per_layer.extend([t, a])
        w, b = self.params[-1]
        rows = a.shape[0] * a.shape[1] * a.shape[2]
        am = a.reshape(rows, a.shape[3])
        wm = w.reshape(w.shape[0], -1)
        if self.ref is not None:
            head = self.ref.gemm_ex(am, wm, bias=b, act=O.LINEAR)
        else:
            head = O.gemm(am, wm, bias=b, act=O.LINEAR)
        head = head.reshape(a.shape[:3] + (w.shape[0],))
        return (head, a) if return_trunk else head

    def timed_forward(self, x, repeats=1):
        """Seconds per forward pass (best of `repeats`, after the weight transforms that __init__ already did)."""
        best = None
        for _ in range(repeats):
            t0 = time.perf_counter()
            self.forward(x)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return best


class CpuQuantizedResNet:
    """The int8 form of the same network on the oracle's restatement of the reference's integer branch (src/layers/Conv2D.cpp:240-308):
    every layer is oracle.int8_conv2d_forward with the layer's quantised weights, per-channel scales, folded bias and the three affine
    transforms (input, residual, output). `layers` is a list of (q_weights, scales, bias, in_qd, ext_qd, out_qd), stem first, head last;
    the head returns fp32."""

    def __init__(self, layers, blocks):
        self.layers = layers
        self.blocks = blocks

    def _conv(self, idx, x, ext, act, out_dtype=O.INT8):
        q, scales, bias, in_qd, ext_qd, out_qd = self.layers[idx]
        return O.int8_conv2d_forward(x, in_qd, q, scales, bias, out_dtype, out_qd, ext, ext_qd, act)

    def forward(self, x_int8, per_layer=None):
        a = self._conv(0, x_int8, None, O.RELU)
        if per_layer is not None:
            per_layer.append(a)
        for blk in range(self.blocks):
            t = self._conv(1 + 2 * blk, a, None, O.RELU)
            a = self._conv(2 + 2 * blk, t, a, O.RELU)
            if per_layer is not None:
                per_layer.extend([t, a])
        return self._conv(len(self.layers) - 1, a, None, O.LINEAR, O.FLOAT32)


class CpuHybridNet:
    """CPU execution of the hybrid network's layers that have a CPU implementation in the reference: the residual trunk (as CpuResNet,
    without its head), then attention half-blocks (RMS normalisation -> dense qkv -> multi-head attention with the relative-position
    table -> dense output with the residual as the product's C operand), then the 1x1 head. `params` has the layout of
    minml_amd.hybridnet.make_hybrid_parameters, already in the storage type. per_layer (a dict) receives every intermediate tensor."""

    def __init__(self, params_storage, blocks, heads):
        self.params = params_storage
        self.blocks = blocks
        self.heads = heads
        self.trunk = CpuResNet(params_storage["trunk"] + [params_storage["head"]], blocks, "oracle")

    def attention_block(self, x, p, per_layer=None, index=0):
        b, h, w, c = x.shape
        rows = b * h * w
        normed = O.rmsnorm_forward(x, p["gamma"])
        qkv = O.gemm(normed.reshape(rows, c), p["w_qkv"], bias=p["b_qkv"], act=O.LINEAR).reshape(b, h, w, 3 * c)
        att = O.multi_head_attention_forward(qkv, self.heads, p["table"], False)
        out = O.gemm(att.reshape(rows, c), p["w_out"], beta=1.0, C=x.reshape(rows, c), bias=p["b_out"], act=O.LINEAR).reshape(b, h, w, c)
        if per_layer is not None:
            per_layer.update({"rmsnorm%d" % index: normed, "qkv%d" % index: qkv, "attention%d" % index: att, "block%d" % index: out})
        return out

    def ffn_block(self, x, p, capacity, per_layer=None, index=0, table=None):
        """The mixture-of-experts half-block (oracle/moe.py). `table` overrides the routing table computed here (used to follow the
        device's choice where two tokens' scores are too close for two different summation orders to agree on their order)."""
        from oracle import moe as M

        b, h, w, c = x.shape
        rows = b * h * w
        normed = O.rmsnorm_forward(x, p["gamma"])
        experts = np.asarray(p["w_router"]).shape[0]
        scores = O.gemm(normed.reshape(rows, c), p["w_router"], bias=p["b_router"], act=O.LINEAR).reshape(b, h, w, experts)
        own_table = M.expert_choice_routing(scores, capacity)
        used = own_table if table is None else table
        gathered = M.gather_tokens(normed, used)
        hidden = M.moe_forward(gathered, p["w_1"], p["b_1"], O.RELU)
        out = M.moe_forward(hidden, p["w_2"], p["b_2"], O.LINEAR)
        y = M.scatter_tokens(out, used, x.shape, beta=1.0, y=x)  # the residual addition rides on the scatter (one rounding)
        if per_layer is not None:
            per_layer.update({"ffn_rmsnorm%d" % index: normed, "scores%d" % index: scores, "table%d" % index: own_table, "hidden%d" % index: hidden,
                              "experts%d" % index: out, "ffn%d" % index: y})
        return y

    def forward(self, x, per_layer=None, moe_capacity=None, tables=None):
        """moe_capacity: slots per expert; None leaves the mixture-of-experts half-blocks out. tables: optional list of routing tables
        (one per block) to use instead of the ones computed here."""
        _, a = self.trunk.forward(x, return_trunk=True)
        if per_layer is not None:
            per_layer["trunk"] = a
        for index, p in enumerate(self.params["attention"]):
            a = self.attention_block(a, p, per_layer, index)
            if moe_capacity is not None:
                a = self.ffn_block(a, self.params["ffn"][index], moe_capacity, per_layer, index, None if tables is None else tables[index])
        w, b = self.params["head"]
        rows = a.shape[0] * a.shape[1] * a.shape[2]
        head = O.gemm(a.reshape(rows, a.shape[3]), w.reshape(w.shape[0], -1), bias=b, act=O.LINEAR)
        return head.reshape(a.shape[:3] + (w.shape[0],))
