"""Writes tests/golden/reference_vectors.npz: inputs and the outputs that the reference's own CPU backend produces for them.

Run in a container where the reference checkout is mounted and `make -C oracle ref` has compiled its CPU backend into
oracle/_ref/libminml_cpu_ref.so (this script calls that library through its cpu_* C entry points; it imports nothing from the
reference). The fixtures let the oracle and the HIP backend be checked against reference results on machines where the reference is
absent. fp16 tensors are stored as uint16 bit patterns. Inputs follow the reference tests' deterministic fill sin(i/10 + shift) * scale
(src/utils/testing_util.cpp:36-55) so that the vectors are reproducible without any random generator.
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
import oracle as O  # noqa: E402


def init_for_test(shape, shift, scale=1.0):
    n = int(np.prod(shape))
    i = np.arange(n, dtype=np.float32)
    return (np.sin(i / np.float32(10.0) + np.float32(shift)) * np.float32(scale)).astype(np.float32).reshape(shape)


def main():
    ref = O.reference()
    if ref is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle ref` where the reference checkout is mounted")
    out = {}
    for tag, conv in (("f32", lambda a: a), ("f16", ref_to_half(ref))):
        # Winograd F(4x4,3x3) on an awkward shape: edge tiles, channel counts that are no multiple of any vector width
        w = conv(init_for_test((13, 3, 3, 19), 0.0))
        x = conv(init_for_test((2, 9, 11, 19), 1.0))
        bias = conv(init_for_test((13,), 1.0))
        ext = conv(init_for_test((2, 9, 11, 13), 2.0))
        wm = ref.winograd_weight_transform(w)
        v = ref.winograd_input_transform(x)
        m = ref.gemm_batched(v, wm)
        y = ref.winograd_output_transform(m, (2, 9, 11, 13), bias, ext, O.RELU)
        # (no bias-less case: with bias == NULL and a channel count that is not a multiple of 16 the reference's AVX-512 tail loop adds whatever
        # its bias register held before — src/backend/cpu/winograd/avx512f_winograd_kernels.cpp UNROLLED1 lacks the vxorps of UNROLLED16)
        y_lin = ref.winograd_output_transform(m, (2, 9, 11, 13), bias, None, O.LINEAR)
        out.update({"wg_w_" + tag: w, "wg_x_" + tag: x, "wg_bias_" + tag: bias, "wg_ext_" + tag: ext, "wg_wm_" + tag: wm, "wg_v_" + tag: v,
                    "wg_m_" + tag: m, "wg_y_relu_" + tag: y, "wg_y_linear_" + tag: y_lin,
                    "wg_wm_inverted_" + tag: ref.winograd_weight_transform(w, True)})
        # gemm_ex 'n','t' with alpha, beta, bias, ReLU (test/backend/test_gemms.cpp sizes) and one K > 1024
        a = conv(init_for_test((23, 67), 0.0))
        b = conv(init_for_test((45, 67), 1.0))
        c = conv(init_for_test((23, 45), 2.0))
        gb = conv(init_for_test((45,), 3.0))
        out.update({"ge_a_" + tag: a, "ge_b_" + tag: b, "ge_c_" + tag: c, "ge_bias_" + tag: gb,
                    "ge_d_" + tag: ref.gemm_ex(a, b, alpha=1.1, beta=0.1, C=c, bias=gb, act=O.RELU)})
        a2 = conv(init_for_test((9, 1200), 0.5, 0.1))
        b2 = conv(init_for_test((7, 1200), 1.5, 0.1))
        out.update({"gk_a_" + tag: a2, "gk_b_" + tag: b2, "gk_d_" + tag: ref.gemm_ex(a2, b2)})
        # 5x5 convolution as im2row + gemm_ex with bias, residual, ReLU (test/backend/test_conv2D.cpp:332-368 pattern)
        cx = conv(init_for_test((2, 7, 6, 8), 1.0))
        cw = conv(init_for_test((12, 5, 5, 8), 0.0, 0.2))
        cb = conv(init_for_test((12,), 1.0))
        ca = conv(init_for_test((2, 7, 6, 12), 2.0))
        out.update({"cv_x_" + tag: cx, "cv_w_" + tag: cw, "cv_bias_" + tag: cb, "cv_add_" + tag: ca, "cv_rows_" + tag: ref.im2row(cx, 5),
                    "cv_y_" + tag: ref.conv2d_forward(cx, cw, cb, ca, O.RELU)})
        out["ab_y_" + tag] = ref.add_bias_act(cx, conv(init_for_test((8,), 0.3)), O.TANH)
        # after the trunk: policy softmax (225 logits), win / draw / loss softmax, global average pooling (136 = 2 x 64 + 8 channels: the
        # reference's vector kernels only; 7 channels: its scalar kernel, which divides by the pixel count instead of multiplying)
        sx = conv(init_for_test((6, 225), 0.0, 3.0))
        s3 = conv(init_for_test((5, 3), 1.0, 2.0))
        px = conv(init_for_test((2, 13, 14, 136), 0.0))
        p7 = conv(init_for_test((2, 5, 5, 7), 1.0))
        out.update({"sm_x_" + tag: sx, "sm_y_" + tag: ref.softmax_forward(sx), "sm3_x_" + tag: s3, "sm3_y_" + tag: ref.softmax_forward(s3),
                    "gap_x_" + tag: px, "gap_y_" + tag: ref.global_average_pooling_forward(px),
                    "gap7_x_" + tag: p7, "gap7_y_" + tag: ref.global_average_pooling_forward(p7)})
    # batch normalisation folded into a convolution [10,3,3,6] and into depthwise weights [3,3,12] (the reference folds in fp32 only)
    for key, wshape, channels in (("fd", (10, 3, 3, 6), 10), ("fd3", (3, 3, 12), 12)):
        fw, fb = init_for_test(wshape, 0.0), init_for_test((channels,), 1.0)
        gamma, beta = init_for_test((channels,), 2.0) + np.float32(1.5), init_for_test((channels,), 3.0)
        stats = np.stack([init_for_test((channels,), 4.0), np.abs(init_for_test((channels,), 5.0)) + np.float32(0.1)])
        folded_w, folded_b = ref.fold_batchnorm(fw, fb, gamma, beta, stats)
        out.update({key + "_w": fw, key + "_b": fb, key + "_gamma": gamma, key + "_beta": beta, key + "_stats": stats, key + "_w_out": folded_w,
                    key + "_b_out": folded_b})
    # transformer-block pieces (the reference computes them in fp32 only): RMS normalisation with and without gamma; attention over a
    # 5x7 board with 4 heads of 8 and a 5x5 position table (clamping active: offsets reach +-6), without table, and in the symmetric layout
    rx, rg = init_for_test((9, 100), 0.0, 2.0), init_for_test((100,), 1.0) + np.float32(1.0)
    out.update({"rms_x": rx, "rms_g": rg, "rms_y": ref.rmsnorm_forward(rx, rg), "rms_y_plain": ref.rmsnorm_forward(rx)})
    ax, at = init_for_test((2, 5, 7, 96), 0.0, 1.5), init_for_test((4, 5, 8), 1.0)
    ax2 = init_for_test((2, 4, 4, 64), 2.0, 1.5)
    out.update({"mha_x": ax, "mha_table": at, "mha_y": ref.multi_head_attention_forward(ax, 4, at),
                "mha_y_plain": ref.multi_head_attention_forward(ax, 4), "mha_sym_x": ax2, "mha_sym_y": ref.multi_head_attention_forward(ax2, 2)})
    # bit-plane unpacking and fp32 -> fp16 narrowing
    packed = (np.arange(3 * 5 * 2, dtype=np.uint64) * 2654435761 % (1 << 32)).astype(np.uint32)
    out["up_packed"] = packed
    out["up_f32"] = ref.unpack_input(packed, (3, 5, 40), O.FLOAT32)
    out["up_f16"] = ref.unpack_input(packed, (3, 5, 40), O.FLOAT16)
    src = np.concatenate([init_for_test((500,), 0.0, 3.0), np.array([0.0, -0.0, 65504.0, 65519.9, 1e-8, -1e-8, 6.0e-5, 5.9e-8, 1.0009765], np.float32)])
    out["cvt_src"] = src
    out["cvt_f16"] = ref.convert(src, O.FLOAT16)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


def ref_to_half(ref):
    return lambda a: ref.convert(np.ascontiguousarray(a, np.float32), O.FLOAT16)


if __name__ == "__main__":
    main()
