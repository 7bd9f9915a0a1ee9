"""Writes tests/golden/reference_int8_conv2d.npz: int8 convolution layers as the reference itself computes them.

For every case this script writes the inputs to a temporary file and runs oracle/_ref/gen_int8_conv2d (tests/golden/gen_int8_conv2d.cpp
linked against the reference's own objects by `make -C oracle fixtures`, where the reference checkout is mounted). That program calls the
reference's quantize_weights (src/layers/quantization.cpp:55-93) and the integer branch of Conv2D::forward on the CPU
(src/layers/Conv2D.cpp:240-308) and returns the quantised weights, channel scales, folded bias and the layer's output. Inputs and
answers are stored together, so the check runs where the reference is absent.

Cases cover: kernel sizes 1 / 3 / 5, with and without an int8 residual, int8 and fp32 outputs, every activation of the branch, and
asymmetric input quantisation (shift != 0, so that the padding value `input_zero` is not 0 and the folded bias differs from the bias).
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.join(HERE, "..", "..")
GENERATOR = os.path.join(ROOT, "oracle", "_ref", "gen_int8_conv2d")

# name: (batch, h, w, cin, cout, k, activation code, has_ext, int8_output, (in), (out), (ext))
CASES = {
    "k3_ext_relu_i8": (2, 7, 6, 12, 10, 3, 3, True, True, (0.05, 0.4), (0.07, -0.3), (0.06, 0.2)),
    "k3_ext_relu_f32": (2, 7, 6, 12, 10, 3, 3, True, False, (0.05, 0.4), (0.07, -0.3), (0.06, 0.2)),
    "k3_noext_relu_i8": (2, 7, 6, 12, 10, 3, 3, False, True, (0.05, -1.3), (0.04, 0.0), (1.0, 0.0)),
    "k3_symmetric_relu_i8": (1, 9, 9, 16, 16, 3, 3, True, True, (0.031, 0.0), (0.043, 0.0), (0.029, 0.0)),
    "k1_ext_relu_i8": (2, 5, 4, 36, 44, 1, 3, True, True, (0.123, 4.56), (0.078, 0.9), (0.078, -0.9)),
    "k1_ext_relu_f32": (2, 5, 4, 36, 44, 1, 3, True, False, (0.123, 4.56), (0.078, 0.9), (0.078, -0.9)),
    "k5_linear_i8": (1, 6, 7, 8, 6, 5, 0, False, True, (0.02, 0.7), (0.05, 0.1), (1.0, 0.0)),
    "k5_sigmoid_i8": (1, 6, 7, 8, 6, 5, 1, True, True, (0.02, 0.7), (0.004, 0.5), (0.01, 0.0)),
    "k3_tanh_f32": (1, 5, 5, 8, 6, 3, 2, False, False, (0.02, -0.2), (1.0, 0.0), (1.0, 0.0)),
    "k3_exp_i8": (1, 5, 5, 8, 6, 3, 5, False, True, (0.02, -0.2), (0.05, 0.0), (1.0, 0.0)),
}


def run_case(spec, seed):
    b, h, w, cin, cout, k, act, has_ext, int8_out, in_qd, out_qd, ext_qd = spec
    rng = np.random.default_rng(seed)
    weights = (rng.standard_normal((cout, k, k, cin)) * np.sqrt(2.0 / (k * k * cin))).astype(np.float32)
    bias = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    x = rng.integers(-128, 128, (b, h, w, cin)).astype(np.int8)
    ext = rng.integers(-128, 128, (b, h, w, cout)).astype(np.int8)
    with tempfile.TemporaryDirectory() as tmp:
        case, result = os.path.join(tmp, "case.bin"), os.path.join(tmp, "result.bin")
        with open(case, "wb") as f:
            f.write(np.array([b, h, w, cin, cout, k, act, int(has_ext), int(int8_out)], np.int32).tobytes())
            f.write(np.array(list(in_qd) + list(out_qd) + list(ext_qd), np.float32).tobytes())
            f.write(weights.tobytes())
            f.write(bias.tobytes())
            f.write(x.tobytes())
            if has_ext:
                f.write(ext.tobytes())
        subprocess.run([GENERATOR, case, result], check=True)
        raw = open(result, "rb").read()
    nw = weights.size
    q = np.frombuffer(raw, np.int8, nw).reshape(weights.shape)
    scales = np.frombuffer(raw, np.float32, cout, nw)
    folded = np.frombuffer(raw, np.float32, cout, nw + 4 * cout)
    out = np.frombuffer(raw, np.int8 if int8_out else np.float32, b * h * w * cout, nw + 8 * cout).reshape(b, h, w, cout)
    return {"weights": weights, "bias": bias, "x": x, "ext": ext if has_ext else np.zeros(0, np.int8), "q": q, "scales": scales, "folded_bias": folded,
            "y": out, "spec": np.array([b, h, w, cin, cout, k, act, int(has_ext), int(int8_out)], np.int32),
            "qd": np.array(list(in_qd) + list(out_qd) + list(ext_qd), np.float32)}


def main():
    if not os.path.exists(GENERATOR):
        raise SystemExit("%s is not built: run `make -C oracle fixtures` where the reference checkout is mounted" % GENERATOR)
    out = {}
    for index, (name, spec) in enumerate(sorted(CASES.items())):
        for key, value in run_case(spec, 100 + index).items():
            out[name + "/" + key] = value
    path = os.path.join(HERE, "reference_int8_conv2d.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, "(%d arrays, %d bytes)" % (len(out), os.path.getsize(path)))


if __name__ == "__main__":
    sys.exit(main())
