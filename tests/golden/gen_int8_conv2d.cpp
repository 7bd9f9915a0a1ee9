/*
 * gen_int8_conv2d.cpp — records what the reference itself computes for an int8 convolution layer: quantize_weights
 * (src/layers/quantization.cpp:55-93, called by Layer::setupQuantization, src/layers/Layer.cpp:147-160) and the integer branch of
 * Conv2D::forward on the CPU (src/layers/Conv2D.cpp:240-308). Linked against the reference's own objects (oracle/Makefile, target
 * `fixtures`); driven by tests/golden/make_int8_fixtures.py, which writes the case file and stores the answers as .npz.
 *
 *   gen_int8_conv2d <case.bin> <result.bin>
 *
 * case.bin:   int32 { batch, height, width, cin, cout, kernel, activation (0 linear, 1 sigmoid, 2 tanh, 3 relu, 5 exp), has_ext, int8_output }
 *             float { in_scale, in_shift, out_scale, out_shift, ext_scale, ext_shift }
 *             float weights [cout, k, k, cin], float bias [cout], int8 input [b, h, w, cin], int8 ext [b, h, w, cout] (if has_ext)
 * result.bin: int8 quantized weights [cout, k, k, cin], float channel_scales [cout], float folded bias [cout],
 *             output [b, h, w, cout] as int8 (int8_output) or float
 */
#include <minml/core/Context.hpp>
#include <minml/core/Tensor.hpp>
#include <minml/layers/Conv2D.hpp>
#include <minml/layers/quantization.hpp>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <memory>
#include <stdexcept>
#include <vector>

using namespace ml;

template<typename T>
static void read_into(std::ifstream &f, T *dst, size_t count)
{
	f.read(reinterpret_cast<char*>(dst), static_cast<std::streamsize>(count * sizeof(T)));
	if (!f)
		throw std::runtime_error("case file too short");
}
template<typename T>
static void write_from(std::ofstream &f, const T *src, size_t count)
{
	f.write(reinterpret_cast<const char*>(src), static_cast<std::streamsize>(count * sizeof(T)));
}

int main(int argc, char **argv)
{
	if (argc != 3)
	{
		std::fprintf(stderr, "usage: %s case.bin result.bin\n", argv[0]);
		return 2;
	}
	try
	{
		std::ifstream in(argv[1], std::ios::binary);
		int32_t h[9];
		float q[6];
		read_into(in, h, 9);
		read_into(in, q, 6);
		const int batch = h[0], height = h[1], width = h[2], cin = h[3], cout = h[4], kernel = h[5], act = h[6];
		const bool has_ext = h[7] != 0, int8_output = h[8] != 0;
		static const char *names[] = { "linear", "sigmoid", "tanh", "relu", "leaky_relu", "gelu" }; /* the reference spells ActivationType::EXP "gelu" (src/layers/Layer.cpp:108-109) */
		const AffineTransform in_t(q[0], q[1]), out_t(q[2], q[3]), ext_t(q[4], q[5]);

		std::shared_ptr<Context> context = std::make_shared<Context>(Device::cpu());
		Conv2D layer(cout, kernel, names[act]);
		const Shape in_shape( { batch, height, width, cin }), out_shape( { batch, height, width, cout });
		if (has_ext)
			layer.setInputShape(std::vector<Shape> { in_shape, out_shape });
		else
			layer.setInputShape(std::vector<Shape> { in_shape });
		layer.changeContext(context);
		Tensor &weights = layer.getWeights().getParam();
		Tensor &bias = layer.getBias().getParam();
		read_into(in, reinterpret_cast<float*>(weights.data()), static_cast<size_t>(weights.volume()));
		read_into(in, reinterpret_cast<float*>(bias.data()), static_cast<size_t>(bias.volume()));
		Tensor input(in_shape, "int8", Device::cpu()), ext(out_shape, "int8", Device::cpu());
		read_into(in, reinterpret_cast<int8_t*>(input.data()), static_cast<size_t>(input.volume()));
		if (has_ext)
			read_into(in, reinterpret_cast<int8_t*>(ext.data()), static_cast<size_t>(ext.volume()));

		/* the layer's own set-up discards the scales into a protected member: record them from the same public function it calls */
		const WeightQuantizer wq = quantize_weights(weights, bias, in_t, "per_first_dim", 8);
		std::vector<AffineTransform> in_transforms { in_t };
		if (has_ext)
			in_transforms.push_back(ext_t);
		layer.setupQuantization(in_transforms, out_t, 8);
		if (int8_output)
			layer.convertTo(DataType::INT8);
		if (std::memcmp(layer.getWeights().getParam().data(), wq.weights.data(), static_cast<size_t>(wq.weights.volume())) != 0)
			throw std::runtime_error("the layer's quantised weights differ from quantize_weights()");

		Tensor output(out_shape, int8_output ? "int8" : "float32", Device::cpu());
		std::vector<Tensor> inputs { input };
		if (has_ext)
			inputs.push_back(ext);
		layer.forward(inputs, output);

		std::ofstream out(argv[2], std::ios::binary);
		write_from(out, reinterpret_cast<const int8_t*>(wq.weights.data()), static_cast<size_t>(wq.weights.volume()));
		write_from(out, reinterpret_cast<const float*>(wq.channel_scales.data()), static_cast<size_t>(cout));
		write_from(out, reinterpret_cast<const float*>(wq.bias.data()), static_cast<size_t>(cout));
		if (int8_output)
			write_from(out, reinterpret_cast<const int8_t*>(output.data()), static_cast<size_t>(output.volume()));
		else
			write_from(out, reinterpret_cast<const float*>(output.data()), static_cast<size_t>(output.volume()));
		return 0;
	} catch (std::exception &e)
	{
		std::fprintf(stderr, "exception: %s\n", e.what());
		return 1;
	}
}
