/*
 * cabi_network.cpp — the benchmark's residual network driven from C++ through the C-ABI only, the way minml's own layers would drive the
 * backend (reference call sequence of a Winograd layer: src/layers/Conv2D.cpp:356-378; of the 1x1 head: src/core/math.cpp:1595-1626).
 *
 *   cabi_network <parameters.bin> <input.bin> <output.bin> <batch> <board> <planes> <channels> <blocks> <mode> <timed passes>
 *
 * parameters.bin: for every layer (stem, 2 * blocks 3x3 convolutions, 1x1 head) the fp16 weights [Cout, k, k, Cin] followed by the fp16
 * bias [Cout]; input.bin: fp16 [batch, board, board, planes]; output.bin receives the fp16 head output [batch, board, board, 1].
 * mode 0 = three calls per layer (input transform, batched product, output transform), 1 = the output transform of every layer inside
 * a residual block merged with the next layer's input transform. Prints the time per pass measured between two host synchronisations.
 */
#include "../include/minml_hip_backend.h"

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <stdexcept>
#include <vector>

static mlTensor_t tensor(void *data, int rank, int d0, int d1 = 0, int d2 = 0, int d3 = 0)
{
	mlTensor_t t;
	std::memset(&t, 0, sizeof(t));
	t.data = data;
	t.dtype = DTYPE_FLOAT16;
	t.rank = rank;
	t.dim[0] = d0;
	t.dim[1] = d1;
	t.dim[2] = d2;
	t.dim[3] = d3;
	return t;
}
static mlShape_t shape(int rank, int d0, int d1 = 0, int d2 = 0, int d3 = 0)
{
	mlShape_t s;
	std::memset(&s, 0, sizeof(s));
	s.rank = rank;
	s.dim[0] = d0;
	s.dim[1] = d1;
	s.dim[2] = d2;
	s.dim[3] = d3;
	return s;
}
static std::vector<uint16_t> read_file(const char *path)
{
	std::ifstream f(path, std::ios::binary | std::ios::ate);
	if (!f)
		throw std::runtime_error(std::string("cannot open ") + path);
	const size_t bytes = static_cast<size_t>(f.tellg());
	std::vector<uint16_t> data(bytes / 2);
	f.seekg(0);
	f.read(reinterpret_cast<char*>(data.data()), static_cast<std::streamsize>(bytes));
	return data;
}

struct Layer
{
		int cout, k, cin;
		void *weights, *bias, *matrices; /* device: [Cout,k,k,Cin], [Cout], [36,Cout,Cin] (3x3 only) */
};

int main(int argc, char **argv)
{
	if (argc != 11)
	{
		std::fprintf(stderr, "usage: %s parameters.bin input.bin output.bin batch board planes channels blocks mode passes\n", argv[0]);
		return 2;
	}
	try
	{
		const int batch = std::atoi(argv[4]), board = std::atoi(argv[5]), planes = std::atoi(argv[6]), channels = std::atoi(argv[7]);
		const int blocks = std::atoi(argv[8]), mode = std::atoi(argv[9]), passes = std::atoi(argv[10]);
		const std::vector<uint16_t> parameters = read_file(argv[1]);
		const std::vector<uint16_t> input = read_file(argv[2]);
		const int tiles = batch * ((board + 3) / 4) * ((board + 3) / 4);
		const size_t pixels = static_cast<size_t>(batch) * board * board;
		if (input.size() != pixels * planes)
			throw std::runtime_error("input.bin does not match the given shape");

		mlContext_t ctx = hip_create_context(0);
		std::vector<Layer> layers;
		size_t offset = 0;
		for (int i = 0; i < 2 * blocks + 2; i++)
		{
			Layer l;
			l.cin = (i == 0) ? planes : channels;
			l.cout = (i == 2 * blocks + 1) ? 1 : channels;
			l.k = (i == 2 * blocks + 1) ? 1 : 3;
			const size_t w_elems = static_cast<size_t>(l.cout) * l.k * l.k * l.cin;
			if (offset + w_elems + l.cout > parameters.size())
				throw std::runtime_error("parameters.bin is too short");
			l.weights = hip_malloc(0, w_elems * 2);
			l.bias = hip_malloc(0, static_cast<size_t>(l.cout) * 2);
			hip_memcpy_from_host(ctx, l.weights, 0, parameters.data() + offset, w_elems * 2);
			hip_memcpy_from_host(ctx, l.bias, 0, parameters.data() + offset + w_elems, static_cast<size_t>(l.cout) * 2);
			offset += w_elems + l.cout;
			l.matrices = nullptr;
			if (l.k == 3)
			{ /* transformed once, like the reference's weight cache (Conv2D.cpp:356-363) */
				l.matrices = hip_malloc(0, static_cast<size_t>(36) * l.cout * l.cin * 2);
				hip_winograd_weight_transform(ctx, 4, tensor(l.weights, 4, l.cout, 3, 3, l.cin), tensor(l.matrices, 3, 36, l.cout, l.cin), false);
			}
			layers.push_back(l);
		}
		/* one workspace with the reference's layout: input matrices at element 0, output matrices behind them (Conv2D.cpp:365-367) */
		const size_t matrix_elems = static_cast<size_t>(36) * tiles * channels;
		uint16_t *workspace = static_cast<uint16_t*>(hip_malloc(0, (2 * matrix_elems + 1024) * 2));
		void *x = hip_malloc(0, input.size() * 2);
		void *act[3] = { hip_malloc(0, pixels * channels * 2), hip_malloc(0, pixels * channels * 2), hip_malloc(0, pixels * channels * 2) };
		void *head = hip_malloc(0, pixels * 2);
		hip_memcpy_from_host(ctx, x, 0, input.data(), input.size() * 2);

		auto input_transform = [&](const Layer &l, void *src)
		{
			hip_winograd_input_transform(ctx, 4, tensor(src, 4, batch, board, board, l.cin), tensor(workspace, 3, 36, tiles, l.cin));
		};
		auto product = [&](const Layer &l)
		{
			uint16_t *out_matrices = workspace + static_cast<size_t>(36) * tiles * l.cin;
			hip_gemm_batched_v2(ctx, 'n', 't', 1.0f, tensor(workspace, 3, 36, tiles, l.cin), tensor(l.matrices, 3, 36, l.cout, l.cin), 0.0f,
					tensor(out_matrices, 3, 36, tiles, l.cout));
		};
		auto output_transform = [&](const Layer &l, void *dst, void *residual)
		{
			uint16_t *out_matrices = workspace + static_cast<size_t>(36) * tiles * l.cin;
			hip_winograd_output_transform(ctx, 4, tensor(out_matrices, 3, 36, tiles, l.cout), tensor(l.bias, 1, l.cout),
					tensor(residual, residual ? 4 : 0, batch, board, board, l.cout), tensor(dst, 4, batch, board, board, l.cout), ACTIVATION_RELU);
		};
		auto output_into_next = [&](const Layer &l, void *dst)
		{
			uint16_t *out_matrices = workspace + static_cast<size_t>(36) * tiles * l.cin;
			hip_winograd_output_input_transform(ctx, 4, tensor(out_matrices, 3, 36, tiles, l.cout), tensor(l.bias, 1, l.cout), tensor(nullptr, 0, 0),
					shape(4, batch, board, board, l.cout), dst, ACTIVATION_RELU, tensor(workspace, 3, 36, tiles, l.cout));
		};
		auto forward = [&]()
		{
			void *a = act[0], *b = act[1], *c = act[2];
			input_transform(layers[0], x);
			product(layers[0]);
			output_transform(layers[0], a, nullptr);
			for (int blk = 0; blk < blocks; blk++)
			{
				const Layer &conv1 = layers[1 + 2 * blk], &conv2 = layers[2 + 2 * blk];
				input_transform(conv1, a);
				product(conv1);
				if (mode == 1 && channels % 64 == 0)
					output_into_next(conv1, nullptr); /* only the second convolution reads this result */
				else
				{
					output_transform(conv1, b, nullptr);
					input_transform(conv2, b);
				}
				product(conv2);
				output_transform(conv2, c, a);
				void *tmp = a;
				a = c;
				c = tmp;
			}
			const Layer &h = layers.back();
			hip_gemm_ex(ctx, DTYPE_FLOAT16, shape(2, static_cast<int>(pixels), 1), head, 1.0f, 'n', shape(2, static_cast<int>(pixels), channels), a, 't',
					shape(2, 1, channels), h.weights, 0.0f, shape(2, static_cast<int>(pixels), 1), head, h.bias, ACTIVATION_LINEAR);
		};

		forward();
		hip_synchronize_with_context(ctx);
		std::vector<uint16_t> result(pixels);
		hip_memcpy_to_host(ctx, result.data(), head, 0, pixels * 2);
		hip_synchronize_with_context(ctx);
		std::ofstream(argv[3], std::ios::binary).write(reinterpret_cast<const char*>(result.data()), static_cast<std::streamsize>(pixels * 2));

		if (passes > 0)
		{
			const auto t0 = std::chrono::steady_clock::now();
			for (int i = 0; i < passes; i++)
				forward();
			hip_synchronize_with_context(ctx);
			const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / passes;
			std::printf("C++ host, batch %d, mode %d: %.3f ms per pass, %.0f positions/s\n", batch, mode, seconds * 1e3, batch / seconds);
		}
		for (Layer &l : layers)
		{
			hip_free(l.weights);
			hip_free(l.bias);
			hip_free(l.matrices);
		}
		hip_free(workspace);
		hip_free(x);
		for (void *p : act)
			hip_free(p);
		hip_free(head);
		hip_destroy_context(ctx);
		std::printf("ALL OK\n");
		return 0;
	} catch (const std::exception &e)
	{
		std::printf("FAIL: %s\n", e.what());
		return 1;
	}
}
