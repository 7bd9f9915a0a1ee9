/*
 * conv.hip — fused convolution forward and im2row for fp16 / fp32 NHWC tensors.
 *
 * hip_convolution_implicit_gemm_forward computes y = act(conv(x, w) + bias + add) with stride 1, zero padding (k-1)/2 and weights
 * [Cout, k, k, Cin]. The reference has this entry point only as a cuDNN / cuBLASLt call (src/backend/cuda/cudnn_math.cpp:374-476) and
 * an empty CPU stub (src/backend/cpu/dispatcher.cpp:249-252); what it must compute is fixed by the reference's own explicit path,
 * explicit_gemm_forward (src/core/math.cpp:1595-1626) = cpu_im2row (src/backend/cpu/conv_im2row.cpp:21-59) followed by gemm_ex('n','t')
 * with beta = 1 on `add` (src/backend/cpu/gemm/gemm.cpp:66-83), equivalently baseline_conv2D_forward in test/backend/test_conv2D.cpp:22-59.
 *
 * On gfx950 the im2row matrix is never written: the MFMA tile engine reads its A operand through an address generator that maps
 * (row = pixel, 16-byte chunk of k) to the input tensor or to padding. 1x1 convolutions are plain GEMMs on the [B*H*W, Cin] view.
 * Channel counts whose rows are not 16-byte multiples fall back to a direct one-thread-per-output kernel.
 */
#include "common.hpp"
#include "gemm_core.hpp"
#include "epilogues.hpp"
#include "gemm_launch.hpp"
#include "gemm_dma.hpp"
#include "conv_window.hpp"
#include "gemm_dma_window.hpp"

#include <algorithm>
#include <cstring>

namespace
{
	using namespace mlhip;

	template<typename T, typename Cfg, typename Epilogue>
	__global__ __launch_bounds__(Cfg::THREADS) void kernel_conv_implicit_gemm(Im2RowRows<T> a_loader, const T *weights, int M, int N, int k_bytes,
			Epilogue epilogue, int tiles_n)
	{
		__shared__ __attribute__((aligned(16))) uint8_t lds[Cfg::LDS_BYTES];
		const unsigned int linear = xcd_contiguous_block_id(blockIdx.x, gridDim.x);
		const int tile_m = linear / tiles_n;
		const int tile_n = linear % tiles_n;
		DenseRows<T> b_loader { weights, N, k_bytes };
		gemm_tile<T, Cfg>(a_loader, b_loader, M, k_bytes, tile_m * Cfg::BM, tile_n * Cfg::BN, lds, epilogue);
	}

	/* Fallback for channel counts the tile engine does not take: one thread per output element. */
	template<typename T>
	__global__ __launch_bounds__(256) void kernel_conv_direct(const T *input, const T *weights, T *output, const T *bias, const T *add, int act,
			int batch, int height, int width, int filters_in, int filters_out, int kernel_h, int kernel_w)
	{
		const size_t total = static_cast<size_t>(batch) * height * width * filters_out;
		const size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
		if (gid >= total)
			return;
		const int out = static_cast<int>(gid % filters_out);
		size_t rest = gid / filters_out;
		const int w = static_cast<int>(rest % width);
		rest /= width;
		const int h = static_cast<int>(rest % height);
		const int b = static_cast<int>(rest / height);
		const int pad_h = (kernel_h - 1) / 2, pad_w = (kernel_w - 1) / 2;

		float acc = 0.0f;
		for (int i = 0; i < kernel_h; i++)
			for (int j = 0; j < kernel_w; j++)
			{
				const int x = h + i - pad_h, y = w + j - pad_w;
				if (x >= 0 && x < height && y >= 0 && y < width)
				{
					const T *src = input + ((static_cast<size_t>(b) * height + x) * width + y) * filters_in;
					const T *wgt = weights + ((static_cast<size_t>(out) * kernel_h + i) * kernel_w + j) * filters_in;
					for (int c = 0; c < filters_in; c++)
						acc += Storage<T>::load(src + c) * Storage<T>::load(wgt + c);
				}
			}
		FloatEpilogue<T> ep;
		ep.D = output;
		ep.C = add;
		ep.bias = bias;
		ep.N = out + 1;
		ep.row_stride = filters_out;
		ep.alpha = 1.0f;
		ep.beta = (add != nullptr) ? 1.0f : 0.0f;
		ep.act = act;
		ep.vectorized = false;
		const float vals[4] = { acc, 0.0f, 0.0f, 0.0f };
		ep(static_cast<int>(gid / filters_out), out, vals);
	}

	/* output [B*H*W][k*k*C] <- input [B][H][W][C]; one thread per 16-byte (or single-element) piece of an output row */
	template<typename V>
	__global__ __launch_bounds__(256) void kernel_im2row(const V *input, V *output, int batch, int height, int width, int vecs_per_pixel, int kernel_size,
			bool invert, V padding)
	{
		const int taps = kernel_size * kernel_size;
		const size_t total = static_cast<size_t>(batch) * height * width * taps * vecs_per_pixel;
		const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
		const int pad = (kernel_size - 1) / 2;
		for (size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < total; gid += stride)
		{
			int c, tap, w, h;
			size_t rest = split_index(gid, vecs_per_pixel, c);
			rest = split_index(rest, taps, tap);
			rest = split_index(rest, width, w);
			const int b = static_cast<int>(split_index(rest, height, h));
			const int i = tap / kernel_size, j = tap % kernel_size;
			const int x = h - pad + (invert ? (kernel_size - 1 - i) : i);
			const int y = w - pad + (invert ? (kernel_size - 1 - j) : j);
			V value = padding;
			if (x >= 0 && x < height && y >= 0 && y < width)
				value = input[((static_cast<size_t>(b) * height + x) * width + y) * vecs_per_pixel + c];
			output[gid] = value;
		}
	}

	/* the same for tensors of fewer than 2^32 pieces, with the four divisions as multiplications (the run-time divisions above are most of
	 * that kernel's instructions: 180 us for the int8 rows of 1024 x 15 x 15 x 256, 590 MB) */
	template<typename V>
	__global__ __launch_bounds__(256) void kernel_im2row_fast(const V *input, V *output, uint32_t total, int height, int width, FastDivisor vecs_per_pixel,
			FastDivisor taps, FastDivisor by_width, FastDivisor by_height, FastDivisor by_kernel, bool invert, V padding)
	{
		constexpr int UNROLL = 4; /* pieces per thread in flight: with one, the launch waits out a memory latency per 32 KB and compute unit */
		const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
		const int kernel_size = static_cast<int>(by_kernel.divisor);
		const int pad = (kernel_size - 1) / 2;
		for (uint64_t first = blockIdx.x * blockDim.x + threadIdx.x; first < total; first += UNROLL * stride)
		{
			V value[UNROLL];
#pragma unroll
			for (int u = 0; u < UNROLL; u++)
			{
				value[u] = padding;
				const uint64_t index = first + u * stride;
				if (index < total)
				{
					uint32_t c, tap, w, h, j;
					uint32_t rest = fast_divide(static_cast<uint32_t>(index), vecs_per_pixel, c);
					rest = fast_divide(rest, taps, tap);
					rest = fast_divide(rest, by_width, w);
					const uint32_t b = fast_divide(rest, by_height, h);
					const int i = static_cast<int>(fast_divide(tap, by_kernel, j));
					const int x = static_cast<int>(h) - pad + (invert ? (kernel_size - 1 - i) : i);
					const int y = static_cast<int>(w) - pad + (invert ? (kernel_size - 1 - static_cast<int>(j)) : static_cast<int>(j));
					if (x >= 0 && x < height && y >= 0 && y < width)
						value[u] = input[((static_cast<size_t>(b) * height + x) * width + y) * vecs_per_pixel.divisor + c];
				}
			}
#pragma unroll
			for (int u = 0; u < UNROLL; u++)
			{
				const uint64_t index = first + u * stride;
				if (index < total)
					output[index] = value[u];
			}
		}
	}

	bool aligned16(const void *p)
	{
		return (reinterpret_cast<uintptr_t>(p) % 16) == 0;
	}

	template<typename T>
	void conv_forward(hipStream_t stream, mlDataType_t dtype, const mlShape_t &in, const mlShape_t &ws, const void *input, const void *weights,
			void *output, const void *bias, const void *add, mlActivationType_t act)
	{
		const int batch = in.dim[0], height = in.dim[1], width = in.dim[2], filters_in = in.dim[3];
		const int filters_out = ws.dim[0], kernel_h = ws.dim[1], kernel_w = ws.dim[2];
		const size_t pixels = static_cast<size_t>(batch) * height * width;
		MLHIP_REQUIRE(pixels <= 0x7fffffffu, "convolution: too many pixels for one launch");
		const int M = static_cast<int>(pixels);

		if (kernel_h == 1 && kernel_w == 1)
		{ /* the [B*H*W, Cin] view of the input is the GEMM operand itself */
			GemmArgs g;
			g.dtype = dtype;
			g.transpose_a = false;
			g.transpose_b = true;
			g.M = M;
			g.N = filters_out;
			g.K = filters_in;
			g.A = input;
			g.B = weights;
			g.C = add;
			g.D = output;
			g.bias = bias;
			g.alpha = 1.0f;
			g.beta = (add != nullptr) ? 1.0f : 0.0f;
			g.act = act;
			launch_gemm(stream, g);
			return;
		}

		const size_t c_bytes = static_cast<size_t>(filters_in) * sizeof(T);
		const size_t k_bytes = c_bytes * kernel_h * kernel_w;
		const bool fast = (c_bytes % 16 == 0) && aligned16(input) && aligned16(weights) && k_bytes <= 0x7fffffffu;
		const auto make_epilogue = [&]()
		{
			FloatEpilogue<T> ep;
			ep.D = reinterpret_cast<T*>(output);
			ep.C = reinterpret_cast<const T*>(add);
			ep.bias = reinterpret_cast<const T*>(bias);
			ep.N = filters_out;
			ep.row_stride = filters_out;
			ep.alpha = 1.0f;
			ep.beta = (add != nullptr) ? 1.0f : 0.0f;
			ep.act = act;
			const size_t vbytes = 4 * sizeof(T);
			ep.vectorized = (filters_out % 4 == 0) && (reinterpret_cast<uintptr_t>(output) % vbytes == 0) && (reinterpret_cast<uintptr_t>(add) % vbytes == 0)
					&& (reinterpret_cast<uintptr_t>(bias) % vbytes == 0);
			return ep;
		};
		if constexpr (sizeof(T) == 2)
		{
			/* a narrow 3x3 layer (64 filters in and out) is bound by HBM: every input pixel through LDS once, the weights in registers */
			const FloatEpilogue<T> ep = make_epilogue();
			/* the forms that specialise_epilogue fixes at compile time: bias with ReLU or no activation, or the bare product */
			const bool fixed_form = ep.vectorized && ((ep.bias != nullptr && (ep.act == ACTIVATION_RELU || ep.act == ACTIVATION_LINEAR))
					|| (ep.bias == nullptr && ep.beta == 0.0f && ep.act == ACTIVATION_LINEAR));
			if (fast && fixed_form && aligned16(output) && aligned16(add) && conv_window_applies(sizeof(T), filters_in, filters_out, kernel_h, kernel_w, height, width, pixels))
			{
				specialise_epilogue(ep, [&](const auto &fixed)
				{
					if constexpr (!std::is_same<typename std::decay<decltype(fixed)>::type, FloatEpilogue<T>>::value)
						launch_conv_window<T>(stream, input, weights, M, height, width, fixed);
				});
				MLHIP_CHECK(hipGetLastError());
				return;
			}
			/* 64 -> 64 filters 5 x 5: the same with the K axis split among the wavefronts */
			if (fast && fixed_form && aligned16(output) && aligned16(add)
					&& conv_window_split_applies<ConvSplit5x5x64>(sizeof(T), filters_in, filters_out, kernel_h, kernel_w, height, width, pixels))
			{
				specialise_epilogue(ep, [&](const auto &fixed)
				{
					if constexpr (!std::is_same<typename std::decay<decltype(fixed)>::type, FloatEpilogue<T>>::value)
						launch_conv_window_split<T, ConvSplit5x5x64>(stream, input, weights, M, height, width, fixed);
				});
				MLHIP_CHECK(hipGetLastError());
				return;
			}
		}
		if (fast && c_bytes % 128 == 0)
		{ /* every 128-byte chunk of K lies within one tap: the direct-to-LDS engine */
			Im2RowDmaRows a_loader;
			a_loader.base = reinterpret_cast<const uint8_t*>(input);
			a_loader.rows = M;
			a_loader.height = height;
			a_loader.width = width;
			a_loader.kernel_h = kernel_h;
			a_loader.kernel_w = kernel_w;
			a_loader.c_bytes = static_cast<int>(c_bytes);
			a_loader.fill = 0;
			const DenseDmaRows b_loader { reinterpret_cast<const uint8_t*>(weights), filters_out, static_cast<int>(k_bytes) };
			if constexpr (sizeof(T) == 2)
				if (conv_dma_window_applies(c_bytes, filters_out, kernel_h, kernel_w, height, width))
				{ /* the tiles' rows are consecutive pixels: the window of pixels they share enters LDS once per 128-byte slice of the channels */
					specialise_epilogue(make_epilogue(), [&](const auto &ep)
					{
						launch_conv_dma_window<T>(stream, input, weights, M, filters_out, height, width, kernel_h, static_cast<int>(c_bytes), 0u, ep);
					});
					MLHIP_CHECK(hipGetLastError());
					return;
				}
			if constexpr (sizeof(T) == 2) /* the fp16 hot path gets its epilogue's common cases fixed at compile time */
				specialise_epilogue(make_epilogue(), [&](const auto &ep)
				{
					launch_gemm_dma<T>(stream, a_loader, b_loader, M, filters_out, static_cast<int>(k_bytes), 1, 0, 0, 0, ep);
				});
			else
				launch_gemm_dma<T>(stream, a_loader, b_loader, M, filters_out, static_cast<int>(k_bytes), 1, 0, 0, 0, make_epilogue());
		}
		else if (fast)
		{
			typedef TileConfig<128, 128, 64, 2, 2> Cfg;
			Im2RowRows<T> a_loader;
			a_loader.base = reinterpret_cast<const T*>(input);
			a_loader.rows = M;
			a_loader.height = height;
			a_loader.width = width;
			a_loader.kernel_h = kernel_h;
			a_loader.kernel_w = kernel_w;
			a_loader.c_bytes = static_cast<int>(c_bytes);
			a_loader.k_bytes = static_cast<int>(k_bytes);
			a_loader.fill = 0u;
			const FloatEpilogue<T> ep = make_epilogue();

			const int tiles_m = ceil_div(M, Cfg::BM), tiles_n = ceil_div(filters_out, Cfg::BN);
			const dim3 grid(static_cast<unsigned int>(tiles_m) * tiles_n);
			hipLaunchKernelGGL((kernel_conv_implicit_gemm<T, Cfg, FloatEpilogue<T>>), grid, dim3(Cfg::THREADS), 0, stream, a_loader,
					reinterpret_cast<const T*>(weights), M, filters_out, static_cast<int>(k_bytes), ep, tiles_n);
		}
		else
		{
			const size_t outputs = pixels * filters_out;
			MLHIP_REQUIRE((outputs + 255) / 256 <= 0x7fffffffu, "convolution: output too large for one launch");
			hipLaunchKernelGGL(kernel_conv_direct<T>, dim3(static_cast<unsigned int>((outputs + 255) / 256)), dim3(256), 0, stream,
					reinterpret_cast<const T*>(input), reinterpret_cast<const T*>(weights), reinterpret_cast<T*>(output), reinterpret_cast<const T*>(bias),
					reinterpret_cast<const T*>(add), static_cast<int>(act), batch, height, width, filters_in, filters_out, kernel_h, kernel_w);
		}
		MLHIP_CHECK(hipGetLastError());
	}

	template<typename V>
	void launch_im2row(hipStream_t stream, const void *input, void *output, int batch, int height, int width, int vecs_per_pixel, int kernel_size,
			bool invert, V padding)
	{
		const size_t total = static_cast<size_t>(batch) * height * width * kernel_size * kernel_size * vecs_per_pixel;
		if (total == 0)
			return;
		const size_t blocks = (total + 255) / 256;
		const unsigned int grid = static_cast<unsigned int>(blocks < (1u << 20) ? blocks : (1u << 20));
		if (total <= 0xffffffffu)
			hipLaunchKernelGGL(kernel_im2row_fast<V>, dim3(static_cast<unsigned int>(std::min<size_t>((blocks + 3) / 4, 1u << 20))), dim3(256), 0, stream, reinterpret_cast<const V*>(input), reinterpret_cast<V*>(output),
					static_cast<uint32_t>(total), height, width, make_fast_divisor(vecs_per_pixel), make_fast_divisor(kernel_size * kernel_size),
					make_fast_divisor(width), make_fast_divisor(height), make_fast_divisor(kernel_size), invert, padding);
		else
			hipLaunchKernelGGL(kernel_im2row<V>, dim3(grid), dim3(256), 0, stream, reinterpret_cast<const V*>(input), reinterpret_cast<V*>(output), batch,
					height, width, vecs_per_pixel, kernel_size, invert, padding);
		MLHIP_CHECK(hipGetLastError());
	}
}

extern "C"
{
	using namespace mlhip;

	void hip_convolution_implicit_gemm_forward(mlContext_t context, mlDataType_t dtype, mlShape_t input_shape, mlShape_t weights_shape,
			const void *input, const void *weights, void *output, const void *bias, const void *add, mlActivationType_t act)
	try
	{
		MLHIP_REQUIRE(input_shape.rank == 4 && weights_shape.rank == 4, "convolution: input must be [B,H,W,Cin] and weights [Cout,k,k,Cin]");
		MLHIP_REQUIRE(input_shape.dim[3] == weights_shape.dim[3], "convolution: input and weights disagree on the number of input filters");
		MLHIP_REQUIRE(dtype == DTYPE_FLOAT16 || dtype == DTYPE_FLOAT32, "convolution: unsupported data type");
		if (volume(input_shape) == 0 || weights_shape.dim[0] == 0)
			return;
		MLHIP_REQUIRE(input != nullptr && weights != nullptr && output != nullptr, "convolution: null tensor");
		if (dtype == DTYPE_FLOAT16)
			conv_forward<half_t>(stream_of(context), dtype, input_shape, weights_shape, input, weights, output, bias, add, act);
		else
			conv_forward<float>(stream_of(context), dtype, input_shape, weights_shape, input, weights, output, bias, add, act);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}

	void hip_im2row(mlContext_t context, mlDataType_t dtype, mlShape_t input_shape, void *output, const void *input, int kernel_size, bool invert,
			const void *padding)
	try
	{
		MLHIP_REQUIRE(input_shape.rank == 4, "im2row: input must be [B,H,W,C]");
		MLHIP_REQUIRE(kernel_size >= 1, "im2row: kernel size must be positive");
		const int esize = size_of(dtype);
		MLHIP_REQUIRE(esize == 1 || esize == 2 || esize == 4 || esize == 8, "im2row: unsupported data type");
		const int batch = input_shape.dim[0], height = input_shape.dim[1], width = input_shape.dim[2], channels = input_shape.dim[3];
		if (volume(input_shape) == 0)
			return;
		MLHIP_REQUIRE(input != nullptr && output != nullptr, "im2row: null tensor");

		uint8_t pad[16] = { 0 };
		if (padding != nullptr)
			for (int i = 0; i < 16; i += esize)
				std::memcpy(pad + i, padding, esize);

		const size_t c_bytes = static_cast<size_t>(channels) * esize;
		if (c_bytes % 16 == 0 && aligned16(input) && aligned16(output))
		{
			uint4_t p;
			std::memcpy(&p, pad, 16);
			launch_im2row<uint4_t>(stream_of(context), input, output, batch, height, width, static_cast<int>(c_bytes / 16), kernel_size, invert, p);
		}
		else
			switch (esize)
			{
				case 1:
				{
					uint8_t p;
					std::memcpy(&p, pad, 1);
					launch_im2row<uint8_t>(stream_of(context), input, output, batch, height, width, channels, kernel_size, invert, p);
					break;
				}
				case 2:
				{
					uint16_t p;
					std::memcpy(&p, pad, 2);
					launch_im2row<uint16_t>(stream_of(context), input, output, batch, height, width, channels, kernel_size, invert, p);
					break;
				}
				case 4:
				{
					uint32_t p;
					std::memcpy(&p, pad, 4);
					launch_im2row<uint32_t>(stream_of(context), input, output, batch, height, width, channels, kernel_size, invert, p);
					break;
				}
				default:
				{
					uint64_t p;
					std::memcpy(&p, pad, 8);
					launch_im2row<uint64_t>(stream_of(context), input, output, batch, height, width, channels, kernel_size, invert, p);
					break;
				}
			}
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(convolution_implicit_gemm_forward)
MLHIP_ALSO_AS_CUDA(im2row)
