/*
 * quantized.hip — the int8 inference path: per-channel requantisation of int32 accumulators and the fused int8 convolution.
 *
 * Arithmetic is that of the reference's CPU int8 convolution (src/layers/Conv2D.cpp:240-308, equal to baseline_int8_conv2D_forward
 * in test/backend/test_quantization.cpp:56-117): int32 accumulation with the input zero point on padded taps, then in fp32 and
 * without fused multiply-adds  tmp = acc * scale[o] + bias[o];  tmp += ext * s_e + sh_e;  act;  q = clamp(round(tmp / s_o - sh_o / s_o))
 * where the inverse transform (1 / s_o, -sh_o / s_o) is formed on the host in fp32 exactly as AffineTransform::get_inverse does
 * (include/minml/layers/quantization.hpp:44-47). The reference's CUDA kernel requantises with round((x - shift) / scale)
 * (src/backend/cuda/kernels/quantized.cu:44-47), which can differ at ties; the CPU form is the one reproduced here.
 *
 * hip_quantized_scale_shift_act is the stand-alone epilogue of the reference's device int8 path (int8 GEMM -> this call,
 * src/layers/Conv2D.cpp:214-239). hip_quantized_conv_forward runs the whole convolution as one int8 MFMA implicit GEMM
 * (v_mfma_i32_32x32x32_i8) with that epilogue fused, so neither the im2row matrix nor the int32 accumulators reach HBM.
 */
#include "common.hpp"
#include "gemm_core.hpp"
#include "epilogues.hpp"
#include "gemm_dma.hpp"

#include <cmath>

namespace
{
	using namespace mlhip;

	/* one thread per 4 consecutive columns of a row; FAST: fewer than 2^32 such groups, the row split by multiplication (four groups in
	 * flight per thread were measured too: 88 against 80 us for 230 400 rows of 256) */
	template<typename OutT, bool FAST>
	__global__ __launch_bounds__(256) void kernel_scale_shift_act(RequantEpilogue<OutT> epilogue, const int32_t *input, int first_dim, int last_dim,
			FastDivisor by_groups)
	{
		const int groups = (last_dim + 3) / 4;
		const size_t total = static_cast<size_t>(first_dim) * groups;
		const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
		for (size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < total; gid += stride)
		{
			int group, m;
			if constexpr (FAST)
			{
				uint32_t remainder;
				m = static_cast<int>(fast_divide(static_cast<uint32_t>(gid), by_groups, remainder));
				group = static_cast<int>(remainder);
			}
			else
				m = static_cast<int>(split_index(gid, groups, group));
			const int n = group * 4;
			const int32_t *src = input + static_cast<size_t>(m) * last_dim + n;
			int acc[4] = { 0, 0, 0, 0 };
			if (epilogue.vectorized)
			{
				const int4_t tmp = *reinterpret_cast<const int4_t*>(src);
#pragma unroll
				for (int e = 0; e < 4; e++)
					acc[e] = tmp[e];
			}
			else
			{
#pragma unroll
				for (int e = 0; e < 4; e++)
					if (n + e < last_dim)
						acc[e] = src[e];
			}
			epilogue(m, n, acc);
		}
	}

	template<typename Cfg, typename Epilogue>
	__global__ __launch_bounds__(Cfg::THREADS) void kernel_int8_conv_implicit_gemm(Im2RowRows<int8_t> a_loader, const int8_t *weights, int M, int N,
			int k_bytes, Epilogue epilogue, int tiles_n)
	{
		__shared__ __attribute__((aligned(16))) uint8_t lds[Cfg::LDS_BYTES];
		const unsigned int linear = xcd_contiguous_block_id(blockIdx.x, gridDim.x);
		const int tile_m = linear / tiles_n;
		const int tile_n = linear % tiles_n;
		DenseRows<int8_t> b_loader { weights, N, k_bytes };
		gemm_tile<int8_t, Cfg>(a_loader, b_loader, M, k_bytes, tile_m * Cfg::BM, tile_n * Cfg::BN, lds, epilogue);
	}

	/* fallback for channel counts that are not multiples of 16: one thread per output */
	template<typename Epilogue>
	__global__ __launch_bounds__(256) void kernel_int8_conv_direct(const int8_t *input, const int8_t *weights, Epilogue epilogue, int input_zero,
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

		int acc = 0;
		for (int i = 0; i < kernel_h; i++)
			for (int j = 0; j < kernel_w; j++)
			{
				const int x = h + i - pad_h, y = w + j - pad_w;
				const int8_t *wgt = weights + ((static_cast<size_t>(out) * kernel_h + i) * kernel_w + j) * filters_in;
				if (x >= 0 && x < height && y >= 0 && y < width)
				{
					const int8_t *src = input + ((static_cast<size_t>(b) * height + x) * width + y) * filters_in;
					for (int c = 0; c < filters_in; c++)
						acc += static_cast<int>(wgt[c]) * static_cast<int>(src[c]);
				}
				else
				{
					for (int c = 0; c < filters_in; c++)
						acc += static_cast<int>(wgt[c]) * input_zero;
				}
			}
		Epilogue local = epilogue;
		local.vectorized = false;
		local.N = out + 1;
		const int vals[4] = { acc, 0, 0, 0 };
		local(static_cast<int>(gid / filters_out), out, vals);
	}

	bool aligned_to(const void *p, size_t bytes)
	{
		return p == nullptr || (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
	}

	template<typename OutT>
	RequantEpilogue<OutT> make_epilogue(void *output, const void *scales, const void *bias, const void *ext, int channels, mlQuantizationData_t output_qd,
			mlQuantizationData_t ext_qd, mlActivationType_t act)
	{
		RequantEpilogue<OutT> ep;
		ep.D = reinterpret_cast<OutT*>(output);
		ep.scales = reinterpret_cast<const float*>(scales);
		ep.bias = reinterpret_cast<const float*>(bias);
		ep.ext = reinterpret_cast<const int8_t*>(ext);
		ep.N = channels;
		ep.row_stride = channels;
		ep.ext_scale = ext_qd.scale;
		ep.ext_shift = ext_qd.shift;
		/* AffineTransform::get_inverse: (1 / scale, -shift / scale), in fp32 */
		ep.inv_scale = 1.0f / output_qd.scale;
		ep.inv_shift = -output_qd.shift / output_qd.scale;
		ep.act = static_cast<int>(act);
		ep.vectorized = (channels % 4 == 0) && aligned_to(output, 4 * sizeof(OutT)) && aligned_to(scales, 16) && aligned_to(bias, 16) && aligned_to(ext, 4);
		return ep;
	}

	template<typename OutT>
	void launch_scale_shift_act(hipStream_t stream, const mlShape_t &shape, void *output, mlQuantizationData_t output_qd, const void *input,
			const void *scales, const void *bias, mlActivationType_t act, const void *ext, mlQuantizationData_t ext_qd)
	{
		const int last = last_dim(shape);
		const size_t first = volume(shape) / last;
		MLHIP_REQUIRE(first <= 0x7fffffffu, "quantized_scale_shift_act: tensor too large");
		RequantEpilogue<OutT> ep = make_epilogue<OutT>(output, scales, bias, ext, last, output_qd, ext_qd, act);
		ep.vectorized = ep.vectorized && aligned_to(input, 16);
		const size_t total = first * ((last + 3) / 4);
		const size_t blocks = (total + 255) / 256;
		const unsigned int grid = static_cast<unsigned int>(blocks < (1u << 20) ? blocks : (1u << 20));
		const FastDivisor by_groups = make_fast_divisor(static_cast<uint32_t>((last + 3) / 4));
		if (total <= 0xffffffffu)
			hipLaunchKernelGGL((kernel_scale_shift_act<OutT, true>), dim3(grid), dim3(256), 0, stream, ep, reinterpret_cast<const int32_t*>(input),
					static_cast<int>(first), last, by_groups);
		else
			hipLaunchKernelGGL((kernel_scale_shift_act<OutT, false>), dim3(grid), dim3(256), 0, stream, ep, reinterpret_cast<const int32_t*>(input),
					static_cast<int>(first), last, by_groups);
		MLHIP_CHECK(hipGetLastError());
	}

	template<typename OutT>
	void launch_quantized_conv(hipStream_t stream, const mlShape_t &in, const mlShape_t &ws, const void *input, mlQuantizationData_t input_qd,
			const void *weights, const void *scales, const void *bias, void *output, mlQuantizationData_t output_qd, const void *ext,
			mlQuantizationData_t ext_qd, mlActivationType_t act)
	{
		const int batch = in.dim[0], height = in.dim[1], width = in.dim[2], filters_in = in.dim[3];
		const int filters_out = ws.dim[0], kernel_h = ws.dim[1], kernel_w = ws.dim[2];
		const size_t pixels = static_cast<size_t>(batch) * height * width;
		MLHIP_REQUIRE(pixels <= 0x7fffffffu, "quantized convolution: too many pixels for one launch");
		const int M = static_cast<int>(pixels);

		/* get_zero<int32_t>: round((0 - shift) / scale) evaluated as 0 * (1/scale) + (-shift/scale) (quantization.hpp:39-47,57-61) */
		const float inv_scale = 1.0f / input_qd.scale;
		const float inv_shift = -input_qd.shift / input_qd.scale;
		const int input_zero = static_cast<int>(std::round(0.0f * inv_scale + inv_shift));

		RequantEpilogue<OutT> ep = make_epilogue<OutT>(output, scales, bias, ext, filters_out, output_qd, ext_qd, act);

		const size_t k_bytes = static_cast<size_t>(filters_in) * kernel_h * kernel_w;
		const bool zero_fits = (input_zero >= -128 && input_zero <= 127) || (kernel_h == 1 && kernel_w == 1);
		const bool fast = (filters_in % 16 == 0) && aligned_to(input, 16) && aligned_to(weights, 16) && k_bytes <= 0x7fffffffu && zero_fits;
		if (fast && kernel_h == 1 && kernel_w == 1 && ep.vectorized && stream_gemm_applies(M, 1, k_bytes))
		{ /* a 1x1 convolution with a short K row is bound by HBM: the persistent streaming kernel on the [B*H*W, Cin] view */
			const StreamGemmArgs sg { input, weights, nullptr, M, filters_out, static_cast<int>(k_bytes), 1, 0, 0, 0 };
			specialise_epilogue(ep, [&](const auto &fixed)
			{
				launch_stream_gemm<int8_t>(stream, sg, fixed);
			});
		}
		else if (fast && filters_in % 128 == 0)
		{ /* every 128-byte chunk of K lies within one tap: the direct-to-LDS engine */
			Im2RowDmaRows a_loader;
			a_loader.base = reinterpret_cast<const uint8_t*>(input);
			a_loader.rows = M;
			a_loader.height = height;
			a_loader.width = width;
			a_loader.kernel_h = kernel_h;
			a_loader.kernel_w = kernel_w;
			a_loader.c_bytes = filters_in;
			a_loader.fill = input_zero & 0xff; /* a 1x1 kernel never pads, so an out-of-range zero point is harmless there */
			const DenseDmaRows b_loader { reinterpret_cast<const uint8_t*>(weights), filters_out, static_cast<int>(k_bytes) };
			specialise_epilogue(ep, [&](const auto &fixed)
			{
				launch_gemm_dma<int8_t>(stream, a_loader, b_loader, M, filters_out, static_cast<int>(k_bytes), 1, 0, 0, 0, fixed);
			});
		}
		else if (fast)
		{
			typedef TileConfig<128, 128, 64, 2, 2> Cfg;
			Im2RowRows<int8_t> a_loader;
			a_loader.base = reinterpret_cast<const int8_t*>(input);
			a_loader.rows = M;
			a_loader.height = height;
			a_loader.width = width;
			a_loader.kernel_h = kernel_h;
			a_loader.kernel_w = kernel_w;
			a_loader.c_bytes = filters_in;
			a_loader.k_bytes = static_cast<int>(k_bytes);
			const uint32_t z = static_cast<uint32_t>(input_zero) & 0xffu;
			a_loader.fill = z | (z << 8) | (z << 16) | (z << 24);
			const int tiles_m = ceil_div(M, Cfg::BM), tiles_n = ceil_div(filters_out, Cfg::BN);
			hipLaunchKernelGGL((kernel_int8_conv_implicit_gemm<Cfg, RequantEpilogue<OutT>>), dim3(static_cast<unsigned int>(tiles_m) * tiles_n),
					dim3(Cfg::THREADS), 0, stream, a_loader, reinterpret_cast<const int8_t*>(weights), M, filters_out, static_cast<int>(k_bytes), ep,
					tiles_n);
		}
		else
		{
			const size_t outputs = pixels * filters_out;
			MLHIP_REQUIRE((outputs + 255) / 256 <= 0x7fffffffu, "quantized convolution: output too large for one launch");
			hipLaunchKernelGGL(kernel_int8_conv_direct<RequantEpilogue<OutT>>, dim3(static_cast<unsigned int>((outputs + 255) / 256)), dim3(256), 0,
					stream, reinterpret_cast<const int8_t*>(input), reinterpret_cast<const int8_t*>(weights), ep, input_zero, batch, height, width,
					filters_in, filters_out, kernel_h, kernel_w);
		}
		MLHIP_CHECK(hipGetLastError());
	}
}

extern "C"
{
	using namespace mlhip;

	void hip_quantized_scale_shift_act(mlContext_t context, mlDataType_t dtype, mlShape_t shape, void *output, mlQuantizationData_t output_qd,
			const void *input, const void *scales, const void *bias, mlActivationType_t act, const void *ext, mlQuantizationData_t ext_qd)
	try
	{
		MLHIP_REQUIRE(shape.rank >= 1, "quantized_scale_shift_act: empty shape");
		if (volume(shape) == 0)
			return;
		MLHIP_REQUIRE(output != nullptr && input != nullptr && scales != nullptr && bias != nullptr, "quantized_scale_shift_act: null tensor");
		switch (dtype)
		{
			case DTYPE_INT8:
				launch_scale_shift_act<int8_t>(stream_of(context), shape, output, output_qd, input, scales, bias, act, ext, ext_qd);
				break;
			case DTYPE_FLOAT32:
				launch_scale_shift_act<float>(stream_of(context), shape, output, output_qd, input, scales, bias, act, ext, ext_qd);
				break;
			case DTYPE_FLOAT16:
				launch_scale_shift_act<half_t>(stream_of(context), shape, output, output_qd, input, scales, bias, act, ext, ext_qd);
				break;
			default:
				fail_logic("HIP backend: quantized_scale_shift_act: output must be INT8, FLOAT16 or FLOAT32");
		}
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}

	void hip_quantized_conv_forward(mlContext_t context, mlShape_t input_shape, mlShape_t weights_shape, const void *input,
			mlQuantizationData_t input_qd, const void *weights, const void *scales, const void *bias, mlDataType_t output_dtype, void *output,
			mlQuantizationData_t output_qd, const void *ext, mlQuantizationData_t ext_qd, mlActivationType_t act)
	try
	{
		MLHIP_REQUIRE(input_shape.rank == 4 && weights_shape.rank == 4, "quantized convolution: input must be [B,H,W,Cin] and weights [Cout,k,k,Cin]");
		MLHIP_REQUIRE(input_shape.dim[3] == weights_shape.dim[3], "quantized convolution: input and weights disagree on the number of input filters");
		if (volume(input_shape) == 0 || weights_shape.dim[0] == 0)
			return;
		MLHIP_REQUIRE(input != nullptr && weights != nullptr && output != nullptr && scales != nullptr && bias != nullptr,
				"quantized convolution: null tensor");
		switch (output_dtype)
		{
			case DTYPE_INT8:
				launch_quantized_conv<int8_t>(stream_of(context), input_shape, weights_shape, input, input_qd, weights, scales, bias, output, output_qd, ext, ext_qd, act);
				break;
			case DTYPE_FLOAT32:
				launch_quantized_conv<float>(stream_of(context), input_shape, weights_shape, input, input_qd, weights, scales, bias, output, output_qd, ext, ext_qd, act);
				break;
			default:
				fail_logic("HIP backend: quantized convolution: output must be INT8 or FLOAT32");
		}
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(quantized_scale_shift_act)
