/*
 * heads.hip — the steps after the convolution trunk that let a served network finish on the device: softmax over the policy logits,
 * global average pooling in front of a value head, batch normalisation in inference mode and its folding into the preceding layer.
 *
 *   softmax_forward:                 y[i, :] = exp(x[i, :] - max_i) / sum_i          reference: src/backend/cpu/avx_misc_kernels.cpp:53-112,
 *                                                                                    device form src/backend/cuda/kernels/softmax.cu:123
 *   global_average_pooling_forward:  y[b, c] = alpha * mean_hw x[b, h, w, c] + beta * y[b, c]
 *                                                                                    src/backend/cpu/kernels/pooling_and_scaling.cpp:142-180,
 *                                                                                    src/backend/cuda/kernels/global_pooling.cu:28-70,269
 *   batchnorm_inference:             y = alpha * act(x * scale + shift) + beta * y, scale = gamma / sqrt(var + 1e-6),
 *                                    shift = bias - mean * scale                     src/backend/cuda/kernels/batchnorm.cu:57-104,400
 *   fold_batchnorm:                  weights *= scale per channel, bias = bias * scale + shift, in place
 *                                                                                    src/backend/cpu/normalization.cpp:296-343,
 *                                                                                    src/backend/cuda/kernels/batchnorm.cu:357-394,606
 * All four are bandwidth bound: 16-byte accesses where the shapes allow, fp32 arithmetic, fp16 results truncated toward zero like every
 * fp16 store of the reference CPU backend.
 */
#include "common.hpp"
#include "device_utils.hpp"

#include <algorithm>
#include <cmath>

namespace
{
	using namespace mlhip;

	__device__ __forceinline__ float wave_max(float v)
	{
#pragma unroll
		for (int offset = 32; offset >= 1; offset >>= 1)
			v = fmaxf(v, __shfl_xor(v, offset));
		return v;
	}
	__device__ __forceinline__ float wave_sum(float v)
	{
#pragma unroll
		for (int offset = 32; offset >= 1; offset >>= 1)
			v += __shfl_xor(v, offset);
		return v;
	}

	/* one wavefront per row, the row held in registers: ITEMS columns per lane, lane-strided so that every access is coalesced */
	template<typename T, int ITEMS>
	__global__ __launch_bounds__(256) void kernel_softmax_in_registers(T *output, const T *input, size_t rows, int columns)
	{
		const int lane = threadIdx.x & 63;
		const size_t stride = static_cast<size_t>(gridDim.x) * 4;
		for (size_t row = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6); row < rows; row += stride)
		{
			const T *src = input + row * columns;
			T *dst = output + row * columns;
			float v[ITEMS];
			float max_value = -INFINITY;
#pragma unroll
			for (int e = 0; e < ITEMS; e++)
			{
				const int j = lane + 64 * e;
				v[e] = (j < columns) ? Storage<T>::load(src + j) : -INFINITY;
				max_value = fmaxf(max_value, v[e]);
			}
			max_value = wave_max(max_value);
			float sum = 0.0f;
#pragma unroll
			for (int e = 0; e < ITEMS; e++)
			{
				const int j = lane + 64 * e;
				v[e] = (j < columns) ? expf(v[e] - max_value) : 0.0f;
				sum += v[e];
			}
			const float scale = 1.0f / wave_sum(sum);
#pragma unroll
			for (int e = 0; e < ITEMS; e++)
			{
				const int j = lane + 64 * e;
				if (j < columns)
					Storage<T>::store(dst + j, v[e] * scale);
			}
		}
	}
	/* the same with VEC consecutive columns per lane and access (16 bytes); the row length must be a multiple of VEC */
	template<typename T, int VEC, int ITEMS>
	__global__ __launch_bounds__(256) void kernel_softmax_in_registers_wide(T *output, const T *input, size_t rows, int columns)
	{
		const int lane = threadIdx.x & 63;
		const size_t stride = static_cast<size_t>(gridDim.x) * 4;
		for (size_t row = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6); row < rows; row += stride)
		{
			const T *src = input + row * columns;
			T *dst = output + row * columns;
			Vec<T, VEC> v[ITEMS];
			float max_value = -INFINITY;
#pragma unroll
			for (int e = 0; e < ITEMS; e++)
			{
				const int j = (lane + 64 * e) * VEC;
				if (j < columns)
				{
					v[e].load(src + j);
#pragma unroll
					for (int k = 0; k < VEC; k++)
						max_value = fmaxf(max_value, v[e].v[k]);
				}
			}
			max_value = wave_max(max_value);
			float sum = 0.0f;
#pragma unroll
			for (int e = 0; e < ITEMS; e++)
				if ((lane + 64 * e) * VEC < columns)
				{
#pragma unroll
					for (int k = 0; k < VEC; k++)
					{
						v[e].v[k] = expf(v[e].v[k] - max_value);
						sum += v[e].v[k];
					}
				}
			const float scale = 1.0f / wave_sum(sum);
#pragma unroll
			for (int e = 0; e < ITEMS; e++)
			{
				const int j = (lane + 64 * e) * VEC;
				if (j < columns)
				{
#pragma unroll
					for (int k = 0; k < VEC; k++)
						v[e].v[k] *= scale;
					v[e].store(dst + j);
				}
			}
		}
	}
	/*
	 * any row length: LANES == 64, one wavefront per row; LANES == 1, one thread per row (short rows such as win / draw / loss).
	 * The row is read three times (maximum, sum, result), the second and third time from cache. In place is allowed: the last pass
	 * reads element j before it writes element j and never reads a written one again.
	 */
	template<typename T, int LANES>
	__global__ __launch_bounds__(256) void kernel_softmax_streaming(T *output, const T *input, size_t rows, int columns)
	{
		constexpr int ROWS_PER_BLOCK = 256 / LANES;
		const int lane = threadIdx.x % LANES;
		const size_t stride = static_cast<size_t>(gridDim.x) * ROWS_PER_BLOCK;
		for (size_t row = static_cast<size_t>(blockIdx.x) * ROWS_PER_BLOCK + threadIdx.x / LANES; row < rows; row += stride)
		{
			const T *src = input + row * columns;
			T *dst = output + row * columns;
			float max_value = -INFINITY;
			for (int j = lane; j < columns; j += LANES)
				max_value = fmaxf(max_value, Storage<T>::load(src + j));
			if (LANES == 64)
				max_value = wave_max(max_value);
			float sum = 0.0f;
			for (int j = lane; j < columns; j += LANES)
				sum += expf(Storage<T>::load(src + j) - max_value);
			if (LANES == 64)
				sum = wave_sum(sum);
			const float scale = 1.0f / sum;
			for (int j = lane; j < columns; j += LANES)
				Storage<T>::store(dst + j, expf(Storage<T>::load(src + j) - max_value) * scale);
		}
	}

	/*
	 * grid (channel slabs, images); 256 threads = 32 channel lanes x 8 pixel lanes. A channel lane owns VEC consecutive channels, a pixel
	 * lane every 8th pixel; the 8 partial sums meet in LDS.
	 */
	template<typename T, int VEC>
	__global__ __launch_bounds__(256) void kernel_global_average_pooling(float beta, T *output, float alpha, const T *input, int hw, int channels)
	{
		constexpr int CHANNEL_LANES = 32, PIXEL_LANES = 8;
		__shared__ float partial[PIXEL_LANES][CHANNEL_LANES * VEC + 1];
		const int channel_lane = threadIdx.x % CHANNEL_LANES;
		const int pixel_lane = threadIdx.x / CHANNEL_LANES;
		const int channel = (blockIdx.x * CHANNEL_LANES + channel_lane) * VEC;
		const T *src = input + static_cast<size_t>(blockIdx.y) * hw * channels + channel;

		float acc[VEC];
#pragma unroll
		for (int e = 0; e < VEC; e++)
			acc[e] = 0.0f;
		if (channel < channels)
		{
#pragma unroll 4
			for (int p = pixel_lane; p < hw; p += PIXEL_LANES)
			{
				Vec<T, VEC> v;
				v.load(src + static_cast<size_t>(p) * channels);
#pragma unroll
				for (int e = 0; e < VEC; e++)
					acc[e] += v.v[e];
			}
		}
#pragma unroll
		for (int e = 0; e < VEC; e++)
			partial[pixel_lane][channel_lane * VEC + e] = acc[e];
		__syncthreads();
		if (pixel_lane == 0 && channel < channels)
		{
			T *dst = output + static_cast<size_t>(blockIdx.y) * channels + channel;
			const float scale = alpha / static_cast<float>(hw);
			Vec<T, VEC> old, result;
			if (beta != 0.0f)
				old.load(dst);
			else
				old.zero();
#pragma unroll
			for (int e = 0; e < VEC; e++)
			{
				float sum = 0.0f;
#pragma unroll
				for (int k = 0; k < PIXEL_LANES; k++)
					sum += partial[k][channel_lane * VEC + e];
				result.v[e] = sum * scale;
				if (beta != 0.0f)
					result.v[e] += beta * old.v[e];
			}
			result.store(dst);
		}
	}

	/*
	 * 256 threads = column_lanes (a power of two up to 64) x row lanes. A thread keeps one group of VEC columns for the whole launch, so
	 * scale and shift (a square root and a division per column) are computed once per thread and not once per element.
	 */
	template<typename T, int VEC>
	__global__ __launch_bounds__(256) void kernel_batchnorm_inference(float beta, T *output, float alpha, const T *input, const T *gamma,
			const T *bias, const float *avg_var, size_t first_dim, int last_dim, int act, int column_lanes)
	{
		const int rows_per_block = 256 / column_lanes;
		const int column = (blockIdx.x * column_lanes + threadIdx.x % column_lanes) * VEC;
		if (column >= last_dim)
			return;
		float scale[VEC], shift[VEC];
		{
			Vec<T, VEC> g, b;
			Vec<float, VEC> mean, variance;
			if (gamma != nullptr)
				g.load(gamma + column);
			if (bias != nullptr)
				b.load(bias + column);
			else
				b.zero();
			mean.load(avg_var + column);
			variance.load(avg_var + last_dim + column);
#pragma unroll
			for (int e = 0; e < VEC; e++)
			{
				scale[e] = ((gamma != nullptr) ? g.v[e] : 1.0f) / sqrtf(variance.v[e] + 1.0e-6f);
				shift[e] = b.v[e] - mean.v[e] * scale[e];
			}
		}
		const size_t stride = static_cast<size_t>(gridDim.y) * rows_per_block;
		for (size_t row = static_cast<size_t>(blockIdx.y) * rows_per_block + threadIdx.x / column_lanes; row < first_dim; row += stride)
		{
			const size_t offset = row * last_dim + column;
			Vec<T, VEC> v, old;
			v.load(input + offset);
			if (beta != 0.0f)
				old.load(output + offset);
			else
				old.zero();
#pragma unroll
			for (int e = 0; e < VEC; e++)
			{
				float t = activate(act, v.v[e] * scale[e] + shift[e]) * alpha;
				if (beta != 0.0f)
					t += beta * old.v[e];
				v.v[e] = t;
			}
			v.store(output + offset);
		}
	}

	/* one workgroup per channel; `other` elements of the weights belong to it, at stride 1 (channel first) or `channels` (channel last) */
	template<typename T>
	__global__ __launch_bounds__(256) void kernel_fold_batchnorm(T *layer_weights, T *layer_bias, const T *bn_weights, const T *bn_bias,
			const float *bn_avg_var, int channels, int other, bool channels_last)
	{
		const int c = blockIdx.x;
		const float gamma = (bn_weights != nullptr) ? Storage<T>::load(bn_weights + c) : 1.0f;
		const float beta = (bn_bias != nullptr) ? Storage<T>::load(bn_bias + c) : 0.0f;
		const float scale = gamma / sqrtf(bn_avg_var[channels + c] + 1.0e-6f);
		const float shift = -bn_avg_var[c] * scale + beta;
		for (int k = threadIdx.x; k < other; k += blockDim.x)
		{
			T *w = layer_weights + (channels_last ? (static_cast<size_t>(k) * channels + c) : (static_cast<size_t>(c) * other + k));
			Storage<T>::store(w, Storage<T>::load(w) * scale);
		}
		if (threadIdx.x == 0)
			Storage<T>::store(layer_bias + c, Storage<T>::load(layer_bias + c) * scale + shift);
	}

	bool aligned_to(const void *p, size_t bytes)
	{
		return p == nullptr || (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
	}
	unsigned int blocks_for(size_t items, unsigned int limit)
	{
		return static_cast<unsigned int>(items < 1 ? 1 : (items < limit ? items : limit));
	}

	template<typename T>
	void launch_softmax(hipStream_t stream, T *output, const T *input, size_t rows, int columns)
	{
		const unsigned int wave_blocks = blocks_for((rows + 3) / 4, 1u << 20);
		constexpr int WIDE = 16 / static_cast<int>(sizeof(T));
		const bool wide = columns % WIDE == 0 && aligned_to(output, 16) && aligned_to(input, 16);
		if (wide && columns > 64 && columns <= 64 * WIDE)
			hipLaunchKernelGGL((kernel_softmax_in_registers_wide<T, WIDE, 1>), dim3(wave_blocks), dim3(256), 0, stream, output, input, rows, columns);
		else if (wide && columns > 64 && columns <= 128 * WIDE)
			hipLaunchKernelGGL((kernel_softmax_in_registers_wide<T, WIDE, 2>), dim3(wave_blocks), dim3(256), 0, stream, output, input, rows, columns);
		else if (wide && columns > 64 && columns <= 256 * WIDE)
			hipLaunchKernelGGL((kernel_softmax_in_registers_wide<T, WIDE, 4>), dim3(wave_blocks), dim3(256), 0, stream, output, input, rows, columns);
		else if (columns <= 16)
			hipLaunchKernelGGL((kernel_softmax_streaming<T, 1>), dim3(blocks_for((rows + 255) / 256, 1u << 20)), dim3(256), 0, stream, output, input, rows,
					columns);
		else if (columns <= 64)
			hipLaunchKernelGGL((kernel_softmax_in_registers<T, 1>), dim3(wave_blocks), dim3(256), 0, stream, output, input, rows, columns);
		else if (columns <= 128)
			hipLaunchKernelGGL((kernel_softmax_in_registers<T, 2>), dim3(wave_blocks), dim3(256), 0, stream, output, input, rows, columns);
		else if (columns <= 256)
			hipLaunchKernelGGL((kernel_softmax_in_registers<T, 4>), dim3(wave_blocks), dim3(256), 0, stream, output, input, rows, columns);
		else if (columns <= 512)
			hipLaunchKernelGGL((kernel_softmax_in_registers<T, 8>), dim3(wave_blocks), dim3(256), 0, stream, output, input, rows, columns);
		else if (columns <= 1024)
			hipLaunchKernelGGL((kernel_softmax_in_registers<T, 16>), dim3(wave_blocks), dim3(256), 0, stream, output, input, rows, columns);
		else
			hipLaunchKernelGGL((kernel_softmax_streaming<T, 64>), dim3(wave_blocks), dim3(256), 0, stream, output, input, rows, columns);
		MLHIP_CHECK(hipGetLastError());
	}

	template<typename T, int VEC>
	void launch_pooling_as(hipStream_t stream, float alpha, const mlTensor_t &x, float beta, mlTensor_t &y)
	{
		const int hw = x.dim[1] * x.dim[2], channels = x.dim[3];
		const dim3 grid(ceil_div(ceil_div(channels, VEC), 32), x.dim[0]);
		hipLaunchKernelGGL((kernel_global_average_pooling<T, VEC>), grid, dim3(256), 0, stream, beta, ptr<T>(y), alpha, ptr<const T>(x), hw, channels);
	}
	template<typename T>
	void launch_pooling(hipStream_t stream, float alpha, const mlTensor_t &x, float beta, mlTensor_t &y)
	{
		constexpr int WIDE = 16 / static_cast<int>(sizeof(T));
		const int channels = x.dim[3];
		const auto fits = [&](int vec) {
			return channels % vec == 0 && aligned_to(x.data, vec * sizeof(T)) && aligned_to(y.data, vec * sizeof(T));
		};
		if (WIDE > 4 && fits(WIDE))
			launch_pooling_as<T, WIDE>(stream, alpha, x, beta, y);
		else if (fits(4))
			launch_pooling_as<T, 4>(stream, alpha, x, beta, y);
		else
			launch_pooling_as<T, 1>(stream, alpha, x, beta, y);
		MLHIP_CHECK(hipGetLastError());
	}

	template<typename T, int VEC>
	void launch_batchnorm_as(hipStream_t stream, float alpha, const mlTensor_t &x, const mlTensor_t &w, const mlTensor_t &b, const mlTensor_t &avg_var,
			float beta, mlTensor_t &y, int act)
	{
		const int last = last_dim(x);
		const size_t first = volume(x) / last;
		const int groups = last / VEC;
		int column_lanes = 1;
		while (column_lanes < 64 && column_lanes < groups)
			column_lanes *= 2;
		const int rows_per_block = 256 / column_lanes;
		const dim3 grid(ceil_div(groups, column_lanes), blocks_for((first + rows_per_block - 1) / rows_per_block, 1024));
		hipLaunchKernelGGL((kernel_batchnorm_inference<T, VEC>), grid, dim3(256), 0, stream, beta, ptr<T>(y), alpha, ptr<const T>(x), ptr<const T>(w),
				ptr<const T>(b), ptr<const float>(avg_var), first, last, act, column_lanes);
	}
	template<typename T>
	void launch_batchnorm(hipStream_t stream, float alpha, const mlTensor_t &x, const mlTensor_t &w, const mlTensor_t &b, const mlTensor_t &avg_var,
			float beta, mlTensor_t &y, int act)
	{
		constexpr int WIDE = 16 / static_cast<int>(sizeof(T));
		const int last = last_dim(x);
		const auto fits = [&](int vec) {
			return last % vec == 0 && aligned_to(x.data, vec * sizeof(T)) && aligned_to(y.data, vec * sizeof(T)) && aligned_to(w.data, vec * sizeof(T))
					&& aligned_to(b.data, vec * sizeof(T)) && aligned_to(avg_var.data, vec * sizeof(float));
		};
		if (WIDE > 4 && fits(WIDE))
			launch_batchnorm_as<T, WIDE>(stream, alpha, x, w, b, avg_var, beta, y, act);
		else if (fits(4))
			launch_batchnorm_as<T, 4>(stream, alpha, x, w, b, avg_var, beta, y, act);
		else
			launch_batchnorm_as<T, 1>(stream, alpha, x, w, b, avg_var, beta, y, act);
		MLHIP_CHECK(hipGetLastError());
	}
}

extern "C"
{
	using namespace mlhip;

	void hip_softmax_forward(mlContext_t context, mlDataType_t dtype, mlShape_t shape, void *output, const void *input)
	try
	{
		if (volume(shape) == 0)
			return;
		MLHIP_REQUIRE(output != nullptr && input != nullptr, "softmax_forward: null pointer");
		const int columns = last_dim(shape);
		const size_t rows = volume(shape) / columns;
		switch (dtype)
		{
			case DTYPE_FLOAT16:
				launch_softmax(stream_of(context), reinterpret_cast<half_t*>(output), reinterpret_cast<const half_t*>(input), rows, columns);
				break;
			case DTYPE_FLOAT32:
				launch_softmax(stream_of(context), reinterpret_cast<float*>(output), reinterpret_cast<const float*>(input), rows, columns);
				break;
			default:
				fail_logic("HIP backend: softmax_forward: unsupported data type");
		}
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_global_average_pooling_forward(mlContext_t context, float alpha, const mlTensor_t x, float beta, mlTensor_t y)
	try
	{
		MLHIP_REQUIRE(x.rank == 4 && y.rank == 2, "global_average_pooling_forward: x must be [B, H, W, C] and y [B, C]");
		MLHIP_REQUIRE(x.dim[0] == y.dim[0] && x.dim[3] == y.dim[1], "global_average_pooling_forward: x and y disagree in batch or channels");
		MLHIP_REQUIRE(x.dtype == y.dtype, "global_average_pooling_forward: x and y must have one data type");
		if (volume(y) == 0)
			return;
		MLHIP_REQUIRE(x.dim[1] > 0 && x.dim[2] > 0, "global_average_pooling_forward: empty spatial extent");
		MLHIP_REQUIRE(x.data != nullptr && y.data != nullptr, "global_average_pooling_forward: null tensor");
		MLHIP_REQUIRE(x.dtype == DTYPE_FLOAT16 || x.dtype == DTYPE_FLOAT32, "global_average_pooling_forward: unsupported data type");
		/* the image index rides in the grid's second dimension: longer batches go slice by slice */
		const size_t esize = size_of(x.dtype), image = static_cast<size_t>(x.dim[1]) * x.dim[2] * x.dim[3] * esize, row = static_cast<size_t>(x.dim[3]) * esize;
		for (int first = 0; first < x.dim[0]; first += 65535)
		{
			mlTensor_t in = x, out = y;
			in.dim[0] = out.dim[0] = std::min(65535, x.dim[0] - first);
			in.data = reinterpret_cast<uint8_t*>(x.data) + first * image;
			out.data = reinterpret_cast<uint8_t*>(y.data) + first * row;
			if (x.dtype == DTYPE_FLOAT16)
				launch_pooling<half_t>(stream_of(context), alpha, in, beta, out);
			else
				launch_pooling<float>(stream_of(context), alpha, in, beta, out);
		}
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_batchnorm_inference(mlContext_t context, float alpha, const mlTensor_t x, const mlTensor_t w, const mlTensor_t b, const mlTensor_t avg_var,
			float beta, mlTensor_t y, mlActivationType_t act)
	try
	{
		if (volume(x) == 0)
			return;
		const int last = last_dim(x);
		MLHIP_REQUIRE(x.dtype == y.dtype && volume(x) == volume(y), "batchnorm_inference: x and y must have one shape and data type");
		MLHIP_REQUIRE(x.data != nullptr && y.data != nullptr, "batchnorm_inference: null tensor");
		MLHIP_REQUIRE(avg_var.data != nullptr && avg_var.dtype == DTYPE_FLOAT32 && volume(avg_var) == 2 * static_cast<size_t>(last),
				"batchnorm_inference: statistics must be fp32 [2, last dim of x]");
		if (w.data != nullptr)
			MLHIP_REQUIRE(w.dtype == x.dtype && volume(w) == static_cast<size_t>(last), "batchnorm_inference: gamma must be [last dim of x]");
		if (b.data != nullptr)
			MLHIP_REQUIRE(b.dtype == x.dtype && volume(b) == static_cast<size_t>(last), "batchnorm_inference: bias must be [last dim of x]");
		mlTensor_t out = y;
		switch (x.dtype)
		{
			case DTYPE_FLOAT16:
				launch_batchnorm<half_t>(stream_of(context), alpha, x, w, b, avg_var, beta, out, act);
				break;
			case DTYPE_FLOAT32:
				launch_batchnorm<float>(stream_of(context), alpha, x, w, b, avg_var, beta, out, act);
				break;
			default:
				fail_logic("HIP backend: batchnorm_inference: unsupported data type");
		}
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_fold_batchnorm(mlContext_t context, mlTensor_t layer_weights, mlTensor_t layer_bias, const mlTensor_t bn_weights, const mlTensor_t bn_bias,
			const mlTensor_t bn_avg_var)
	try
	{
		if (volume(layer_weights) == 0)
			return;
		/* rank 3 = depthwise weights [k, k, channels]; otherwise channels lead (src/backend/cpu/normalization.cpp:304,327) */
		const bool channels_last = (layer_weights.rank == 3);
		const int channels = channels_last ? last_dim(layer_weights) : layer_weights.dim[0];
		const size_t other = volume(layer_weights) / channels;
		MLHIP_REQUIRE(layer_weights.data != nullptr && layer_bias.data != nullptr, "fold_batchnorm: null layer tensor");
		MLHIP_REQUIRE(layer_bias.dtype == layer_weights.dtype && volume(layer_bias) == static_cast<size_t>(channels),
				"fold_batchnorm: layer bias must be [channels] in the weights' data type");
		MLHIP_REQUIRE(bn_avg_var.data != nullptr && bn_avg_var.dtype == DTYPE_FLOAT32 && volume(bn_avg_var) == 2 * static_cast<size_t>(channels),
				"fold_batchnorm: statistics must be fp32 [2, channels]");
		if (bn_weights.data != nullptr)
			MLHIP_REQUIRE(bn_weights.dtype == layer_weights.dtype && volume(bn_weights) == static_cast<size_t>(channels),
					"fold_batchnorm: gamma must be [channels] in the weights' data type");
		if (bn_bias.data != nullptr)
			MLHIP_REQUIRE(bn_bias.dtype == layer_weights.dtype && volume(bn_bias) == static_cast<size_t>(channels),
					"fold_batchnorm: batchnorm bias must be [channels] in the weights' data type");
		MLHIP_REQUIRE(other <= 0x7fffffffu, "fold_batchnorm: weights too large");
		const hipStream_t stream = stream_of(context);
		switch (layer_weights.dtype)
		{
			case DTYPE_FLOAT16:
				hipLaunchKernelGGL(kernel_fold_batchnorm<half_t>, dim3(channels), dim3(256), 0, stream, ptr<half_t>(layer_weights), ptr<half_t>(layer_bias),
						ptr<const half_t>(bn_weights), ptr<const half_t>(bn_bias), ptr<const float>(bn_avg_var), channels, static_cast<int>(other),
						channels_last);
				break;
			case DTYPE_FLOAT32:
				hipLaunchKernelGGL(kernel_fold_batchnorm<float>, dim3(channels), dim3(256), 0, stream, ptr<float>(layer_weights), ptr<float>(layer_bias),
						ptr<const float>(bn_weights), ptr<const float>(bn_bias), ptr<const float>(bn_avg_var), channels, static_cast<int>(other),
						channels_last);
				break;
			default:
				fail_logic("HIP backend: fold_batchnorm: unsupported data type");
		}
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(softmax_forward)
MLHIP_ALSO_AS_CUDA(global_average_pooling_forward)
MLHIP_ALSO_AS_CUDA(batchnorm_inference)
MLHIP_ALSO_AS_CUDA(fold_batchnorm)
