/*
 * elementwise.hip — the bandwidth-bound neighbours of the convolution path: non-fused bias + activation, activation,
 * weighted tensor sum, dtype conversion and bit-plane unpacking of the network input.
 *
 *   add_bias_act:        y = act(x + b) * alpha + beta * y        reference: src/backend/cuda/kernels/activations.cu:64-84
 *                                                                 (CPU form y = act(x + b): src/backend/cpu/dispatcher.cpp:267-290)
 *   activation_forward:  y = act(x) * alpha + beta * y; LINEAR is a plain copy        activations.cu:36-48,190-214
 *   add_tensors:         y = a1*x1 + a2*x2 + a3*x3 + beta*y, absent terms skipped     src/backend/cuda/kernels/tensor_op.cu:289-363
 *   convert_type:        fp16 <-> fp32, truncating toward zero on narrowing          src/backend/cpu/dispatcher.cpp:175-188, fp16.hpp:61-68
 *   unpack_input:        bit j of word (i, j / 32) -> 1 or 0 in the destination type  src/backend/cpu/dispatcher.cpp:112-123,143-174
 * fp16 results are truncated toward zero like every fp16 store of the reference CPU backend.
 */
#include "common.hpp"
#include "device_utils.hpp"

namespace
{
	using namespace mlhip;

	template<typename T, int VEC>
	__global__ __launch_bounds__(256) void kernel_add_bias_act(float beta, T *y, float alpha, const T *x, const T *bias, size_t first_dim, int last_dim,
			int act)
	{
		const int groups = last_dim / VEC;
		const size_t total = first_dim * groups;
		const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
		for (size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < total; gid += stride)
		{
			const int col = static_cast<int>(gid % groups) * VEC;
			const size_t offset = (gid / groups) * last_dim + col;
			Vec<T, VEC> vx, vb, vy;
			vx.load(x + offset);
			if (bias != nullptr)
				vb.load(bias + col);
			else
				vb.zero();
			if (beta != 0.0f)
				vy.load(y + offset);
			else
				vy.zero();
#pragma unroll
			for (int e = 0; e < VEC; e++)
			{
				float t = activate(act, vx.v[e] + vb.v[e]) * alpha;
				if (beta != 0.0f)
					t += beta * vy.v[e];
				vx.v[e] = t;
			}
			vx.store(y + offset);
		}
	}

	template<typename T, int VEC>
	__global__ __launch_bounds__(256) void kernel_axpy3(float alpha1, const T *x1, float alpha2, const T *x2, float alpha3, const T *x3, float beta, T *y,
			size_t elements)
	{
		const bool use1 = (alpha1 != 0.0f) && (x1 != nullptr);
		const bool use2 = (alpha2 != 0.0f) && (x2 != nullptr);
		const bool use3 = (alpha3 != 0.0f) && (x3 != nullptr);
		const bool use_y = (beta != 0.0f);
		const size_t total = elements / VEC;
		const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
		for (size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < total; gid += stride)
		{
			const size_t offset = gid * VEC;
			Vec<T, VEC> v1, v2, v3, vy;
			v1.zero();
			v2.zero();
			v3.zero();
			vy.zero();
			if (use1)
				v1.load(x1 + offset);
			if (use2)
				v2.load(x2 + offset);
			if (use3)
				v3.load(x3 + offset);
			if (use_y)
				vy.load(y + offset);
#pragma unroll
			for (int e = 0; e < VEC; e++)
				vy.v[e] = alpha1 * v1.v[e] + alpha2 * v2.v[e] + alpha3 * v3.v[e] + beta * vy.v[e];
			vy.store(y + offset);
		}
	}

	template<typename DstT, typename SrcT>
	__global__ __launch_bounds__(256) void kernel_convert(DstT *dst, const SrcT *src, size_t elements)
	{
		const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
		for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < elements; i += stride)
			Storage<DstT>::store(dst + i, Storage<SrcT>::load(src + i));
	}

	template<typename T>
	__device__ __forceinline__ T one_or_zero(bool b)
	{
		return b ? static_cast<T>(1) : static_cast<T>(0);
	}
	template<typename T>
	__global__ __launch_bounds__(256) void kernel_unpack_input(T *dst, const uint32_t *src, size_t first_dim, int last_dim)
	{
		const int words = (last_dim + 31) / 32;
		const size_t total = first_dim * last_dim;
		const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
		for (size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < total; gid += stride)
		{
			const size_t i = gid / last_dim;
			const int j = static_cast<int>(gid % last_dim);
			const uint32_t word = src[i * words + j / 32];
			dst[gid] = one_or_zero<T>((word >> (j % 32)) & 1u);
		}
	}

	unsigned int grid_for(size_t items)
	{
		const size_t blocks = (items + 255) / 256;
		return static_cast<unsigned int>(blocks < 1 ? 1 : (blocks < (1u << 20) ? blocks : (1u << 20)));
	}
	bool aligned_to(const void *p, size_t bytes)
	{
		return p == nullptr || (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
	}

	template<typename T>
	void launch_add_bias_act(hipStream_t stream, float alpha, const mlTensor_t &x, const mlTensor_t &b, float beta, mlTensor_t &y, int act)
	{
		const int last = last_dim(x);
		const size_t first = volume(x) / last;
		const bool vec4 = (last % 4 == 0) && aligned_to(x.data, 4 * sizeof(T)) && aligned_to(y.data, 4 * sizeof(T)) && aligned_to(b.data, 4 * sizeof(T));
		if (vec4)
			hipLaunchKernelGGL((kernel_add_bias_act<T, 4>), dim3(grid_for(first * (last / 4))), dim3(256), 0, stream, beta, ptr<T>(y), alpha, ptr<const T>(x),
					ptr<const T>(b), first, last, act);
		else
			hipLaunchKernelGGL((kernel_add_bias_act<T, 1>), dim3(grid_for(first * last)), dim3(256), 0, stream, beta, ptr<T>(y), alpha, ptr<const T>(x),
					ptr<const T>(b), first, last, act);
		MLHIP_CHECK(hipGetLastError());
	}
	template<typename T>
	void launch_axpy3(hipStream_t stream, float a1, const mlTensor_t &x1, float a2, const mlTensor_t &x2, float a3, const mlTensor_t &x3, float beta,
			mlTensor_t &y)
	{
		const size_t elements = volume(y);
		const bool vec4 = (elements % 4 == 0) && aligned_to(x1.data, 4 * sizeof(T)) && aligned_to(x2.data, 4 * sizeof(T))
				&& aligned_to(x3.data, 4 * sizeof(T)) && aligned_to(y.data, 4 * sizeof(T));
		if (vec4)
			hipLaunchKernelGGL((kernel_axpy3<T, 4>), dim3(grid_for(elements / 4)), dim3(256), 0, stream, a1, ptr<const T>(x1), a2, ptr<const T>(x2), a3,
					ptr<const T>(x3), beta, ptr<T>(y), elements);
		else
			hipLaunchKernelGGL((kernel_axpy3<T, 1>), dim3(grid_for(elements)), dim3(256), 0, stream, a1, ptr<const T>(x1), a2, ptr<const T>(x2), a3,
					ptr<const T>(x3), beta, ptr<T>(y), elements);
		MLHIP_CHECK(hipGetLastError());
	}
}

extern "C"
{
	using namespace mlhip;

	void hip_add_bias_act(mlContext_t context, float alpha, const mlTensor_t x, const mlTensor_t b, float beta, mlTensor_t y, mlActivationType_t act)
	{
		if (volume(x) == 0)
			return;
		MLHIP_REQUIRE(x.dtype == y.dtype && volume(x) == volume(y), "add_bias_act: x and y must have one shape and data type");
		MLHIP_REQUIRE(x.data != nullptr && y.data != nullptr, "add_bias_act: null tensor");
		if (b.data != nullptr)
			MLHIP_REQUIRE(b.dtype == x.dtype && volume(b) == static_cast<size_t>(last_dim(x)), "add_bias_act: bias must be [last dim of x]");
		mlTensor_t out = y;
		switch (x.dtype)
		{
			case DTYPE_FLOAT16:
				launch_add_bias_act<half_t>(stream_of(context), alpha, x, b, beta, out, act);
				break;
			case DTYPE_FLOAT32:
				launch_add_bias_act<float>(stream_of(context), alpha, x, b, beta, out, act);
				break;
			default:
				fail_logic("HIP backend: add_bias_act: unsupported data type");
		}
	}
	void hip_activation_forward(mlContext_t context, float alpha, const mlTensor_t x, float beta, mlTensor_t y, mlActivationType_t act)
	{
		if (volume(x) == 0)
			return;
		MLHIP_REQUIRE(x.dtype == y.dtype && volume(x) == volume(y), "activation_forward: x and y must have one shape and data type");
		if (act == ACTIVATION_LINEAR)
		{ /* the reference copies and ignores alpha / beta in this case */
			if (x.data != y.data)
				hip_memcpy_within_device(context, y.data, 0, x.data, 0, volume(x) * size_of(x.dtype));
			return;
		}
		mlTensor_t flat = x;
		flat.rank = 1;
		flat.dim[0] = static_cast<int>(volume(x));
		mlTensor_t flat_y = y;
		flat_y.rank = 1;
		flat_y.dim[0] = flat.dim[0];
		mlTensor_t no_bias;
		no_bias.data = nullptr;
		no_bias.dtype = x.dtype;
		no_bias.rank = 0;
		/* view as [elements / 4, 4] when possible so that the vector path applies */
		if (flat.dim[0] % 4 == 0)
		{
			flat.rank = flat_y.rank = 2;
			flat.dim[1] = flat_y.dim[1] = 4;
			flat.dim[0] = flat_y.dim[0] = flat.dim[0] / 4;
		}
		hip_add_bias_act(context, alpha, flat, no_bias, beta, flat_y, act);
	}
	void hip_add_tensors(mlContext_t context, float alpha1, const mlTensor_t x1, float alpha2, const mlTensor_t x2, float alpha3, const mlTensor_t x3,
			float beta, mlTensor_t y)
	{
		if (volume(y) == 0 || y.data == nullptr)
			return;
		mlTensor_t out = y;
		switch (y.dtype)
		{
			case DTYPE_FLOAT16:
				launch_axpy3<half_t>(stream_of(context), alpha1, x1, alpha2, x2, alpha3, x3, beta, out);
				break;
			case DTYPE_FLOAT32:
				launch_axpy3<float>(stream_of(context), alpha1, x1, alpha2, x2, alpha3, x3, beta, out);
				break;
			default:
				fail_logic("HIP backend: add_tensors: unsupported data type");
		}
	}
	void hip_scale_tensor(mlContext_t context, float alpha, mlTensor_t x)
	{ /* x *= alpha (reference: src/backend/cuda/kernels/tensor_op.cu:318-321) */
		mlTensor_t none;
		none.data = nullptr;
		none.dtype = x.dtype;
		none.rank = 0;
		hip_add_tensors(context, 0.0f, none, 0.0f, none, 0.0f, none, alpha, x);
	}
	void hip_convert_type(mlContext_t context, void *dst, mlDataType_t dst_dtype, const void *src, mlDataType_t src_dtype, int elements)
	{
		if (elements <= 0)
			return;
		MLHIP_REQUIRE(dst != nullptr && src != nullptr, "convert_type: null pointer");
		if (dst_dtype == src_dtype)
		{
			if (dst != src)
				hip_memcpy_within_device(context, dst, 0, src, 0, static_cast<size_t>(elements) * size_of(dst_dtype));
			return;
		}
		const size_t n = static_cast<size_t>(elements);
		if (src_dtype == DTYPE_FLOAT32 && dst_dtype == DTYPE_FLOAT16)
			hipLaunchKernelGGL((kernel_convert<half_t, float>), dim3(grid_for(n)), dim3(256), 0, stream_of(context), reinterpret_cast<half_t*>(dst),
					reinterpret_cast<const float*>(src), n);
		else if (src_dtype == DTYPE_FLOAT16 && dst_dtype == DTYPE_FLOAT32)
			hipLaunchKernelGGL((kernel_convert<float, half_t>), dim3(grid_for(n)), dim3(256), 0, stream_of(context), reinterpret_cast<float*>(dst),
					reinterpret_cast<const half_t*>(src), n);
		else
			fail_logic("unsupported conversion");
		MLHIP_CHECK(hipGetLastError());
	}
	void hip_unpack_input(mlContext_t context, mlShape_t shape, mlDataType_t dst_dtype, void *dst, const void *src)
	{
		if (volume(shape) == 0)
			return;
		MLHIP_REQUIRE(dst != nullptr && src != nullptr, "unpack_input: null pointer");
		const int last = last_dim(shape);
		const size_t first = volume(shape) / last;
		const dim3 grid(grid_for(first * last)), block(256);
		const uint32_t *in = reinterpret_cast<const uint32_t*>(src);
		switch (dst_dtype)
		{
			case DTYPE_FLOAT16:
				hipLaunchKernelGGL(kernel_unpack_input<half_t>, grid, block, 0, stream_of(context), reinterpret_cast<half_t*>(dst), in, first, last);
				break;
			case DTYPE_FLOAT32:
				hipLaunchKernelGGL(kernel_unpack_input<float>, grid, block, 0, stream_of(context), reinterpret_cast<float*>(dst), in, first, last);
				break;
			case DTYPE_UINT8:
				hipLaunchKernelGGL(kernel_unpack_input<uint8_t>, grid, block, 0, stream_of(context), reinterpret_cast<uint8_t*>(dst), in, first, last);
				break;
			case DTYPE_INT8:
				hipLaunchKernelGGL(kernel_unpack_input<int8_t>, grid, block, 0, stream_of(context), reinterpret_cast<int8_t*>(dst), in, first, last);
				break;
			case DTYPE_INT16:
				hipLaunchKernelGGL(kernel_unpack_input<int16_t>, grid, block, 0, stream_of(context), reinterpret_cast<int16_t*>(dst), in, first, last);
				break;
			case DTYPE_INT32:
				hipLaunchKernelGGL(kernel_unpack_input<int32_t>, grid, block, 0, stream_of(context), reinterpret_cast<int32_t*>(dst), in, first, last);
				break;
			default:
				fail_logic("HIP backend: unpack_input: unsupported destination type");
		}
		MLHIP_CHECK(hipGetLastError());
	}
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(add_bias_act)
MLHIP_ALSO_AS_CUDA(activation_forward)
MLHIP_ALSO_AS_CUDA(add_tensors)
MLHIP_ALSO_AS_CUDA(scale_tensor)
MLHIP_ALSO_AS_CUDA(convert_type)
MLHIP_ALSO_AS_CUDA(unpack_input)
