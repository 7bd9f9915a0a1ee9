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
			const size_t offset = gid * VEC; /* rows are contiguous and last_dim == groups * VEC */
			Vec<T, VEC> vx, vb, vy;
			vx.load(x + offset);
			if (bias != nullptr)
			{
				int group;
				split_index(gid, groups, group);
				vb.load(bias + group * VEC);
			}
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

	/* VEC elements per thread and step: 8 gives one 16-byte access on the fp16 side and two on the fp32 side. */
	template<typename DstT, typename SrcT, int VEC>
	__global__ __launch_bounds__(256) void kernel_convert(DstT *dst, const SrcT *src, size_t elements)
	{
		const size_t total = elements / VEC;
		const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
		for (size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < total; gid += stride)
		{
			Vec<SrcT, VEC> in;
			in.load(src + gid * VEC);
			Vec<DstT, VEC> out;
#pragma unroll
			for (int e = 0; e < VEC; e++)
				out.v[e] = in.v[e];
			out.store(dst + gid * VEC);
		}
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
			int j;
			const size_t i = split_index(gid, last_dim, j);
			const uint32_t word = src[i * words + j / 32];
			dst[gid] = one_or_zero<T>((word >> (j % 32)) & 1u);
		}
	}
	/*
	 * last_dim a multiple of GROUP (a power of two up to 32, GROUP * sizeof(T) == 16 where the type allows): one thread
	 * expands GROUP consecutive bits of one word and writes them with 16-byte stores.
	 */
	template<typename T, int GROUP>
	__global__ __launch_bounds__(256) void kernel_unpack_input_grouped(T *dst, const uint32_t *src, size_t first_dim, int last_dim)
	{
		typedef T vt __attribute__((ext_vector_type(GROUP)));
		const int words = (last_dim + 31) / 32;
		const int groups = last_dim / GROUP;
		const size_t total = first_dim * groups;
		const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
		for (size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < total; gid += stride)
		{
			int group;
			const size_t i = split_index(gid, groups, group);
			const int j = group * GROUP;
			const uint32_t bits = src[i * words + j / 32] >> (j % 32);
			vt out;
#pragma unroll
			for (int e = 0; e < GROUP; e++)
				out[e] = one_or_zero<T>((bits >> e) & 1u);
			*reinterpret_cast<vt*>(dst + i * last_dim + j) = out;
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

	template<typename DstT, typename SrcT>
	void launch_convert(hipStream_t stream, DstT *dst, const SrcT *src, size_t elements)
	{
		constexpr int VEC = 8;
		const size_t body = (aligned_to(dst, VEC * sizeof(DstT)) && aligned_to(src, VEC * sizeof(SrcT))) ? (elements / VEC) * VEC : 0;
		if (body > 0)
			hipLaunchKernelGGL((kernel_convert<DstT, SrcT, VEC>), dim3(grid_for(body / VEC)), dim3(256), 0, stream, dst, src, body);
		if (body < elements)
			hipLaunchKernelGGL((kernel_convert<DstT, SrcT, 1>), dim3(grid_for(elements - body)), dim3(256), 0, stream, dst + body, src + body,
					elements - body);
	}
	template<typename T>
	void launch_unpack_input(hipStream_t stream, T *dst, const uint32_t *src, size_t first, int last)
	{
		constexpr int GROUP = (sizeof(T) >= 4) ? 4 : static_cast<int>(16 / sizeof(T));
		if (last % GROUP == 0 && aligned_to(dst, GROUP * sizeof(T)))
			hipLaunchKernelGGL((kernel_unpack_input_grouped<T, GROUP>), dim3(grid_for(first * (last / GROUP))), dim3(256), 0, stream, dst, src, first,
					last);
		else
			hipLaunchKernelGGL(kernel_unpack_input<T>, dim3(grid_for(first * last)), dim3(256), 0, stream, dst, src, first, last);
	}

	template<typename T>
	void launch_add_bias_act(hipStream_t stream, float alpha, const mlTensor_t &x, const mlTensor_t &b, float beta, mlTensor_t &y, int act)
	{
		const int last = last_dim(x);
		const size_t first = volume(x) / last;
		constexpr int WIDE = 16 / static_cast<int>(sizeof(T)); /* elements of one 16-byte access */
		const auto fits = [&](int vec) {
			return (last % vec == 0) && aligned_to(x.data, vec * sizeof(T)) && aligned_to(y.data, vec * sizeof(T)) && aligned_to(b.data, vec * sizeof(T));
		};
		if (WIDE > 4 && fits(WIDE))
			hipLaunchKernelGGL((kernel_add_bias_act<T, WIDE>), dim3(grid_for(first * (last / WIDE))), dim3(256), 0, stream, beta, ptr<T>(y), alpha,
					ptr<const T>(x), ptr<const T>(b), first, last, act);
		else if (fits(4))
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
		constexpr int WIDE = 16 / static_cast<int>(sizeof(T)); /* elements of one 16-byte access */
		const auto fits = [&](int vec) {
			return (elements % vec == 0) && aligned_to(x1.data, vec * sizeof(T)) && aligned_to(x2.data, vec * sizeof(T))
					&& aligned_to(x3.data, vec * sizeof(T)) && aligned_to(y.data, vec * sizeof(T));
		};
		if (WIDE > 4 && fits(WIDE))
			hipLaunchKernelGGL((kernel_axpy3<T, WIDE>), dim3(grid_for(elements / WIDE)), dim3(256), 0, stream, a1, ptr<const T>(x1), a2, ptr<const T>(x2),
					a3, ptr<const T>(x3), beta, ptr<T>(y), elements);
		else if (fits(4))
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
	try
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
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_activation_forward(mlContext_t context, float alpha, const mlTensor_t x, float beta, mlTensor_t y, mlActivationType_t act)
	try
	{
		if (volume(x) == 0)
			return;
		MLHIP_REQUIRE(x.dtype == y.dtype && volume(x) == volume(y), "activation_forward: x and y must have one shape and data type");
		mlhip::NestedEntryCalls nested;
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
		/* one row of all elements: the widest vector form that divides the length applies */
		hip_add_bias_act(context, alpha, flat, no_bias, beta, flat_y, act);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_add_tensors(mlContext_t context, float alpha1, const mlTensor_t x1, float alpha2, const mlTensor_t x2, float alpha3, const mlTensor_t x3,
			float beta, mlTensor_t y)
	try
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
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_scale_tensor(mlContext_t context, float alpha, mlTensor_t x)
	try
	{ /* x *= alpha (reference: src/backend/cuda/kernels/tensor_op.cu:318-321) */
		mlhip::NestedEntryCalls nested;
		mlTensor_t none;
		none.data = nullptr;
		none.dtype = x.dtype;
		none.rank = 0;
		hip_add_tensors(context, 0.0f, none, 0.0f, none, 0.0f, none, alpha, x);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_convert_type(mlContext_t context, void *dst, mlDataType_t dst_dtype, const void *src, mlDataType_t src_dtype, int elements)
	try
	{
		if (elements <= 0)
			return;
		MLHIP_REQUIRE(dst != nullptr && src != nullptr, "convert_type: null pointer");
		mlhip::NestedEntryCalls nested;
		if (dst_dtype == src_dtype)
		{
			if (dst != src)
				hip_memcpy_within_device(context, dst, 0, src, 0, static_cast<size_t>(elements) * size_of(dst_dtype));
			return;
		}
		const size_t n = static_cast<size_t>(elements);
		if (src_dtype == DTYPE_FLOAT32 && dst_dtype == DTYPE_FLOAT16)
			launch_convert(stream_of(context), reinterpret_cast<half_t*>(dst), reinterpret_cast<const float*>(src), n);
		else if (src_dtype == DTYPE_FLOAT16 && dst_dtype == DTYPE_FLOAT32)
			launch_convert(stream_of(context), reinterpret_cast<float*>(dst), reinterpret_cast<const half_t*>(src), n);
		else
			fail_logic("unsupported conversion");
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_unpack_input(mlContext_t context, mlShape_t shape, mlDataType_t dst_dtype, void *dst, const void *src)
	try
	{
		if (volume(shape) == 0)
			return;
		MLHIP_REQUIRE(dst != nullptr && src != nullptr, "unpack_input: null pointer");
		const int last = last_dim(shape);
		const size_t first = volume(shape) / last;
		const uint32_t *in = reinterpret_cast<const uint32_t*>(src);
		const hipStream_t stream = stream_of(context);
		switch (dst_dtype)
		{
			case DTYPE_FLOAT16:
				launch_unpack_input(stream, reinterpret_cast<half_t*>(dst), in, first, last);
				break;
			case DTYPE_FLOAT32:
				launch_unpack_input(stream, reinterpret_cast<float*>(dst), in, first, last);
				break;
			case DTYPE_UINT8:
				launch_unpack_input(stream, reinterpret_cast<uint8_t*>(dst), in, first, last);
				break;
			case DTYPE_INT8:
				launch_unpack_input(stream, reinterpret_cast<int8_t*>(dst), in, first, last);
				break;
			case DTYPE_INT16:
				launch_unpack_input(stream, reinterpret_cast<int16_t*>(dst), in, first, last);
				break;
			case DTYPE_INT32:
				launch_unpack_input(stream, reinterpret_cast<int32_t*>(dst), in, first, last);
				break;
			default:
				fail_logic("HIP backend: unpack_input: unsupported destination type");
		}
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(add_bias_act)
MLHIP_ALSO_AS_CUDA(activation_forward)
MLHIP_ALSO_AS_CUDA(add_tensors)
MLHIP_ALSO_AS_CUDA(scale_tensor)
MLHIP_ALSO_AS_CUDA(convert_type)
MLHIP_ALSO_AS_CUDA(unpack_input)
