/*
 * device_utils.hpp — device-side vector types, fp16 conversions and small helpers shared by the gfx950 kernels.
 *
 * fp32 -> fp16 conversion truncates toward zero everywhere, because that is what the reference CPU backend does on every
 * fp16 store (reference: src/backend/cpu/fp16.hpp:61-68, vcvtps2ph imm 0x03 in src/backend/cpu/winograd/avx2_winograd_kernels.cpp:135-141
 * and src/backend/cpu/gemm/avx512f_kernels.cpp:219-243). gfx9 has that conversion as one packed instruction (v_cvt_pkrtz_f16_f32).
 */
#ifndef MINML_AMD_DEVICE_UTILS_HPP_
#define MINML_AMD_DEVICE_UTILS_HPP_

#include "../../include/minml_hip_backend.h"

#include <hip/hip_runtime.h>
#include <cstdint>

namespace mlhip
{
	typedef _Float16 half_t;
	typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
	typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
	typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
	typedef float float2_t __attribute__((ext_vector_type(2)));
	typedef float float4_t __attribute__((ext_vector_type(4)));
	typedef float float16_t __attribute__((ext_vector_type(16)));
	typedef int int2_t __attribute__((ext_vector_type(2)));
	typedef int int4_t __attribute__((ext_vector_type(4)));
	typedef int int16_t_v __attribute__((ext_vector_type(16)));
	typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
	typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

	/* two floats -> packed pair of halfs, round toward zero */
	__device__ __forceinline__ uint32_t pack_rtz(float lo, float hi)
	{
		typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));
		const fp16x2 tmp = __builtin_amdgcn_cvt_pkrtz(lo, hi);
		return __builtin_bit_cast(uint32_t, tmp);
	}
	__device__ __forceinline__ uint16_t half_bits_rtz(float x)
	{
		return static_cast<uint16_t>(pack_rtz(x, 0.0f) & 0xffffu);
	}
	__device__ __forceinline__ float half_bits_to_float(uint16_t h)
	{
		return static_cast<float>(__builtin_bit_cast(half_t, h));
	}
	__device__ __forceinline__ float lo_half(uint32_t packed)
	{
		return half_bits_to_float(static_cast<uint16_t>(packed & 0xffffu));
	}
	__device__ __forceinline__ float hi_half(uint32_t packed)
	{
		return half_bits_to_float(static_cast<uint16_t>(packed >> 16));
	}

	/* storage-type traits: T = float or half_t; compute type is always float */
	template<typename T>
	struct Storage;
	template<>
	struct Storage<float>
	{
			__device__ static __forceinline__ float load(const float *p)
			{
				return *p;
			}
			__device__ static __forceinline__ void store(float *p, float x)
			{
				*p = x;
			}
	};
	template<>
	struct Storage<half_t>
	{
			__device__ static __forceinline__ float load(const half_t *p)
			{
				return static_cast<float>(*p);
			}
			__device__ static __forceinline__ void store(half_t *p, float x)
			{
				*reinterpret_cast<uint16_t*>(p) = half_bits_rtz(x);
			}
	};

	/* Vector of N storage elements moved with one memory instruction; N * sizeof(T) is 4, 8 or 16 bytes. */
	template<typename T, int N>
	struct Vec
	{
			float v[N];

			__device__ __forceinline__ void load(const T *p)
			{
				if constexpr (sizeof(T) == 4)
				{
					typedef float vt __attribute__((ext_vector_type(N)));
					const vt tmp = *reinterpret_cast<const vt*>(p);
#pragma unroll
					for (int i = 0; i < N; i++)
						v[i] = tmp[i];
				}
				else
				{
					typedef _Float16 vt __attribute__((ext_vector_type(N)));
					const vt tmp = *reinterpret_cast<const vt*>(p);
#pragma unroll
					for (int i = 0; i < N; i++)
						v[i] = static_cast<float>(tmp[i]);
				}
			}
			__device__ __forceinline__ void store(T *p) const
			{
				if constexpr (sizeof(T) == 4)
				{
					typedef float vt __attribute__((ext_vector_type(N)));
					vt tmp;
#pragma unroll
					for (int i = 0; i < N; i++)
						tmp[i] = v[i];
					*reinterpret_cast<vt*>(p) = tmp;
				}
				else
				{
					static_assert(sizeof(T) == 4 || N % 2 == 0, "half vectors are stored in pairs");
					typedef uint32_t vt __attribute__((ext_vector_type(N / 2)));
					vt tmp;
#pragma unroll
					for (int i = 0; i < N / 2; i++)
						tmp[i] = pack_rtz(v[2 * i], v[2 * i + 1]);
					*reinterpret_cast<vt*>(p) = tmp;
				}
			}
			/* the same store marked non-temporal: the line is not meant to be kept in the caches */
			__device__ __forceinline__ void store_streaming(T *p) const
			{
				if constexpr (sizeof(T) == 4)
				{
					typedef float vt __attribute__((ext_vector_type(N)));
					vt tmp;
#pragma unroll
					for (int i = 0; i < N; i++)
						tmp[i] = v[i];
					__builtin_nontemporal_store(tmp, reinterpret_cast<vt*>(p));
				}
				else
				{
					typedef uint32_t vt __attribute__((ext_vector_type(N / 2)));
					vt tmp;
#pragma unroll
					for (int i = 0; i < N / 2; i++)
						tmp[i] = pack_rtz(v[2 * i], v[2 * i + 1]);
					__builtin_nontemporal_store(tmp, reinterpret_cast<vt*>(p));
				}
			}
			__device__ __forceinline__ void zero()
			{
#pragma unroll
				for (int i = 0; i < N; i++)
					v[i] = 0.0f;
			}
	};
	template<typename T>
	struct Vec<T, 1>
	{
			float v[1];
			__device__ __forceinline__ void load(const T *p)
			{
				v[0] = Storage<T>::load(p);
			}
			__device__ __forceinline__ void store(T *p) const
			{
				Storage<T>::store(p, v[0]);
			}
			__device__ __forceinline__ void store_streaming(T *p) const
			{
				Storage<T>::store(p, v[0]);
			}
			__device__ __forceinline__ void zero()
			{
				v[0] = 0.0f;
			}
	};

	/*
	 * quotient and remainder of a flat index by a 32-bit extent. 64-bit integer division is a long instruction sequence on this
	 * hardware and dominates a bandwidth-bound kernel that does one per 16 bytes; indices below 2^32 take the 32-bit form.
	 */
	__device__ __forceinline__ size_t split_index(size_t index, int extent, int &remainder)
	{
		if ((index >> 32) == 0)
		{
			const uint32_t i = static_cast<uint32_t>(index), d = static_cast<uint32_t>(extent);
			const uint32_t q = i / d;
			remainder = static_cast<int>(i - q * d);
			return q;
		}
		const size_t q = index / static_cast<size_t>(extent);
		remainder = static_cast<int>(index - q * static_cast<size_t>(extent));
		return q;
	}

	/*
	 * Division of a 32-bit number by a divisor that is fixed for a launch: a multiplication, two additions and two shifts (the
	 * branch-free multiply-and-shift form: q = hi(magic * n), result = (((n - q) >> 1) + q) >> shift) instead of the ~30 instructions
	 * of a division by a run-time value. Exact for every n < 2^32 and every divisor >= 1.
	 */
	struct FastDivisor
	{
			uint32_t divisor, magic, shift;
	};
	inline FastDivisor make_fast_divisor(uint32_t divisor)
	{
		FastDivisor f { divisor, 0u, 0u };
		if (divisor < 2)
			return f; /* 1 is handled by the device side */
		uint32_t log2_floor = 31;
		while (((divisor >> log2_floor) & 1u) == 0)
			log2_floor--;
		if ((divisor & (divisor - 1)) == 0)
			f.shift = log2_floor - 1; /* a power of two: magic 0 */
		else
		{
			const uint64_t numerator = (static_cast<uint64_t>(1) << log2_floor) << 32;
			uint32_t proposed = static_cast<uint32_t>(numerator / divisor);
			const uint64_t rest = numerator % divisor;
			proposed += proposed;
			if (rest + rest >= divisor)
				proposed += 1;
			f.magic = proposed + 1;
			f.shift = log2_floor;
		}
		return f;
	}
	__device__ __forceinline__ uint32_t fast_divide(uint32_t n, const FastDivisor &f, uint32_t &remainder)
	{
		const uint32_t q = __umulhi(f.magic, n);
		const uint32_t quotient = (f.divisor == 1u) ? n : ((((n - q) >> 1) + q) >> f.shift);
		remainder = n - quotient * f.divisor;
		return quotient;
	}

	/* activations of the reference (src/backend/cpu/common_math.hpp:40-55, src/backend/cpu/def_misc_kernels.cpp:52-72) */
	__device__ __forceinline__ float activate(int act, float x)
	{
		switch (act)
		{
			default:
			case 0: /* LINEAR */
				return x;
			case 1: /* SIGMOID */
				return 1.0f / (1.0f + expf(-x));
			case 2: /* TANH */
				return tanhf(x);
			case 3: /* RELU */
				return fmaxf(0.0f, x);
			case 4: /* LEAKY_RELU */
				return (x > 0.0f) ? x : 0.1f * x;
			case 5: /* EXP */
				return expf(x);
		}
	}

	/*
	 * Workgroup ids are handed to the 8 XCDs round-robin (id % 8); each XCD has its own L2. This remap gives every XCD a
	 * contiguous range of logical ids so that neighbouring work (which shares input rows / operand tiles) meets in one L2.
	 */
	__device__ __forceinline__ unsigned int xcd_contiguous_block_id(unsigned int id, unsigned int count)
	{
		constexpr unsigned int XCDS = 8;
		const unsigned int full = (count / XCDS) * XCDS;
		if (id >= full)
			return id; /* tail blocks keep their id */
		return (id % XCDS) * (full / XCDS) + id / XCDS;
	}
	/*
	 * The other way to keep neighbouring work in one L2: runs of `run` consecutive logical ids go to one XCD, and the runs go round
	 * the 8 XCDs, so that the whole chip works on one dense window of the logical range at any moment. Ids beyond the last whole
	 * group of 8 runs keep their value.
	 */
	__device__ __forceinline__ unsigned int xcd_run_block_id(unsigned int id, unsigned int count, unsigned int run)
	{
		constexpr unsigned int XCDS = 8;
		const unsigned int span = XCDS * run, full = count / span * span;
		if (id >= full)
			return id;
		const unsigned int xcd = id % XCDS, seq = id / XCDS;
		return (seq / run) * span + xcd * run + seq % run;
	}
} /* namespace mlhip */

#endif /* MINML_AMD_DEVICE_UTILS_HPP_ */
