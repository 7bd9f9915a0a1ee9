/*
 * epilogues.hpp — per-element tails applied to GEMM accumulators before they leave registers: the reference's fused
 * "alpha, + bias, + beta*C, activation" (src/backend/cpu/gemm/def_kernels.cpp:237-275, avx512f_kernels.cpp:798-857) and the
 * int8 requantisation of src/layers/Conv2D.cpp:284-306.
 */
#ifndef MINML_AMD_EPILOGUES_HPP_
#define MINML_AMD_EPILOGUES_HPP_

#include "device_utils.hpp"

#include <type_traits>

namespace mlhip
{
	/*
	 * D[m][n] = act(alpha * acc + bias[n] + beta * C[m][n]); C is not read when beta == 0 (the Winograd workspace it may point to is
	 * uninitialised). Activations other than LINEAR / RELU are applied to the value rounded to the storage type, because the reference
	 * runs them as a second pass over the stored matrix (src/backend/cpu/gemm/gemm.cpp:81-82).
	 */
	/*
	 * Which parts of an epilogue are known when the kernel is compiled. A kernel whose epilogue decides activation / bias / residual at
	 * run time carries the code of every activation and a branch per decision in its innermost store loop; with the common cases fixed
	 * at compile time (ReLU or linear, bias present, residual present or not) that loop is straight-line code. EPILOGUE_RUNTIME keeps
	 * the decision in the functor's fields; `specialise_epilogue` picks the compile-time form that matches them.
	 */
	constexpr int EPILOGUE_RUNTIME = -1;

	template<typename T, int ACT = EPILOGUE_RUNTIME, int WITH_C = EPILOGUE_RUNTIME, int WITH_BIAS = EPILOGUE_RUNTIME>
	struct FloatEpilogue
	{
			T *D;
			const T *C;
			const T *bias;
			int N; /* columns n >= N are not written */
			int row_stride; /* elements between consecutive rows of C and D */
			float alpha, beta;
			int act;
			bool vectorized; /* N % 4 == 0 and D, C, bias 4-element aligned */
			int bias_batch_stride = 0; /* elements between the biases of consecutive matrices of a batch (0: one bias for all) */
			static constexpr bool has_c = true;
			static constexpr bool no_side_input = (WITH_C == 0); /* known at compile time: nothing is read per output element */

			__device__ __forceinline__ int activation() const
			{
				if constexpr (ACT == EPILOGUE_RUNTIME)
					return act;
				else
					return ACT;
			}
			__device__ __forceinline__ bool with_c() const
			{
				if constexpr (WITH_C == EPILOGUE_RUNTIME)
					return beta != 0.0f;
				else
					return WITH_C != 0;
			}
			__device__ __forceinline__ bool with_bias() const
			{
				if constexpr (WITH_BIAS == EPILOGUE_RUNTIME)
					return bias != nullptr;
				else
					return WITH_BIAS != 0;
			}
			/* the same epilogue for the columns first .. first + count - 1 only, addressed as columns 0 .. count - 1 */
			FloatEpilogue columns(int first, int count) const
			{
				FloatEpilogue e = *this;
				e.D += first;
				if (e.C != nullptr)
					e.C += first;
				if (e.bias != nullptr)
					e.bias += first;
				e.N = count;
				return e;
			}
			/* the same epilogue with other parts fixed at compile time (the caller guarantees that they agree with the fields) */
			template<int A, int C, int B>
			FloatEpilogue<T, A, C, B> fixed() const
			{
				FloatEpilogue<T, A, C, B> e;
				e.D = D;
				e.C = this->C;
				e.bias = bias;
				e.N = N;
				e.row_stride = row_stride;
				e.alpha = alpha;
				e.beta = beta;
				e.act = act;
				e.vectorized = vectorized;
				e.bias_batch_stride = bias_batch_stride;
				return e;
			}
			__device__ __forceinline__ float finish(float x) const
			{
				const int a = activation();
				if (a == ACTIVATION_RELU)
					return fmaxf(x, 0.0f);
				if (a != ACTIVATION_LINEAR)
				{
					if constexpr (sizeof(T) == 2)
						x = half_bits_to_float(half_bits_rtz(x));
					return activate(a, x);
				}
				return x;
			}
			/*
			 * Split form for kernels that want the side inputs in flight early (only when `vectorized`): the per-column constants of 4
			 * consecutive n, the per-element side input (beta * C) of one group, and the tail that consumes both. Same arithmetic and
			 * order as operator().
			 */
			struct Column
			{
					float bias[4];
			};
			struct Extra
			{
					typename std::conditional<sizeof(T) == 2, uint2_t, float4_t>::type raw; /* 4 elements of C, unconverted */
			};
			__device__ __forceinline__ bool has_extra() const
			{
				return with_c();
			}
			__device__ __forceinline__ Column load_column(int n) const
			{
				Column col;
				Vec<T, 4> b;
				b.zero();
				if (with_bias())
					b.load(bias + n);
#pragma unroll
				for (int e = 0; e < 4; e++)
					col.bias[e] = b.v[e];
				return col;
			}
			/* only when has_extra(): an unconditional load, kept raw so that nothing waits for it before apply() */
			__device__ __forceinline__ Extra load_extra(int m, int n) const
			{
				Extra x;
				x.raw = *reinterpret_cast<const decltype(x.raw)*>(C + static_cast<size_t>(m) * row_stride + n);
				return x;
			}
			/* only when nothing is read per element (no_side_input): the 4 finished results, same arithmetic and order as apply() */
			__device__ __forceinline__ Vec<T, 4> value(const float (&acc)[4], const Column &col) const
			{
				Vec<T, 4> out;
#pragma unroll
				for (int e = 0; e < 4; e++)
					out.v[e] = acc[e] * alpha;
				if (with_bias())
				{
#pragma unroll
					for (int e = 0; e < 4; e++)
						out.v[e] += col.bias[e];
				}
#pragma unroll
				for (int e = 0; e < 4; e++)
					out.v[e] = finish(out.v[e]);
				return out;
			}
			/* the 4 finished results of apply(), for kernels that store them themselves */
			__device__ __forceinline__ Vec<T, 4> result(const float (&acc)[4], const Column &col, const Extra &x) const
			{
				Vec<T, 4> out;
#pragma unroll
				for (int e = 0; e < 4; e++)
					out.v[e] = acc[e] * alpha;
				if (with_bias())
				{
#pragma unroll
					for (int e = 0; e < 4; e++)
						out.v[e] += col.bias[e];
				}
				if (with_c())
				{
					float c[4];
					if constexpr (sizeof(T) == 2)
					{
						c[0] = lo_half(x.raw[0]);
						c[1] = hi_half(x.raw[0]);
						c[2] = lo_half(x.raw[1]);
						c[3] = hi_half(x.raw[1]);
					}
					else
					{
#pragma unroll
						for (int e = 0; e < 4; e++)
							c[e] = x.raw[e];
					}
#pragma unroll
					for (int e = 0; e < 4; e++)
						out.v[e] += beta * c[e];
				}
#pragma unroll
				for (int e = 0; e < 4; e++)
					out.v[e] = finish(out.v[e]);
				return out;
			}
			__device__ __forceinline__ void apply(int m, int n, const float (&acc)[4], const Column &col, const Extra &x) const
			{
				result(acc, col, x).store(D + static_cast<size_t>(m) * row_stride + n);
			}
			__device__ __forceinline__ void operator()(int m, int n, const float (&acc)[4]) const
			{
				if (n >= N)
					return;
				const size_t offset = static_cast<size_t>(m) * row_stride + n;
				if (vectorized)
				{
					Vec<T, 4> out;
#pragma unroll
					for (int e = 0; e < 4; e++)
						out.v[e] = acc[e] * alpha;
					if (with_bias())
					{
						Vec<T, 4> b;
						b.load(bias + n);
#pragma unroll
						for (int e = 0; e < 4; e++)
							out.v[e] += b.v[e];
					}
					if (with_c())
					{
						Vec<T, 4> c;
						c.load(C + offset);
#pragma unroll
						for (int e = 0; e < 4; e++)
							out.v[e] += beta * c.v[e];
					}
#pragma unroll
					for (int e = 0; e < 4; e++)
						out.v[e] = finish(out.v[e]);
					out.store(D + offset);
				}
				else
				{
#pragma unroll
					for (int e = 0; e < 4; e++)
						if (n + e < N)
						{
							float x = acc[e] * alpha;
							if (with_bias())
								x += Storage<T>::load(bias + n + e);
							if (with_c())
								x += beta * Storage<T>::load(C + offset + e);
							Storage<T>::store(D + offset + e, finish(x));
						}
				}
			}
	};

	/* int8 x int8 -> int32 product stored as is (reference: src/backend/cuda/gemms.cpp:119-130, alpha = 1, beta = 0) */
	struct Int32Epilogue
	{
			int32_t *D;
			int N;
			int row_stride;
			bool vectorized;
			static constexpr bool has_c = false;
			static constexpr bool no_side_input = false;

			Int32Epilogue columns(int first, int count) const
			{
				Int32Epilogue e = *this;
				e.D += first;
				e.N = count;
				return e;
			}
			struct Column
			{
			};
			struct Extra
			{
			};
			__device__ __forceinline__ Column load_column(int) const
			{
				return Column { };
			}
			__device__ __forceinline__ bool has_extra() const
			{
				return false;
			}
			__device__ __forceinline__ Extra load_extra(int, int) const
			{
				return Extra { };
			}
			__device__ __forceinline__ void apply(int m, int n, const int (&acc)[4], const Column&, const Extra&) const
			{
				*reinterpret_cast<int4_t*>(D + static_cast<size_t>(m) * row_stride + n) = int4_t { acc[0], acc[1], acc[2], acc[3] };
			}
			__device__ __forceinline__ void operator()(int m, int n, const int (&acc)[4]) const
			{
				if (n >= N)
					return;
				const size_t offset = static_cast<size_t>(m) * row_stride + n;
				if (vectorized)
					*reinterpret_cast<int4_t*>(D + offset) = int4_t { acc[0], acc[1], acc[2], acc[3] };
				else
				{
#pragma unroll
					for (int e = 0; e < 4; e++)
						if (n + e < N)
							D[offset + e] = acc[e];
				}
			}
	};

	/*
	 * The float tail of the reference's int8 convolution, evaluated in its order and without fused multiply-adds
	 * (src/layers/Conv2D.cpp:284-306, include/minml/layers/quantization.hpp:39-47, src/layers/quantization.cpp:39-43):
	 *   tmp = float(acc) * scale[n] + bias[n];  tmp += float(ext) * ext_scale + ext_shift;  tmp = act(tmp);
	 *   q = clamp(round_half_away(tmp * inv_scale + inv_shift), -128, 127)      with inv_scale = 1 / out_scale, inv_shift = -out_shift / out_scale
	 */
	__device__ __forceinline__ float requant_value(int acc, float scale, float bias, bool has_ext, int ext, float ext_scale, float ext_shift, int act)
	{
#pragma clang fp contract(off)
		float tmp = static_cast<float>(acc) * scale;
		tmp = tmp + bias;
		if (has_ext)
		{
			float e = static_cast<float>(ext) * ext_scale;
			e = e + ext_shift;
			tmp = tmp + e;
		}
		switch (act)
		{
			case ACTIVATION_SIGMOID:
				tmp = 1.0f / (1.0f + expf(-tmp));
				break;
			case ACTIVATION_TANH:
				tmp = tanhf(tmp);
				break;
			case ACTIVATION_RELU:
				tmp = fmaxf(0.0f, tmp);
				break;
			case ACTIVATION_EXP:
				tmp = expf(tmp);
				break;
			default:
				break;
		}
		return tmp;
	}
	__device__ __forceinline__ int quantize_to_int8(float x, float inv_scale, float inv_shift)
	{
#pragma clang fp contract(off)
		float q = x * inv_scale;
		q = q + inv_shift;
		/*
		 * std::round (halves away from zero), then the clamp to [-128, 127], as: add the largest float below one half with the sign of q,
		 * clamp, and let the conversion truncate. Equal to the reference's order for every float: checked exhaustively for |q| <= 300
		 * (above that both forms saturate); an exact half k + 0.5 plus 0.49999997 rounds up to k + 1 in fp32, anything below it does not.
		 */
		q = q + copysignf(0x1.fffffep-2f, q);
		q = fmaxf(-128.0f, fminf(127.0f, q));
		return static_cast<int>(q);
	}

	/* four values already within [-128, 127] -> four bytes, first value lowest: two saturating 16-bit packs and one byte shuffle */
	__device__ __forceinline__ uint32_t pack_int8x4(const int (&q)[4])
	{
		typedef short short2_t __attribute__((ext_vector_type(2)));
		const short2_t lo = __builtin_amdgcn_cvt_pk_i16(q[0], q[1]), hi = __builtin_amdgcn_cvt_pk_i16(q[2], q[3]);
		return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo), 0x06040200u);
	}

	template<typename OutT, int ACT = EPILOGUE_RUNTIME, int WITH_EXT = EPILOGUE_RUNTIME> /* OutT: int8_t (requantised), float or half_t (dequantised) */
	struct RequantEpilogue
	{
			OutT *D;
			const float *scales;
			const float *bias;
			const int8_t *ext;
			int N;
			int row_stride;
			float ext_scale, ext_shift;
			float inv_scale, inv_shift;
			int act;
			bool vectorized; /* N % 4 == 0 and all pointers 4-element aligned */
			static constexpr bool has_c = false;
			static constexpr bool no_side_input = false;

			__device__ __forceinline__ int activation() const
			{
				if constexpr (ACT == EPILOGUE_RUNTIME)
					return act;
				else
					return ACT;
			}
			__device__ __forceinline__ bool with_ext() const
			{
				if constexpr (WITH_EXT == EPILOGUE_RUNTIME)
					return ext != nullptr;
				else
					return WITH_EXT != 0;
			}
			RequantEpilogue columns(int first, int count) const
			{
				RequantEpilogue e = *this;
				e.D += first;
				e.scales += first;
				e.bias += first;
				if (e.ext != nullptr)
					e.ext += first;
				e.N = count;
				return e;
			}
			template<int A, int E>
			RequantEpilogue<OutT, A, E> fixed() const
			{
				RequantEpilogue<OutT, A, E> e;
				e.D = D;
				e.scales = scales;
				e.bias = bias;
				e.ext = ext;
				e.N = N;
				e.row_stride = row_stride;
				e.ext_scale = ext_scale;
				e.ext_shift = ext_shift;
				e.inv_scale = inv_scale;
				e.inv_shift = inv_shift;
				e.act = act;
				e.vectorized = vectorized;
				return e;
			}
			struct Column
			{
					float4_t scales, bias;
			};
			struct Extra
			{
					uint32_t packed;
			};
			__device__ __forceinline__ Column load_column(int n) const
			{
				Column col;
				col.scales = *reinterpret_cast<const float4_t*>(scales + n);
				col.bias = *reinterpret_cast<const float4_t*>(bias + n);
				return col;
			}
			__device__ __forceinline__ bool has_extra() const
			{
				return with_ext();
			}
			__device__ __forceinline__ Extra load_extra(int m, int n) const
			{
				Extra x;
				x.packed = *reinterpret_cast<const uint32_t*>(ext + static_cast<size_t>(m) * row_stride + n);
				return x;
			}
			__device__ __forceinline__ void apply(int m, int n, const int (&acc)[4], const Column &col, const Extra &x) const
			{
				const size_t offset = static_cast<size_t>(m) * row_stride + n;
				float vals[4];
#pragma unroll
				for (int e = 0; e < 4; e++)
				{
					const int ext_val = static_cast<int>(static_cast<int8_t>((x.packed >> (8 * e)) & 0xffu));
					vals[e] = requant_value(acc[e], col.scales[e], col.bias[e], with_ext(), ext_val, ext_scale, ext_shift, activation());
				}
				if constexpr (sizeof(OutT) == 1)
				{
					int q[4];
#pragma unroll
					for (int e = 0; e < 4; e++)
						q[e] = quantize_to_int8(vals[e], inv_scale, inv_shift);
					*reinterpret_cast<uint32_t*>(D + offset) = pack_int8x4(q);
				}
				else
				{
					Vec<OutT, 4> out;
#pragma unroll
					for (int e = 0; e < 4; e++)
						out.v[e] = vals[e];
					out.store(D + offset);
				}
			}
			__device__ __forceinline__ void operator()(int m, int n, const int (&acc)[4]) const
			{
				if (n >= N)
					return;
				const size_t offset = static_cast<size_t>(m) * row_stride + n;
				float vals[4];
				if (vectorized)
				{
					const float4_t s = *reinterpret_cast<const float4_t*>(scales + n);
					const float4_t b = *reinterpret_cast<const float4_t*>(bias + n);
					uint32_t e_packed = 0;
					if (with_ext())
						e_packed = *reinterpret_cast<const uint32_t*>(ext + offset);
#pragma unroll
					for (int e = 0; e < 4; e++)
					{
						const int ext_val = static_cast<int>(static_cast<int8_t>((e_packed >> (8 * e)) & 0xffu));
						vals[e] = requant_value(acc[e], s[e], b[e], with_ext(), ext_val, ext_scale, ext_shift, activation());
					}
					if constexpr (sizeof(OutT) == 1)
					{
						int q[4];
#pragma unroll
						for (int e = 0; e < 4; e++)
							q[e] = quantize_to_int8(vals[e], inv_scale, inv_shift);
						*reinterpret_cast<uint32_t*>(D + offset) = pack_int8x4(q);
					}
					else
					{
						Vec<OutT, 4> out;
#pragma unroll
						for (int e = 0; e < 4; e++)
							out.v[e] = vals[e];
						out.store(D + offset);
					}
				}
				else
				{
#pragma unroll
					for (int e = 0; e < 4; e++)
						if (n + e < N)
						{
							const int ext_val = with_ext() ? static_cast<int>(ext[offset + e]) : 0;
							const float v = requant_value(acc[e], scales[n + e], bias[n + e], with_ext(), ext_val, ext_scale, ext_shift, activation());
							if constexpr (sizeof(OutT) == 1)
								D[offset + e] = static_cast<OutT>(quantize_to_int8(v, inv_scale, inv_shift));
							else
								Storage<OutT>::store(D + offset + e, v);
						}
				}
			}
	};

	/*
	 * Calls launch(e') with e' = `e` whose activation and optional inputs are compile-time constants where they are the hot path's
	 * (ReLU or linear; bias present; residual present or not; 4-element groups whole and aligned), and with `e` itself otherwise.
	 * `launch` is a generic lambda: every form it is called with is a kernel instantiation of its own.
	 */
	template<typename T, typename Launch>
	inline void specialise_epilogue(const FloatEpilogue<T> &e, Launch &&launch)
	{
		const bool eligible = e.vectorized && e.bias != nullptr && (e.act == ACTIVATION_RELU || e.act == ACTIVATION_LINEAR);
		if (e.vectorized && e.bias == nullptr && e.beta == 0.0f && e.act == ACTIVATION_LINEAR)
			launch(e.template fixed<ACTIVATION_LINEAR, 0, 0>()); /* the bare product (times alpha) */
		else if (!eligible)
			launch(e);
		else if (e.act == ACTIVATION_RELU)
		{
			if (e.beta != 0.0f)
				launch(e.template fixed<ACTIVATION_RELU, 1, 1>());
			else
				launch(e.template fixed<ACTIVATION_RELU, 0, 1>());
		}
		else
		{
			if (e.beta != 0.0f)
				launch(e.template fixed<ACTIVATION_LINEAR, 1, 1>());
			else
				launch(e.template fixed<ACTIVATION_LINEAR, 0, 1>());
		}
	}
	template<typename OutT, typename Launch>
	inline void specialise_epilogue(const RequantEpilogue<OutT> &e, Launch &&launch)
	{
		const bool eligible = e.vectorized && (e.act == ACTIVATION_RELU || e.act == ACTIVATION_LINEAR);
		if (!eligible)
			launch(e);
		else if (e.act == ACTIVATION_RELU)
		{
			if (e.ext != nullptr)
				launch(e.template fixed<ACTIVATION_RELU, 1>());
			else
				launch(e.template fixed<ACTIVATION_RELU, 0>());
		}
		else
		{
			if (e.ext != nullptr)
				launch(e.template fixed<ACTIVATION_LINEAR, 1>());
			else
				launch(e.template fixed<ACTIVATION_LINEAR, 0>());
		}
	}
} /* namespace mlhip */

#endif /* MINML_AMD_EPILOGUES_HPP_ */
