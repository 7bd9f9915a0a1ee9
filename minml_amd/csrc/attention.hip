/*
 * attention.hip — the two pieces of a transformer block that the reference's CPU backend defines and that follow the convolution trunk
 * in the hybrid networks: RMS normalisation and multi-head self-attention over the board's tokens with a 2-D relative-position bias.
 *
 *   rmsnorm_forward:               y[i, :] = (gamma * x[i, :]) / (1e-6 + sqrt(mean_j x[i, j]^2))
 *                                  reference: src/backend/cpu/normalization.cpp:452-486, device form src/backend/cuda/kernels/rmsnorm.cu:219
 *   multi_head_attention_forward:  per image b and head h, with q, k, v the head's slices of the token vectors
 *                                  x[b, token, {q | k | v}, h, :] (k = q in the symmetric layout):
 *                                      s = q k^T / sqrt(head_dim) + table[h][r + clamp(dh, -r, r)][r + clamp(dw, -r, r)]
 *                                      y[b, token, h, :] = softmax_rows(s) v
 *                                  reference: src/backend/cpu/attention.cpp:142-214,395-431 (the reference runs it as a batched product
 *                                  into a [B, heads, T, T] workspace, a softmax pass over it and a second batched product; device form
 *                                  src/backend/cuda/kernels/attention.cu:509-568)
 *
 * Attention here is one launch that never writes the T x T scores: a workgroup owns one (image, head), stages the head's keys
 * (row-major) and values (transposed) in LDS, and each wavefront walks its 32 query rows over the keys in blocks of 32 with a running
 * maximum and sum ("online" softmax), both products on MFMA. The scores come out of the first product with one query row per lane
 * (the other half of the row's keys in lane + 32), which is the operand layout that the second product wants, so the probabilities
 * go from accumulator registers straight into the next MFMA. Shapes outside that kernel's reach (head sizes that are not multiples of
 * 32, more keys than fit LDS) run on a plain kernel with one wavefront per query row.
 */
#include "common.hpp"
#include "device_utils.hpp"
#include "gemm_core.hpp"

#include <algorithm>
#include <cmath>

namespace
{
	using namespace mlhip;

	__device__ __forceinline__ float wave_sum(float v)
	{
#pragma unroll
		for (int offset = 32; offset >= 1; offset >>= 1)
			v += __shfl_xor(v, offset);
		return v;
	}
	__device__ __forceinline__ float wave_max(float v)
	{
#pragma unroll
		for (int offset = 32; offset >= 1; offset >>= 1)
			v = fmaxf(v, __shfl_xor(v, offset));
		return v;
	}

	/* ------------------------------------------------------------------------------------------------------------------------
	 * RMS normalisation: one wavefront per row, two passes over the row (the second one hits the cache)
	 * ---------------------------------------------------------------------------------------------------------------------- */
	template<typename T, int VEC>
	__global__ __launch_bounds__(256) void kernel_rmsnorm_forward(T *output, const T *input, const T *weights, size_t rows, int columns)
	{
		const int lane = threadIdx.x & 63;
		const size_t stride = static_cast<size_t>(gridDim.x) * 4;
		const float inv_columns = 1.0f / static_cast<float>(columns);
		for (size_t row = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6); row < rows; row += stride)
		{
			const T *src = input + row * columns;
			T *dst = output + row * columns;
			float sum_square = 0.0f;
			for (int j = lane * VEC; j < columns; j += 64 * VEC)
			{
				Vec<T, VEC> x;
				x.load(src + j);
#pragma unroll
				for (int e = 0; e < VEC; e++)
					sum_square = fmaf(x.v[e], x.v[e], sum_square);
			}
			sum_square = wave_sum(sum_square);
			const float rms = sqrtf(sum_square * inv_columns);
			const float inv_rms = 1.0f / (1.0e-6f + rms);
			for (int j = lane * VEC; j < columns; j += 64 * VEC)
			{
				Vec<T, VEC> x;
				x.load(src + j);
				if (weights != nullptr)
				{
					Vec<T, VEC> g;
					g.load(weights + j);
#pragma unroll
					for (int e = 0; e < VEC; e++)
						x.v[e] = g.v[e] * x.v[e];
				}
#pragma unroll
				for (int e = 0; e < VEC; e++)
					x.v[e] = x.v[e] * inv_rms;
				x.store(dst + j);
			}
		}
	}
	/*
	 * The same with the row held in registers between the two passes: ITEMS vectors of VEC elements per lane, columns <= 64 * VEC * ITEMS.
	 * A wavefront takes UNROLL rows at a time and requests all of them before it reduces the first: with one row per wavefront the
	 * launch is a procession of short-lived wavefronts that each wait out one memory latency (19.5 us for 57 600 rows of 256 halfs,
	 * 3.0 TB/s).
	 */
	template<typename T, int VEC, int ITEMS, int UNROLL>
	__global__ __launch_bounds__(256) void kernel_rmsnorm_in_registers(T *output, const T *input, const T *weights, size_t rows, int columns)
	{
		const int lane = threadIdx.x & 63;
		const size_t stride = static_cast<size_t>(gridDim.x) * 4 * UNROLL;
		const float inv_columns = 1.0f / static_cast<float>(columns);
		Vec<T, VEC> gamma[ITEMS];
#pragma unroll
		for (int i = 0; i < ITEMS; i++)
		{
			const int j = (lane + 64 * i) * VEC;
#pragma unroll
			for (int e = 0; e < VEC; e++)
				gamma[i].v[e] = 1.0f;
			if (weights != nullptr && j < columns)
				gamma[i].load(weights + j);
		}
		for (size_t first = (static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6)) * UNROLL; first < rows; first += stride)
		{
			Vec<T, VEC> x[UNROLL][ITEMS];
#pragma unroll
			for (int u = 0; u < UNROLL; u++)
			{
				const T *src = input + (first + u) * columns;
#pragma unroll
				for (int i = 0; i < ITEMS; i++)
				{
					const int j = (lane + 64 * i) * VEC;
					x[u][i].zero();
					if (j < columns && first + u < rows)
						x[u][i].load(src + j);
				}
			}
#pragma unroll
			for (int u = 0; u < UNROLL; u++)
			{
				float sum_square = 0.0f;
#pragma unroll
				for (int i = 0; i < ITEMS; i++)
#pragma unroll
					for (int e = 0; e < VEC; e++)
						sum_square = fmaf(x[u][i].v[e], x[u][i].v[e], sum_square);
				sum_square = wave_sum(sum_square);
				const float rms = sqrtf(sum_square * inv_columns);
				const float inv_rms = 1.0f / (1.0e-6f + rms);
				T *dst = output + (first + u) * columns;
#pragma unroll
				for (int i = 0; i < ITEMS; i++)
				{
					const int j = (lane + 64 * i) * VEC;
#pragma unroll
					for (int e = 0; e < VEC; e++)
						x[u][i].v[e] = (gamma[i].v[e] * x[u][i].v[e]) * inv_rms;
					if (j < columns && first + u < rows)
						x[u][i].store(dst + j);
				}
			}
		}
	}
	template<typename T>
	void launch_rmsnorm(hipStream_t stream, T *output, const T *input, const T *weights, size_t rows, int columns)
	{
		constexpr int WIDE = 16 / sizeof(T);
		const unsigned int groups = static_cast<unsigned int>(std::min<size_t>((rows + 3) / 4, 65536));
		/* the in-register kernels take 4 rows (2 for the longest rows) per wavefront at a time */
		const unsigned int groups4 = static_cast<unsigned int>(std::min<size_t>((rows + 15) / 16, 65536));
		const unsigned int groups2 = static_cast<unsigned int>(std::min<size_t>((rows + 7) / 8, 65536));
		const bool aligned = (reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(output) | reinterpret_cast<uintptr_t>(weights)) % 16 == 0;
		/* rows of up to 64 * WIDE * 4 elements stay in registers; the vector width shrinks for short rows so that all 64 lanes have work */
		if (aligned && columns % WIDE == 0 && columns > 64 * WIDE / 2 && columns <= 64 * WIDE)
			hipLaunchKernelGGL((kernel_rmsnorm_in_registers<T, WIDE, 1, 4>), dim3(groups4), dim3(256), 0, stream, output, input, weights, rows, columns);
		else if (aligned && columns % WIDE == 0 && columns > 64 * WIDE && columns <= 64 * WIDE * 2)
			hipLaunchKernelGGL((kernel_rmsnorm_in_registers<T, WIDE, 2, 4>), dim3(groups4), dim3(256), 0, stream, output, input, weights, rows, columns);
		else if (aligned && columns % WIDE == 0 && columns > 64 * WIDE * 2 && columns <= 64 * WIDE * 4)
			hipLaunchKernelGGL((kernel_rmsnorm_in_registers<T, WIDE, 4, 2>), dim3(groups2), dim3(256), 0, stream, output, input, weights, rows, columns);
		else if (aligned && columns % (WIDE / 2) == 0 && columns <= 64 * WIDE / 2)
			hipLaunchKernelGGL((kernel_rmsnorm_in_registers<T, WIDE / 2, 1, 4>), dim3(groups4), dim3(256), 0, stream, output, input, weights, rows, columns);
		else if (aligned && columns % WIDE == 0)
			hipLaunchKernelGGL((kernel_rmsnorm_forward<T, WIDE>), dim3(groups), dim3(256), 0, stream, output, input, weights, rows, columns);
		else
			hipLaunchKernelGGL((kernel_rmsnorm_forward<T, 1>), dim3(groups), dim3(256), 0, stream, output, input, weights, rows, columns);
		MLHIP_CHECK(hipGetLastError());
	}

	/* ------------------------------------------------------------------------------------------------------------------------
	 * attention
	 * ---------------------------------------------------------------------------------------------------------------------- */
	struct AttentionShape
	{
			int tokens, width; /* tokens = height * width */
			int heads;
			int embedding; /* heads * head_dim */
			int token_stride; /* elements between two tokens of the input: (3 - symmetric) * embedding */
			int k_offset, v_offset; /* element offsets of the k and v parts inside a token vector */
			int table_size; /* 2 r - 1 positions per direction, 0 = no bias */
			int table_row; /* table_size rounded up to a multiple of 4 */
			float scale; /* 1 / sqrt(head_dim) */
	};

	__device__ __forceinline__ int clamp_int(int x, int lower, int upper)
	{
		return max(lower, min(upper, x));
	}
	/* by value on purpose: a bit cast applied directly to an element of a vector register reads element 0 whatever the index */
	__device__ __forceinline__ uint32_t float_bits(float x)
	{
		return __builtin_bit_cast(uint32_t, x);
	}
	/* round to nearest: the probabilities are an MFMA operand here, not a stored result */
	__device__ __forceinline__ uint32_t pack_halfs(float lo, float hi)
	{
		const half2_t tmp = { static_cast<half_t>(lo), static_cast<half_t>(hi) };
		return __builtin_bit_cast(uint32_t, tmp);
	}

	/*
	 * LDS of the MFMA kernel, in this order (all offsets multiples of 16 bytes):
	 *   keys    [tokens_padded][D * sizeof(T) + 16]          row-major, rows past `tokens` zero
	 *   values  [D][tokens_padded * sizeof(T) + 16]          transposed, columns past `tokens` zero
	 *   place   [tokens_padded] uint32                        (row << 16) | column of every key on the board
	 *   table   [table_size][table_row] float                 the head's bias table
	 * The 16 bytes of padding per row spread 16-byte fragment reads of consecutive rows over the banks.
	 */
	template<typename T, int D>
	struct AttentionLds
	{
			static constexpr int KEY_ROW = D * sizeof(T) + 16;
			__host__ __device__ static int tokens_padded(int tokens)
			{
				return (tokens + 31) / 32 * 32;
			}
			__host__ __device__ static int value_row(int tokens)
			{
				return tokens_padded(tokens) * static_cast<int>(sizeof(T)) + 16;
			}
			__host__ __device__ static int values_offset(int tokens)
			{
				return tokens_padded(tokens) * KEY_ROW;
			}
			__host__ __device__ static int place_offset(int tokens)
			{
				return values_offset(tokens) + D * value_row(tokens);
			}
			__host__ __device__ static int table_offset(int tokens)
			{
				return place_offset(tokens) + tokens_padded(tokens) * 4;
			}
			__host__ __device__ static int bytes(int tokens, int table_size, int table_row)
			{
				return table_offset(tokens) + table_size * table_row * 4;
			}
	};

	/* how the kernel finds a score's bias */
	enum
	{
		BIAS_NONE = 0, /* no table */
		BIAS_DIRECT = 1, /* the table spans every offset that occurs on the board (2r - 1 >= 2 max(H, W) - 1): no clamping, and the table index
		 splits into a per-key and a per-query part, so that one addition per score finds the entry */
		BIAS_CLAMPED = 2 /* offsets beyond the table's range use its border entries */
	};
	constexpr float LOG2_E = 1.4426950408889634f;

	template<typename T, int D, int BIAS>
	__global__ __launch_bounds__(256) void kernel_attention_mfma(const T *__restrict__ input, T *__restrict__ output, const T *__restrict__ table,
			AttentionShape shape)
	{
		typedef AttentionLds<T, D> Lds;
		typedef MfmaTraits<T> Traits;
		constexpr int ES = sizeof(T);
		constexpr int Q_CHUNKS = D * ES / 32; /* 16-byte operand chunks per lane that cover the head dimension */
		constexpr int P_GROUPS = 32 * ES / 32; /* MFMA groups that cover the 32 keys of a block: 2 for fp16, 4 for fp32 */
		constexpr int D_BLOCKS = D / 32;
		constexpr int ROW_CHUNKS = D * ES / 16;
		extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

		const int tokens = shape.tokens;
		const int tokens_padded = Lds::tokens_padded(tokens);
		const int value_row = Lds::value_row(tokens);
		uint8_t *keys = lds;
		uint8_t *values = lds + Lds::values_offset(tokens);
		uint32_t *place = reinterpret_cast<uint32_t*>(lds + Lds::place_offset(tokens));
		float *bias = reinterpret_cast<float*>(lds + Lds::table_offset(tokens));

		/* the heads of one image run on one XCD (images go round the XCDs): their q / k / v parts are neighbouring pieces of the same
		 * token rows, which then meet in one L2 instead of being fetched through eight */
		const unsigned int lin = (shape.heads > 1) ? xcd_run_block_id(blockIdx.x, gridDim.x, shape.heads) : blockIdx.x;
		const int image = lin / shape.heads;
		const int head = lin - image * shape.heads;
		const T *tokens_base = input + static_cast<size_t>(image) * tokens * shape.token_stride + head * D;
		const int range = (shape.table_size - 1) / 2;
		/* scores are kept in units of ln 2 (scale and table carry the factor log2 e) so that the exponential is the hardware's exp2 */
		const float scale = shape.scale * LOG2_E;

		/* ---- stage keys, transposed values, key places and the head's table ---- */
		for (int i = threadIdx.x; i < tokens_padded * ROW_CHUNKS; i += 256)
		{
			const int token = i / ROW_CHUNKS;
			const int chunk = i - token * ROW_CHUNKS;
			uint4_t k = { 0u, 0u, 0u, 0u }, v = { 0u, 0u, 0u, 0u };
			if (token < tokens)
			{
				const T *row = tokens_base + static_cast<size_t>(token) * shape.token_stride;
				k = *reinterpret_cast<const uint4_t*>(reinterpret_cast<const uint8_t*>(row + shape.k_offset) + chunk * 16);
				v = *reinterpret_cast<const uint4_t*>(reinterpret_cast<const uint8_t*>(row + shape.v_offset) + chunk * 16);
			}
			*reinterpret_cast<uint4_t*>(keys + token * Lds::KEY_ROW + chunk * 16) = k;
			if constexpr (ES == 2)
			{
#pragma unroll
				for (int e = 0; e < 8; e++)
				{
					const uint32_t word = v[e / 2];
					*reinterpret_cast<uint16_t*>(values + (chunk * 8 + e) * value_row + token * 2) = static_cast<uint16_t>((e & 1) ? (word >> 16) : (word & 0xffffu));
				}
			}
			else
			{
#pragma unroll
				for (int e = 0; e < 4; e++)
					*reinterpret_cast<uint32_t*>(values + (chunk * 4 + e) * value_row + token * 4) = v[e];
			}
		}
		for (int i = threadIdx.x; i < tokens_padded; i += 256)
		{
			const int token = (i < tokens) ? i : 0; /* padding keys are masked later; they only need a harmless place */
			const int row = token / shape.width;
			const int column = token - row * shape.width;
			if constexpr (BIAS == BIAS_DIRECT)
				place[i] = static_cast<uint32_t>(row * shape.table_row + column) * 4u; /* the key's part of the entry's byte offset */
			else
				place[i] = (static_cast<uint32_t>(row) << 16) | static_cast<uint32_t>(column);
		}
		if constexpr (BIAS != BIAS_NONE)
		{
			const T *head_table = table + static_cast<size_t>(head) * shape.table_size * shape.table_row;
			for (int i = threadIdx.x; i < shape.table_size * shape.table_row; i += 256)
				bias[i] = Storage<T>::load(head_table + i) * LOG2_E;
		}
		__syncthreads();

		const int wave = threadIdx.x >> 6;
		const int lane = threadIdx.x & 63;
		const int lane_row = lane & 31; /* the query row (or key row, or output column) this lane addresses inside a block of 32 */
		const int half_sel = lane >> 5;
		const int key_blocks = tokens_padded / 32;

		for (int query_block = wave; query_block < key_blocks; query_block += 4)
		{
			const int query = query_block * 32 + lane_row;
			const bool query_valid = query < tokens;
			uint4_t q_frag[Q_CHUNKS];
#pragma unroll
			for (int t = 0; t < Q_CHUNKS; t++)
			{
				q_frag[t] = uint4_t { 0u, 0u, 0u, 0u };
				if (query_valid)
					q_frag[t] = *reinterpret_cast<const uint4_t*>(reinterpret_cast<const uint8_t*>(tokens_base + static_cast<size_t>(query) * shape.token_stride)
							+ (2 * t + half_sel) * 16);
			}
			const int query_place = query_valid ? query : 0;
			const int query_h = query_place / shape.width;
			const int query_w = query_place - query_h * shape.width;
			/* BIAS_DIRECT: entry (r + key_h - query_h, r + key_w - query_w) = this lane's base + the key's part */
			const uint8_t *bias_base = reinterpret_cast<const uint8_t*>(bias) + ((range - query_h) * shape.table_row + (range - query_w)) * 4;

			float running_max = -INFINITY, running_sum = 0.0f;
			float16_t out[D_BLOCKS];
#pragma unroll
			for (int db = 0; db < D_BLOCKS; db++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					out[db][r] = 0.0f;

			for (int key_block = 0; key_block < key_blocks; key_block++)
			{
				/* scores of 32 queries x 32 keys: lane (query lane_row), register r: key 8 (r / 4) + 4 half_sel + r % 4 of the block */
				float16_t s;
#pragma unroll
				for (int r = 0; r < 16; r++)
					s[r] = 0.0f;
				const uint8_t *key_row = keys + (key_block * 32 + lane_row) * Lds::KEY_ROW + half_sel * 16;
#pragma unroll
				for (int t = 0; t < Q_CHUNKS; t++)
				{
					const uint4_t k_frag = *reinterpret_cast<const uint4_t*>(key_row + t * 32);
					Traits::mma(k_frag, q_frag[t], s);
				}
				float block_max = -INFINITY;
#pragma unroll
				for (int g = 0; g < 4; g++)
				{
					const int key0 = key_block * 32 + 8 * g + 4 * half_sel;
					const uint4_t key_place = *reinterpret_cast<const uint4_t*>(place + key0);
#pragma unroll
					for (int e = 0; e < 4; e++)
					{
						float value = s[4 * g + e] * scale;
						if constexpr (BIAS == BIAS_DIRECT)
							value = value + *reinterpret_cast<const float*>(bias_base + key_place[e]);
						else if constexpr (BIAS == BIAS_CLAMPED)
						{
							const int dh = clamp_int(static_cast<int>(key_place[e] >> 16) - query_h, -range, range);
							const int dw = clamp_int(static_cast<int>(key_place[e] & 0xffffu) - query_w, -range, range);
							value = value + bias[(range + dh) * shape.table_row + range + dw];
						}
						s[4 * g + e] = value;
					}
				}
				if (key_block == key_blocks - 1 && tokens != tokens_padded) /* the ragged last block: keys past the end do not take part */
				{
#pragma unroll
					for (int r = 0; r < 16; r++)
						s[r] = (key_block * 32 + 8 * (r / 4) + 4 * half_sel + (r % 4) < tokens) ? s[r] : -INFINITY;
				}
#pragma unroll
				for (int r = 0; r < 16; r++)
					block_max = fmaxf(block_max, s[r]);
				block_max = fmaxf(block_max, __shfl_xor(block_max, 32));
				const float new_max = fmaxf(running_max, block_max);
				const float rescale = __builtin_amdgcn_exp2f(running_max - new_max);
				float block_sum = 0.0f;
#pragma unroll
				for (int r = 0; r < 16; r++)
				{
					s[r] = __builtin_amdgcn_exp2f(s[r] - new_max);
					block_sum += s[r];
				}
				block_sum += __shfl_xor(block_sum, 32);
				running_sum = running_sum * rescale + block_sum;
				running_max = new_max;
#pragma unroll
				for (int db = 0; db < D_BLOCKS; db++)
#pragma unroll
					for (int r = 0; r < 16; r++)
						out[db][r] *= rescale;

				/* out[query][d] += sum over the block's keys of p[query][key] * v[key][d]; the values are the MFMA's first operand so that
				 * the result keeps one query row per lane: lane (query lane_row), register r: d = 8 (r / 4) + 4 half_sel + r % 4 */
#pragma unroll
				for (int g = 0; g < P_GROUPS; g++)
				{
					uint4_t p_frag;
					int first_key, second_key; /* where this lane's two runs of keys of the group start */
					if constexpr (ES == 2)
					{
						p_frag = uint4_t { pack_halfs(s[8 * g + 0], s[8 * g + 1]), pack_halfs(s[8 * g + 2], s[8 * g + 3]), pack_halfs(s[8 * g + 4], s[8 * g + 5]),
								pack_halfs(s[8 * g + 6], s[8 * g + 7]) };
						first_key = key_block * 32 + 16 * g + 4 * half_sel;
						second_key = first_key + 8;
					}
					else
					{
						p_frag = uint4_t { float_bits(s[4 * g + 0]), float_bits(s[4 * g + 1]), float_bits(s[4 * g + 2]), float_bits(s[4 * g + 3]) };
						first_key = key_block * 32 + 8 * g + 4 * half_sel;
						second_key = first_key + 2; /* the second half of the 16 bytes */
					}
#pragma unroll
					for (int db = 0; db < D_BLOCKS; db++)
					{
						const uint8_t *value_line = values + (db * 32 + lane_row) * value_row;
						const uint2_t lo = *reinterpret_cast<const uint2_t*>(value_line + first_key * ES);
						const uint2_t hi = *reinterpret_cast<const uint2_t*>(value_line + second_key * ES);
						const uint4_t v_frag = { lo[0], lo[1], hi[0], hi[1] };
						Traits::mma(v_frag, p_frag, out[db]);
					}
				}
			}

			if (query_valid)
			{
				const float inv_sum = 1.0f / running_sum;
				T *dst = output + (static_cast<size_t>(image) * tokens + query) * shape.embedding + head * D;
#pragma unroll
				for (int db = 0; db < D_BLOCKS; db++)
#pragma unroll
					for (int g = 0; g < 4; g++)
					{
						Vec<T, 4> y;
#pragma unroll
						for (int e = 0; e < 4; e++)
							y.v[e] = out[db][4 * g + e] * inv_sum;
						y.store(dst + db * 32 + 8 * g + 4 * half_sel);
					}
			}
		}
	}

	/*
	 * Plain kernel for every other shape: one wavefront per query row; the row of scores lives in LDS ([4 wavefronts][tokens] floats), the
	 * keys and values are read from memory (an image's head fits the caches).
	 */
	template<typename T>
	__global__ __launch_bounds__(256) void kernel_attention_plain(const T *__restrict__ input, T *__restrict__ output, const T *__restrict__ table,
			AttentionShape shape, int head_dim, int rows_total)
	{
		extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
		const int wave = threadIdx.x >> 6;
		const int lane = threadIdx.x & 63;
		const int tokens = shape.tokens;
		float *scores = reinterpret_cast<float*>(lds) + wave * tokens;
		const int range = (shape.table_size - 1) / 2;
		for (int row = blockIdx.x * 4 + wave; row < rows_total; row += gridDim.x * 4)
		{
			/* row = (image * heads + head) * tokens + query */
			const int query = row % tokens;
			const int head = (row / tokens) % shape.heads;
			const int image = row / (tokens * shape.heads);
			const T *tokens_base = input + static_cast<size_t>(image) * tokens * shape.token_stride + head * head_dim;
			const T *q = tokens_base + static_cast<size_t>(query) * shape.token_stride;
			const int query_h = query / shape.width, query_w = query - query_h * shape.width;
			const T *head_table = (shape.table_size > 0) ? table + static_cast<size_t>(head) * shape.table_size * shape.table_row : nullptr;
			float max_value = -INFINITY;
			for (int key = lane; key < tokens; key += 64)
			{
				const T *k = tokens_base + static_cast<size_t>(key) * shape.token_stride + shape.k_offset;
				float dot = 0.0f;
				for (int d = 0; d < head_dim; d++)
					dot = fmaf(Storage<T>::load(q + d), Storage<T>::load(k + d), dot);
				float value = dot * shape.scale;
				if (head_table != nullptr)
				{
					const int key_h = key / shape.width, key_w = key - key_h * shape.width;
					const int dh = clamp_int(key_h - query_h, -range, range), dw = clamp_int(key_w - query_w, -range, range);
					value = value + Storage<T>::load(head_table + (range + dh) * shape.table_row + range + dw);
				}
				scores[key] = value;
				max_value = fmaxf(max_value, value);
			}
			max_value = wave_max(max_value);
			float sum = 0.0f;
			for (int key = lane; key < tokens; key += 64)
			{
				const float p = expf(scores[key] - max_value);
				scores[key] = p;
				sum += p;
			}
			sum = wave_sum(sum);
			const float inv_sum = 1.0f / sum;
			T *dst = output + (static_cast<size_t>(image) * tokens + query) * shape.embedding + head * head_dim;
			for (int d = lane; d < head_dim; d += 64)
			{
				float acc = 0.0f;
				const T *v = tokens_base + shape.v_offset + d;
				for (int key = 0; key < tokens; key++)
					acc = fmaf(scores[key] * inv_sum, Storage<T>::load(v + static_cast<size_t>(key) * shape.token_stride), acc);
				Storage<T>::store(dst + d, acc);
			}
		}
	}

	constexpr int MAX_ATTENTION_LDS = 160 * 1024;

	template<typename T, int D>
	bool try_launch_attention_mfma(hipStream_t stream, const T *input, T *output, const T *table, const AttentionShape &shape, int batch)
	{
		typedef AttentionLds<T, D> Lds;
		const int bytes = Lds::bytes(shape.tokens, shape.table_size, shape.table_row);
		if (bytes > MAX_ATTENTION_LDS)
			return false;
		const int height = shape.tokens / shape.width;
		const int bias = (shape.table_size == 0) ? BIAS_NONE : ((shape.table_size >= 2 * std::max(height, shape.width) - 1) ? BIAS_DIRECT : BIAS_CLAMPED);
		const void *kernel = nullptr;
		switch (bias)
		{
			case BIAS_NONE:
				kernel = reinterpret_cast<const void*>(&kernel_attention_mfma<T, D, BIAS_NONE>);
				break;
			case BIAS_DIRECT:
				kernel = reinterpret_cast<const void*>(&kernel_attention_mfma<T, D, BIAS_DIRECT>);
				break;
			default:
				kernel = reinterpret_cast<const void*>(&kernel_attention_mfma<T, D, BIAS_CLAMPED>);
				break;
		}
		ensure_dynamic_lds(kernel, bytes);
		AttentionShape shape_arg = shape;
		void *args[] = { static_cast<void*>(&input), static_cast<void*>(&output), static_cast<void*>(&table), static_cast<void*>(&shape_arg) };
		MLHIP_CHECK(hipLaunchKernel(kernel, dim3(batch * shape.heads), dim3(256), args, bytes, stream));
		return true;
	}
	template<typename T>
	void launch_attention(hipStream_t stream, const T *input, T *output, const T *table, const AttentionShape &shape, int batch, int head_dim)
	{
		const bool aligned = (reinterpret_cast<uintptr_t>(input) % 16 == 0) && (reinterpret_cast<uintptr_t>(output) % 16 == 0)
				&& (static_cast<size_t>(shape.token_stride) * sizeof(T)) % 16 == 0;
		bool done = false;
		if (aligned && shape.tokens < 65536 && shape.width < 65536)
		{
			if (head_dim == 32)
				done = try_launch_attention_mfma<T, 32>(stream, input, output, table, shape, batch);
			else if (head_dim == 64)
				done = try_launch_attention_mfma<T, 64>(stream, input, output, table, shape, batch);
			else if (head_dim == 128)
				done = try_launch_attention_mfma<T, 128>(stream, input, output, table, shape, batch);
		}
		if (done)
			return;
		const int bytes = 4 * shape.tokens * static_cast<int>(sizeof(float));
		MLHIP_REQUIRE(bytes <= MAX_ATTENTION_LDS, "multi_head_attention_forward: too many tokens");
		const long long rows_total = static_cast<long long>(batch) * shape.heads * shape.tokens;
		MLHIP_REQUIRE(rows_total < (1ll << 31), "multi_head_attention_forward: too many rows");
		const void *kernel = reinterpret_cast<const void*>(&kernel_attention_plain<T>);
		ensure_dynamic_lds(kernel, bytes);
		const unsigned int groups = static_cast<unsigned int>(std::min<long long>((rows_total + 3) / 4, 65536));
		hipLaunchKernelGGL((kernel_attention_plain<T>), dim3(groups), dim3(256), bytes, stream, input, output, table, shape, head_dim,
				static_cast<int>(rows_total));
		MLHIP_CHECK(hipGetLastError());
	}
}

extern "C"
{
	using namespace mlhip;

	void hip_rmsnorm_forward(mlContext_t context, mlShape_t shape, mlDataType_t dtype, const void *input, void *output, const void *weights)
	try
	{
		if (volume(shape) == 0)
			return;
		MLHIP_REQUIRE(input != nullptr && output != nullptr, "rmsnorm_forward: null pointer");
		const int columns = last_dim(shape);
		const size_t rows = volume(shape) / columns;
		switch (dtype)
		{
			case DTYPE_FLOAT16:
				launch_rmsnorm(stream_of(context), reinterpret_cast<half_t*>(output), reinterpret_cast<const half_t*>(input),
						reinterpret_cast<const half_t*>(weights), rows, columns);
				break;
			case DTYPE_FLOAT32:
				launch_rmsnorm(stream_of(context), reinterpret_cast<float*>(output), reinterpret_cast<const float*>(input),
						reinterpret_cast<const float*>(weights), rows, columns);
				break;
			default:
				fail_logic("HIP backend: rmsnorm_forward: unsupported data type");
		}
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}

	/* elements of the caller's workspace: inference needs none here (the scores never leave the chip); the training count is the
	 * reference's (src/backend/cuda/kernels/attention.cu, src/backend/cpu/attention.cpp:303-313) for callers that size buffers by it */
	int hip_multi_head_attention_get_workspace_size(mlShape_t input_shape, mlShape_t weights_shape, int num_heads, bool training)
	try
	{
		if (!training)
			return 0;
		MLHIP_REQUIRE(input_shape.rank == 4, "multi_head_attention_get_workspace_size: input must be [B, H, W, C]");
		const int tokens = input_shape.dim[1] * input_shape.dim[2];
		return 2 * input_shape.dim[0] * num_heads * tokens * tokens;
	}
	catch (...)
	{
		return mlhip::entry_failed<int>();
	}

	void hip_multi_head_attention_forward(mlContext_t context, mlShape_t input_shape, mlShape_t weights_shape, mlShape_t bias_shape, mlDataType_t dtype,
			const void *input, void *output, const void *weights, const void *bias, void *workspace, void *backward_data, int num_heads, bool symmetric)
	try
	{
		MLHIP_REQUIRE(input_shape.rank == 4, "multi_head_attention_forward: input must be [B, H, W, C]");
		MLHIP_REQUIRE(num_heads > 0, "multi_head_attention_forward: number of heads must be positive");
		const int parts = symmetric ? 2 : 3;
		MLHIP_REQUIRE(input_shape.dim[3] % parts == 0, "multi_head_attention_forward: channels must hold q, k and v (q and v when symmetric)");
		const int embedding = input_shape.dim[3] / parts;
		MLHIP_REQUIRE(embedding % num_heads == 0, "multi_head_attention_forward: embedding must be divisible by the number of heads");
		if (backward_data != nullptr)
			fail_runtime("HIP backend: multi_head_attention_forward: keeping the attention matrix for a backward pass is not implemented (inference only)");
		if (volume(input_shape) == 0)
			return;
		MLHIP_REQUIRE(input != nullptr && output != nullptr, "multi_head_attention_forward: null pointer");
		AttentionShape shape;
		shape.tokens = input_shape.dim[1] * input_shape.dim[2];
		shape.width = input_shape.dim[2];
		shape.heads = num_heads;
		shape.embedding = embedding;
		shape.token_stride = input_shape.dim[3];
		shape.k_offset = symmetric ? 0 : embedding;
		shape.v_offset = (parts - 1) * embedding;
		shape.table_size = 0;
		shape.table_row = 0;
		if (weights != nullptr)
		{
			MLHIP_REQUIRE(weights_shape.rank == 3 && weights_shape.dim[0] == num_heads && weights_shape.dim[1] % 2 == 1
					&& weights_shape.dim[2] == (weights_shape.dim[1] + 3) / 4 * 4,
					"multi_head_attention_forward: the position table must be [heads, 2r-1, round_up(2r-1, 4)]");
			shape.table_size = weights_shape.dim[1];
			shape.table_row = weights_shape.dim[2];
		}
		const int head_dim = embedding / num_heads;
		shape.scale = static_cast<float>(1.0 / std::sqrt(static_cast<double>(head_dim))); /* the reference takes the root of an int: in double */
		switch (dtype)
		{
			case DTYPE_FLOAT16:
				launch_attention(stream_of(context), reinterpret_cast<const half_t*>(input), reinterpret_cast<half_t*>(output),
						reinterpret_cast<const half_t*>(weights), shape, input_shape.dim[0], head_dim);
				break;
			case DTYPE_FLOAT32:
				launch_attention(stream_of(context), reinterpret_cast<const float*>(input), reinterpret_cast<float*>(output),
						reinterpret_cast<const float*>(weights), shape, input_shape.dim[0], head_dim);
				break;
			default:
				fail_logic("HIP backend: multi_head_attention_forward: unsupported data type");
		}
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}

	MLHIP_ALSO_AS_CUDA(rmsnorm_forward)
	MLHIP_ALSO_AS_CUDA(multi_head_attention_get_workspace_size)
	MLHIP_ALSO_AS_CUDA(multi_head_attention_forward)
}
