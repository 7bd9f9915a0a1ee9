/*
 * moe.hip — mixture-of-experts steps of the hybrid networks' feed-forward blocks: routing (expert choice, token choice, hash),
 * gathering the routed tokens per expert, the per-expert dense layers, and scattering the experts' results back to their tokens.
 *
 * Interface and tensor layouts follow the reference's device backend (declarations: include/minml/backend/cuda_backend.h:245-265;
 * kernels: src/backend/cuda/kernels/moe.cu; callers: src/layers/{Router,GatherTokens,MixtureOfExperts,ScatterTokens}.cpp). The reference
 * has no CPU implementation of these operations (src/core/math.cpp:1328-1491), so their arithmetic is fixed here where its kernels
 * leave it open: equal scores are ordered by ascending token index (the reference: by its sorting network), and the scatter sums a
 * token's contributions in fp32 in ascending expert order and rounds once (the reference: atomic additions in the storage type).
 *
 *   scores                 [B, H, W, E]      one router logit per token and expert
 *   indices_and_values     [B, 2, E, K]      storage type; plane 0 = token index of slot k of expert e (as a number, -1 = empty), plane 1 = gate
 *   gathered tokens        [B, K, E, C]
 *   expert weights / bias  [E, N, C] / [E, N]
 */
#include "common.hpp"
#include "device_utils.hpp"
#include "epilogues.hpp"
#include "gemm_dma.hpp"
#include "gemm_stream.hpp"

namespace
{
	using namespace mlhip;

	constexpr int MAX_ROUTED_TOKENS = 2048; /* tokens per image that the in-LDS sorts take */

	__device__ __forceinline__ uint32_t ascending_bits(float v)
	{
		const uint32_t u = __builtin_bit_cast(uint32_t, v);
		return u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
	}
	__device__ __forceinline__ float from_ascending_bits(uint32_t s)
	{
		const uint32_t u = s ^ ((s >> 31) ? 0x80000000u : 0xffffffffu);
		return __builtin_bit_cast(float, u);
	}
	/* in-place bitonic sort of `count` (a power of two) 64-bit keys in LDS, ascending; all threads of the workgroup take part */
	__device__ __forceinline__ void sort_keys(uint64_t *keys, int count)
	{
		for (int k = 2; k <= count; k <<= 1)
			for (int j = k >> 1; j > 0; j >>= 1)
			{
				for (int i = threadIdx.x; i < count; i += blockDim.x)
				{
					const int partner = i ^ j;
					if (partner > i)
					{
						const bool ascending = ((i & k) == 0);
						const uint64_t a = keys[i], b = keys[partner];
						if ((a > b) == ascending)
						{
							keys[i] = b;
							keys[partner] = a;
						}
					}
				}
				__syncthreads();
			}
	}
	__device__ __forceinline__ int next_power_of_two(int n)
	{
		int p = 1;
		while (p < n)
			p <<= 1;
		return p;
	}

	/* one workgroup per (expert, image): the expert's `capacity` best tokens, best first, gate = sigmoid(score) */
	template<typename T>
	__global__ __launch_bounds__(256) void kernel_expert_choice_routing(const T *scores, T *indices_and_values, int tokens, int experts, int capacity)
	{
		__shared__ uint64_t keys[MAX_ROUTED_TOKENS];
		const int e = blockIdx.x, b = blockIdx.y;
		const int padded = next_power_of_two(tokens);
		for (int t = threadIdx.x; t < padded; t += blockDim.x)
		{
			uint64_t key = ~0ull;
			if (t < tokens)
			{
				const float s = Storage<T>::load(scores + (static_cast<size_t>(b) * tokens + t) * experts + e);
				key = (static_cast<uint64_t>(~ascending_bits(s)) << 32) | static_cast<uint32_t>(t); /* score descending, then token ascending */
			}
			keys[t] = key;
		}
		__syncthreads();
		sort_keys(keys, padded);
		T *index_row = indices_and_values + ((static_cast<size_t>(b) * 2 + 0) * experts + e) * capacity;
		T *value_row = indices_and_values + ((static_cast<size_t>(b) * 2 + 1) * experts + e) * capacity;
		for (int k = threadIdx.x; k < capacity; k += blockDim.x)
		{
			if (k < tokens)
			{
				const uint64_t key = keys[k];
				const float s = from_ascending_bits(~static_cast<uint32_t>(key >> 32));
				Storage<T>::store(index_row + k, static_cast<float>(static_cast<uint32_t>(key)));
				Storage<T>::store(value_row + k, 1.0f / (1.0f + expf(-s)));
			}
			else
			{
				Storage<T>::store(index_row + k, -1.0f);
				Storage<T>::store(value_row + k, 0.0f);
			}
		}
	}

	/*
	 * One workgroup per image. Every token takes the expert with the largest score + bias (the lowest index among equals); its gate is
	 * softmax(scores)[that expert] with the maximum of score + bias as the shift, kept in the storage type; the tokens are then sorted
	 * by (expert, gate descending, token) and every expert keeps the first `capacity` of its run.
	 */
	template<typename T>
	__global__ __launch_bounds__(256) void kernel_token_choice_routing(const T *scores, const T *bias, T *indices_and_values, int tokens, int experts,
			int capacity)
	{
		__shared__ uint64_t keys[MAX_ROUTED_TOKENS];
		__shared__ int first[4096 + 1]; /* first[e] = position of expert e's run in the sorted keys, -1 if it has none; count in last[e] */
		__shared__ int last[4096 + 1];
		const int b = blockIdx.x;
		const int padded = next_power_of_two(tokens);
		for (int e = threadIdx.x; e < experts; e += blockDim.x)
		{
			first[e] = -1;
			last[e] = -1;
		}
		for (int t = threadIdx.x; t < padded; t += blockDim.x)
		{
			uint64_t key = ~0ull;
			if (t < tokens)
			{
				const T *row = scores + (static_cast<size_t>(b) * tokens + t) * experts;
				float best = 0.0f;
				int choice = 0;
				for (int e = 0; e < experts; e++)
				{
					const float plus = Storage<T>::load(row + e) + ((bias != nullptr) ? Storage<T>::load(bias + e) : 0.0f);
					if (e == 0 || plus > best)
					{
						best = plus;
						choice = e;
					}
				}
				float total = 0.0f;
				for (int e = 0; e < experts; e++)
					total = total + expf(Storage<T>::load(row + e) - best);
				float gate = expf(Storage<T>::load(row + choice) - best) / total;
				if constexpr (sizeof(T) == 2)
					gate = half_bits_to_float(half_bits_rtz(gate));
				key = (static_cast<uint64_t>(choice) << 52) | (static_cast<uint64_t>(~ascending_bits(gate)) << 20) | static_cast<uint64_t>(t);
			}
			keys[t] = key;
		}
		__syncthreads();
		sort_keys(keys, padded);
		for (int p = threadIdx.x; p < tokens; p += blockDim.x)
		{
			const int e = static_cast<int>(keys[p] >> 52);
			if (p == 0 || static_cast<int>(keys[p - 1] >> 52) != e)
				first[e] = p;
			if (p + 1 == tokens || static_cast<int>(keys[p + 1] >> 52) != e)
				last[e] = p;
		}
		__syncthreads();
		for (int i = threadIdx.x; i < experts * capacity; i += blockDim.x)
		{
			const int e = i / capacity, k = i - e * capacity;
			T *index_slot = indices_and_values + ((static_cast<size_t>(b) * 2 + 0) * experts + e) * capacity + k;
			T *value_slot = indices_and_values + ((static_cast<size_t>(b) * 2 + 1) * experts + e) * capacity + k;
			if (first[e] >= 0 && first[e] + k <= last[e])
			{
				const uint64_t key = keys[first[e] + k];
				Storage<T>::store(index_slot, static_cast<float>(static_cast<uint32_t>(key & 0xfffffu)));
				Storage<T>::store(value_slot, from_ascending_bits(~static_cast<uint32_t>(key >> 20)));
			}
			else
			{
				Storage<T>::store(index_slot, -1.0f);
				Storage<T>::store(value_slot, 0.0f);
			}
		}
	}

	template<typename T>
	__global__ __launch_bounds__(256) void kernel_hash_routing(T *indices_and_values, int batch, int tokens, int experts, int capacity)
	{
		const size_t total = static_cast<size_t>(batch) * experts * capacity;
		for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += static_cast<size_t>(gridDim.x) * blockDim.x)
		{
			const int k = static_cast<int>(i % capacity);
			const int e = static_cast<int>((i / capacity) % experts);
			const size_t b = i / (static_cast<size_t>(capacity) * experts);
			const int token = k * experts + e;
			const bool filled = token < tokens;
			Storage<T>::store(indices_and_values + ((b * 2 + 0) * experts + e) * capacity + k, filled ? static_cast<float>(token) : -1.0f);
			Storage<T>::store(indices_and_values + ((b * 2 + 1) * experts + e) * capacity + k, filled ? 1.0f : 0.0f);
		}
	}

	/* one thread per group of VEC channels of one gathered row (b, k, e) */
	template<typename T, int VEC>
	__global__ __launch_bounds__(256) void kernel_gather_tokens(const T *x, const T *indices_and_values, T *y, float beta, size_t groups, int tokens, int channels,
			int experts, int capacity)
	{
		const int per_row = channels / VEC;
		for (size_t g = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; g < groups; g += static_cast<size_t>(gridDim.x) * blockDim.x)
		{
			const size_t row = g / per_row; /* (b * K + k) * E + e */
			const int c = static_cast<int>(g - row * per_row) * VEC;
			const int e = static_cast<int>(row % experts);
			const size_t bk = row / experts;
			const int k = static_cast<int>(bk % capacity);
			const size_t b = bk / capacity;
			const int token = static_cast<int>(Storage<T>::load(indices_and_values + ((b * 2 + 0) * experts + e) * capacity + k));
			Vec<T, VEC> out;
			out.zero();
			if (beta != 0.0f)
			{
				out.load(y + row * channels + c);
#pragma unroll
				for (int i = 0; i < VEC; i++)
					out.v[i] *= beta;
			}
			if (token >= 0)
			{
				Vec<T, VEC> in;
				in.load(x + (b * tokens + token) * channels + c);
#pragma unroll
				for (int i = 0; i < VEC; i++)
					out.v[i] = in.v[i] + out.v[i];
			}
			out.store(y + row * channels + c);
		}
	}

	/* the same for fewer than 2^32 groups: the flat index is split by multiplications instead of 64-bit divisions, which were most of
	 * the instructions of a thread that moves 16 bytes; whether the old value takes part is fixed at compile time */
	template<typename T, int VEC, bool WITH_BETA>
	__global__ __launch_bounds__(256) void kernel_gather_tokens_fast(const T *x, const T *indices_and_values, T *y, float beta, uint32_t groups, int tokens,
			int channels, FastDivisor by_pieces, FastDivisor by_experts, FastDivisor by_capacity)
	{
		const uint32_t experts = by_experts.divisor, capacity = by_capacity.divisor;
		for (uint64_t g64 = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; g64 < groups; g64 += static_cast<uint64_t>(gridDim.x) * blockDim.x)
		{
			uint32_t piece, e, k;
			const uint32_t row = fast_divide(static_cast<uint32_t>(g64), by_pieces, piece); /* (b * K + k) * E + e */
			const uint32_t bk = fast_divide(row, by_experts, e);
			const uint32_t b = fast_divide(bk, by_capacity, k);
			const int c = static_cast<int>(piece) * VEC;
			const int token = static_cast<int>(Storage<T>::load(indices_and_values + (static_cast<size_t>(b * 2u) * experts + e) * capacity + k));
			Vec<T, VEC> out;
			out.zero();
			T *y_piece = y + static_cast<size_t>(row) * channels + c;
			if constexpr (WITH_BETA)
			{
				out.load(y_piece);
#pragma unroll
				for (int i = 0; i < VEC; i++)
					out.v[i] *= beta;
			}
			if (token >= 0)
			{
				Vec<T, VEC> in;
				in.load(x + (static_cast<size_t>(b) * tokens + token) * channels + c);
#pragma unroll
				for (int i = 0; i < VEC; i++)
					out.v[i] = in.v[i] + out.v[i];
			}
			out.store(y_piece);
		}
	}

	/*
	 * One wavefront per token and block of 64 * VEC channels: the slots that hold the token are found by scanning the image's index
	 * table expert by expert (a token occupies at most one slot per expert), and their gated rows are summed in fp32 in that order.
	 */
	template<typename T, int VEC>
	__global__ __launch_bounds__(256) void kernel_scatter_tokens(const T *x, const T *indices_and_values, T *y, float beta, size_t total_tokens, int tokens,
			int channels, int experts, int capacity)
	{
#pragma clang fp contract(off)
		const int lane = threadIdx.x & 63;
		const size_t slot = static_cast<size_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
		const int channel_blocks = (channels + 64 * VEC - 1) / (64 * VEC);
		const size_t global_token = slot / channel_blocks;
		if (global_token >= total_tokens)
			return;
		const int c = (static_cast<int>(slot % channel_blocks) * 64 + lane) * VEC;
		const size_t b = global_token / tokens;
		const int token = static_cast<int>(global_token - b * tokens);
		const bool active = c < channels;
		Vec<T, VEC> acc;
		acc.zero();
		if (beta != 0.0f && active)
		{
			acc.load(y + global_token * channels + c);
#pragma unroll
			for (int i = 0; i < VEC; i++)
				acc.v[i] *= beta;
		}
		/*
		 * Experts are taken eight at a time: first the index rows of all eight are scanned (independent loads, one ballot each per 64
		 * slots), then their gates and rows are requested together, then the rows are added in expert order. A wavefront that looked
		 * for one expert's slot, loaded its row and only then turned to the next expert spent its time waiting for eight chains of
		 * dependent loads.
		 */
		constexpr int GROUP = 8;
		const T *index_plane = indices_and_values + (b * 2 + 0) * experts * capacity;
		const T *gate_plane = indices_and_values + (b * 2 + 1) * experts * capacity;
		for (int e0 = 0; e0 < experts && capacity > 0; e0 += GROUP)
		{
			int found[GROUP];
#pragma unroll
			for (int i = 0; i < GROUP; i++)
				found[i] = -1;
			for (int k0 = 0; k0 < capacity; k0 += 64)
			{
				const int k = min(k0 + lane, capacity - 1);
				int index[GROUP];
#pragma unroll
				for (int i = 0; i < GROUP; i++)
					index[i] = static_cast<int>(Storage<T>::load(index_plane + static_cast<size_t>(min(e0 + i, experts - 1)) * capacity + k));
#pragma unroll
				for (int i = 0; i < GROUP; i++)
				{
					const unsigned long long hits = __ballot(k0 + lane < capacity && e0 + i < experts && index[i] == token);
					if (hits != 0ull && found[i] < 0) /* a token holds at most one slot per expert; of duplicates in a hand-made table the lowest counts */
						found[i] = k0 + __builtin_ctzll(hits);
				}
			}
			float gate[GROUP];
			Vec<T, VEC> in[GROUP];
#pragma unroll
			for (int i = 0; i < GROUP; i++)
			{
				const int e = min(e0 + i, experts - 1), slot_k = max(found[i], 0);
				gate[i] = Storage<T>::load(gate_plane + static_cast<size_t>(e) * capacity + slot_k);
				in[i].zero();
				if (active)
					in[i].load(x + ((b * capacity + slot_k) * experts + e) * channels + c);
			}
#pragma unroll
			for (int i = 0; i < GROUP; i++)
				if (found[i] >= 0)
				{
#pragma unroll
					for (int v = 0; v < VEC; v++)
					{
						const float scaled = gate[i] * in[i].v[v];
						acc.v[v] = acc.v[v] + scaled;
					}
				}
		}
		if (active)
			acc.store(y + global_token * channels + c);
	}

	/*
	 * The same sum with the search taken out of the wavefronts' critical path. One workgroup serves a range of the tokens of ONE image.
	 * It first inverts the image's routing table for its tokens in LDS (inverse[token][expert] = the lowest slot of that expert holding
	 * the token, or "none") and compacts every token's row of that table into a list of (row of the expert outputs, gate) in expert
	 * order; then every wavefront walks its tokens: it reads a token's count and list from LDS into scalar registers and requests all
	 * of the token's rows at once (up to four per step; the count selects a fully unrolled form). Same additions in the same order as
	 * kernel_scatter_tokens, hence the same bits.
	 *
	 * The kernel is bound by the number of instructions a wavefront issues per token, not by memory: a version that requested all
	 * `experts` rows of every token (absent ones at an offset outside the buffer, skipped by a select) took as long with every request
	 * outside the buffer as with the real ones. Hence the compact lists (no work for absent experts), the rows' addresses as scalar
	 * offsets of a buffer descriptor (no per-lane address arithmetic) and no division in the token loop.
	 */
	constexpr int SCATTER_NONE = 0x7fffffff;
	constexpr int SCATTER_OUTSIDE = 0x40000000; /* offset that lies past the end of the descriptor used here */
	template<typename T, int VEC>
	__device__ __forceinline__ Vec<T, VEC> scatter_load_row(__amdgpu_buffer_rsrc_t r, int lane_offset, int row_offset)
	{
		Vec<T, VEC> out;
		if constexpr (VEC == 1 && sizeof(T) == 4)
			out.v[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, lane_offset, row_offset, 0));
		else if constexpr (VEC == 1)
			out.v[0] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(__builtin_amdgcn_raw_buffer_load_b16(r, lane_offset, row_offset, 0))));
		else if constexpr (sizeof(T) == 4)
		{
			static_assert(VEC == 4, "rows move 16 bytes per lane");
			typedef uint32_t words __attribute__((ext_vector_type(4)));
			const words w = __builtin_amdgcn_raw_buffer_load_b128(r, lane_offset, row_offset, 0);
#pragma unroll
			for (int i = 0; i < 4; i++)
				out.v[i] = __builtin_bit_cast(float, static_cast<uint32_t>(w[i]));
		}
		else
		{
			static_assert(VEC == 4, "rows move 8 bytes per lane");
			typedef _Float16 halves __attribute__((ext_vector_type(4)));
			const halves h = __builtin_bit_cast(halves, __builtin_amdgcn_raw_buffer_load_b64(r, lane_offset, row_offset, 0));
#pragma unroll
			for (int i = 0; i < 4; i++)
				out.v[i] = static_cast<float>(h[i]);
		}
		return out;
	}
	/* adds N listed contributions to acc: all rows requested before the first is used */
	template<typename T, int VEC, int N>
	__device__ __forceinline__ void scatter_add_listed(Vec<T, VEC> &acc, const int *list, __amdgpu_buffer_rsrc_t rows, int lane_offset, int row_bytes)
	{
#pragma clang fp contract(off)
		int row[N];
		float gate[N];
		Vec<T, VEC> in[N];
#pragma unroll
		for (int i = 0; i < N; i++)
		{
			row[i] = __builtin_amdgcn_readfirstlane(list[2 * i]);
			gate[i] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(list[2 * i + 1]));
		}
#pragma unroll
		for (int i = 0; i < N; i++)
			in[i] = scatter_load_row<T, VEC>(rows, lane_offset, row[i] * row_bytes);
#pragma unroll
		for (int i = 0; i < N; i++)
#pragma unroll
			for (int v = 0; v < VEC; v++)
			{
				const float scaled = gate[i] * in[i].v[v];
				acc.v[v] = acc.v[v] + scaled;
			}
	}
	/* dynamic LDS of kernel_scatter_tokens_by_image for `per_part` tokens per workgroup: inverse table, lists of (row, gate), counts */
	inline size_t scatter_by_image_lds_bytes(int per_part, int experts)
	{
		return static_cast<size_t>(per_part) * (static_cast<size_t>(experts) * 3 + 1) * sizeof(int);
	}
	template<typename T, int VEC, bool WITH_BETA>
	__global__ __launch_bounds__(256) void kernel_scatter_tokens_by_image(const T *x, const T *indices_and_values, T *y, float beta, int tokens, int channels,
			int experts, int capacity, int splits)
	{
#pragma clang fp contract(off)
		extern __shared__ int scatter_lds[];
		const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
		const size_t b = blockIdx.x / splits;
		const int part = blockIdx.x % splits;
		const int per_part = (tokens + splits - 1) / splits;
		const int first = part * per_part, mine = max(min(tokens, first + per_part) - first, 0); /* this workgroup's tokens: first ... first + mine - 1 */
		int *inverse = scatter_lds; /* [per_part][experts] */
		int *lists = inverse + per_part * experts; /* [per_part][experts][2]: row of the image's expert outputs, gate as fp32 bits */
		int *count = lists + per_part * experts * 2; /* [per_part] */
		const T *index_plane = indices_and_values + (b * 2 + 0) * experts * capacity;
		const T *gate_plane = indices_and_values + (b * 2 + 1) * experts * capacity;
		for (int i = threadIdx.x; i < mine * experts; i += blockDim.x)
			inverse[i] = SCATTER_NONE;
		__syncthreads();
		for (int i = threadIdx.x; i < experts * capacity; i += blockDim.x)
		{
			const int e = i / capacity, k = i - e * capacity;
			const int token = static_cast<int>(Storage<T>::load(index_plane + i)) - first;
			if (token >= 0 && token < mine)
				atomicMin(&inverse[token * experts + e], k); /* of duplicates in a hand-made table the lowest slot counts */
		}
		__syncthreads();
		for (int t = threadIdx.x; t < mine; t += blockDim.x)
		{
			int n = 0;
			for (int e = 0; e < experts; e++)
			{
				const int slot = inverse[t * experts + e];
				if (slot != SCATTER_NONE)
				{
					lists[(t * experts + n) * 2 + 0] = slot * experts + e;
					lists[(t * experts + n) * 2 + 1] = __builtin_bit_cast(int, Storage<T>::load(gate_plane + e * capacity + slot));
					n++;
				}
			}
			count[t] = n;
		}
		__syncthreads();
		/* the image's expert outputs [capacity][experts][channels] behind a buffer descriptor: a row is a scalar offset, a lane's place in
		 * it the vector offset, and a lane past the end of the row asks outside the buffer, which returns zeros and moves nothing */
		const int row_bytes = channels * static_cast<int>(sizeof(T));
		const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(x + b * capacity * experts * channels), 0,
				capacity * experts * row_bytes, 0x00020000);
		const int channel_blocks = (channels + 64 * VEC - 1) / (64 * VEC);
		const int waves = blockDim.x >> 6;
		for (int t = wave; t < mine; t += waves)
		{
			const int n = __builtin_amdgcn_readfirstlane(count[t]);
			T *y_row = y + (b * tokens + first + t) * channels;
			for (int block = 0; block < channel_blocks; block++)
			{
				const int c = (block * 64 + lane) * VEC;
				const bool active = c < channels;
				const int lane_offset = active ? c * static_cast<int>(sizeof(T)) : SCATTER_OUTSIDE;
				Vec<T, VEC> acc;
				acc.zero();
				if constexpr (WITH_BETA)
				{
					acc.load(y_row + (active ? c : 0));
#pragma unroll
					for (int i = 0; i < VEC; i++)
						acc.v[i] *= beta;
				}
				for (int j = 0; j < n; j += 4)
				{
					const int *list = lists + (t * experts + j) * 2;
					switch (min(n - j, 4))
					{
						case 1:
							scatter_add_listed<T, VEC, 1>(acc, list, rows, lane_offset, row_bytes);
							break;
						case 2:
							scatter_add_listed<T, VEC, 2>(acc, list, rows, lane_offset, row_bytes);
							break;
						case 3:
							scatter_add_listed<T, VEC, 3>(acc, list, rows, lane_offset, row_bytes);
							break;
						default:
							scatter_add_listed<T, VEC, 4>(acc, list, rows, lane_offset, row_bytes);
							break;
					}
				}
				if (active)
					acc.store(y_row + c);
			}
		}
	}

	/* fallback of the expert layers for shapes the tile engine does not take: one thread per output element */
	template<typename T>
	__global__ __launch_bounds__(256) void kernel_moe_generic(const T *x, const T *w, const T *bias, T *y, float beta, size_t outputs, int experts, int neurons,
			int channels, int act)
	{
		for (size_t o = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; o < outputs; o += static_cast<size_t>(gridDim.x) * blockDim.x)
		{
			const int n = static_cast<int>(o % neurons);
			const size_t row = o / neurons; /* (b * K + k) * E + e */
			const int e = static_cast<int>(row % experts);
			const T *a = x + row * channels;
			const T *wr = w + (static_cast<size_t>(e) * neurons + n) * channels;
			float acc = 0.0f;
			for (int c = 0; c < channels; c++)
				acc = fmaf(Storage<T>::load(a + c), Storage<T>::load(wr + c), acc);
			if (bias != nullptr)
				acc += Storage<T>::load(bias + static_cast<size_t>(e) * neurons + n);
			if (beta != 0.0f)
				acc += beta * Storage<T>::load(y + o);
			if (act == ACTIVATION_RELU)
				acc = fmaxf(acc, 0.0f);
			else if (act != ACTIVATION_LINEAR)
			{
				if constexpr (sizeof(T) == 2)
					acc = half_bits_to_float(half_bits_rtz(acc));
				acc = activate(act, acc);
			}
			Storage<T>::store(y + o, acc);
		}
	}

	unsigned int grid_for(size_t items)
	{
		const size_t blocks = (items + 255) / 256;
		return static_cast<unsigned int>(blocks < 65536 * 16 ? (blocks > 0 ? blocks : 1) : 65536 * 16);
	}
	void require_routing_tensors(const mlTensor_t &x, const mlTensor_t &iv, const char *what)
	{
		MLHIP_REQUIRE(x.rank == 4 && iv.rank == 4 && iv.dim[1] == 2, std::string(what) + ": scores must be [B, H, W, E] and the routing table [B, 2, E, K]");
		MLHIP_REQUIRE(x.dim[0] == iv.dim[0] && x.dim[3] == iv.dim[2], std::string(what) + ": batch size or number of experts differ");
		MLHIP_REQUIRE(x.dtype == iv.dtype && (x.dtype == DTYPE_FLOAT16 || x.dtype == DTYPE_FLOAT32), std::string(what) + ": fp16 or fp32 tensors of one type");
		MLHIP_REQUIRE(x.dim[1] * x.dim[2] <= MAX_ROUTED_TOKENS, std::string(what) + ": at most 2048 tokens per image");
		MLHIP_REQUIRE(iv.dim[2] <= 4096 && x.dim[1] * x.dim[2] < (1 << 20), std::string(what) + ": too many experts");
	}
	template<typename T>
	bool vector_ok(int channels, int vec, const void *a, const void *b)
	{
		const size_t bytes = sizeof(T) * vec;
		return channels % vec == 0 && reinterpret_cast<uintptr_t>(a) % bytes == 0 && reinterpret_cast<uintptr_t>(b) % bytes == 0;
	}
}

extern "C"
{
	using namespace mlhip;

	void hip_expert_choice_routing_forward(mlContext_t context, const mlTensor_t x, mlTensor_t indices_and_values)
	try
	{
		require_routing_tensors(x, indices_and_values, "expert_choice_routing_forward");
		const int batch = x.dim[0], tokens = x.dim[1] * x.dim[2], experts = x.dim[3], capacity = indices_and_values.dim[3];
		if (batch == 0 || experts == 0 || capacity == 0)
			return;
		MLHIP_REQUIRE(x.data != nullptr && indices_and_values.data != nullptr && batch <= 65535, "expert_choice_routing_forward: null tensor or batch above 65535");
		const dim3 grid(experts, batch);
		if (x.dtype == DTYPE_FLOAT16)
			hipLaunchKernelGGL(kernel_expert_choice_routing<half_t>, grid, dim3(256), 0, stream_of(context), ptr<const half_t>(x), ptr<half_t>(indices_and_values),
					tokens, experts, capacity);
		else
			hipLaunchKernelGGL(kernel_expert_choice_routing<float>, grid, dim3(256), 0, stream_of(context), ptr<const float>(x), ptr<float>(indices_and_values),
					tokens, experts, capacity);
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_token_choice_routing_forward(mlContext_t context, const mlTensor_t x, const mlTensor_t bias, mlTensor_t indices_and_values)
	try
	{
		require_routing_tensors(x, indices_and_values, "token_choice_routing_forward");
		const int batch = x.dim[0], tokens = x.dim[1] * x.dim[2], experts = x.dim[3], capacity = indices_and_values.dim[3];
		if (batch == 0 || experts == 0 || capacity == 0)
			return;
		if (bias.data != nullptr)
			MLHIP_REQUIRE(bias.dtype == x.dtype && volume(bias) == static_cast<size_t>(experts), "token_choice_routing_forward: bias must be [E] of the scores' type");
		MLHIP_REQUIRE(x.data != nullptr && indices_and_values.data != nullptr, "token_choice_routing_forward: null tensor");
		if (x.dtype == DTYPE_FLOAT16)
			hipLaunchKernelGGL(kernel_token_choice_routing<half_t>, dim3(batch), dim3(256), 0, stream_of(context), ptr<const half_t>(x), ptr<const half_t>(bias),
					ptr<half_t>(indices_and_values), tokens, experts, capacity);
		else
			hipLaunchKernelGGL(kernel_token_choice_routing<float>, dim3(batch), dim3(256), 0, stream_of(context), ptr<const float>(x), ptr<const float>(bias),
					ptr<float>(indices_and_values), tokens, experts, capacity);
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_hash_routing(mlContext_t context, const mlTensor_t x, mlTensor_t indices_and_values)
	try
	{
		require_routing_tensors(x, indices_and_values, "hash_routing");
		const int batch = x.dim[0], tokens = x.dim[1] * x.dim[2], experts = x.dim[3], capacity = indices_and_values.dim[3];
		const size_t total = static_cast<size_t>(batch) * experts * capacity;
		if (total == 0)
			return;
		MLHIP_REQUIRE(indices_and_values.data != nullptr, "hash_routing: null tensor");
		if (x.dtype == DTYPE_FLOAT16)
			hipLaunchKernelGGL(kernel_hash_routing<half_t>, dim3(grid_for(total)), dim3(256), 0, stream_of(context), ptr<half_t>(indices_and_values), batch, tokens,
					experts, capacity);
		else
			hipLaunchKernelGGL(kernel_hash_routing<float>, dim3(grid_for(total)), dim3(256), 0, stream_of(context), ptr<float>(indices_and_values), batch, tokens,
					experts, capacity);
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}

	void hip_gather_tokens_forward(mlContext_t context, const mlTensor_t x, const mlTensor_t indices_and_values, float beta, mlTensor_t y)
	try
	{
		MLHIP_REQUIRE(x.rank == 4 && y.rank == 4 && indices_and_values.rank == 4 && indices_and_values.dim[1] == 2,
				"gather_tokens_forward: x [B, H, W, C], routing table [B, 2, E, K], y [B, K, E, C]");
		const int batch = x.dim[0], tokens = x.dim[1] * x.dim[2], channels = x.dim[3], capacity = y.dim[1], experts = y.dim[2];
		MLHIP_REQUIRE(y.dim[0] == batch && y.dim[3] == channels && indices_and_values.dim[0] == batch && indices_and_values.dim[2] == experts
				&& indices_and_values.dim[3] == capacity, "gather_tokens_forward: shapes do not agree");
		MLHIP_REQUIRE(x.dtype == y.dtype && x.dtype == indices_and_values.dtype && (x.dtype == DTYPE_FLOAT16 || x.dtype == DTYPE_FLOAT32),
				"gather_tokens_forward: fp16 or fp32 tensors of one type");
		const size_t rows = static_cast<size_t>(batch) * capacity * experts;
		if (rows == 0 || channels == 0)
			return;
		MLHIP_REQUIRE(x.data != nullptr && y.data != nullptr && indices_and_values.data != nullptr, "gather_tokens_forward: null tensor");
		const hipStream_t stream = stream_of(context);
#define MLHIP_GATHER(T, VEC) \
		do { \
			const size_t groups = rows * (channels / VEC); \
			if (groups <= 0xffffffffu) \
			{ \
				const FastDivisor by_pieces = make_fast_divisor(static_cast<uint32_t>(channels / VEC)), by_experts = make_fast_divisor(static_cast<uint32_t>(experts)), \
						by_capacity = make_fast_divisor(static_cast<uint32_t>(capacity)); \
				if (beta != 0.0f) \
					hipLaunchKernelGGL((kernel_gather_tokens_fast<T, VEC, true>), dim3(grid_for(groups)), dim3(256), 0, stream, ptr<const T>(x), \
							ptr<const T>(indices_and_values), ptr<T>(y), beta, static_cast<uint32_t>(groups), tokens, channels, by_pieces, by_experts, by_capacity); \
				else \
					hipLaunchKernelGGL((kernel_gather_tokens_fast<T, VEC, false>), dim3(grid_for(groups)), dim3(256), 0, stream, ptr<const T>(x), \
							ptr<const T>(indices_and_values), ptr<T>(y), beta, static_cast<uint32_t>(groups), tokens, channels, by_pieces, by_experts, by_capacity); \
			} \
			else \
				hipLaunchKernelGGL((kernel_gather_tokens<T, VEC>), dim3(grid_for(groups)), dim3(256), 0, stream, ptr<const T>(x), \
						ptr<const T>(indices_and_values), ptr<T>(y), beta, groups, tokens, channels, experts, capacity); \
		} while (0)
		if (x.dtype == DTYPE_FLOAT16)
		{
			if (vector_ok<half_t>(channels, 8, x.data, y.data))
				MLHIP_GATHER(half_t, 8);
			else
				MLHIP_GATHER(half_t, 1);
		}
		else
		{
			if (vector_ok<float>(channels, 4, x.data, y.data))
				MLHIP_GATHER(float, 4);
			else
				MLHIP_GATHER(float, 1);
		}
#undef MLHIP_GATHER
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_scatter_tokens_forward(mlContext_t context, const mlTensor_t x, const mlTensor_t indices_and_values, float beta, mlTensor_t y)
	try
	{
		MLHIP_REQUIRE(x.rank == 4 && y.rank == 4 && indices_and_values.rank == 4 && indices_and_values.dim[1] == 2,
				"scatter_tokens_forward: x [B, K, E, C], routing table [B, 2, E, K], y [B, H, W, C]");
		const int batch = y.dim[0], tokens = y.dim[1] * y.dim[2], channels = y.dim[3], capacity = x.dim[1], experts = x.dim[2];
		MLHIP_REQUIRE(x.dim[0] == batch && x.dim[3] == channels && indices_and_values.dim[0] == batch && indices_and_values.dim[2] == experts
				&& indices_and_values.dim[3] == capacity, "scatter_tokens_forward: shapes do not agree");
		MLHIP_REQUIRE(x.dtype == y.dtype && x.dtype == indices_and_values.dtype && (x.dtype == DTYPE_FLOAT16 || x.dtype == DTYPE_FLOAT32),
				"scatter_tokens_forward: fp16 or fp32 tensors of one type");
		const size_t total_tokens = static_cast<size_t>(batch) * tokens;
		if (total_tokens == 0 || channels == 0)
			return;
		MLHIP_REQUIRE(x.data != nullptr && y.data != nullptr && indices_and_values.data != nullptr, "scatter_tokens_forward: null tensor");
		const hipStream_t stream = stream_of(context);
		/* the by-image form needs a grid of (images x parts) workgroups, the tables of a part's tokens in LDS, and the expert outputs of
		 * one image within reach of a buffer descriptor's 32-bit offsets */
		const int splits = std::max(1, std::min(8, tokens / 16));
		const size_t lds_bytes = scatter_by_image_lds_bytes((tokens + splits - 1) / splits, experts);
		const size_t image_bytes = static_cast<size_t>(capacity) * experts * channels * size_of(x.dtype);
		const bool by_image = experts > 0 && capacity > 0 && lds_bytes <= 48 * 1024 && static_cast<size_t>(batch) * splits <= 0x7fffffffu
				&& image_bytes < 0x40000000u;
#define MLHIP_SCATTER(T, VEC) \
		do { \
			if (by_image) \
			{ \
				if (beta != 0.0f) \
					hipLaunchKernelGGL((kernel_scatter_tokens_by_image<T, VEC, true>), dim3(static_cast<unsigned int>(batch) * splits), dim3(256), lds_bytes, \
							stream, ptr<const T>(x), ptr<const T>(indices_and_values), ptr<T>(y), beta, tokens, channels, experts, capacity, splits); \
				else \
					hipLaunchKernelGGL((kernel_scatter_tokens_by_image<T, VEC, false>), dim3(static_cast<unsigned int>(batch) * splits), dim3(256), lds_bytes, \
							stream, ptr<const T>(x), ptr<const T>(indices_and_values), ptr<T>(y), beta, tokens, channels, experts, capacity, splits); \
				break; \
			} \
			const size_t wavefronts = total_tokens * ((channels + 64 * VEC - 1) / (64 * VEC)); \
			MLHIP_REQUIRE((wavefronts + 3) / 4 <= 0x7fffffffu, "scatter_tokens_forward: tensor too large for one launch"); \
			hipLaunchKernelGGL((kernel_scatter_tokens<T, VEC>), dim3(static_cast<unsigned int>((wavefronts + 3) / 4)), dim3(256), 0, stream, ptr<const T>(x), \
					ptr<const T>(indices_and_values), ptr<T>(y), beta, total_tokens, tokens, channels, experts, capacity); \
		} while (0)
		if (x.dtype == DTYPE_FLOAT16)
		{
			if (vector_ok<half_t>(channels, 4, x.data, y.data))
				MLHIP_SCATTER(half_t, 4);
			else
				MLHIP_SCATTER(half_t, 1);
		}
		else
		{
			if (vector_ok<float>(channels, 4, x.data, y.data))
				MLHIP_SCATTER(float, 4);
			else
				MLHIP_SCATTER(float, 1);
		}
#undef MLHIP_SCATTER
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}

	void hip_moe_forward(mlContext_t context, const mlTensor_t x, const mlTensor_t w, const mlTensor_t b, float beta, mlTensor_t y, mlActivationType_t act)
	try
	{
		MLHIP_REQUIRE(x.rank == 4 && y.rank == 4 && w.rank == 3, "moe_forward: x [B, K, E, C], weights [E, N, C], y [B, K, E, N]");
		const int batch = x.dim[0], capacity = x.dim[1], experts = x.dim[2], channels = x.dim[3], neurons = w.dim[1];
		MLHIP_REQUIRE(w.dim[0] == experts && w.dim[2] == channels && y.dim[0] == batch && y.dim[1] == capacity && y.dim[2] == experts && y.dim[3] == neurons,
				"moe_forward: shapes do not agree");
		MLHIP_REQUIRE(x.dtype == y.dtype && x.dtype == w.dtype && (x.dtype == DTYPE_FLOAT16 || x.dtype == DTYPE_FLOAT32),
				"moe_forward: fp16 or fp32 tensors of one type");
		if (b.data != nullptr)
			MLHIP_REQUIRE(b.dtype == x.dtype && volume(b) == static_cast<size_t>(experts) * neurons, "moe_forward: bias must be [E, N] of the tensors' type");
		const size_t rows = static_cast<size_t>(batch) * capacity;
		if (rows == 0 || experts == 0 || neurons == 0)
			return;
		MLHIP_REQUIRE(x.data != nullptr && y.data != nullptr && w.data != nullptr && rows <= 0x7fffffffu && experts <= 65535, "moe_forward: null tensor or too large");
		const hipStream_t stream = stream_of(context);
		const int esize = size_of(x.dtype);
		const size_t k_bytes = static_cast<size_t>(channels) * esize;
		const auto aligned = [](const void *p, size_t a) { return reinterpret_cast<uintptr_t>(p) % a == 0; };
		const bool vectorized = neurons % 4 == 0 && aligned(y.data, 4 * esize) && aligned(b.data, 4 * esize);
		const bool dma = channels > 0 && k_bytes % 128 == 0 && aligned(x.data, 16) && aligned(w.data, 16) && static_cast<size_t>(experts) * k_bytes <= 0x7fffffffu;
		if (dma)
		{
			/* expert e multiplies the rows (b, k) of x, which lie E * C elements apart, by its own [N, C] weights into rows E * N apart */
			DenseDmaRows a_loader { reinterpret_cast<const uint8_t*>(x.data), static_cast<int>(rows), static_cast<int>(k_bytes) };
			a_loader.row_stride_bytes = static_cast<int>(static_cast<size_t>(experts) * k_bytes);
			const DenseDmaRows b_loader { reinterpret_cast<const uint8_t*>(w.data), neurons, static_cast<int>(k_bytes) };
			const auto launch = [&](auto zero)
			{
				typedef decltype(zero) T;
				FloatEpilogue<T> ep;
				ep.D = reinterpret_cast<T*>(y.data);
				ep.C = reinterpret_cast<const T*>(y.data);
				ep.bias = reinterpret_cast<const T*>(b.data);
				ep.N = neurons;
				ep.row_stride = experts * neurons;
				ep.alpha = 1.0f;
				ep.beta = beta;
				ep.act = act;
				ep.vectorized = vectorized;
				ep.bias_batch_stride = neurons;
				/* the epilogue's common cases (ReLU / linear, bias present, beta = 0 or not) are fixed at compile time: with K of only a few
				 * chunks the epilogue is most of a tile's time, and its run-time form is twice as slow */
				if constexpr (sizeof(T) == 2)
					specialise_epilogue(ep, [&](const auto &fixed)
					{
						if (vectorized && stream_gemm_half_applies(static_cast<int>(rows), experts, k_bytes))
						{
							/* short K rows (the layer that widens 256 channels to the hidden width): the streaming kernel, whose B operand
							 * stays in registers; the experts are the matrices of its batch, their rows E * C elements apart */
							StreamGemmArgs sg { x.data, w.data, y.data, static_cast<int>(rows), neurons, static_cast<int>(k_bytes), experts,
									static_cast<size_t>(channels), static_cast<size_t>(neurons) * channels, static_cast<size_t>(neurons) };
							sg.a_row_bytes = static_cast<size_t>(experts) * k_bytes;
							launch_stream_gemm<T>(stream, sg, fixed);
						}
						else
							launch_gemm_dma<T>(stream, a_loader, b_loader, static_cast<int>(rows), neurons, static_cast<int>(k_bytes), experts, k_bytes,
									static_cast<size_t>(neurons) * k_bytes, static_cast<size_t>(neurons), fixed);
					});
				else
					launch_gemm_dma<T>(stream, a_loader, b_loader, static_cast<int>(rows), neurons, static_cast<int>(k_bytes), experts, k_bytes,
							static_cast<size_t>(neurons) * k_bytes, static_cast<size_t>(neurons), ep);
			};
			if (x.dtype == DTYPE_FLOAT16)
				launch(half_t(0));
			else
				launch(0.0f);
		}
		else
		{
			const size_t outputs = rows * experts * neurons;
			if (x.dtype == DTYPE_FLOAT16)
				hipLaunchKernelGGL(kernel_moe_generic<half_t>, dim3(grid_for(outputs)), dim3(256), 0, stream, ptr<const half_t>(x), ptr<const half_t>(w),
						ptr<const half_t>(b), ptr<half_t>(y), beta, outputs, experts, neurons, channels, static_cast<int>(act));
			else
				hipLaunchKernelGGL(kernel_moe_generic<float>, dim3(grid_for(outputs)), dim3(256), 0, stream, ptr<const float>(x), ptr<const float>(w),
						ptr<const float>(b), ptr<float>(y), beta, outputs, experts, neurons, channels, static_cast<int>(act));
		}
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(expert_choice_routing_forward)
MLHIP_ALSO_AS_CUDA(token_choice_routing_forward)
MLHIP_ALSO_AS_CUDA(hash_routing)
MLHIP_ALSO_AS_CUDA(gather_tokens_forward)
MLHIP_ALSO_AS_CUDA(scatter_tokens_forward)
MLHIP_ALSO_AS_CUDA(moe_forward)
