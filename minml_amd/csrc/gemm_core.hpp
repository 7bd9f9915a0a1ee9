/*
 * gemm_core.hpp — the MFMA tile engine shared by every GEMM-shaped kernel of the backend (plain / batched GEMM, gemm_ex,
 * implicit-GEMM convolution in fp16 / fp32 / int8).
 *
 * Problem form: ACC[m][n] = sum_k A[m][k] * B[n][k]  — both operands K-contiguous ("n","t" in the reference's notation,
 * src/backend/cpu/gemm/gemm.cpp:39-83); accumulation in fp32 (int32 for int8 operands) over the whole K extent, as the
 * reference does (src/backend/cpu/gemm/gemm_runtime.cpp:360, def_kernels.cpp:214-282).
 *
 * Mapping to gfx950:
 *   - a workgroup of WAVES_M x WAVES_N wavefronts (64 lanes each) owns a BM x BN tile of ACC; every wavefront owns a
 *     (BM/WAVES_M) x (BN/WAVES_N) sub-tile as a grid of 32x32 MFMA blocks held in accumulator registers;
 *   - operand tiles of BKB bytes of K per row are staged through LDS, double buffered: the global loads of step i+1 are in
 *     flight while the MFMAs of step i run; rows are padded by 16 bytes so that 16-byte fragment reads of 16 consecutive lanes hit
 *     64 distinct banks;
 *   - one MFMA operand fragment is 16 bytes per lane: 8 halfs for v_mfma_f32_32x32x16_f16, 16 bytes for v_mfma_i32_32x32x32_i8,
 *     4 floats feeding four v_mfma_f32_32x32x2_f32;
 *   - B rows are fed as the MFMA's first operand, so that each lane ends up with 4 consecutive n of one row m, and the epilogue
 *     moves 4 consecutive output elements per lane through an LDS slab to fully coalesced global stores.
 *
 * The A operand is produced by a loader object, which is how the same engine serves a dense matrix and the implicit (never
 * materialised) im2row matrix of a convolution; the epilogue is a functor applied to 4 consecutive n of one row.
 */
#ifndef MINML_AMD_GEMM_CORE_HPP_
#define MINML_AMD_GEMM_CORE_HPP_

#include "device_utils.hpp"

namespace mlhip
{
	template<typename T>
	struct MfmaTraits;
	template<>
	struct MfmaTraits<half_t>
	{
			typedef float acc_t;
			typedef float16_t acc_vec;
			__device__ static __forceinline__ void mma(const uint4_t &a, const uint4_t &b, acc_vec &c)
			{
				c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
			}
	};
	template<>
	struct MfmaTraits<float>
	{
			typedef float acc_t;
			typedef float16_t acc_vec;
			__device__ static __forceinline__ void mma(const uint4_t &a, const uint4_t &b, acc_vec &c)
			{
				const float4_t fa = __builtin_bit_cast(float4_t, a);
				const float4_t fb = __builtin_bit_cast(float4_t, b);
#pragma unroll
				for (int e = 0; e < 4; e++)
					c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[e], fb[e], c, 0, 0, 0);
			}
	};
	template<>
	struct MfmaTraits<int8_t>
	{
			typedef int acc_t;
			typedef int16_t_v acc_vec;
			__device__ static __forceinline__ void mma(const uint4_t &a, const uint4_t &b, acc_vec &c)
			{
				c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(int4_t, a), __builtin_bit_cast(int4_t, b), c, 0, 0, 0);
			}
	};

	/* Dense row-major operand [rows][K] with leading dimension K (elements); rows >= `rows` and chunks beyond K read as zero. */
	template<typename T>
	struct DenseRows
	{
			const T *base;
			int rows;
			int k_bytes; /* K * sizeof(T), a multiple of 16 */

			struct RowState
			{
					const uint8_t *ptr; /* nullptr => row out of range */
			};
			__device__ __forceinline__ RowState begin_row(int row) const
			{
				RowState s;
				s.ptr = (row < rows) ? reinterpret_cast<const uint8_t*>(base) + static_cast<size_t>(row) * k_bytes : nullptr;
				return s;
			}
			__device__ __forceinline__ uint4_t load(const RowState &s, int byte_offset) const
			{
				if (s.ptr != nullptr && byte_offset < k_bytes)
					return *reinterpret_cast<const uint4_t*>(s.ptr + byte_offset);
				return uint4_t { 0u, 0u, 0u, 0u };
			}
	};

	/*
	 * Implicit im2row operand of a stride-1, "same"-padded convolution over an NHWC tensor: row m = (b, h, w), column
	 * k = ((i * kw) + j) * Cin + c reads input[b][h + i - ph][w + j - pw][c], or `fill` (replicated byte pattern) outside the image
	 * (reference: src/backend/cpu/conv_im2row.cpp:21-59; the fill value is the int8 zero point of src/layers/Conv2D.cpp:245,266-270).
	 * Cin * sizeof(T) must be a multiple of 16 so that a 16-byte chunk never straddles two taps.
	 */
	template<typename T>
	struct Im2RowRows
	{
			const T *base;
			int rows; /* B * H * W */
			int height, width;
			int kernel_h, kernel_w;
			int c_bytes; /* Cin * sizeof(T) */
			int k_bytes; /* kernel_h * kernel_w * c_bytes */
			uint32_t fill;

			struct RowState
			{
					const uint8_t *image; /* start of image b, nullptr => row out of range */
					int h, w;
			};
			__device__ __forceinline__ RowState begin_row(int row) const
			{
				RowState s;
				if (row < rows)
				{
					const int hw = height * width;
					const int b = row / hw;
					const int rem = row - b * hw;
					s.h = rem / width;
					s.w = rem - s.h * width;
					s.image = reinterpret_cast<const uint8_t*>(base) + static_cast<size_t>(b) * hw * c_bytes;
				}
				else
				{
					s.image = nullptr;
					s.h = 0;
					s.w = 0;
				}
				return s;
			}
			__device__ __forceinline__ uint4_t load(const RowState &s, int byte_offset) const
			{
				if (s.image == nullptr || byte_offset >= k_bytes)
					return uint4_t { 0u, 0u, 0u, 0u };
				const int tap = byte_offset / c_bytes;
				const int c = byte_offset - tap * c_bytes;
				const int i = tap / kernel_w;
				const int j = tap - i * kernel_w;
				const int x = s.h + i - (kernel_h - 1) / 2;
				const int y = s.w + j - (kernel_w - 1) / 2;
				if (x >= 0 && x < height && y >= 0 && y < width)
					return *reinterpret_cast<const uint4_t*>(s.image + (static_cast<size_t>(x) * width + y) * c_bytes + c);
				return uint4_t { fill, fill, fill, fill };
			}
	};

	template<int BM_, int BN_, int BKB_, int WAVES_M_, int WAVES_N_>
	struct TileConfig
	{
			static constexpr int BM = BM_;
			static constexpr int BN = BN_;
			static constexpr int BKB = BKB_; /* bytes of K per row per pipeline step: 64 or 128 */
			static constexpr int WAVES_M = WAVES_M_;
			static constexpr int WAVES_N = WAVES_N_;
			static constexpr int THREADS = 64 * WAVES_M * WAVES_N;
			static constexpr int WM = BM / WAVES_M; /* wavefront sub-tile */
			static constexpr int WN = BN / WAVES_N;
			static constexpr int BLOCKS_M = WM / 32;
			static constexpr int BLOCKS_N = WN / 32;
			static constexpr int ROW_STRIDE = BKB + 16; /* padded LDS row, bytes */
			static constexpr int CHUNKS_PER_ROW = BKB / 16;
			static constexpr int A_STAGE_BYTES = BM * ROW_STRIDE;
			static constexpr int B_STAGE_BYTES = BN * ROW_STRIDE;
			static constexpr int STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
			static constexpr int A_LOADS = (BM * CHUNKS_PER_ROW) / THREADS;
			static constexpr int B_LOADS = (BN * CHUNKS_PER_ROW) / THREADS;
			static constexpr int SLAB_STRIDE = WN + 4; /* epilogue slab row, in 4-byte words */
			static constexpr int SLAB_BYTES = 32 * SLAB_STRIDE * 4; /* one 32-row slab per wavefront */
			static constexpr int EPILOGUE_BYTES = WAVES_M * WAVES_N * SLAB_BYTES;
			static constexpr int LDS_BYTES = (2 * STAGE_BYTES > EPILOGUE_BYTES) ? 2 * STAGE_BYTES : EPILOGUE_BYTES;
			static_assert(WM % 32 == 0 && WN % 32 == 0, "wavefront sub-tile must be a grid of 32x32 MFMA blocks");
			static_assert((BM * CHUNKS_PER_ROW) % THREADS == 0 && (BN * CHUNKS_PER_ROW) % THREADS == 0, "tile rows must divide evenly over the threads");
			static_assert(BKB == 64 || BKB == 128, "BKB must be 64 or 128 bytes");
	};

	/*
	 * Computes one BM x BN tile: rows [m0, m0+BM) of the A loader against rows [n0, n0+BN) of the B loader, then hands every group of
	 * 4 consecutive n of one row m to epilogue(m, n, acc[4]) (only for m < M; the functor masks n itself).
	 */
	template<typename T, typename Cfg, typename ALoader, typename BLoader, typename Epilogue>
	__device__ __forceinline__ void gemm_tile(const ALoader &a_loader, const BLoader &b_loader, int M, int k_bytes, int m0, int n0, uint8_t *lds,
			const Epilogue &epilogue)
	{
		typedef MfmaTraits<T> Traits;
		typedef typename Traits::acc_vec acc_vec;
		typedef typename Traits::acc_t acc_t;

		const int tid = threadIdx.x;
		const int lane = tid & 63;
		const int wave = tid >> 6;
		const int wave_m = wave / Cfg::WAVES_N;
		const int wave_n = wave % Cfg::WAVES_N;

		/* which 16-byte chunks of the A and B tiles this thread moves each step */
		typename ALoader::RowState a_rows[Cfg::A_LOADS];
		typename BLoader::RowState b_rows[Cfg::B_LOADS];
		int a_lds[Cfg::A_LOADS], a_kc[Cfg::A_LOADS];
		int b_lds[Cfg::B_LOADS], b_kc[Cfg::B_LOADS];
#pragma unroll
		for (int i = 0; i < Cfg::A_LOADS; i++)
		{
			const int chunk = tid + i * Cfg::THREADS;
			const int row = chunk / Cfg::CHUNKS_PER_ROW;
			a_kc[i] = (chunk % Cfg::CHUNKS_PER_ROW) * 16;
			a_rows[i] = a_loader.begin_row(m0 + row);
			a_lds[i] = row * Cfg::ROW_STRIDE + a_kc[i];
		}
#pragma unroll
		for (int i = 0; i < Cfg::B_LOADS; i++)
		{
			const int chunk = tid + i * Cfg::THREADS;
			const int row = chunk / Cfg::CHUNKS_PER_ROW;
			b_kc[i] = (chunk % Cfg::CHUNKS_PER_ROW) * 16;
			b_rows[i] = b_loader.begin_row(n0 + row);
			b_lds[i] = Cfg::A_STAGE_BYTES + row * Cfg::ROW_STRIDE + b_kc[i];
		}

		acc_vec acc[Cfg::BLOCKS_M][Cfg::BLOCKS_N];
#pragma unroll
		for (int i = 0; i < Cfg::BLOCKS_M; i++)
#pragma unroll
			for (int j = 0; j < Cfg::BLOCKS_N; j++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					acc[i][j][r] = 0;

		uint4_t a_regs[Cfg::A_LOADS], b_regs[Cfg::B_LOADS];
		const int steps = (k_bytes + Cfg::BKB - 1) / Cfg::BKB;

		/* prologue: stage 0 */
#pragma unroll
		for (int i = 0; i < Cfg::A_LOADS; i++)
			a_regs[i] = a_loader.load(a_rows[i], a_kc[i]);
#pragma unroll
		for (int i = 0; i < Cfg::B_LOADS; i++)
			b_regs[i] = b_loader.load(b_rows[i], b_kc[i]);
#pragma unroll
		for (int i = 0; i < Cfg::A_LOADS; i++)
			*reinterpret_cast<uint4_t*>(lds + a_lds[i]) = a_regs[i];
#pragma unroll
		for (int i = 0; i < Cfg::B_LOADS; i++)
			*reinterpret_cast<uint4_t*>(lds + b_lds[i]) = b_regs[i];
		__syncthreads();

		const int frag_lane_offset = (lane & 31) * Cfg::ROW_STRIDE + (lane >> 5) * 16;
		for (int step = 0; step < steps; step++)
		{
			const int cur = (step & 1) * Cfg::STAGE_BYTES;
			const int nxt = Cfg::STAGE_BYTES - cur;
			const bool has_next = (step + 1) < steps;
			if (has_next)
			{
				const int kb = (step + 1) * Cfg::BKB;
#pragma unroll
				for (int i = 0; i < Cfg::A_LOADS; i++)
					a_regs[i] = a_loader.load(a_rows[i], kb + a_kc[i]);
#pragma unroll
				for (int i = 0; i < Cfg::B_LOADS; i++)
					b_regs[i] = b_loader.load(b_rows[i], kb + b_kc[i]);
			}

			const uint8_t *a_tile = lds + cur + (wave_m * Cfg::WM) * Cfg::ROW_STRIDE + frag_lane_offset;
			const uint8_t *b_tile = lds + cur + Cfg::A_STAGE_BYTES + (wave_n * Cfg::WN) * Cfg::ROW_STRIDE + frag_lane_offset;
#pragma unroll
			for (int ks = 0; ks < Cfg::BKB / 32; ks++)
			{
				uint4_t fa[Cfg::BLOCKS_M], fb[Cfg::BLOCKS_N];
#pragma unroll
				for (int i = 0; i < Cfg::BLOCKS_M; i++)
					fa[i] = *reinterpret_cast<const uint4_t*>(a_tile + i * 32 * Cfg::ROW_STRIDE + ks * 32);
#pragma unroll
				for (int j = 0; j < Cfg::BLOCKS_N; j++)
					fb[j] = *reinterpret_cast<const uint4_t*>(b_tile + j * 32 * Cfg::ROW_STRIDE + ks * 32);
#pragma unroll
				for (int i = 0; i < Cfg::BLOCKS_M; i++)
#pragma unroll
					for (int j = 0; j < Cfg::BLOCKS_N; j++)
						Traits::mma(fb[j], fa[i], acc[i][j]); /* B rows as first operand: lane gets 4 consecutive n */
			}

			if (has_next)
			{
#pragma unroll
				for (int i = 0; i < Cfg::A_LOADS; i++)
					*reinterpret_cast<uint4_t*>(lds + nxt + a_lds[i]) = a_regs[i];
#pragma unroll
				for (int i = 0; i < Cfg::B_LOADS; i++)
					*reinterpret_cast<uint4_t*>(lds + nxt + b_lds[i]) = b_regs[i];
			}
			__syncthreads();
		}

		/*
		 * Epilogue. With B as the first MFMA operand, lane l, register r of block (i, j) holds
		 *   n = 32*j + 8*(r/4) + 4*(l/32) + r%4,   m = 32*i + l%32      (relative to the wavefront sub-tile).
		 * Each wavefront transposes one 32-row slab at a time through its private LDS slab [32][WN + 4] and reads it back row-wise,
		 * 4 consecutive n per lane, so that global traffic of the epilogue is contiguous along n.
		 */
		acc_t *slab = reinterpret_cast<acc_t*>(lds + wave * Cfg::SLAB_BYTES);
		constexpr int LANES_PER_ROW = Cfg::WN / 4;
		constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
		static_assert(64 % LANES_PER_ROW == 0 && 32 % ROWS_PER_PASS == 0, "unsupported wavefront tile width");
#pragma unroll
		for (int i = 0; i < Cfg::BLOCKS_M; i++)
		{
#pragma unroll
			for (int j = 0; j < Cfg::BLOCKS_N; j++)
#pragma unroll
				for (int q = 0; q < 4; q++)
				{
					typedef acc_t vec4 __attribute__((ext_vector_type(4)));
					vec4 tmp;
#pragma unroll
					for (int e = 0; e < 4; e++)
						tmp[e] = acc[i][j][q * 4 + e];
					const int n = 32 * j + 8 * q + 4 * (lane >> 5);
					*reinterpret_cast<vec4*>(slab + (lane & 31) * Cfg::SLAB_STRIDE + n) = tmp;
				}
			__builtin_amdgcn_s_waitcnt(0xc07f); /* lgkmcnt(0): the slab is private to this wavefront, whose LDS operations complete in order */
			__builtin_amdgcn_wave_barrier();
#pragma unroll
			for (int pass = 0; pass < 32 / ROWS_PER_PASS; pass++)
			{
				const int row = pass * ROWS_PER_PASS + lane / LANES_PER_ROW;
				const int col = (lane % LANES_PER_ROW) * 4;
				typedef acc_t vec4 __attribute__((ext_vector_type(4)));
				const vec4 tmp = *reinterpret_cast<const vec4*>(slab + row * Cfg::SLAB_STRIDE + col);
				const int m = m0 + wave_m * Cfg::WM + 32 * i + row;
				const int n = n0 + wave_n * Cfg::WN + col;
				if (m < M)
				{
					acc_t vals[4] = { tmp[0], tmp[1], tmp[2], tmp[3] };
					epilogue(m, n, vals);
				}
			}
			__builtin_amdgcn_s_waitcnt(0xc07f);
			__builtin_amdgcn_wave_barrier();
		}
	}
} /* namespace mlhip */

#endif /* MINML_AMD_GEMM_CORE_HPP_ */
