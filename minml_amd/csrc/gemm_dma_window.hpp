/*
 * gemm_dma_window.hpp — the tile engine of gemm_dma.hpp for stride-1, "same"-padded k x k convolutions whose input pixels are whole
 * multiples of 128 bytes, with the A operand taken from a WINDOW of input pixels instead of from the im2row gather.
 *
 * The im2row form of the engine fetches every tap of every row as its own 128-byte request: per chunk of K a 256 x 256 tile moves 32 KB
 * of A and 32 KB of B from L2 to LDS, and delivering those 64 KB takes about as long as multiplying them. But the rows of a tile are 256
 * consecutive pixels, and tap (i, j) of pixel m is pixel m + (i - pad) * W + (j - pad): the k * k taps of a tile read the same
 * 256 + 2 * pad * (W + 1) pixels over and over. So K is walked slice-major (a slice = 128 bytes of the channels, i.e. 64 halfs): for each
 * slice the window of pixels enters LDS once (one of two buffers; the next slice's window arrives while this one is multiplied), and the
 * k * k chunks of the slice read their A fragments from it at per-tap offsets (a tap outside the image reads a row holding the padding
 * byte). Only the B operand still streams through the slots: 32 KB per chunk instead of 64.
 *
 * The sum over K runs in the order (slice, tap) instead of (tap, slice); everything else (fragment layout, swizzle, epilogue) is the
 * engine's.
 */
#ifndef MINML_AMD_GEMM_DMA_WINDOW_HPP_
#define MINML_AMD_GEMM_DMA_WINDOW_HPP_

#include "gemm_dma.hpp"

namespace mlhip
{
	/* B operand [rows][k * k][Cin] read slice-major: chunk (slice, tap) is the 128 bytes at tap * c_bytes + slice * 128 of a row */
	struct SliceMajorDmaRows
	{
			const uint8_t *base;
			int rows;
			int c_bytes, taps;

			struct Row
			{
					const uint8_t *ptr;
			};
			struct Step
			{
					int tap, slice_bytes;
			};
			__device__ __forceinline__ Row begin_row(int row) const
			{
				return Row { base + static_cast<size_t>(min(row, rows - 1)) * c_bytes * taps };
			}
			__device__ __forceinline__ Step first_step() const
			{
				return Step { 0, 0 };
			}
			__device__ __forceinline__ void advance(Step &s) const
			{
				s.tap++;
				if (s.tap >= taps)
				{
					s.tap = 0;
					s.slice_bytes += 128;
				}
			}
			__device__ __forceinline__ const uint8_t* chunk(const Row &r, const Step &s, int chunk_bytes) const
			{
				return r.ptr + s.tap * c_bytes + s.slice_bytes + chunk_bytes;
			}
	};

	template<typename Cfg>
	struct WindowTileLds
	{
			static constexpr int WINDOW_PIXELS = 352; /* 256 rows + 2 * 44 pixels of halo + rounding to 8 */
			static constexpr int WINDOW_BYTES = WINDOW_PIXELS * 128;
			static constexpr int SLOTS = 2;
			static constexpr int WINDOWS = SLOTS * Cfg::B_SLOT_BYTES; /* offset of the two window buffers */
			static constexpr int PADDING = WINDOWS + 2 * WINDOW_BYTES; /* 256 bytes of the padding value, one bank cycle */
			static constexpr int BYTES = (PADDING + 256 > Cfg::EPILOGUE_BYTES) ? PADDING + 256 : Cfg::EPILOGUE_BYTES;
			static constexpr int WINDOW_LOADS = (WINDOW_PIXELS / 8 + Cfg::WAVES - 1) / Cfg::WAVES; /* 1 KB requests of a window per wavefront */
			static constexpr int MAX_HALO = (WINDOW_PIXELS - Cfg::BM - 8) / 2;
			static_assert(Cfg::BM == 256 && Cfg::SLOTS == 2 && BYTES <= 160 * 1024, "the window form needs tiles of 256 rows and two slots");
	};

	/* one BM x BN tile of the convolution; rows m0 ... are consecutive pixels of the flattened [B * H * W] tensor */
	template<typename T, typename Cfg, typename Epilogue>
	__device__ __forceinline__ void conv_tile_dma_window(const uint8_t *input, const SliceMajorDmaRows &b_loader, int M, int height, int width, int kernel_size,
			uint32_t fill_word, int m0, int n0, uint8_t *lds, const Epilogue &epilogue)
	{
		typedef MfmaTraits<T> Traits;
		typedef typename Traits::acc_vec acc_vec;
		typedef WindowTileLds<Cfg> Lds;
		constexpr int KSTEPS = Cfg::KSTEPS;

		const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
		const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;
		const int c_bytes = b_loader.c_bytes, taps = b_loader.taps;
		const int slices = c_bytes / 128;
		const int chunks = slices * taps;
		const int pad = kernel_size / 2;
		const int halo = pad * (width + 1);
		const int window_first = ((m0 - halo) >> 3) << 3; /* flattened number of the pixel in position 0 of a window (may be negative) */

		if (tid < 64)
			reinterpret_cast<uint32_t*>(lds + Lds::PADDING)[tid] = fill_word;

		/* window loader: wavefront w moves the groups of 8 pixels w, w + WAVES, ... of a window */
		auto request_window_group = [&](int slice, int t)
		{
			const int group = wave + Cfg::WAVES * t;
			if (group < Lds::WINDOW_PIXELS / 8)
			{
				const int position = group * 8 + (lane >> 3);
				const int pixel = min(max(window_first + position, 0), M - 1); /* pixels before the tensor or past its end are never valid taps */
				const int chunk = (lane & 7) ^ dma_swizzle(position);
				__builtin_amdgcn_global_load_lds((global_ptr_t) (input + static_cast<size_t>(pixel) * c_bytes + slice * 128 + chunk * 16),
						(lds_ptr_t) (lds + Lds::WINDOWS + (slice & 1) * Lds::WINDOW_BYTES + group * 1024), 16, 0, 0);
			}
		};
		/* B loader geometry, as in gemm_tile_dma */
		SliceMajorDmaRows::Row b_rows[Cfg::B_LOADS];
		int b_chunk[Cfg::B_LOADS];
#pragma unroll
		for (int i = 0; i < Cfg::B_LOADS; i++)
		{
			const int row = (wave + Cfg::WAVES * i) * 8 + (lane >> 3);
			b_chunk[i] = ((lane & 7) ^ dma_swizzle(row)) * 16;
			b_rows[i] = b_loader.begin_row(n0 + row);
		}
		SliceMajorDmaRows::Step b_step = b_loader.first_step();
		auto request_b = [&](int c)
		{
			uint8_t *slot = lds + (c & 1) * Cfg::B_SLOT_BYTES;
#pragma unroll
			for (int l = 0; l < Cfg::B_LOADS; l++)
				__builtin_amdgcn_global_load_lds((global_ptr_t) b_loader.chunk(b_rows[l], b_step, b_chunk[l]), (lds_ptr_t) (slot + (wave + Cfg::WAVES * l) * 1024), 16, 0, 0);
			b_loader.advance(b_step);
		};

		/* where this lane's pixel of each 32-row block lies in its image, which taps of it are inside, and its position in the window */
		uint32_t inside[Cfg::BLOCKS_M];
		int centre[Cfg::BLOCKS_M];
#pragma unroll
		for (int i = 0; i < Cfg::BLOCKS_M; i++)
		{
			const int m = m0 + wave_m * Cfg::WM + 32 * i + (lane & 31);
			const int r = min(m, M - 1) % (height * width);
			const int h = r / width, w = r - h * width;
			uint32_t rows_inside = 0, columns_inside = 0; /* bit k * di: row h + di - pad exists; bit dj: column w + dj - pad exists */
			for (int d = 0; d < kernel_size; d++)
			{
				rows_inside |= (static_cast<unsigned>(h + d - pad) < static_cast<unsigned>(height)) ? (1u << (kernel_size * d)) : 0u;
				columns_inside |= (static_cast<unsigned>(w + d - pad) < static_cast<unsigned>(width)) ? (1u << d) : 0u;
			}
			inside[i] = (m < M) ? rows_inside * columns_inside : 0u; /* bit k * di + dj; rows past the end read padding only */
			centre[i] = m - window_first;
		}
		int b_frag[Cfg::BLOCKS_N];
#pragma unroll
		for (int j = 0; j < Cfg::BLOCKS_N; j++)
		{
			const int row = wave_n * Cfg::WN + 32 * j + (lane & 31);
			b_frag[j] = row * Cfg::BKB + (((lane >> 5) ^ dma_swizzle(row)) * 16);
		}
		/*
		 * LDS addresses of this lane's A fragments (k step 0) of one chunk = tap (di, dj) of a slice, whose window starts at `window`;
		 * k step kk is at (address ^ (kk * 32)). A tap outside the image reads the padding area at the offset that has the banks of the
		 * address it replaces (the area holds the padding in all 16 positions of a 256-byte bank cycle), so that the padded lanes of a
		 * read collide with no lane that reads the window.
		 */
		auto compute_a_fragments = [&](int window, int di, int dj, int (&address)[Cfg::BLOCKS_M])
		{
			const int offset = (di - pad) * width + (dj - pad);
			const int bit = di * kernel_size + dj;
#pragma unroll
			for (int i = 0; i < Cfg::BLOCKS_M; i++)
			{
				const int position = centre[i] + offset;
				const int in_window = position * 128 + (((lane >> 5) ^ dma_swizzle(position)) * 16);
				address[i] = ((inside[i] >> bit) & 1u) ? window + in_window : Lds::PADDING + (in_window & 0xf0);
			}
		};

		acc_vec acc[Cfg::BLOCKS_M][Cfg::BLOCKS_N];
#pragma unroll
		for (int i = 0; i < Cfg::BLOCKS_M; i++)
#pragma unroll
			for (int j = 0; j < Cfg::BLOCKS_N; j++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					acc[i][j][r] = 0;

		/* the first slice's window and the first chunk of B */
		for (int t = 0; t < Lds::WINDOW_LOADS; t++)
			request_window_group(0, t);
		request_b(0);

		uint4_t fa[2][Cfg::BLOCKS_M], fb[2][Cfg::BLOCKS_N];
		auto read_fragments = [&](int c, int kk, const int (&address)[Cfg::BLOCKS_M], uint4_t (&a_regs)[Cfg::BLOCKS_M], uint4_t (&b_regs)[Cfg::BLOCKS_N])
		{
			const uint8_t *slot = lds + (c & 1) * Cfg::B_SLOT_BYTES;
#pragma unroll
			for (int i = 0; i < Cfg::BLOCKS_M; i++)
				a_regs[i] = *reinterpret_cast<const uint4_t*>(lds + (address[i] ^ (kk * 32)));
#pragma unroll
			for (int j = 0; j < Cfg::BLOCKS_N; j++)
				b_regs[j] = *reinterpret_cast<const uint4_t*>(slot + (b_frag[j] ^ (kk * 32)));
		};
		/* chunk c becomes readable: with two slots every load issued so far (the chunk's B rows, and window groups requested before them)
		 * has to have landed in every wavefront; the slot of chunk c - 1 is free for chunk c + 1 */
		auto open_chunk = [&]()
		{
			wait_lgkmcnt<0>();
			wait_vmcnt<0>();
			barrier_no_fence();
		};
		auto multiply = [&](auto lo, auto hi, auto buffer)
		{
			constexpr int cur = decltype(buffer)::value;
			static_for<decltype(hi)::value - decltype(lo)::value>([&](auto index)
			{
				constexpr int idx = decltype(lo)::value + decltype(index)::value;
				constexpr int i = idx / Cfg::BLOCKS_N, j = idx % Cfg::BLOCKS_N;
				Traits::mma(fb[cur][j], fa[cur][i], acc[i][j]);
			});
		};
		constexpr int MFMAS = Cfg::BLOCKS_M * Cfg::BLOCKS_N;

		int a_frag[Cfg::BLOCKS_M], a_next[Cfg::BLOCKS_M];
		open_chunk();
		compute_a_fragments(Lds::WINDOWS, 0, 0, a_frag);
		read_fragments(0, 0, a_frag, fa[0], fb[0]);

		/* position of chunk c + 1 in K: its slice's number and window, its tap */
		int next_slice = 0, next_window = Lds::WINDOWS, next_di = 0, next_dj = 0, next_tap = 0;
		auto process_chunk = [&](int c) __attribute__((always_inline))
		{
			const int slice = next_slice, tap = next_tap;
			next_tap++;
			next_dj++;
			if (next_dj == kernel_size)
			{
				next_dj = 0;
				next_di++;
			}
			if (next_tap == taps)
			{
				next_tap = next_di = 0;
				next_slice++;
				next_window ^= Lds::WINDOWS ^ (Lds::WINDOWS + Lds::WINDOW_BYTES);
			}
			const bool more = (c + 1 < chunks);
			static_for<KSTEPS>([&](auto kstep)
			{
				constexpr int kk = decltype(kstep)::value;
				constexpr int cur = kk & 1, nxt = 1 - cur;
				constexpr int HEAD = (kk + 1 < KSTEPS) ? 1 : (MFMAS > Cfg::TAIL_MFMAS ? MFMAS - Cfg::TAIL_MFMAS : 1);
				multiply(std::integral_constant<int, 0>(), std::integral_constant<int, HEAD>(), std::integral_constant<int, cur>());
				__builtin_amdgcn_sched_barrier(0);
				if constexpr (kk == 0)
				{
					/* one group of the next slice's window per chunk, during the slice's first chunks; then the B rows of chunk c + 1,
					 * into the slot freed by the barrier that opened chunk c */
					if (tap < Lds::WINDOW_LOADS && slice + 1 < slices)
						request_window_group(slice + 1, tap);
					if (more)
						request_b(c + 1);
				}
				if constexpr (kk == 1)
					compute_a_fragments(next_window, next_di, next_dj, a_next);
				if constexpr (kk + 1 < KSTEPS)
					read_fragments(c, kk + 1, a_frag, fa[nxt], fb[nxt]);
				else
				{
					if (more)
					{
						open_chunk();
						read_fragments(c + 1, 0, a_next, fa[nxt], fb[nxt]);
					}
#pragma unroll
					for (int i = 0; i < Cfg::BLOCKS_M; i++)
						a_frag[i] = a_next[i];
				}
				__builtin_amdgcn_sched_barrier(0);
				multiply(std::integral_constant<int, HEAD>(), std::integral_constant<int, MFMAS>(), std::integral_constant<int, cur>());
				__builtin_amdgcn_sched_barrier(0);
			});
		};
		for (int c = 0; c + 1 < chunks; c++)
			process_chunk(c);
		/* the last chunk has been opened with an empty load queue: the epilogue's first loads go out now and land while it is multiplied */
		SlabEpilogue<T, Cfg, Epilogue> store;
		store.begin(M, m0, n0, epilogue);
		process_chunk(chunks - 1);

		/* the slots become the epilogue's slabs: every wavefront must have finished reading fragments */
		__builtin_amdgcn_s_waitcnt(0xc07f);
		barrier_no_fence();
		store.finish(acc, lds, M, epilogue);
	}

	template<typename T, typename Cfg, typename Epilogue>
	__global__ __launch_bounds__(Cfg::THREADS, 1) void kernel_conv_dma_window(const uint8_t *input, SliceMajorDmaRows b_loader, int M, int height, int width,
			int kernel_size, uint32_t fill_word, Epilogue epilogue, int tiles_n)
	{
		extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
		const unsigned int linear = xcd_contiguous_block_id(blockIdx.x, gridDim.x);
		const int tile_m = linear / tiles_n;
		const int tile_n = linear % tiles_n;
		conv_tile_dma_window<T, Cfg>(input, b_loader, M, height, width, kernel_size, fill_word, tile_m * Cfg::BM, tile_n * Cfg::BN, lds, epilogue);
	}

	/*
	 * Whether the window form takes a convolution: a square kernel of 3 x 3 or 5 x 5 taps, pixels of whole 128-byte slices, an image
	 * narrow enough for the window, and an output width of 128 or of a multiple of 192 that is not one of 256. Measured at batch 512 of
	 * 19 x 19 boards in fp16: 128 filters 3 x 3 78 -> 73 us and 5 x 5 179 -> 170 us, 384 filters 5 x 5 1477 -> 1424 us (3 x 3 level);
	 * on the 256-column tiles (wavefront sub-tiles of 128 x 64, four A blocks whose addresses change with every tap) the per-tap
	 * arithmetic costs what the lighter operand stream saves (256 filters: 3 x 3 240 -> 254 us, 5 x 5 642 -> 660 us), so those stay
	 * on the gathering loader.
	 */
	inline bool conv_dma_window_applies(size_t c_bytes, int filters_out, int kernel_h, int kernel_w, int height, int width)
	{
		typedef WindowTileLds<DmaTileMedium> Lds;
		const int halo = (kernel_h / 2) * (width + 1);
		return kernel_h == kernel_w && (kernel_h == 3 || kernel_h == 5) && c_bytes % 128 == 0 && c_bytes > 0 && height >= 1 && halo <= Lds::MAX_HALO
				&& filters_out % 256 != 0 && (filters_out % 192 == 0 || filters_out == 128);
	}
	template<typename T, typename Cfg, typename Epilogue>
	inline void launch_conv_dma_window_as(hipStream_t stream, const void *input, const void *weights, int M, int N, int height, int width, int kernel_size,
			int c_bytes, uint32_t fill_word, const Epilogue &epilogue)
	{
		typedef WindowTileLds<Cfg> Lds;
		auto kernel = kernel_conv_dma_window<T, Cfg, Epilogue>;
		ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), Lds::BYTES);
		const SliceMajorDmaRows b_loader { reinterpret_cast<const uint8_t*>(weights), N, c_bytes, kernel_size * kernel_size };
		const int tiles_m = ceil_div(M, Cfg::BM), tiles_n = ceil_div(N, Cfg::BN);
		hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned int>(tiles_m) * tiles_n), dim3(Cfg::THREADS), Lds::BYTES, stream,
				reinterpret_cast<const uint8_t*>(input), b_loader, M, height, width, kernel_size, fill_word, epilogue, tiles_n);
	}
	template<typename T, typename Epilogue>
	inline void launch_conv_dma_window(hipStream_t stream, const void *input, const void *weights, int M, int N, int height, int width, int kernel_size,
			int c_bytes, uint32_t fill_word, const Epilogue &epilogue)
	{
		if (N % 192 == 0)
			launch_conv_dma_window_as<T, DmaTile192>(stream, input, weights, M, N, height, width, kernel_size, c_bytes, fill_word, epilogue);
		else
			launch_conv_dma_window_as<T, DmaTileMedium>(stream, input, weights, M, N, height, width, kernel_size, c_bytes, fill_word, epilogue);
	}
} /* namespace mlhip */

#endif /* MINML_AMD_GEMM_DMA_WINDOW_HPP_ */
