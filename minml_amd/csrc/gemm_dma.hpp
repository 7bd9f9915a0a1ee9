/*
 * gemm_dma.hpp — the compute-bound MFMA tile engine: ACC[m][n] = sum_k A[m][k] * B[n][k] for tiles of 256 rows, with both operands
 * moved L2 -> LDS by direct-to-LDS loads (global_load_lds_dwordx4, no staging registers).
 *
 * Serves the implicit-GEMM convolution (fp16 / fp32 / int8: the A operand is the never-materialised im2row matrix of reference
 * src/backend/cpu/conv_im2row.cpp:21-59) and dense GEMMs whose K rows are multiples of 128 bytes (gemm / gemm_ex / batched GEMM,
 * reference src/backend/cpu/gemm/gemm.cpp:39-83). Arithmetic is the same as the smaller engine in gemm_core.hpp: fp32 (int32)
 * accumulation over the whole K extent in 32x32 MFMA blocks, B rows as the first MFMA operand, epilogue functor on 4 consecutive n.
 *
 * How it keeps the matrix cores fed (per workgroup of 4 wavefronts, one workgroup per CU):
 *   - a wavefront owns up to 128 x 128 of the tile (16 accumulator blocks = 256 AGPRs), so one 16-byte fragment feeds 4 MFMAs; a
 *     256 x 256 tile needs (256 + 256) * 2 bytes of operands per 2 * 256 * 256 flops, the least a CU's register file allows;
 *   - K is consumed in chunks of 128 bytes per row, i.e. whole 128-byte cache lines per row and request (64-byte pieces made every line
 *     cross the L2 -> L1 path twice and capped the operand stream at 8 TB/s); a chunk of all rows of the A and B tiles is one LDS slot;
 *     chunk c + SLOTS - 1 is requested while chunk c is consumed, its loads spread over the chunk's four k steps;
 *   - completion is tracked by hand (s_waitcnt vmcnt + a fence-free s_barrier per chunk; a __syncthreads() fence would drain the queue);
 *   - per-lane global addresses make the DMA do the im2row gather: a lane whose tap falls outside the image points at a 16-byte row of
 *     a constant table holding the padding byte (zero, or the int8 zero point), so padding costs no branch and no LDS write path;
 *   - the fragment reads of k step t + 1 are issued before the MFMAs of k step t (register double buffer, at most 8 reads outstanding
 *     so that the 4-bit lgkmcnt can express "all but the newest"), so LDS latency is covered by arithmetic;
 *   - a slot is written linearly by the DMA (1 KB per instruction per wavefront: 8 rows x 128 bytes) and read through an XOR swizzle
 *     of the 16-byte chunk index, conflict-free for both.
 */
#ifndef MINML_AMD_GEMM_DMA_HPP_
#define MINML_AMD_GEMM_DMA_HPP_

#include "common.hpp"
#include "gemm_core.hpp"
#include "gemm_stream.hpp"

#include <type_traits>
#include <utility>

namespace mlhip
{
	/* 256 rows of 16 bytes: row v holds the byte v sixteen times (the target of padding lanes) */
	struct PadTable
	{
			uint8_t bytes[256][16];
	};
	constexpr PadTable make_pad_table()
	{
		PadTable t { };
		for (int v = 0; v < 256; v++)
			for (int b = 0; b < 16; b++)
				t.bytes[v][b] = static_cast<uint8_t>(v);
		return t;
	}
	static __device__ const PadTable dma_pad_table = make_pad_table();

	/*
	 * Swizzle of the 16-byte chunk index within a 128-byte LDS row. Measured on gfx950 for the MFMA fragment access (lane l reads row
	 * l % 32, chunk 2 kk + l / 32, 16 bytes): XOR with row / 2 sustains 182 bytes per clock per CU, as fast as a linear read (190);
	 * XOR with row, row / 4 or row + row / 8 only ~118, no swizzle 32.
	 */
	__device__ __forceinline__ int dma_swizzle(int row)
	{
		return (row >> 1) & 7;
	}

	template<int BM_, int BN_, int WAVES_M_, int WAVES_N_, int SLOTS_, int REQUEST_PARTS_ = (SLOTS_ >= 3 ? 4 : 2), int TAIL_MFMAS_ = 4>
	struct DmaTileConfig
	{
			static constexpr int REQUEST_PARTS = REQUEST_PARTS_; /* k steps of a chunk over which the loads of a later chunk are issued */
			static constexpr int TAIL_MFMAS = TAIL_MFMAS_; /* MFMAs of a chunk's last k step issued after the next chunk has been opened */
			static constexpr int BM = BM_;
			static constexpr int BN = BN_;
			static constexpr int BKB = 128; /* bytes of K per row per chunk */
			static constexpr int KSTEPS = BKB / 32; /* MFMA k steps per chunk */
			static constexpr int WAVES_M = WAVES_M_;
			static constexpr int WAVES_N = WAVES_N_;
			static constexpr int WAVES = WAVES_M * WAVES_N;
			static constexpr int THREADS = 64 * WAVES;
			static constexpr int SLOTS = SLOTS_;
			static constexpr int DISTANCE = SLOTS - 1; /* chunks requested ahead of the one being consumed */
			static constexpr int WM = BM / WAVES_M;
			static constexpr int WN = BN / WAVES_N;
			static constexpr int BLOCKS_M = WM / 32;
			static constexpr int BLOCKS_N = WN / 32;
			static constexpr int A_SLOT_BYTES = BM * BKB;
			static constexpr int B_SLOT_BYTES = BN * BKB;
			static constexpr int SLOT_BYTES = A_SLOT_BYTES + B_SLOT_BYTES;
			static constexpr int A_LOADS = BM / 8 / WAVES; /* direct-to-LDS instructions per thread per chunk */
			static constexpr int B_LOADS = BN / 8 / WAVES;
			static constexpr int LOADS_PER_CHUNK = A_LOADS + B_LOADS;
			static constexpr int SLAB_STRIDE = WN + 4; /* epilogue slab row, in 4-byte words */
			static constexpr int SLAB_BYTES = 32 * SLAB_STRIDE * 4;
			static constexpr int EPILOGUE_BYTES = WAVES * SLAB_BYTES;
			static constexpr int LDS_BYTES = (SLOTS * SLOT_BYTES > EPILOGUE_BYTES) ? SLOTS * SLOT_BYTES : EPILOGUE_BYTES;
			static_assert(WM % 32 == 0 && WN % 32 == 0, "wavefront sub-tile must be a grid of 32x32 MFMA blocks");
			static_assert(BM % (8 * WAVES) == 0 && BN % (8 * WAVES) == 0, "tile rows must divide evenly over the wavefronts' 8-row DMA blocks");
			static_assert(SLOTS >= 2 && (SLOTS - 2) * LOADS_PER_CHUNK <= 63, "queue depth must fit the 6-bit vmcnt");
			static_assert(BLOCKS_M + BLOCKS_N <= 15, "fragment reads of one k step must fit the 4-bit lgkmcnt");
			static_assert(LDS_BYTES <= 160 * 1024, "slots must fit the 160 KB of LDS");
	};

	/* Dense operand [rows][K] with K-contiguous rows of k_bytes bytes (a multiple of 128); rows past the end re-read the last row (their products are never stored). */
	struct DenseDmaRows
	{
			const uint8_t *base;
			int rows;
			int k_bytes;
			int row_stride_bytes = 0; /* bytes between consecutive rows; 0 = rows are contiguous (k_bytes apart) */

			struct Row
			{
					const uint8_t *ptr;
			};
			struct Step
			{
					int kb;
			};
			__device__ __forceinline__ Row begin_row(int row) const
			{
				return Row { base + static_cast<size_t>(min(row, rows - 1)) * (row_stride_bytes != 0 ? row_stride_bytes : k_bytes) };
			}
			__device__ __forceinline__ Step first_step() const
			{
				return Step { 0 };
			}
			__device__ __forceinline__ void advance(Step &s) const
			{
				s.kb += 128;
			}
			__device__ __forceinline__ const uint8_t* chunk(const Row &r, const Step &s, int chunk_bytes) const
			{
				return r.ptr + s.kb + chunk_bytes;
			}
	};

	/*
	 * Implicit im2row operand of a stride-1, "same"-padded convolution over an NHWC tensor (row m = pixel (b, h, w); column
	 * k = ((i * kw) + j) * Cin + c reads input[b][h + i - ph][w + j - pw][c], the padding byte outside the image). Cin * sizeof(T) must be
	 * a multiple of 128 so that a chunk never straddles two taps: tap and channel offset of a chunk are then the same for all lanes.
	 */
	struct Im2RowDmaRows
	{
			const uint8_t *base;
			int rows; /* B * H * W */
			int height, width;
			int kernel_h, kernel_w;
			int c_bytes; /* Cin * sizeof(T) */
			int fill; /* padding byte, 0..255 */

			struct Row
			{
					const uint8_t *image;
					int h, w;
			};
			struct Step
			{
					int i, j, c; /* tap row, tap column, byte offset within the tap */
			};
			__device__ __forceinline__ Row begin_row(int row) const
			{
				Row r;
				if (row < rows)
				{
					const int hw = height * width;
					const int b = row / hw;
					const int rem = row - b * hw;
					r.h = rem / width;
					r.w = rem - r.h * width;
					r.image = base + static_cast<size_t>(b) * hw * c_bytes;
				}
				else
				{ /* always outside the image: reads padding */
					r.image = base;
					r.h = -64; /* kernels are far smaller than 64 taps */
					r.w = 0;
				}
				return r;
			}
			__device__ __forceinline__ Step first_step() const
			{
				return Step { 0, 0, 0 };
			}
			__device__ __forceinline__ void advance(Step &s) const
			{
				s.c += 128;
				if (s.c >= c_bytes)
				{
					s.c = 0;
					s.j++;
					if (s.j >= kernel_w)
					{
						s.j = 0;
						s.i++;
					}
				}
			}
			__device__ __forceinline__ const uint8_t* chunk(const Row &r, const Step &s, int chunk_bytes) const
			{
				const int x = r.h + s.i - (kernel_h - 1) / 2;
				const int y = r.w + s.j - (kernel_w - 1) / 2;
				const bool inside = (static_cast<unsigned int>(x) < static_cast<unsigned int>(height))
						&& (static_cast<unsigned int>(y) < static_cast<unsigned int>(width));
				const uint8_t *p = r.image + ((x * width + y) * c_bytes + s.c + chunk_bytes);
				return inside ? p : &dma_pad_table.bytes[fill][0];
			}
	};

	/* f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), expanded at compile time */
	template<typename F, int ... I>
	__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>)
	{
		(f(std::integral_constant<int, I>()), ...);
	}
	template<int N, typename F>
	__device__ __forceinline__ void static_for(F &&f)
	{
		static_for_impl(f, std::make_integer_sequence<int, N>());
	}

	template<int LOADS>
	__device__ __forceinline__ void wait_vmcnt_chunks(int chunks_outstanding)
	{
		switch (chunks_outstanding)
		{
			case 0:
				wait_vmcnt<0>();
				break;
			case 1:
				wait_vmcnt<LOADS>();
				break;
			default:
				wait_vmcnt<2 * LOADS>();
				break;
		}
	}
	template<int N>
	__device__ __forceinline__ void wait_lgkmcnt()
	{
		/* s_waitcnt immediate: lgkmcnt in bits [11:8]; vmcnt (bits [3:0], [15:14]) and expcnt [6:4] left at "no wait" */
		__builtin_amdgcn_s_waitcnt(0xc07f | ((N & 15) << 8));
	}

	/*
	 * Epilogue shared by the tile functions. Lane l, register r of block (i, j) holds n = 32*j + 8*(r/4) + 4*(l/32) + r%4,
	 * m = 32*i + l%32 (relative to the wavefront sub-tile). Each wavefront transposes one 32-row slab at a time through its private LDS
	 * slab [32][WN + 4] and reads it back row-wise, 4 consecutive n per lane, so that the epilogue's global traffic is contiguous along n.
	 */
	/*
	 * The columns of a wavefront's sub-tile that one pass scheme covers: WIDTH / 4 lanes per slab row (4 consecutive n each), hence
	 * 64 / (WIDTH / 4) rows per pass. Sub-tiles 32, 64 or 128 columns wide are one such part; a 96-column sub-tile is a 64-column part
	 * followed by a 32-column part.
	 */
	template<typename Epilogue, int OFFSET_, int WIDTH_>
	struct SlabColumns
	{
			static constexpr int OFFSET = OFFSET_, WIDTH = WIDTH_;
			static constexpr int LANES_PER_ROW = WIDTH / 4, ROWS_PER_PASS = 64 / LANES_PER_ROW, PASSES = 32 / ROWS_PER_PASS;
			static_assert(64 % LANES_PER_ROW == 0 && 32 % ROWS_PER_PASS == 0, "unsupported width of a slab part");
			int row_in_pass, col, n, n_safe;
			bool n_valid;
			typename Epilogue::Column column;
			typename Epilogue::Extra extra[2][PASSES];
	};

	/*
	 * The epilogue of a tile in two steps. begin() places the wavefront's lanes on the slab's columns, fetches the per-column constants
	 * and requests the side inputs (residual) of the first 32-row block; the tile function calls it BEFORE the last chunk of K is
	 * multiplied (the load queue is empty then: the last chunk's operands have landed and nothing else is requested), so that these
	 * loads fly under the last chunk's MFMAs instead of at the head of an epilogue that nothing overlaps. finish() transposes the
	 * accumulators through the slabs and stores. The early requests use clamped addresses (rows past M re-read row M - 1, columns past N
	 * column 0), so they are valid for edge tiles as well.
	 */
	template<typename T, typename Cfg, typename Epilogue>
	struct SlabEpilogue
	{
			typedef typename MfmaTraits<T>::acc_t acc_t;
			typedef acc_t vec4 __attribute__((ext_vector_type(4)));
			static constexpr bool TWO_PARTS = (Cfg::WN == 96);
			typedef SlabColumns<Epilogue, 0, TWO_PARTS ? 64 : Cfg::WN> First;
			typedef SlabColumns<Epilogue, 64, 32> Second;
			First first;
			Second second; /* used only by 96-column sub-tiles */
			int m_wave, n_wave;

			template<typename F>
			__device__ __forceinline__ void for_parts(F &&f)
			{
				f(first);
				if constexpr (TWO_PARTS)
					f(second);
			}
			template<typename Part, int I, int BUF, bool CLAMP>
			__device__ __forceinline__ void request_extras(Part &part, const Epilogue &epilogue, int M, std::integral_constant<int, I>, std::integral_constant<int, BUF>,
					std::integral_constant<bool, CLAMP>)
			{
				if (!epilogue.has_extra())
					return;
#pragma unroll
				for (int pass = 0; pass < Part::PASSES; pass++)
				{
					const int m = m_wave + part.row_in_pass + 32 * I + pass * Part::ROWS_PER_PASS;
					part.extra[BUF][pass] = epilogue.load_extra(CLAMP ? min(m, M - 1) : m, part.n_safe);
				}
			}
			__device__ __forceinline__ void begin(int M, int m0, int n0, const Epilogue &epilogue)
			{
				const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
				m_wave = m0 + (wave / Cfg::WAVES_N) * Cfg::WM;
				n_wave = n0 + (wave % Cfg::WAVES_N) * Cfg::WN;
				for_parts([&](auto &part)
				{
					typedef typename std::decay<decltype(part)>::type Part;
					part.row_in_pass = lane / Part::LANES_PER_ROW;
					part.col = Part::OFFSET + (lane % Part::LANES_PER_ROW) * 4;
					part.n = n_wave + part.col;
					part.n_valid = part.n < epilogue.N;
					part.n_safe = part.n_valid ? part.n : 0;
				});
				if (epilogue.vectorized)
					for_parts([&](auto &part)
					{
						part.column = epilogue.load_column(part.n_safe);
						request_extras(part, epilogue, M, std::integral_constant<int, 0>(), std::integral_constant<int, 0>(), std::true_type());
					});
			}
			template<typename Acc>
			__device__ __forceinline__ void finish(Acc &acc, uint8_t *lds, int M, const Epilogue &epilogue)
			{
				const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
				acc_t *slab = reinterpret_cast<acc_t*>(lds + wave * Cfg::SLAB_BYTES);
				auto fill_slab = [&](auto block)
				{
					constexpr int i = decltype(block)::value;
#pragma unroll
					for (int j = 0; j < Cfg::BLOCKS_N; j++)
#pragma unroll
						for (int q = 0; q < 4; q++)
						{
							vec4 tmp;
#pragma unroll
							for (int e = 0; e < 4; e++)
								tmp[e] = acc[i][j][q * 4 + e];
							*reinterpret_cast<vec4*>(slab + (lane & 31) * Cfg::SLAB_STRIDE + 32 * j + 8 * q + 4 * (lane >> 5)) = tmp;
						}
					__builtin_amdgcn_s_waitcnt(0xc07f); /* lgkmcnt(0): the slab is private to this wavefront, whose LDS operations complete in order */
					__builtin_amdgcn_wave_barrier();
				};
				auto release_slab = [&]()
				{
					__builtin_amdgcn_s_waitcnt(0xc07f);
					__builtin_amdgcn_wave_barrier();
				};
				if (epilogue.vectorized)
				{
					/*
					 * Fast path (4-element groups are whole and aligned). A wavefront is alone on its SIMD, so nothing hides the latency of
					 * the epilogue's own loads: the per-column constants and the first block's side inputs were requested by begin(), and
					 * the side inputs of row block i + 1 are requested before row block i is processed, all passes of a block at once,
					 * from clamped addresses so that no load sits behind a branch.
					 * A wavefront whose whole sub-tile lies inside the matrix (all but the last row / column tiles) runs the UNCHECKED
					 * form: no per-pass range test, hence no branch between the side-input loads and their use, so the compiler counts
					 * the outstanding loads exactly instead of draining them all (vmcnt(0)) in front of every pass.
					 */
					const bool inside = __builtin_amdgcn_readfirstlane(static_cast<int>(m_wave + Cfg::WM <= M && n_wave + Cfg::WN <= epilogue.N)) != 0;
					auto run = [&](auto checked_tag)
					{
						constexpr bool CHECKED = decltype(checked_tag)::value;
						static_for<Cfg::BLOCKS_M>([&](auto block)
						{
							constexpr int i = decltype(block)::value;
							fill_slab(block);
							if constexpr (i + 1 < Cfg::BLOCKS_M)
								for_parts([&](auto &part)
								{
									request_extras(part, epilogue, M, std::integral_constant<int, i + 1>(), std::integral_constant<int, (i + 1) & 1>(),
											std::integral_constant<bool, CHECKED>());
								});
							for_parts([&](auto &part)
							{
								typedef typename std::decay<decltype(part)>::type Part;
#pragma unroll
								for (int pass = 0; pass < Part::PASSES; pass++)
								{
									const int row = pass * Part::ROWS_PER_PASS + part.row_in_pass;
									const vec4 tmp = *reinterpret_cast<const vec4*>(slab + row * Cfg::SLAB_STRIDE + part.col);
									const int m = m_wave + part.row_in_pass + 32 * i + pass * Part::ROWS_PER_PASS;
									if (!CHECKED || (m < M && part.n_valid))
									{
										acc_t vals[4] = { tmp[0], tmp[1], tmp[2], tmp[3] };
										epilogue.apply(m, part.n, vals, part.column, part.extra[i & 1][pass]);
									}
								}
							});
							release_slab();
						});
					};
					if (inside)
						run(std::false_type());
					else
						run(std::true_type());
				}
				else
				{
					/* general path: the functor handles ragged and unaligned groups element by element; the passes stay a rolled loop */
					static_for<Cfg::BLOCKS_M>([&](auto block)
					{
						constexpr int i = decltype(block)::value;
						fill_slab(block);
						for_parts([&](auto &part)
						{
							typedef typename std::decay<decltype(part)>::type Part;
#pragma clang loop unroll(disable)
							for (int pass = 0; pass < Part::PASSES; pass++)
							{
								const int row = pass * Part::ROWS_PER_PASS + part.row_in_pass;
								const vec4 tmp = *reinterpret_cast<const vec4*>(slab + row * Cfg::SLAB_STRIDE + part.col);
								const int m = m_wave + part.row_in_pass + 32 * i + pass * Part::ROWS_PER_PASS;
								if (m < M)
								{
									acc_t vals[4] = { tmp[0], tmp[1], tmp[2], tmp[3] };
									epilogue(m, part.n, vals);
								}
							}
						});
						release_slab();
					});
				}
			}
	};

	/*
	 * Computes one BM x BN tile and hands every group of 4 consecutive n of one row m < M to epilogue(m, n, acc[4]) (the functor masks
	 * n itself). k_bytes must be a positive multiple of 128. `lds` is the workgroup's dynamic LDS block of Cfg::LDS_BYTES bytes.
	 */
	template<typename T, typename Cfg, typename ALoader, typename BLoader, typename Epilogue>
	__device__ __forceinline__ void gemm_tile_dma(const ALoader &a_loader, const BLoader &b_loader, int M, int k_bytes, int m0, int n0, uint8_t *lds,
			const Epilogue &epilogue)
	{
		typedef MfmaTraits<T> Traits;
		typedef typename Traits::acc_vec acc_vec;
		typedef typename Traits::acc_t acc_t;
		constexpr int SLOTS = Cfg::SLOTS, DISTANCE = Cfg::DISTANCE, KSTEPS = Cfg::KSTEPS;

		const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
		const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;

		/* loader geometry: wavefront w fills the 1 KB blocks w, w + WAVES, ... of each operand; lane l fills position l of a block, i.e.
		 * row l / 8 of the block's 8 rows and position l % 8 of that row, and fetches the chunk the swizzle assigns to that position */
		typename ALoader::Row a_rows[Cfg::A_LOADS];
		typename BLoader::Row b_rows[Cfg::B_LOADS];
		int a_chunk[Cfg::A_LOADS], b_chunk[Cfg::B_LOADS];
#pragma unroll
		for (int i = 0; i < Cfg::A_LOADS; i++)
		{
			const int row = (wave + Cfg::WAVES * i) * 8 + (lane >> 3);
			a_chunk[i] = ((lane & 7) ^ dma_swizzle(row)) * 16;
			a_rows[i] = a_loader.begin_row(m0 + row);
		}
#pragma unroll
		for (int i = 0; i < Cfg::B_LOADS; i++)
		{
			const int row = (wave + Cfg::WAVES * i) * 8 + (lane >> 3);
			b_chunk[i] = ((lane & 7) ^ dma_swizzle(row)) * 16;
			b_rows[i] = b_loader.begin_row(n0 + row);
		}
		/* K position of the chunk whose loads are being issued (chunks are requested in order) */
		typename ALoader::Step a_step = a_loader.first_step();
		typename BLoader::Step b_step = b_loader.first_step();
		const int chunks = k_bytes / Cfg::BKB;

		/* The loads of a chunk are issued in PARTS portions, one per k step of the chunk being consumed: spread over all four k steps
		 * when the queue is deep enough, in the first two when the chunk is needed right after this one (SLOTS == 2). Portion `part`
		 * holds the loads whose index l (A loads first, then B loads) has l % PARTS == part. */
		constexpr int PARTS = Cfg::REQUEST_PARTS;
		auto request_part = [&](int c, int part)
		{
			uint8_t *slot = lds + (c % SLOTS) * Cfg::SLOT_BYTES;
#pragma unroll
			for (int l = 0; l < Cfg::LOADS_PER_CHUNK; l++)
				if (l % PARTS == part)
				{
					if (l < Cfg::A_LOADS)
						__builtin_amdgcn_global_load_lds((global_ptr_t) a_loader.chunk(a_rows[l], a_step, a_chunk[l]),
								(lds_ptr_t) (slot + (wave + Cfg::WAVES * l) * 1024), 16, 0, 0);
					else
						__builtin_amdgcn_global_load_lds((global_ptr_t) b_loader.chunk(b_rows[l - Cfg::A_LOADS], b_step, b_chunk[l - Cfg::A_LOADS]),
								(lds_ptr_t) (slot + Cfg::A_SLOT_BYTES + (wave + Cfg::WAVES * (l - Cfg::A_LOADS)) * 1024), 16, 0, 0);
				}
			if (part == PARTS - 1)
			{
				a_loader.advance(a_step);
				b_loader.advance(b_step);
			}
		};

		/* fragment geometry: lane l supplies row l % 32 of a 32-row block and the 16-byte half l / 32 of each 32-byte k step; the byte
		 * offset of k step kk within the row is ((2 kk + l / 32) ^ swizzle) * 16 = (first ^ (kk * 32)) because kk only sets bits 5..6 */
		int a_frag[Cfg::BLOCKS_M], b_frag[Cfg::BLOCKS_N];
#pragma unroll
		for (int i = 0; i < Cfg::BLOCKS_M; i++)
		{
			const int row = wave_m * Cfg::WM + 32 * i + (lane & 31);
			a_frag[i] = row * Cfg::BKB + (((lane >> 5) ^ dma_swizzle(row)) * 16);
		}
#pragma unroll
		for (int j = 0; j < Cfg::BLOCKS_N; j++)
		{
			const int row = wave_n * Cfg::WN + 32 * j + (lane & 31);
			b_frag[j] = Cfg::A_SLOT_BYTES + row * Cfg::BKB + (((lane >> 5) ^ dma_swizzle(row)) * 16);
		}

		acc_vec acc[Cfg::BLOCKS_M][Cfg::BLOCKS_N];
#pragma unroll
		for (int i = 0; i < Cfg::BLOCKS_M; i++)
#pragma unroll
			for (int j = 0; j < Cfg::BLOCKS_N; j++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					acc[i][j][r] = 0;

		for (int c = 0; c < DISTANCE; c++)
			if (c < chunks)
				for (int part = 0; part < PARTS; part++)
					request_part(c, part);

		/* fragments of one k step: (BLOCKS_M + BLOCKS_N) x 16 bytes per lane; two copies alternate between consecutive k steps */
		uint4_t fa[2][Cfg::BLOCKS_M], fb[2][Cfg::BLOCKS_N];
		auto read_fragments = [&](int c, int kk, uint4_t (&a_regs)[Cfg::BLOCKS_M], uint4_t (&b_regs)[Cfg::BLOCKS_N])
		{
			const uint8_t *slot = lds + (c % SLOTS) * Cfg::SLOT_BYTES;
#pragma unroll
			for (int i = 0; i < Cfg::BLOCKS_M; i++)
				a_regs[i] = *reinterpret_cast<const uint4_t*>(slot + (a_frag[i] ^ (kk * 32)));
#pragma unroll
			for (int j = 0; j < Cfg::BLOCKS_N; j++)
				b_regs[j] = *reinterpret_cast<const uint4_t*>(slot + (b_frag[j] ^ (kk * 32)));
		};
		/* chunk c becomes readable: its loads have landed in every wavefront, and the slot of chunk c - 1 is free for chunk c + DISTANCE */
		auto open_chunk = [&](int c)
		{
			wait_lgkmcnt<0>(); /* this wavefront's reads of chunk c - 1 are complete before anyone may overwrite its slot */
			wait_vmcnt_chunks<Cfg::LOADS_PER_CHUNK>(min(DISTANCE - 1, chunks - 1 - c));
			barrier_no_fence();
		};

		if (chunks > 0)
		{
			open_chunk(0);
			read_fragments(0, 0, fa[0], fb[0]);
		}
		/* MFMAs number lo .. hi - 1 of a k step, in the order i-major over the accumulator blocks */
		auto multiply = [&](auto lo, auto hi, auto buffer)
		{
			constexpr int cur = decltype(buffer)::value;
						static_for<decltype(hi)::value - decltype(lo)::value>([&](auto index)
			{
				constexpr int idx = decltype(lo)::value + decltype(index)::value;
				constexpr int i = idx / Cfg::BLOCKS_N, j = idx % Cfg::BLOCKS_N;
				Traits::mma(fb[cur][j], fa[cur][i], acc[i][j]); /* B rows as first operand: lane gets 4 consecutive n */
			});
		};
		constexpr int MFMAS = Cfg::BLOCKS_M * Cfg::BLOCKS_N;
		auto process_chunk = [&](int c) __attribute__((always_inline))
		{
			const bool request = (c + DISTANCE < chunks);
			static_for<KSTEPS>([&](auto kstep)
			{
				constexpr int kk = decltype(kstep)::value;
				constexpr int cur = kk & 1, nxt = 1 - cur;
				/*
				 * Order within a k step: a few MFMAs first, then the fragment reads of the next k step, then the remaining MFMAs. The
				 * compiler guards the first MFMA with a full lgkmcnt(0) (it does not count in-order LDS returns across the loop), which
				 * is free here because this k step's fragments were requested a whole k step ago and nothing newer is outstanding yet;
				 * the reads issued after it then have the remaining MFMAs to complete. The scheduling barriers keep the scheduler
				 * from sinking the reads below the MFMAs (it would, to shorten register live ranges). The last k step of a chunk issues
				 * more MFMAs up front, so that the matrix pipe has work queued while this wavefront waits at the chunk's barrier.
				 */
				constexpr int HEAD = (kk + 1 < KSTEPS) ? 1 : (MFMAS > Cfg::TAIL_MFMAS ? MFMAS - Cfg::TAIL_MFMAS : 1);
				multiply(std::integral_constant<int, 0>(), std::integral_constant<int, HEAD>(), std::integral_constant<int, cur>());
				__builtin_amdgcn_sched_barrier(0);
				/* a portion of the loads of the chunk DISTANCE ahead, into the slot freed by the barrier that opened chunk c */
				if (request && kk < PARTS)
					request_part(c + DISTANCE, kk);
				/* fragment reads of the next k step (the first one of the next chunk after that chunk has been opened) */
				if (kk + 1 < KSTEPS)
					read_fragments(c, kk + 1, fa[nxt], fb[nxt]);
				else if (c + 1 < chunks)
				{
					open_chunk(c + 1);
					read_fragments(c + 1, 0, fa[nxt], fb[nxt]);
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
		if (chunks > 0)
			process_chunk(chunks - 1);

		/* the slots become the epilogue's slabs: every wavefront must have finished reading fragments */
		__builtin_amdgcn_s_waitcnt(0xc07f);
		barrier_no_fence();

		store.finish(acc, lds, M, epilogue);
	}

	/* tile shapes by output width: wavefront sub-tiles of 128x128, 128x64 and 64x64 */
	typedef DmaTileConfig<256, 256, 2, 4, 2, 2, 4> DmaTileWide;
	typedef DmaTileConfig<256, 128, 4, 2, 2, 2, 2> DmaTileMedium;
	typedef DmaTileConfig<256, 64, 4, 2, 3, 4, 2> DmaTileNarrow;
	typedef DmaTileConfig<256, 192, 4, 2, 2, 2, 2> DmaTile192; /* wavefront sub-tiles of 64 x 96: widths that are multiples of 192 but not of 256 (384 channels) */

	/*
	 * One workgroup per tile; blockIdx.y selects the matrix of a batch (operand bases advance by the given byte strides, D and C of the
	 * epilogue by stride_c elements). Column tiles of one row tile get consecutive ids on one XCD, so the A rows they share meet in L2.
	 */
	template<typename T, typename Cfg, typename ALoader, typename Epilogue>
	__global__ __launch_bounds__(Cfg::THREADS, 1) void kernel_gemm_dma(ALoader a_loader, DenseDmaRows b_loader, int M, int k_bytes, size_t stride_a_bytes,
			size_t stride_b_bytes, size_t stride_c, Epilogue epilogue, int tiles_n)
	{
		extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
		const unsigned int linear = xcd_contiguous_block_id(blockIdx.x, gridDim.x);
		const int tile_m = linear / tiles_n;
		const int tile_n = linear % tiles_n;
		const size_t batch = blockIdx.y;
		a_loader.base += batch * stride_a_bytes;
		b_loader.base += batch * stride_b_bytes;
		epilogue.D += batch * stride_c;
		if constexpr (Epilogue::has_c)
		{
			epilogue.C += batch * stride_c;
			if (epilogue.bias != nullptr)
				epilogue.bias += batch * epilogue.bias_batch_stride; /* 0 unless every matrix of the batch has its own bias */
		}
		gemm_tile_dma<T, Cfg>(a_loader, b_loader, M, k_bytes, tile_m * Cfg::BM, tile_n * Cfg::BN, lds, epilogue);
	}

	template<typename T, typename Cfg, typename ALoader, typename Epilogue>
	inline void launch_gemm_dma_as(hipStream_t stream, const ALoader &a_loader, const DenseDmaRows &b_loader, int M, int N, int k_bytes, int batch,
			size_t stride_a_bytes, size_t stride_b_bytes, size_t stride_c, const Epilogue &epilogue)
	{
		auto kernel = kernel_gemm_dma<T, Cfg, ALoader, Epilogue>;
		ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), Cfg::LDS_BYTES);
		const int tiles_m = ceil_div(M, Cfg::BM), tiles_n = ceil_div(N, Cfg::BN);
		hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned int>(tiles_m) * tiles_n, batch), dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream, a_loader,
				b_loader, M, k_bytes, stride_a_bytes, stride_b_bytes, stride_c, epilogue, tiles_n);
	}
	/* picks the tile width that pads N least (ties go to the wider tile, whose fragments feed more MFMAs) */
	template<typename T, typename ALoader, typename Epilogue>
	inline void launch_gemm_dma(hipStream_t stream, const ALoader &a_loader, const DenseDmaRows &b_loader, int M, int N, int k_bytes, int batch,
			size_t stride_a_bytes, size_t stride_b_bytes, size_t stride_c, const Epilogue &epilogue)
	{
		const int wide = ceil_div(N, 256) * 256, medium = ceil_div(N, 128) * 128, narrow = ceil_div(N, 64) * 64;
		if (N % 192 == 0 && N % 256 != 0)
			launch_gemm_dma_as<T, DmaTile192>(stream, a_loader, b_loader, M, N, k_bytes, batch, stride_a_bytes, stride_b_bytes, stride_c, epilogue);
		else if (N > 256 && N % 256 != 0)
		{
			/* e.g. N = 384: the first 256 columns on wide tiles (more flops per operand byte and per fragment read), the remaining
			 * columns on the tile width that pads them least, instead of narrower tiles throughout */
			const int first = N / 256 * 256;
			DenseDmaRows head = b_loader, tail = b_loader;
			head.rows = first;
			tail.rows = N - first;
			tail.base += static_cast<size_t>(first) * (b_loader.row_stride_bytes != 0 ? b_loader.row_stride_bytes : b_loader.k_bytes);
			launch_gemm_dma_as<T, DmaTileWide>(stream, a_loader, head, M, first, k_bytes, batch, stride_a_bytes, stride_b_bytes, stride_c,
					epilogue.columns(0, first));
			launch_gemm_dma<T>(stream, a_loader, tail, M, N - first, k_bytes, batch, stride_a_bytes, stride_b_bytes, stride_c,
					epilogue.columns(first, N - first));
		}
		else if (wide <= medium && wide <= narrow)
			launch_gemm_dma_as<T, DmaTileWide>(stream, a_loader, b_loader, M, N, k_bytes, batch, stride_a_bytes, stride_b_bytes, stride_c, epilogue);
		else if (medium <= narrow)
			launch_gemm_dma_as<T, DmaTileMedium>(stream, a_loader, b_loader, M, N, k_bytes, batch, stride_a_bytes, stride_b_bytes, stride_c, epilogue);
		else
			launch_gemm_dma_as<T, DmaTileNarrow>(stream, a_loader, b_loader, M, N, k_bytes, batch, stride_a_bytes, stride_b_bytes, stride_c, epilogue);
	}
} /* namespace mlhip */

#endif /* MINML_AMD_GEMM_DMA_HPP_ */
