/*
 * gemm_stream.hpp — the streaming batched GEMM of the Winograd path:  C[i] = A[i] * B[i]^T  for rows of exactly 512 bytes of K
 * (256 halfs or 128 floats: the channel counts of the benchmark networks), plain store of the product (alpha = 1, beta = 0).
 *
 * This product is bound by HBM, not by the matrix cores: one matrix pair moves T*512 bytes in and T*N*s bytes out for only
 * 2*T*N*K flops, and the 36 B operands together are a few megabytes. The kernel is therefore organised around the A stream:
 *   - persistent workgroups (one per CU), each owning a set of "units" (128 rows of A of one matrix; 64 rows for the plain batched
 *     products on the 8-wavefront layout, see launch_stream_gemm_as) and, with 8
 *     wavefronts of 32 columns each, all 256 columns of N, so that every row of A is fetched by exactly one workgroup (for wider N the
 *     column slices of one row range sit on one XCD and share its L2);
 *   - every wavefront keeps ITS part of the B operand (32 columns x full K = 64 VGPRs) in registers for the whole run of units that
 *     share a matrix, so B costs neither LDS space nor LDS bandwidth;
 *   - A moves HBM -> LDS with direct-to-LDS loads (global_load_lds_dwordx4, no staging registers) into a ring of 128-byte-per-row
 *     stages that runs ahead across unit boundaries (STAGES - 1 stages of 16 KB, or of 8 KB for units of 64 rows), so loads never stop for an epilogue or for the next
 *     unit's prologue; completion is tracked with explicit vmcnt waits and fence-free barriers (a fence would drain the whole ring);
 *   - two wavefronts per SIMD: one that waits (full memory pipeline, stage barrier, store epilogue) leaves the SIMD to the other;
 *   - fragment reads of k step t + 1 are in flight while k step t is multiplied (register double buffer);
 *   - LDS stages are written linearly by the DMA and read through an XOR swizzle of the 16-byte chunk index (row / 2: measured to be
 *     the placement that sustains full LDS read bandwidth for the MFMA fragment access on gfx950);
 *   - accumulators leave through a per-wavefront LDS slab so that global stores are 16 bytes per lane, 64 bytes contiguous per row.
 */
#ifndef MINML_AMD_GEMM_STREAM_HPP_
#define MINML_AMD_GEMM_STREAM_HPP_

#include "common.hpp"
#include "gemm_core.hpp"
#include "epilogues.hpp"

#include <type_traits>

namespace mlhip
{
	typedef __attribute__((address_space(3))) void *lds_ptr_t;
	typedef __attribute__((address_space(1))) const void *global_ptr_t;

	template<int N>
	__device__ __forceinline__ void wait_vmcnt()
	{
		/* s_waitcnt immediate: vmcnt in bits [3:0] and [15:14], expcnt [6:4] and lgkmcnt [11:8] left at "no wait" */
		__builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
	}
	__device__ __forceinline__ void wait_lgkmcnt_zero()
	{
		__builtin_amdgcn_s_waitcnt(0xc07f);
	}
	/* s_barrier without a memory fence: the waits above already order the direct-to-LDS loads this kernel cares about */
	__device__ __forceinline__ void barrier_no_fence()
	{
		asm volatile("" ::: "memory");
		__builtin_amdgcn_s_barrier();
		asm volatile("" ::: "memory");
	}

	struct StreamGemmConfig
	{
			static constexpr int BM = 128; /* rows of A per unit */
			static constexpr int BN = 128; /* columns per workgroup */
			static constexpr int K_BYTES = 512;
			static constexpr int STAGE_K_BYTES = 128; /* bytes of K per row per stage */
			static constexpr int STAGE_BYTES = BM * STAGE_K_BYTES; /* 16 KB */
			static constexpr int STAGES_PER_UNIT = K_BYTES / STAGE_K_BYTES; /* 4 */
	};

	/* at most `stages` stages of LOADS vector-memory operations each may remain outstanding (stages <= MAX; the counter holds up to 63) */
	template<int LOADS, int MAX = 14>
	__device__ __forceinline__ void wait_vmcnt_stages(int stages)
	{
		if constexpr (MAX == 0)
			wait_vmcnt<0>();
		else
		{
			if (stages >= MAX)
				wait_vmcnt<(MAX * LOADS <= 63) ? MAX * LOADS : 63>();
			else
				wait_vmcnt_stages<LOADS, MAX - 1>(stages);
		}
	}
	template<int N, typename F>
	__device__ __forceinline__ void stream_static_for(F &&f)
	{
		if constexpr (N > 0)
		{
			stream_static_for<N - 1>(f);
			f(std::integral_constant<int, N - 1>());
		}
	}

	/* tag: store the product as is (alpha = 1, beta = 0, no bias, linear), 16 bytes per lane */
	struct PlainStore
	{
	};
	/* epilogues that read nothing per output element (PlainStore; functors whose residual is absent at compile time): their results are
	 * finished in the accumulator registers and cross the slab in the output type, 16 bytes per lane on the way out */
	template<typename Epilogue>
	struct stream_epilogue_reads_nothing
	{
			static constexpr bool value = Epilogue::no_side_input;
	};
	template<>
	struct stream_epilogue_reads_nothing<PlainStore>
	{
			static constexpr bool value = true;
	};

	/*
	 * One workgroup of WAVES_M x WAVES_N wavefronts covers a unit of 128 rows x 32 * WAVES_N columns; a wavefront owns 128 / WAVES_M
	 * rows x 32 columns, keeps the B operand of its 32 columns (KB bytes of K each) in KB / 8 VGPRs and accumulates in 32x32 blocks; the
	 * pipeline is one k step deep. KB = 128, 256 or 512 bytes per K row. Epilogue: PlainStore, or a functor with the split protocol of
	 * epilogues.hpp (load_column / load_extra / apply on 4 consecutive n, vectorized case only; value() instead of apply() for functors
	 * that read nothing per element), whose D / C pointers advance by stride_c and whose bias advances by its bias_batch_stride per
	 * matrix of the batch. Consecutive rows of A lie a_row_bytes apart (KB for a dense matrix; more when the matrices of the batch are
	 * interleaved row by row, as the experts' tokens are).
	 */
	template<typename T, int KB, int WAVES_M, int WAVES_N, int STAGES, typename Epilogue, int BM = StreamGemmConfig::BM>
	__global__ __launch_bounds__(64 * WAVES_M * WAVES_N, 1) void kernel_gemm_stream_wide_nt(const T *A, const T *B, T *C, int M, int N, size_t stride_a,
			size_t stride_b, size_t stride_c, int batch, int tiles_m, int n_tiles, int units_per_group, int sweep, size_t a_row_bytes, Epilogue epilogue)
	{
		typedef StreamGemmConfig Cfg;
		typedef MfmaTraits<T> Traits;
		typedef typename Traits::acc_vec acc_vec;
		typedef typename Traits::acc_t acc_t;
		constexpr bool PLAIN = std::is_same<Epilogue, PlainStore>::value;
		constexpr bool PACKED = stream_epilogue_reads_nothing<Epilogue>::value;
		constexpr int WAVES = WAVES_M * WAVES_N;
		constexpr int BN = 32 * WAVES_N;
		constexpr int STAGE_BYTES = BM * Cfg::STAGE_K_BYTES; /* one stage: 128 bytes of K of every row of a unit */
		constexpr int ROWS = BM / WAVES_M; /* rows of a unit owned by one wavefront */
		constexpr int BLOCKS = ROWS / 32;
		constexpr int STAGES_PER_UNIT = KB / Cfg::STAGE_K_BYTES;
		constexpr int DISTANCE = STAGES - 1; /* stages requested ahead of the one being multiplied */
		constexpr int LOADS = (STAGE_BYTES / 1024) / WAVES; /* 1 KB blocks of a stage moved by one wavefront */
		constexpr int SLAB_STRIDE = 32 * (PACKED ? sizeof(T) : 4) + 16;
		constexpr int KSTEPS = 4; /* MFMA k steps per stage */
		static_assert(KB % Cfg::STAGE_K_BYTES == 0 && ROWS % 32 == 0, "unsupported unit shape");
		static_assert(LOADS >= 1 && (STAGE_BYTES / 1024) % WAVES == 0 && DISTANCE >= 2 && DISTANCE <= 16 && (DISTANCE - 2) * LOADS <= 63, "unsupported workgroup shape");
		extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
		uint8_t *ring = lds;
		uint8_t *slab = lds + STAGES * STAGE_BYTES + (threadIdx.x >> 6) * (32 * SLAB_STRIDE);

		const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
		const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
		int group, n_tile;
		if (gridDim.x % (8 * n_tiles) == 0)
		{ /* ids congruent mod 8 share an XCD: give the column slices of one group consecutive slots of one XCD */
			const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
			group = (slot / n_tiles) * 8 + xcd;
			n_tile = slot % n_tiles;
		}
		else
		{
			group = blockIdx.x / n_tiles;
			n_tile = blockIdx.x % n_tiles;
		}
		const int n0 = n_tile * BN + wave_n * 32; /* first column of this wavefront */
		const int total_units = batch * tiles_m;
		/*
		 * Which units this workgroup owns. Default: a contiguous range of units_per_group units, ascending. Sweep form (sweep > 0
		 * workgroups per matrix): workgroup j of a matrix takes its row blocks j, j + sweep, ... and walks them from the last to the
		 * first, so that all workgroups move through the rows of their matrices together, from the end to the beginning. A producer
		 * that wrote these rows in ascending order left the last ones in the last-level cache, and a consumer that reads the product
		 * in ascending order finds the rows written last by this kernel there.
		 */
		const int sweep_matrix = (sweep > 0) ? group / sweep : 0;
		const int sweep_lane = (sweep > 0) ? group % sweep : 0;
		const int unit_begin = (sweep > 0) ? sweep_matrix * tiles_m : group * units_per_group;
		const int unit_end = (sweep > 0) ? ((sweep_matrix < batch && sweep_lane < tiles_m) ? unit_begin + 1 : unit_begin)
				: min(total_units, unit_begin + units_per_group);
		if (unit_begin >= unit_end)
			return;

		int load_row[LOADS], load_chunk_bytes[LOADS];
#pragma unroll
		for (int i = 0; i < LOADS; i++)
		{
			const int row = (wave + WAVES * i) * 8 + (lane >> 3);
			load_row[i] = row;
			load_chunk_bytes[i] = ((lane & 7) ^ ((row >> 1) & 7)) * 16;
		}
		const int frag_row = lane & 31;
		const int half_sel = lane >> 5;
		int frag_first[BLOCKS]; /* byte offset within a stage of this lane's fragment of k step 0, per 32-row block */
#pragma unroll
		for (int i = 0; i < BLOCKS; i++)
		{
			const int row = wave_m * ROWS + 32 * i + frag_row;
			frag_first[i] = row * Cfg::STAGE_K_BYTES + ((half_sel ^ ((row >> 1) & 7)) * 16);
		}

		int unit = unit_begin;
		while (unit < unit_end)
		{
			/* ---- a run of units of one matrix ---- */
			const int matrix = unit / tiles_m;
			const int run_end = min(unit_end, (matrix + 1) * tiles_m);
			const int run_units = (sweep > 0) ? (tiles_m - sweep_lane + sweep - 1) / sweep : run_end - unit;
			const int run_stages = run_units * STAGES_PER_UNIT;
			/* row block of the u-th unit of this run: tile_base + u * tile_step */
			const int tile_base = (sweep > 0) ? sweep_lane + (run_units - 1) * sweep : unit - matrix * tiles_m;
			const int tile_step = (sweep > 0) ? -sweep : 1;
			const uint8_t *a_base = reinterpret_cast<const uint8_t*>(A + static_cast<size_t>(matrix) * stride_a);
			const uint8_t *b_base = reinterpret_cast<const uint8_t*>(B + static_cast<size_t>(matrix) * stride_b);
			T *c_base = C + static_cast<size_t>(matrix) * stride_c;
			Epilogue local = epilogue;
			if constexpr (!PLAIN)
			{
				local.D += static_cast<size_t>(matrix) * stride_c;
				if constexpr (Epilogue::has_c)
				{
					local.C += static_cast<size_t>(matrix) * stride_c;
					if (local.bias != nullptr)
						local.bias += static_cast<size_t>(matrix) * local.bias_batch_stride; /* 0 unless every matrix has its own bias */
				}
			}

			wait_vmcnt<0>();
			wait_lgkmcnt_zero();
			barrier_no_fence(); /* nobody reads stages of the previous run any more */

			uint4_t b_regs[KB / 32]; /* 32 columns x KB / 32 k steps, 16 bytes per lane each */
			{
				const int n = min(n0 + frag_row, N - 1);
				const uint8_t *row = b_base + static_cast<size_t>(n) * KB + half_sel * 16;
#pragma unroll
				for (int k = 0; k < KB / 32; k++)
					b_regs[k] = *reinterpret_cast<const uint4_t*>(row + k * 32);
			}
			auto request_stage = [&](int g) __attribute__((always_inline))
			{
				const int u = g / STAGES_PER_UNIT, ks = g - u * STAGES_PER_UNIT;
				const int m_first = (tile_base + u * tile_step) * BM;
				uint8_t *stage = ring + (g % STAGES) * STAGE_BYTES;
#pragma unroll
				for (int i = 0; i < LOADS; i++)
				{
					const int m = min(m_first + load_row[i], M - 1); /* rows past the end re-read the last row; their products are never stored */
					__builtin_amdgcn_global_load_lds((global_ptr_t) (a_base + static_cast<size_t>(m) * a_row_bytes + ks * Cfg::STAGE_K_BYTES + load_chunk_bytes[i]),
							(lds_ptr_t) (stage + (wave + WAVES * i) * 1024), 16, 0, 2); /* non-temporal: every row of A is read once */
				}
			};
			uint4_t frags[2][BLOCKS];
			auto read_fragments = [&](int g, int kk, uint4_t (&regs)[BLOCKS]) __attribute__((always_inline))
			{
				const uint8_t *stage = ring + (g % STAGES) * STAGE_BYTES;
#pragma unroll
				for (int i = 0; i < BLOCKS; i++)
					regs[i] = *reinterpret_cast<const uint4_t*>(stage + (frag_first[i] ^ (kk * 32)));
			};
			acc_vec acc[BLOCKS];
			auto clear_accumulators = [&]() __attribute__((always_inline))
			{
#pragma unroll
				for (int i = 0; i < BLOCKS; i++)
#pragma unroll
					for (int r = 0; r < 16; r++)
						acc[i][r] = 0;
			};
			/*
			 * Side inputs of the epilogue (per-column constants, residual of every pass of the unit). Loads return in order, so a load
			 * issued at store time would have to wait for the whole ring in front of it; the residual of unit u is therefore requested
			 * when unit u starts, from clamped addresses, and is old by the time it is used.
			 */
			struct NoSide
			{
					struct Column
					{
					};
					struct Extra
					{
					};
			};
			struct Side
			{
					typename std::conditional<PLAIN, NoSide, Epilogue>::type::Column column;
					typename std::conditional<PLAIN, NoSide, Epilogue>::type::Extra extra[BLOCKS][4];
			};
			typename std::conditional<PLAIN, NoSide, Side>::type side;
			const int side_n = (n0 + (lane & 7) * 4 < N) ? n0 + (lane & 7) * 4 : 0;
			auto request_side_inputs = [&](int u) __attribute__((always_inline))
			{
				if constexpr (!PLAIN)
				{
					if (!local.has_extra())
						return;
					const int m_first = (tile_base + u * tile_step) * BM + wave_m * ROWS;
#pragma unroll
					for (int i = 0; i < BLOCKS; i++)
#pragma unroll
						for (int pass = 0; pass < 4; pass++)
							side.extra[i][pass] = local.load_extra(min(m_first + 32 * i + pass * 8 + (lane >> 3), M - 1), side_n);
				}
			};
			if constexpr (!PACKED)
				side.column = local.load_column(side_n);
			/* packed form: the constants of this lane's 4 consecutive n in each of the 4 register groups of an accumulator block */
			typename std::conditional<PLAIN, NoSide, Epilogue>::type::Column packed_columns[4];
			if constexpr (PACKED && !PLAIN)
			{
#pragma unroll
				for (int q = 0; q < 4; q++)
				{
					const int n = n0 + 8 * q + 4 * half_sel;
					packed_columns[q] = local.load_column(n < local.N ? n : 0);
				}
			}
			auto store_unit = [&](int u) __attribute__((always_inline))
			{
				/* lane l, register r of block i: m = 32 i + l % 32, n = 8 (r / 4) + 4 (l / 32) + r % 4 */
				const int m_first = (tile_base + u * tile_step) * BM + wave_m * ROWS;
				if constexpr (PACKED)
				{
					T *out_base;
					size_t out_stride;
					int out_n;
					if constexpr (PLAIN)
					{
						out_base = c_base;
						out_stride = N;
						out_n = N;
					}
					else
					{
						out_base = local.D;
						out_stride = local.row_stride;
						out_n = local.N;
					}
					constexpr int ELEMS_PER_16B = 16 / sizeof(T);
					constexpr int LANES_PER_ROW = 32 / ELEMS_PER_16B;
					constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
					const int col = (lane % LANES_PER_ROW) * ELEMS_PER_16B;
#pragma unroll
					for (int i = 0; i < BLOCKS; i++)
					{
#pragma unroll
						for (int q = 0; q < 4; q++)
						{
							Vec<T, 4> v;
							if constexpr (PLAIN)
							{
#pragma unroll
								for (int e = 0; e < 4; e++)
									v.v[e] = acc[i][4 * q + e];
							}
							else
							{
								const acc_t vals[4] = { acc[i][4 * q + 0], acc[i][4 * q + 1], acc[i][4 * q + 2], acc[i][4 * q + 3] };
								v = local.value(vals, packed_columns[q]);
							}
							v.store(reinterpret_cast<T*>(slab + frag_row * SLAB_STRIDE) + 8 * q + 4 * half_sel);
						}
						wait_lgkmcnt_zero(); /* the slab is private to this wavefront */
						__builtin_amdgcn_wave_barrier();
#pragma unroll
						for (int pass = 0; pass < 32 / ROWS_PER_PASS; pass++)
						{
							const int row = pass * ROWS_PER_PASS + lane / LANES_PER_ROW;
							const uint4_t v = *reinterpret_cast<const uint4_t*>(slab + row * SLAB_STRIDE + col * sizeof(T));
							const int m = m_first + 32 * i + row;
							if (m < M && n0 + col < out_n) /* the width is a multiple of the 16-byte vector (checked by the launcher) */
								*reinterpret_cast<uint4_t*>(out_base + static_cast<size_t>(m) * out_stride + n0 + col) = v;
						}
						wait_lgkmcnt_zero();
						__builtin_amdgcn_wave_barrier();
					}
				}
				else
				{
					/* accumulators cross the slab unconverted; every lane then owns 4 consecutive n of one row per pass */
					typedef acc_t vec4 __attribute__((ext_vector_type(4)));
					constexpr int ROWS_PER_PASS = 8, PASSES = 4;
					const int col = (lane & 7) * 4;
					const int n = n0 + col;
					const bool n_valid = n < local.N;
#pragma unroll
					for (int i = 0; i < BLOCKS; i++)
					{
#pragma unroll
						for (int q = 0; q < 4; q++)
						{
							vec4 v;
#pragma unroll
							for (int e = 0; e < 4; e++)
								v[e] = acc[i][4 * q + e];
							*reinterpret_cast<vec4*>(slab + frag_row * SLAB_STRIDE + (8 * q + 4 * half_sel) * 4) = v;
						}
						wait_lgkmcnt_zero();
						__builtin_amdgcn_wave_barrier();
#pragma unroll
						for (int pass = 0; pass < PASSES; pass++)
						{
							const int row = pass * ROWS_PER_PASS + (lane >> 3);
							const vec4 v = *reinterpret_cast<const vec4*>(slab + row * SLAB_STRIDE + col * 4);
							const int m = m_first + 32 * i + row;
							if (m < M && n_valid)
							{
								const acc_t vals[4] = { v[0], v[1], v[2], v[3] };
								local.apply(m, n, vals, side.column, side.extra[i][pass]);
							}
						}
						wait_lgkmcnt_zero();
						__builtin_amdgcn_wave_barrier();
					}
				}
			};

			for (int g = 0; g < DISTANCE; g++)
				if (g < run_stages)
					request_stage(g);
			/* Loads return in order: once at most the stages requested after stage 0 are outstanding, the B operand (requested first) and
			 * stage 0 have landed, and the first k steps run while the rest of the ring is still filling (no change where HBM bounds the
			 * launch; 59 -> 57 us for the fp32 products of 4096 tiles at 128 channels). The explicit wait also tells the compiler that no
			 * register load is outstanding any more, so it guards nothing inside the loop. */
			wait_vmcnt_stages<LOADS>(min(DISTANCE, run_stages) - 1);
			barrier_no_fence();
			clear_accumulators();
			read_fragments(0, 0, frags[0]);

			/*
			 * One unit: its k steps, then its epilogue. In the STEADY form every stage opening and every request is unconditional, so the
			 * body is straight-line code and the compiler can count the vector-memory operations between the side-input loads and
			 * their first use exactly (with branches in between it falls back to vmcnt(0), which drains the ring once per unit); the
			 * general form serves the last units of a run.
			 */
			auto process_unit = [&](int u, auto steady_tag) __attribute__((always_inline))
			{
				constexpr bool STEADY = decltype(steady_tag)::value;
				request_side_inputs(u);
				stream_static_for<STAGES_PER_UNIT * KSTEPS>([&](auto step)
				{
					constexpr int t = decltype(step)::value; /* k step within the unit */
					constexpr int ks = t / KSTEPS, kk = t % KSTEPS;
					constexpr int cur = t & 1, nxt = 1 - cur;
					const int g = u * STAGES_PER_UNIT + ks;
					/* the first MFMA is guarded by the compiler with lgkmcnt(0): this k step's fragments were requested one k step ago */
					Traits::mma(b_regs[t], frags[cur][0], acc[0]);
					__builtin_amdgcn_sched_barrier(0);
					if constexpr (kk + 1 < KSTEPS)
						read_fragments(g, kk + 1, frags[nxt]);
					else if (STEADY || g + 1 < run_stages)
					{
						/* stage g + 1 has landed once at most the loads of the stages requested after it (g + 2 .. g + DISTANCE - 1) are
						 * outstanding; after the barrier every wavefront has all of stage g in registers, so the buffers of stages <= g
						 * are free and stage g + DISTANCE takes that of stage g + DISTANCE - STAGES */
						wait_lgkmcnt_zero();
						if constexpr (STEADY)
							wait_vmcnt<(DISTANCE - 2) * LOADS>();
						else
							wait_vmcnt_stages<LOADS>(min(DISTANCE - 2, run_stages - 2 - g));
						barrier_no_fence();
						if (STEADY || g + DISTANCE < run_stages)
							request_stage(g + DISTANCE);
						read_fragments(g + 1, 0, frags[nxt]);
					}
					__builtin_amdgcn_sched_barrier(0);
#pragma unroll
					for (int i = 1; i < BLOCKS; i++)
						Traits::mma(b_regs[t], frags[cur][i], acc[i]);
					__builtin_amdgcn_sched_barrier(0);
				});
				store_unit(u);
				clear_accumulators();
			};
			/* steady while the last stage of the unit can still request DISTANCE stages ahead */
			const int steady_units = max(0, (run_stages - DISTANCE) / STAGES_PER_UNIT);
			int u = 0;
			for (; u < steady_units; u++)
				process_unit(u, std::true_type());
			for (; u < run_units; u++)
				process_unit(u, std::false_type());
			unit = run_end;
		}
	}
	/* operands of one streaming launch: `batch` products C[i] = A[i] * B[i]^T with K rows of k_bytes bytes (strides in elements) */
	struct StreamGemmArgs
	{
			const void *A, *B;
			void *C; /* used by PlainStore only; functors carry their own pointers */
			int M, N, k_bytes, batch;
			size_t stride_a, stride_b, stride_c;
			size_t a_row_bytes = 0; /* bytes between consecutive rows of A; 0 = dense rows of k_bytes */
	};
	/*
	 * A K row length the kernel is instantiated for. There is no lower bound on the size of the product: with a single unit per
	 * workgroup the kernel still starts faster than the tile engine (its B operand goes straight to registers and its first stage is one
	 * 16 KB request), e.g. 10 against 19 us for the 36 products of one 15x15 position.
	 */
	inline bool stream_gemm_applies(int M, int batch, size_t k_bytes)
	{
		return (k_bytes == 128 || k_bytes == 256 || k_bytes == 512) && M > 0 && batch > 0;
	}
	/* the fp16 forms are also instantiated for 768-byte rows (384 halfs), whose B operand still fits the registers */
	inline bool stream_gemm_half_applies(int M, int batch, size_t k_bytes)
	{
		return stream_gemm_applies(M, batch, k_bytes) || (k_bytes == 768 && M > 0 && batch > 0);
	}
	inline bool stream_gemm_plain_applies(int M, int batch, size_t k_bytes, int element_size)
	{
		return (element_size == 2) ? stream_gemm_half_applies(M, batch, k_bytes) : stream_gemm_applies(M, batch, k_bytes);
	}
	/*
	 * How one launch divides its row blocks ("units" of BM rows of one matrix) among the workgroups. The grid is `groups` row-range groups
	 * x n_tiles column slices. Two ways to hand out units: contiguous (group j takes units [j * units_per_group, ...) of the concatenated
	 * (matrix, row block) sequence, ascending, crossing into the next matrix where its range does), or the sweep form (sweep > 0 groups per
	 * matrix, group j of a matrix takes that matrix's row blocks j, j + sweep, ... from the last to the first). `rows_of_busiest_group`
	 * is what the launch waits for: the rows the group with most units multiplies.
	 */
	struct StreamGemmPlan
	{
			int bm, tiles_m, groups, units_per_group, sweep;
			long long rows_of_busiest_group;
	};
	inline StreamGemmPlan plan_stream_gemm(int M, int batch, int n_tiles, int bm, bool allow_sweep)
	{
		StreamGemmPlan p;
		p.bm = bm;
		p.tiles_m = ceil_div(M, bm);
		const int total_units = batch * p.tiles_m;
		int groups = device_compute_units() / n_tiles;
		if (groups >= 8)
			groups -= groups % 8; /* keeps the grid a multiple of 8 * n_tiles so that the column slices of a group share an XCD */
		if (groups < 1)
			groups = 1;
		if (groups > total_units)
			groups = total_units;
		p.groups = groups;
		p.units_per_group = ceil_div(total_units, groups);
		p.sweep = 0;
		p.rows_of_busiest_group = static_cast<long long>(p.units_per_group) * bm;
		/*
		 * Sweep form for batched products whose matrices each get at least two workgroups (the 36 Winograd matrices on 256 compute
		 * units: 7 each, 252 workgroups): measured 1.3 % to 2.8 % more positions per second on the 20-block network than the
		 * contiguous split of the same units, although it leaves 4 compute units idle, because the rows meet the last-level cache in
		 * the right order.
		 */
		if (allow_sweep && n_tiles == 1 && batch > 1 && groups / batch >= 2)
		{
			const int per_matrix = min(groups / batch, p.tiles_m);
			if ((groups - per_matrix * batch) * 16 <= groups) /* only when at most 1 / 16 of the compute units stay idle */
			{
				p.sweep = per_matrix;
				p.groups = per_matrix * batch;
				p.rows_of_busiest_group = static_cast<long long>(ceil_div(p.tiles_m, per_matrix)) * bm;
			}
		}
		return p;
	}
	template<typename T, int KB, int WAVES_M, int WAVES_N, typename Epilogue, int BM>
	inline void launch_stream_gemm_planned(hipStream_t stream, const StreamGemmArgs &g, const Epilogue &epilogue, const StreamGemmPlan &plan)
	{
		typedef StreamGemmConfig Cfg;
		constexpr int WAVES = WAVES_M * WAVES_N;
		constexpr int SLAB_BYTES = WAVES * 32 * (32 * (stream_epilogue_reads_nothing<Epilogue>::value ? sizeof(T) : 4) + 16);
		constexpr int STAGE_BYTES = BM * Cfg::STAGE_K_BYTES;
		constexpr int RING_STAGES = 128 * 1024 / STAGE_BYTES; /* 128 KB of ring where the slabs leave room for it: 8 stages of 128 rows, 16 of 64 */
		constexpr int STAGES = (RING_STAGES * STAGE_BYTES + SLAB_BYTES <= 160 * 1024) ? RING_STAGES : RING_STAGES - RING_STAGES / 8;
		constexpr int LDS = STAGES * STAGE_BYTES + SLAB_BYTES;
		static_assert(LDS <= 160 * 1024, "ring and slabs must fit the 160 KB of LDS");
		auto kernel = kernel_gemm_stream_wide_nt<T, KB, WAVES_M, WAVES_N, STAGES, Epilogue, BM>;
		ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), LDS);
		const int n_tiles = ceil_div(g.N, 32 * WAVES_N);
		hipLaunchKernelGGL(kernel, dim3(plan.groups * n_tiles), dim3(64 * WAVES), LDS, stream, reinterpret_cast<const T*>(g.A), reinterpret_cast<const T*>(g.B),
				reinterpret_cast<T*>(g.C), g.M, g.N, g.stride_a, g.stride_b, g.stride_c, g.batch, plan.tiles_m, n_tiles, plan.units_per_group, plan.sweep,
				g.a_row_bytes != 0 ? g.a_row_bytes : static_cast<size_t>(KB), epilogue);
	}
	template<typename T, int KB, int WAVES_M, int WAVES_N, typename Epilogue>
	inline void launch_stream_gemm_as(hipStream_t stream, const StreamGemmArgs &g, const Epilogue &epilogue)
	{
		constexpr bool PLAIN = std::is_same<Epilogue, PlainStore>::value;
		const int n_tiles = ceil_div(g.N, 32 * WAVES_N);
		const StreamGemmPlan wide = plan_stream_gemm(g.M, g.batch, n_tiles, 128, true);
		/*
		 * Units of 64 rows for the plain batched products on the 1 x 8 wavefront layout (a wavefront then owns two 32-row blocks instead
		 * of four: 32 accumulator registers less, half as long an epilogue per unit, a ring of 16 stages of 8 KB), in the sweep form and
		 * where the busiest workgroup gets no more rows than with units of 128. Measured on MI355X, stand-alone, 256 -> 256 channels in
		 * fp16: 16384 tiles 132 -> 120 us, 12800 tiles 107 -> 92 us, 4096 tiles 40 -> 38 us; 20 x 256 network 99.9 k -> 102.4 k positions/s
		 * on the same box. The 2 x 4 layout (64 < N <= 128, or N = 384 as three slices) would own a single 32-row block per wavefront and
		 * measures slower with it (128 channels 45 -> 46 us, 384 channels 206 -> 227 us, fp32 at 128 channels 57 -> 63 us), and the
		 * contiguous split of 64-row units, although it balances 36 x 16384 rows perfectly over 256 workgroups, loses the sweep's order
		 * through the last-level cache (96.0 k positions/s). Products with an epilogue functor (1x1 convolutions, the experts' layers)
		 * measured level with units of 64 rows and keep units of 128.
		 */
		if constexpr (PLAIN && WAVES_M == 1)
		{
			const StreamGemmPlan fine = plan_stream_gemm(g.M, g.batch, n_tiles, 64, true);
			if (fine.sweep > 0 && fine.rows_of_busiest_group <= wide.rows_of_busiest_group)
			{
				launch_stream_gemm_planned<T, KB, WAVES_M, WAVES_N, Epilogue, 64>(stream, g, epilogue, fine);
				return;
			}
		}
		launch_stream_gemm_planned<T, KB, WAVES_M, WAVES_N, Epilogue, 128>(stream, g, epilogue, wide);
	}
	/* wavefront layout by output width: 8 x 32 columns for N > 128, 2 x 4 for N > 64, 4 x 2 below */
	template<typename T, int KB, typename Epilogue>
	inline void launch_stream_gemm_kb(hipStream_t stream, const StreamGemmArgs &g, const Epilogue &epilogue)
	{
		constexpr bool PLAIN = std::is_same<Epilogue, PlainStore>::value;
		/* else B-operand registers + side inputs + a 128-row accumulator exceed 256 VGPRs (at 512 bytes an epilogue that reads nothing per
		 * element still fits: 233) */
		constexpr bool WIDE_FITS = PLAIN || KB < 512 || (KB == 512 && stream_epilogue_reads_nothing<Epilogue>::value);
		/* slices of 256 columns unless slices of 128 pad N less (N = 384: two wide slices multiply 512 columns, three narrow ones 384;
		 * measured 252 -> 206 us for the Winograd product at 384 channels) */
		const bool wide_pads_more = ceil_div(g.N, 256) * 256 > ceil_div(g.N, 128) * 128;
		if (g.N > 128 && WIDE_FITS && !wide_pads_more)
		{
			if constexpr (WIDE_FITS)
				launch_stream_gemm_as<T, KB, 1, 8>(stream, g, epilogue);
		}
		else if (g.N > 128) /* column slices of 128: every row of A is then fetched by ceil(N / 128) workgroups of one XCD */
			launch_stream_gemm_as<T, KB, 2, 4>(stream, g, epilogue);
		else if (g.N > 64)
			launch_stream_gemm_as<T, KB, 2, 4>(stream, g, epilogue);
		else
			launch_stream_gemm_as<T, KB, 4, 2>(stream, g, epilogue);
	}
	template<typename T, typename Epilogue>
	inline void launch_stream_gemm(hipStream_t stream, const StreamGemmArgs &g, const Epilogue &epilogue)
	{
		if constexpr (!std::is_same<Epilogue, PlainStore>::value && stream_epilogue_reads_nothing<Epilogue>::value)
		{
			/* the packed form stores 16 bytes per lane: rows and widths that do not allow it take the functor's run-time form */
			const auto sixteen = [](size_t elements) { return (elements * sizeof(T)) % 16 == 0; };
			if (!(sixteen(epilogue.N) && sixteen(epilogue.row_stride) && sixteen(g.stride_c) && reinterpret_cast<uintptr_t>(epilogue.D) % 16 == 0))
			{
				launch_stream_gemm<T>(stream, g, epilogue.template fixed<EPILOGUE_RUNTIME, EPILOGUE_RUNTIME, EPILOGUE_RUNTIME>());
				return;
			}
		}
		switch (g.k_bytes)
		{
			case 128:
				launch_stream_gemm_kb<T, 128>(stream, g, epilogue);
				break;
			case 256:
				launch_stream_gemm_kb<T, 256>(stream, g, epilogue);
				break;
			case 512:
				launch_stream_gemm_kb<T, 512>(stream, g, epilogue);
				break;
			case 768:
				if constexpr (std::is_same<T, half_t>::value)
				{
					launch_stream_gemm_kb<T, 768>(stream, g, epilogue);
					break;
				}
				[[fallthrough]];
			default:
				fail_logic("HIP backend: streaming GEMM: unsupported K row length");
		}
	}
} /* namespace mlhip */

#endif /* MINML_AMD_GEMM_STREAM_HPP_ */
