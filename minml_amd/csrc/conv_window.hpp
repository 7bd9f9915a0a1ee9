/*
 * conv_window.hpp — stride-1, "same"-padded 3 x 3 convolution over an NHWC tensor for NARROW layers: 64 halfs per pixel in (128 bytes), 64
 * filters out. The computation is the implicit GEMM of the reference (src/backend/cpu/conv_im2row.cpp:21-59 followed by the product with the
 * [Cout][k][k][Cin] weights and the fused tail of src/backend/cpu/gemm/def_kernels.cpp:237-275), organised for a layer that HBM bounds:
 *   - a row of the implicit matrix is one output pixel, its K axis the 9 taps of 128 bytes each. The tile engine fetches every tap of every
 *     row through L2 (9 times the input); here each input pixel enters LDS ONCE, into a ring indexed by the flattened pixel number, and the
 *     tap (i, j) of pixel m is read from the slot of pixel m + (i - 1) * W + (j - 1). A tap outside the image reads a row of zeros kept
 *     beside the ring;
 *   - persistent workgroups own a contiguous range of pixels, so the ring slides: direct-to-LDS loads of the next blocks of pixels run
 *     ahead of the multiplication across unit boundaries, with one workgroup barrier per unit of 128 pixels (not per 128 bytes of K);
 *   - the residual ("add" tensor, same shape as the output) travels the same way into a second ring, so it costs no registers, never
 *     makes a wavefront wait for a load at store time, and is read in the accumulators' own layout;
 *   - every wavefront keeps its 32 filters x 9 taps of the weights in registers (36 x 16 bytes per lane): the B operand costs neither
 *     LDS space nor LDS bandwidth;
 *   - fragment reads run five k steps ahead of the multiplication (a wavefront's 36 k steps are one chain of dependent MFMAs, so nothing
 *     else hides the LDS latency); results leave through per-wavefront LDS slabs, 16 bytes per lane;
 *   - the two wavefronts of a SIMD run half a unit out of step, so that the one's multiplication meets the other's tail and address
 *     arithmetic instead of its multiplication.
 * Measured on MI355X for 512 x 19 x 19 pixels, bias + residual + ReLU: 27 us against 37 us on the tile engine (71 MB: 2.6 TB/s); of a
 * workgroup's 23 us, 5 are the start (weights, first pixels), the rest 6 units of 3 us in which each wavefront multiplies for 1.1 us.
 */
#ifndef MINML_AMD_CONV_WINDOW_HPP_
#define MINML_AMD_CONV_WINDOW_HPP_

#include "gemm_stream.hpp"

namespace mlhip
{
	struct ConvWindowConfig
	{
			static constexpr int KS = 3, TAPS = KS * KS, PAD = KS / 2;
			static constexpr int PIXEL_BYTES = 128; /* of the input, and of a row of the output and of the residual (64 halfs) */
			static constexpr int FILTERS = 64;
			static constexpr int KSTEPS_PER_TAP = 4; /* 32 bytes of K per MFMA step */
			static constexpr int WAVES_M = 4, WAVES_N = 2, WAVES = WAVES_M * WAVES_N;
			static constexpr int BM = 32 * WAVES_M; /* pixels per unit: one 32-row block per wavefront */
			static constexpr int RING_PIXELS = 512; /* 64 KB, 4 blocks of BM pixels */
			static constexpr int RING_BLOCKS = RING_PIXELS / BM;
			static constexpr int LOADS = (BM / 8) / WAVES; /* 1 KB requests (8 pixels) of a block moved by one wavefront */
			static constexpr int ZERO_ROW = RING_PIXELS * PIXEL_BYTES; /* LDS offset of the slot after the ring's last: 128 bytes that stand for a tap outside the image */
			static constexpr int RESIDUAL_RING = ZERO_ROW + 1024;
			static constexpr int SLABS = RESIDUAL_RING + RING_PIXELS * PIXEL_BYTES;
			static constexpr int SLAB_STRIDE = 80; /* 64 bytes of payload per row + 16 of padding */
			static constexpr int LDS_BYTES = SLABS + WAVES * 32 * SLAB_STRIDE;
			static constexpr int DEPTH = 6; /* fragment registers in rotation: a read is issued 5 k steps before its use */
	};

	/*
	 * Workgroup j takes the pixels [j * rows_per_group, (j + 1) * rows_per_group) (a multiple of 32, so that a wavefront's block lies wholly
	 * inside the range or wholly outside). Pixels are requested in blocks of BM: input block s holds the pixels first + s * BM ... of the
	 * flattened tensor, where first = (range begin - halo) rounded down to 8 and halo = W + 1; unit v (BM pixels from range begin + v * BM)
	 * needs the input blocks v ... v + lead and the residual rows of its own pixels, which are requested together with input block v + lead;
	 * `ahead` further blocks are in flight. Epilogue: FloatEpilogue in a form fixed at compile time; WITH_RESIDUAL says whether it reads C.
	 */
	template<typename T, bool WITH_RESIDUAL, typename Epilogue>
	__global__ __launch_bounds__(64 * ConvWindowConfig::WAVES, 1) void kernel_conv_window(const uint8_t *input, const uint8_t *weights, int M, int height,
			int width, int rows_per_group, int ahead, uint32_t fill, Epilogue epilogue)
	{
		typedef ConvWindowConfig Cfg;
		typedef MfmaTraits<T> Traits;
		typedef typename Traits::acc_vec acc_vec;
		typedef typename Traits::acc_t acc_t;
		constexpr int KS = Cfg::KS, TAPS = Cfg::TAPS, PAD = Cfg::PAD, BM = Cfg::BM, WAVES = Cfg::WAVES, LOADS = Cfg::LOADS, RING = Cfg::RING_PIXELS;
		constexpr int KB = TAPS * Cfg::PIXEL_BYTES; /* bytes of one row of the weights */
		constexpr int GROUP_LOADS = LOADS * (WITH_RESIDUAL ? 2 : 1); /* vector-memory operations of one request group of one wavefront */
		constexpr int STEPS = TAPS * Cfg::KSTEPS_PER_TAP, DEPTH = Cfg::DEPTH;
		static_assert(sizeof(T) == 2 && (BM / 8) % WAVES == 0 && WITH_RESIDUAL == !Epilogue::no_side_input, "unsupported instantiation");
		extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
		uint8_t *slab = lds + Cfg::SLABS + (threadIdx.x >> 6) * (32 * Cfg::SLAB_STRIDE);

		const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
		const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;
		const int range_begin = blockIdx.x * rows_per_group;
		const int range_end = min(M, range_begin + rows_per_group);
		if (range_begin >= range_end)
			return;
		const int halo = PAD * (width + 1);
		const int first = ((range_begin - halo) >> 3) << 3; /* flattened number of the pixel in ring position 0 (may be negative) */
		const int lead = 1 + (range_begin - first + halo - 1) / BM;
		const int units = (range_end - range_begin + BM - 1) / BM;
		const int groups = units + lead; /* request groups: input block g, and the residual of unit g - lead */
		const int n0 = wave_n * 32;
		const int frag_row = lane & 31, half_sel = lane >> 5;

		Epilogue local = epilogue;
		const uint8_t *residual = nullptr;
		if constexpr (WITH_RESIDUAL)
			residual = reinterpret_cast<const uint8_t*>(local.C);
		auto request_residual = [&](int g) __attribute__((always_inline))
		{
			if constexpr (WITH_RESIDUAL)
			{
				if (g >= lead)
				{
#pragma unroll
					for (int i = 0; i < LOADS; i++)
					{
						const int q = (g - lead) * BM + (wave + WAVES * i) * 8; /* range-relative number of the first of 8 rows */
						const int slot = (q & (RING - 1)) + (lane >> 3);
						const int m = min(range_begin + q + (lane >> 3), M - 1);
						const int chunk = (lane & 7) ^ ((slot >> 1) & 7);
						__builtin_amdgcn_global_load_lds((global_ptr_t) (residual + static_cast<size_t>(m) * Cfg::PIXEL_BYTES + chunk * 16),
								(lds_ptr_t) (lds + Cfg::RESIDUAL_RING + (q & (RING - 1)) * Cfg::PIXEL_BYTES), 16, 0, 2); /* read once */
					}
				}
			}
		};
		auto request_input = [&](int g) __attribute__((always_inline))
		{
#pragma unroll
			for (int i = 0; i < LOADS; i++)
			{
				const int q = g * BM + (wave + WAVES * i) * 8; /* ring-relative number of the first of 8 pixels */
				const int slot = (q & (RING - 1)) + (lane >> 3);
				const int p = min(max(first + q + (lane >> 3), 0), M - 1); /* pixels before the tensor or past its end are never used */
				const int chunk = (lane & 7) ^ ((slot >> 1) & 7);
				__builtin_amdgcn_global_load_lds((global_ptr_t) (input + static_cast<size_t>(p) * Cfg::PIXEL_BYTES + chunk * 16),
						(lds_ptr_t) (lds + (q & (RING - 1)) * Cfg::PIXEL_BYTES), 16, 0, 0);
			}
		};
		auto request_group = [&](int g) __attribute__((always_inline))
		{
			request_residual(g);
			request_input(g);
		};
		const int prologue_groups = min(groups, lead + ahead);
#pragma unroll
		for (int g = 0; g < Cfg::RING_BLOCKS - 1; g++)
			if (g < prologue_groups)
				request_input(g);

		/*
		 * The weights of this wavefront's 32 filters: TAPS * 4 k steps of 16 bytes per lane, lane (r, h) holding bytes 32 k + 16 h ... of
		 * filter row r. Read straight from memory that is 36 requests of 32 cache lines each per wavefront (the rows are 1152 bytes apart),
		 * 4 us of address processing per compute unit. Instead the four wavefronts that share a filter block fetch it once, 16 contiguous
		 * bytes per lane (9 requests each), and pass it through LDS, in rows padded to 1168 bytes so that the 32 rows of a fragment read
		 * spread over all banks. The staging area is the residual ring and the slabs, which nothing uses yet: the residual of the first
		 * units is requested once the weights are in registers (staging one filter block at a time beside the first units' residual was
		 * measured: two more barriers and a longer start, 26 against 23 us; so was the barrier-free way of the K-split kernel below,
		 * through the wavefront's own slab: 28.5 against 26 us for the launch).
		 */
		constexpr int STAGE_ROW = KB + 16, STAGE_REQUESTS = (32 * KB / 1024) / Cfg::WAVES_M;
		static_assert((32 * KB) % (1024 * Cfg::WAVES_M) == 0 && Cfg::RESIDUAL_RING + Cfg::WAVES_N * 32 * STAGE_ROW <= Cfg::LDS_BYTES, "weights do not fit the staging area");
		uint4_t staged[STAGE_REQUESTS];
#pragma unroll
		for (int j = 0; j < STAGE_REQUESTS; j++)
			staged[j] = *reinterpret_cast<const uint4_t*>(weights + static_cast<size_t>(n0) * KB + (wave_m * STAGE_REQUESTS + j) * 1024 + lane * 16);
		typename Epilogue::Column columns[4];
#pragma unroll
		for (int q = 0; q < 4; q++)
			columns[q] = local.load_column(n0 + 8 * q + 4 * half_sel);
		wait_vmcnt<0>(); /* also the first input blocks: from here on no load into a register is outstanding, and the waits below count ring requests */
		uint8_t *staging = lds + Cfg::RESIDUAL_RING + wave_n * (32 * STAGE_ROW);
#pragma unroll
		for (int j = 0; j < STAGE_REQUESTS; j++)
		{
			const int byte = (wave_m * STAGE_REQUESTS + j) * 1024 + lane * 16;
			*reinterpret_cast<uint4_t*>(staging + (byte / KB) * STAGE_ROW + byte % KB) = staged[j];
		}
		wait_lgkmcnt_zero();
		barrier_no_fence();
		uint4_t b_regs[KB / 32];
#pragma unroll
		for (int k = 0; k < KB / 32; k++)
			b_regs[k] = *reinterpret_cast<const uint4_t*>(staging + frag_row * STAGE_ROW + k * 32 + half_sel * 16);
		wait_lgkmcnt_zero();
		barrier_no_fence(); /* the staging area is free again */
		if (tid < 32)
			reinterpret_cast<uint32_t*>(lds + Cfg::ZERO_ROW)[tid] = fill;
#pragma unroll
		for (int g = 0; g < Cfg::RING_BLOCKS - 1; g++)
			if (g < prologue_groups)
				request_residual(g);
		/* vector-memory operations of a group that may still be outstanding when a later wait counts them: the prologue's groups have their input already */
		auto group_operations = [&](int g) __attribute__((always_inline))
		{
			return (g < prologue_groups) ? GROUP_LOADS - LOADS : GROUP_LOADS;
		};

		/*
		 * The results of a unit are stored after the next unit's wait and barrier: a store issued just before that wait would count as
		 * outstanding there and hold the wavefront until it is acknowledged.
		 */
		uint4_t held[2];
		int held_first = -1; /* first pixel of the block whose results wait in `held` (uniform over the wavefront) */
		const int col = (lane & 3) * 8; /* 4 lanes x 16 bytes per row of 32 halfs, 16 rows per pass */
		auto store_held = [&]() __attribute__((always_inline))
		{
			if (held_first < 0)
				return;
#pragma unroll
			for (int pass = 0; pass < 2; pass++)
			{
				const int row = pass * 16 + (lane >> 2);
				if (held_first + row < range_end)
					*reinterpret_cast<uint4_t*>(local.D + static_cast<size_t>(held_first + row) * Cfg::FILTERS + n0 + col) = held[pass];
			}
			held_first = -1;
		};
		/*
		 * Where this lane's pixel lies in its image, kept from unit to unit without a division: the number within the image advances by
		 * BM modulo H * W, and the row is the product with 1 / W, which is exact below 2^20 pixels per image (checked by the launcher).
		 */
		const int image_pixels = height * width;
		const int image_step = BM % image_pixels;
		const float inverse_width = 1.0f / static_cast<float>(width);
		int in_image = (range_begin + wave_m * 32 + frag_row) % image_pixels;
		int address[TAPS]; /* LDS address of this lane's 16 bytes of k step 0 of each tap; k step kk of the same tap is at (address ^ (kk * 32)) */
		/* for unit v, called once per unit in ascending order. Pixels past the end of the tensor compute something that is never stored. */
		auto compute_addresses = [&](int v) __attribute__((always_inline))
		{
			const int h = static_cast<int>((static_cast<float>(in_image) + 0.5f) * inverse_width), w = in_image - h * width;
			uint32_t rows_inside = 0, columns_inside = 0; /* bit KS * di: row h + di - PAD exists; bit dj: column w + dj - PAD exists */
#pragma unroll
			for (int d = 0; d < KS; d++)
			{
				rows_inside |= (static_cast<unsigned>(h + d - PAD) < static_cast<unsigned>(height)) ? (1u << (KS * d)) : 0u;
				columns_inside |= (static_cast<unsigned>(w + d - PAD) < static_cast<unsigned>(width)) ? (1u << d) : 0u;
			}
			const uint32_t inside = rows_inside * columns_inside; /* bit KS * di + dj: which taps lie inside the image */
			const int centre = range_begin + v * BM + wave_m * 32 + frag_row - first; /* ring-relative number of the pixel */
			in_image += image_step;
			in_image -= (in_image >= image_pixels) ? image_pixels : 0;
#pragma unroll
			for (int tap = 0; tap < TAPS; tap++)
			{
				/* a tap outside the image reads slot RING, the row of zeros, whose swizzle term is 0 */
				const int offset = (tap / KS - PAD) * width + (tap % KS - PAD);
				const int slot = ((inside >> tap) & 1u) ? ((centre + offset) & (RING - 1)) : RING;
				address[tap] = slot * Cfg::PIXEL_BYTES + ((half_sel ^ ((slot >> 1) & 7)) * 16);
			}
		};
		acc_vec acc;
		/* 8 bytes of the residual row of this lane's pixel per register group q: bytes 2 * (n0 + 8 q + 4 half_sel) ..., in the ring's chunk order */
		typename Epilogue::Extra extra[4];
		auto read_residual = [&](int block_first) __attribute__((always_inline))
		{
			if constexpr (WITH_RESIDUAL)
			{
				const int res_slot = (block_first - range_begin + frag_row) & (RING - 1);
#pragma unroll
				for (int q = 0; q < 4; q++)
				{
					const int chunk = (wave_n * 4 + q) ^ ((res_slot >> 1) & 7);
					extra[q].raw = *reinterpret_cast<const decltype(extra[q].raw)*>(lds + Cfg::RESIDUAL_RING + res_slot * Cfg::PIXEL_BYTES + chunk * 16 + half_sel * 8);
				}
			}
		};
		/* residual_of >= 0: the residual rows of the block that starts there are read while the last k steps are multiplied */
		auto multiply = [&](int residual_of) __attribute__((always_inline))
		{
			uint4_t frags[DEPTH];
#pragma unroll
			for (int t = 0; t < DEPTH - 1; t++)
				frags[t] = *reinterpret_cast<const uint4_t*>(lds + (address[t / Cfg::KSTEPS_PER_TAP] ^ ((t % Cfg::KSTEPS_PER_TAP) * 32)));
			stream_static_for<STEPS>([&](auto step)
			{
				constexpr int t = decltype(step)::value;
				constexpr int ahead_t = t + DEPTH - 1;
				if constexpr (ahead_t < STEPS)
					frags[ahead_t % DEPTH] = *reinterpret_cast<const uint4_t*>(lds + (address[ahead_t / Cfg::KSTEPS_PER_TAP] ^ ((ahead_t % Cfg::KSTEPS_PER_TAP) * 32)));
				if constexpr (t == 0)
				{
#pragma unroll
					for (int e = 0; e < 16; e++)
						acc[e] = 0;
				}
				if constexpr (t == STEPS - DEPTH + 1)
				{
					if (residual_of >= 0)
						read_residual(residual_of);
				}
				/* keeps the read DEPTH - 1 steps ahead of its use: left to itself the scheduler pairs reads and waits for each pair */
				__builtin_amdgcn_sched_barrier(0);
				Traits::mma(b_regs[t], frags[t % DEPTH], acc);
				__builtin_amdgcn_sched_barrier(0);
			});
		};
		/* the tail of the block that starts at pixel block_first: lane l, accumulator register e holds m = l % 32, n = 8 (e / 4) + 4 (l / 32) + e % 4 */
		auto finish = [&](int block_first) __attribute__((always_inline))
		{
#pragma unroll
			for (int q = 0; q < 4; q++)
			{
				const acc_t vals[4] = { acc[4 * q + 0], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3] };
				Vec<T, 4> out;
				if constexpr (WITH_RESIDUAL)
					out = local.result(vals, columns[q], extra[q]);
				else
					out = local.value(vals, columns[q]);
				out.store(reinterpret_cast<T*>(slab + frag_row * Cfg::SLAB_STRIDE) + 8 * q + 4 * half_sel);
			}
			wait_lgkmcnt_zero(); /* the slab is private to this wavefront */
			__builtin_amdgcn_wave_barrier();
#pragma unroll
			for (int pass = 0; pass < 2; pass++)
				held[pass] = *reinterpret_cast<const uint4_t*>(slab + (pass * 16 + (lane >> 2)) * Cfg::SLAB_STRIDE + col * sizeof(T));
			held_first = block_first;
		};
		/*
		 * The two wavefronts of a SIMD run half a unit out of step, so that the one's multiplication meets the other's tail and address
		 * arithmetic instead of its multiplication: the first four ("early") finish a block right after multiplying it, the other four
		 * ("late") after the next unit's barrier, before they multiply that unit. The residual of unit v - 1 is therefore still read during
		 * unit v, which the ring allows while at most 2 groups are requested ahead.
		 */
		const bool late = __builtin_amdgcn_readfirstlane(wave) >= WAVES / 2;
		int unfinished = -1; /* late wavefronts: first pixel of the block whose sums still sit in the accumulators */
		if (!late)
			compute_addresses(0);
		for (int v = 0; v < units; v++)
		{
			const int m_first = __builtin_amdgcn_readfirstlane(range_begin + v * BM + wave_m * 32); /* first pixel of this wavefront's block */
			/*
			 * Group v + lead has landed once at most the groups requested after it are outstanding (loads return in order); after the
			 * barrier nobody multiplies unit v - 1 any more, so the group that takes its ring positions may be requested.
			 */
			int allowed = 0;
			for (int g = v + lead + 1; g < min(groups, v + lead + ahead); g++)
				allowed += group_operations(g);
			wait_lgkmcnt_zero();
			wait_vmcnt_stages<1>(allowed);
			barrier_no_fence();
			if (v + lead + ahead < groups)
				request_group(v + lead + ahead);
			store_held();
			if (late)
			{
				if (unfinished >= 0)
				{
					read_residual(unfinished);
					finish(unfinished);
					store_held();
					unfinished = -1;
				}
				compute_addresses(v);
			}
			if (m_first < range_end) /* else this wavefront's block lies beyond the range (uniform over the wavefront) */
			{
				multiply(late ? -1 : m_first);
				if (late)
					unfinished = m_first;
				else
					finish(m_first);
			}
			if (!late && v + 1 < units)
				compute_addresses(v + 1);
		}
		if (late && unfinished >= 0)
		{
			read_residual(unfinished);
			finish(unfinished);
		}
		store_held();
	}

	/*
	 * The same scheme for layers whose filter bank exceeds what one pair of wavefront columns can hold (64 -> 64 filters 5 x 5: 200 KB;
	 * 128 -> 128 filters 3 x 3: 288 KB; the registers of a workgroup hold 512 KB): the K axis is SPLIT among the wavefronts. The 8
	 * wavefronts are N_BLOCKS blocks of 32 filters x K_SPLIT ranges of the k * k * PIXEL_BYTES / 128 chunks (128 bytes of K each); a
	 * wavefront keeps its block's weights for its chunks in registers, multiplies EVERY pixel of a unit (BM = 64 pixels, two 32-row
	 * blocks, two independent chains of MFMAs) by them, and the K_SPLIT partial sums of an output meet in LDS: each wavefront hands the
	 * accumulator registers it does not finish to the wavefront that does, which adds them in ascending order of the K ranges (so the
	 * result does not depend on timing), applies the tail and stores 4 consecutive filters of one pixel per lane. Two workgroup
	 * barriers per unit: pixels landed / partial sums written. The residual is read straight into registers at the start of the unit.
	 * Measured on MI355X at 512 x 19 x 19 pixels with bias + residual + ReLU: 64 -> 64 filters 5 x 5 57 us against 73 us on the tile engine;
	 * the form for 128 -> 128 filters 3 x 3 (pixels of 256 bytes, 4 filter blocks x 2 K ranges, 144 registers of weights per lane) spills
	 * registers and takes 151 us against 78 us, so it is not instantiated.
	 */
	template<int KS_, int PIXEL_BYTES_, int N_BLOCKS_, int K_SPLIT_>
	struct ConvSplitConfig
	{
			static constexpr int KS = KS_, TAPS = KS * KS, PAD = KS / 2, PIXEL_BYTES = PIXEL_BYTES_, N_BLOCKS = N_BLOCKS_, K_SPLIT = K_SPLIT_;
			static constexpr int CHUNKS_PER_PIXEL = PIXEL_BYTES / 128, CHUNKS = TAPS * CHUNKS_PER_PIXEL;
			static constexpr int MAX_CHUNKS = (CHUNKS + K_SPLIT - 1) / K_SPLIT; /* per wavefront */
			static constexpr int FILTERS = 32 * N_BLOCKS, WAVES = N_BLOCKS * K_SPLIT;
			static constexpr int BLOCKS = 2, BM = 32 * BLOCKS;
			static constexpr int RING_PIXELS = 65536 / PIXEL_BYTES; /* 64 KB */
			static constexpr int RING_BLOCKS = RING_PIXELS / BM;
			static constexpr int LOADS = (BM * PIXEL_BYTES / 1024) / WAVES; /* 1 KB requests of a block of pixels moved by one wavefront */
			static constexpr int ZERO_ROW = RING_PIXELS * PIXEL_BYTES; /* the slot after the ring's last stands for a tap outside the image */
			static constexpr int PARTIALS = ZERO_ROW + 1024;
			static constexpr int Q_PER = 4 / K_SPLIT; /* groups of 4 accumulator registers (8 filters) that a wavefront finishes */
			static constexpr int PARTIAL_BYTES = N_BLOCKS * K_SPLIT * (K_SPLIT - 1) * Q_PER * BLOCKS * 1024;
			static constexpr int STAGING_BYTES = WAVES * 32 * 144; /* the weights' way into registers at the start, in the same place */
			static constexpr int LDS_BYTES = PARTIALS + (PARTIAL_BYTES > STAGING_BYTES ? PARTIAL_BYTES : STAGING_BYTES);
			static constexpr int DEPTH = (MAX_CHUNKS > 7) ? 3 : 4; /* fragment registers in rotation, per block */
			static constexpr int SWIZZLE_MASK = (PIXEL_BYTES == 128) ? 7 : 15, SWIZZLE_SHIFT = (PIXEL_BYTES == 128) ? 1 : 0;
			static_assert(WAVES == 8 && (PIXEL_BYTES == 128 || PIXEL_BYTES == 256) && 4 % K_SPLIT == 0 && (BM * PIXEL_BYTES / 1024) % WAVES == 0
					&& LDS_BYTES <= 160 * 1024, "unsupported shape");
	};
	template<typename T, typename Cfg, bool WITH_RESIDUAL, typename Epilogue>
	__global__ __launch_bounds__(64 * Cfg::WAVES, 1) void kernel_conv_window_split(const uint8_t *input, const uint8_t *weights, int M, int height, int width,
			int rows_per_group, int ahead, uint32_t fill, Epilogue epilogue)
	{
		typedef MfmaTraits<T> Traits;
		typedef typename Traits::acc_vec acc_vec;
		typedef typename Traits::acc_t acc_t;
		typedef acc_t vec4 __attribute__((ext_vector_type(4)));
		constexpr int KS = Cfg::KS, PAD = Cfg::PAD, BM = Cfg::BM, BLOCKS = Cfg::BLOCKS, WAVES = Cfg::WAVES, LOADS = Cfg::LOADS, RING = Cfg::RING_PIXELS;
		constexpr int P = Cfg::PIXEL_BYTES, CPP = Cfg::CHUNKS_PER_PIXEL, K_SPLIT = Cfg::K_SPLIT, Q_PER = Cfg::Q_PER, MAX_CHUNKS = Cfg::MAX_CHUNKS;
		constexpr int KB = Cfg::TAPS * P; /* bytes of one row of the weights */
		constexpr int DEPTH = Cfg::DEPTH, STEPS = MAX_CHUNKS * 4;
		constexpr int PIXELS_PER_REQUEST = 1024 / P, LANES_PER_PIXEL = P / 16;
		static_assert(sizeof(T) == 2 && WITH_RESIDUAL == !Epilogue::no_side_input, "unsupported instantiation");
		extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

		const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
		const int block_n = wave % Cfg::N_BLOCKS, split = __builtin_amdgcn_readfirstlane(wave / Cfg::N_BLOCKS);
		const int range_begin = blockIdx.x * rows_per_group;
		const int range_end = min(M, range_begin + rows_per_group);
		if (range_begin >= range_end)
			return;
		const int halo = PAD * (width + 1);
		const int first = ((range_begin - halo) >> 3) << 3; /* flattened number of the pixel in ring position 0 (may be negative) */
		const int lead = 1 + (range_begin - first + halo - 1) / BM; /* unit v needs the blocks of pixels up to v + lead */
		const int units = (range_end - range_begin + BM - 1) / BM;
		const int groups = units + lead;
		const int n0 = block_n * 32;
		const int frag_row = lane & 31, half_sel = lane >> 5;
		/* this wavefront's chunks of K: [chunk_begin, chunk_end) */
		const int chunk_begin = (Cfg::CHUNKS * split) / K_SPLIT, chunk_end = (Cfg::CHUNKS * (split + 1)) / K_SPLIT;
		const int chunks = chunk_end - chunk_begin;

		if (tid < P / 4)
			reinterpret_cast<uint32_t*>(lds + Cfg::ZERO_ROW)[tid] = fill;
		Epilogue local = epilogue;
		auto request_group = [&](int g) __attribute__((always_inline))
		{
#pragma unroll
			for (int i = 0; i < LOADS; i++)
			{
				const int q = g * BM + (wave + WAVES * i) * PIXELS_PER_REQUEST; /* ring-relative number of the first pixel of the request */
				const int slot = (q & (RING - 1)) + lane / LANES_PER_PIXEL;
				const int p = min(max(first + q + lane / LANES_PER_PIXEL, 0), M - 1); /* pixels before the tensor or past its end are never used */
				const int chunk = (lane % LANES_PER_PIXEL) ^ ((slot >> Cfg::SWIZZLE_SHIFT) & Cfg::SWIZZLE_MASK);
				__builtin_amdgcn_global_load_lds((global_ptr_t) (input + static_cast<size_t>(p) * P + chunk * 16), (lds_ptr_t) (lds + (q & (RING - 1)) * P), 16, 0, 0);
			}
		};
		const int prologue_groups = min(groups, lead + ahead);
#pragma unroll
		for (int g = 0; g < Cfg::RING_BLOCKS - 1; g++)
			if (g < prologue_groups)
				request_group(g);

		/*
		 * The weights of this wavefront's 32 filters for its chunks: 4 k steps of 16 bytes per lane and chunk, lane (r, h) holding bytes
		 * 32 kk + 16 h ... of chunk c of filter row r; chunks past its range hold zeros. Read in that layout, a request touches 32 cache
		 * lines (the rows are KB bytes apart) and the address processing of 28 or 36 such requests per wavefront takes microseconds.
		 * They are read 128 contiguous bytes per 8 lanes instead (8 rows per request) and turned into the fragment layout through a
		 * private piece of LDS, chunk by chunk, with no workgroup barrier.
		 */
		uint4_t b_regs[MAX_CHUNKS * 4];
		{
			constexpr int STAGE_STRIDE = 144;
			static_assert(Cfg::PARTIALS + WAVES * 32 * STAGE_STRIDE <= Cfg::LDS_BYTES, "no room to stage the weights");
			uint8_t *stage = lds + Cfg::PARTIALS + wave * (32 * STAGE_STRIDE);
			const uint8_t *block = weights + static_cast<size_t>(n0) * KB + static_cast<size_t>(chunk_begin) * 128;
			uint4_t staged[MAX_CHUNKS][4]; /* lane l, register j: row l / 8 + 8 j, bytes 16 (l % 8) ... of the chunk */
#pragma unroll
			for (int c = 0; c < MAX_CHUNKS; c++)
#pragma unroll
				for (int j = 0; j < 4; j++)
				{
					staged[c][j] = uint4_t { 0u, 0u, 0u, 0u };
					if (c < chunks)
						staged[c][j] = *reinterpret_cast<const uint4_t*>(block + static_cast<size_t>((lane >> 3) + 8 * j) * KB + c * 128 + (lane & 7) * 16);
				}
#pragma unroll
			for (int c = 0; c < MAX_CHUNKS; c++)
			{
#pragma unroll
				for (int j = 0; j < 4; j++)
					*reinterpret_cast<uint4_t*>(stage + ((lane >> 3) + 8 * j) * STAGE_STRIDE + (lane & 7) * 16) = staged[c][j];
				wait_lgkmcnt_zero();
				__builtin_amdgcn_wave_barrier();
#pragma unroll
				for (int kk = 0; kk < 4; kk++)
					b_regs[c * 4 + kk] = *reinterpret_cast<const uint4_t*>(stage + frag_row * STAGE_STRIDE + (2 * kk + half_sel) * 16);
				wait_lgkmcnt_zero();
				__builtin_amdgcn_wave_barrier();
			}
		}
		/* this wavefront finishes the register groups q = split * Q_PER ... of every block: filters n0 + 8 q + 4 half_sel ... + 3 of pixel 32 b + lane % 32 */
		typename Epilogue::Column columns[Q_PER];
#pragma unroll
		for (int qq = 0; qq < Q_PER; qq++)
			columns[qq] = local.load_column(n0 + 8 * (split * Q_PER + qq) + 4 * half_sel);
		wait_vmcnt<0>(); /* also the first groups of pixels: from here on the waits below count ring requests and residual loads */

		const int image_pixels = height * width;
		const int image_step = BM % image_pixels;
		const float inverse_width = 1.0f / static_cast<float>(width);
		int in_image[BLOCKS];
#pragma unroll
		for (int b = 0; b < BLOCKS; b++)
			in_image[b] = (range_begin + 32 * b + frag_row) % image_pixels;
		/* LDS address of this lane's 16 bytes of k step 0 of each of its chunks, per block; k step kk is at (address ^ (kk * 32)) */
		int address[MAX_CHUNKS][BLOCKS];
		auto compute_addresses = [&](int v) __attribute__((always_inline))
		{
#pragma unroll
			for (int b = 0; b < BLOCKS; b++)
			{
				const int h = static_cast<int>((static_cast<float>(in_image[b]) + 0.5f) * inverse_width), w = in_image[b] - h * width;
				const int centre = range_begin + v * BM + 32 * b + frag_row - first; /* ring-relative number of the pixel */
				in_image[b] += image_step;
				in_image[b] -= (in_image[b] >= image_pixels) ? image_pixels : 0;
#pragma unroll
				for (int c = 0; c < MAX_CHUNKS; c++)
				{
					const int chunk = chunk_begin + c; /* uniform over the wavefront */
					const int tap = chunk / CPP, part = chunk - tap * CPP;
					const int di = tap / KS, dj = tap - di * KS;
					const bool inside = (static_cast<unsigned>(h + di - PAD) < static_cast<unsigned>(height)) && (static_cast<unsigned>(w + dj - PAD) < static_cast<unsigned>(width))
							&& c < chunks;
					/* a tap outside the image reads slot RING, the row of zeros, whose swizzle term is 0 */
					const int slot = inside ? ((centre + (di - PAD) * width + (dj - PAD)) & (RING - 1)) : RING;
					address[c][b] = slot * P + (((part * 8 + half_sel) ^ ((slot >> Cfg::SWIZZLE_SHIFT) & Cfg::SWIZZLE_MASK)) * 16);
				}
			}
		};
		typename std::conditional<WITH_RESIDUAL, typename Epilogue::Extra, int>::type extra[Q_PER][BLOCKS];
		/* where source wavefront (block_n, from) leaves register group qq of block b of a unit for the wavefront (block_n, to) that finishes it */
		auto partial_slot = [&](int unit, int to, int from, int qq, int b) __attribute__((always_inline))
		{
			const int source = (from < to) ? from : from - 1;
			return lds + Cfg::PARTIALS + (((((block_n * K_SPLIT + to) * (K_SPLIT - 1) + source) * Q_PER + qq) * BLOCKS + b) * 64 + lane) * 16;
		};
		auto request_residual = [&](int unit) __attribute__((always_inline))
		{
			if constexpr (WITH_RESIDUAL)
			{
#pragma unroll
				for (int qq = 0; qq < Q_PER; qq++)
#pragma unroll
					for (int b = 0; b < BLOCKS; b++)
						extra[qq][b] = local.load_extra(min(range_begin + unit * BM + 32 * b + frag_row, range_end - 1), n0 + 8 * (split * Q_PER + qq) + 4 * half_sel);
			}
		};
		acc_vec acc[BLOCKS];
		vec4 own[Q_PER][BLOCKS]; /* the register groups this wavefront finishes itself, kept while it multiplies the next unit */
		auto multiply = [&]() __attribute__((always_inline))
		{
			uint4_t frags[DEPTH][BLOCKS];
#pragma unroll
			for (int t = 0; t < DEPTH - 1; t++)
#pragma unroll
				for (int b = 0; b < BLOCKS; b++)
					frags[t][b] = *reinterpret_cast<const uint4_t*>(lds + (address[t / 4][b] ^ ((t % 4) * 32)));
			stream_static_for<STEPS>([&](auto step)
			{
				constexpr int t = decltype(step)::value;
				constexpr int ahead_t = t + DEPTH - 1;
				if constexpr (ahead_t < STEPS)
				{
#pragma unroll
					for (int b = 0; b < BLOCKS; b++)
						frags[ahead_t % DEPTH][b] = *reinterpret_cast<const uint4_t*>(lds + (address[ahead_t / 4][b] ^ ((ahead_t % 4) * 32)));
				}
				if constexpr (t == 0)
				{
#pragma unroll
					for (int b = 0; b < BLOCKS; b++)
#pragma unroll
						for (int e = 0; e < 16; e++)
							acc[b][e] = 0;
				}
				__builtin_amdgcn_sched_barrier(0);
#pragma unroll
				for (int b = 0; b < BLOCKS; b++)
					Traits::mma(b_regs[t], frags[t % DEPTH][b], acc[b]);
				__builtin_amdgcn_sched_barrier(0);
			});
		};
		/* leaves the register groups of unit `unit` that other wavefronts finish in its buffer, keeps this wavefront's own */
		auto hand_over = [&](int unit) __attribute__((always_inline))
		{
			stream_static_for<K_SPLIT>([&](auto to_tag)
			{
				constexpr int to = decltype(to_tag)::value;
#pragma unroll
				for (int qq = 0; qq < Q_PER; qq++)
#pragma unroll
					for (int b = 0; b < BLOCKS; b++)
					{
						vec4 part;
#pragma unroll
						for (int e = 0; e < 4; e++)
							part[e] = acc[b][4 * (to * Q_PER + qq) + e];
						if (to != split)
							*reinterpret_cast<vec4*>(partial_slot(unit, to, split, qq, b)) = part;
						else
							own[qq][b] = part;
					}
			});
		};
		/* adds the partial sums of unit `unit` in ascending order of the K ranges, applies the tail, stores */
		auto finish = [&](int unit) __attribute__((always_inline))
		{
#pragma unroll
			for (int qq = 0; qq < Q_PER; qq++)
#pragma unroll
				for (int b = 0; b < BLOCKS; b++)
				{
					vec4 sum;
#pragma unroll
					for (int from = 0; from < K_SPLIT; from++)
					{
						vec4 part = own[qq][b];
						if (from != split)
							part = *reinterpret_cast<const vec4*>(partial_slot(unit, split, from, qq, b));
						if (from == 0)
							sum = part;
						else
							sum += part;
					}
					const acc_t vals[4] = { sum[0], sum[1], sum[2], sum[3] };
					Vec<T, 4> out;
					if constexpr (WITH_RESIDUAL)
						out = local.result(vals, columns[qq], extra[qq][b]);
					else
						out = local.value(vals, columns[qq]);
					const int m = range_begin + unit * BM + 32 * b + frag_row;
					if (m < range_end)
						out.store(local.D + static_cast<size_t>(m) * Cfg::FILTERS + n0 + 8 * (split * Q_PER + qq) + 4 * half_sel);
				}
		};

		/*
		 * The two wavefronts of a SIMD share its matrix pipe, so one of them multiplies later than the other anyway: the later four
		 * ("late") do their address arithmetic at the start of the unit, while the first four multiply, instead of after their own
		 * multiplication, where it would hold up the barrier. (Adding the partial sums of unit v during unit v + 1, from two buffers in
		 * turn and with one barrier per unit, was measured slower: 63 against 57 us for 512 x 19 x 19 pixels, 64 -> 64 filters 5 x 5.)
		 */
		const bool late = __builtin_amdgcn_readfirstlane(wave) >= WAVES / 2;
		if (!late)
			compute_addresses(0);
		for (int v = 0; v < units; v++)
		{
			/*
			 * Group v + lead has landed once at most the LOADS requested after it are outstanding (loads return in order; stores are not
			 * counted, they may be acknowledged early): the later groups and the residual loads of the units since. After the barrier
			 * nobody multiplies unit v - 1 or adds its partial sums any more.
			 */
			const int later_groups = min(groups, v + lead + ahead) - (v + lead + 1);
			const int later_units = min(v, ahead); /* units whose residual was requested after group v + lead was */
			wait_lgkmcnt_zero();
			wait_vmcnt_stages<1>(max(later_groups, 0) * LOADS + (WITH_RESIDUAL ? later_units * Q_PER * BLOCKS : 0));
			barrier_no_fence();
			if (v + lead + ahead < groups)
				request_group(v + lead + ahead);
			request_residual(v);
			if (late)
				compute_addresses(v);
			multiply();
			if (!late && v + 1 < units)
				compute_addresses(v + 1);
			hand_over(v);
			wait_lgkmcnt_zero();
			barrier_no_fence();
			finish(v);
		}
	}

	/* whether the windowed kernel takes a convolution: fp16, 64 filters in and out, 3 x 3, an image narrow enough for the pixel ring */
	inline bool conv_window_applies(int element_size, int filters_in, int filters_out, int kernel_h, int kernel_w, int height, int width, size_t pixels)
	{
		typedef ConvWindowConfig Cfg;
		const int halo = Cfg::PAD * (width + 1);
		const int lead_max = 1 + (2 * halo + 6) / Cfg::BM;
		return element_size == 2 && filters_in * element_size == Cfg::PIXEL_BYTES && filters_out == Cfg::FILTERS && kernel_h == Cfg::KS && kernel_w == Cfg::KS
				&& Cfg::RING_BLOCKS - 1 - lead_max >= 1 && pixels < (1u << 30) && static_cast<size_t>(height) * width < (1u << 20);
	}
	typedef ConvSplitConfig<5, 128, 2, 4> ConvSplit5x5x64;
	template<typename Cfg>
	inline bool conv_window_split_applies(int element_size, int filters_in, int filters_out, int kernel_h, int kernel_w, int height, int width, size_t pixels)
	{
		const int halo = Cfg::PAD * (width + 1);
		const int lead_max = 1 + (2 * halo + 6) / Cfg::BM;
		return element_size == 2 && filters_in * element_size == Cfg::PIXEL_BYTES && filters_out == Cfg::FILTERS && kernel_h == Cfg::KS && kernel_w == Cfg::KS
				&& Cfg::RING_BLOCKS - 1 - lead_max >= 1 && pixels < (1u << 30) && static_cast<size_t>(height) * width < (1u << 20);
	}
	template<typename T, typename Cfg, typename Epilogue>
	inline void launch_conv_window_split(hipStream_t stream, const void *input, const void *weights, int pixels, int height, int width, const Epilogue &epilogue)
	{
		constexpr bool WITH_RESIDUAL = !Epilogue::no_side_input;
		auto kernel = kernel_conv_window_split<T, Cfg, WITH_RESIDUAL, Epilogue>;
		ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), Cfg::LDS_BYTES);
		const int halo = Cfg::PAD * (width + 1);
		const int lead_max = 1 + (2 * halo + 6) / Cfg::BM;
		const int ahead = min(Cfg::RING_BLOCKS - 1 - lead_max, 3);
		int groups = device_compute_units();
		const int rows_per_group = ceil_div(ceil_div(pixels, groups), 32) * 32;
		groups = ceil_div(pixels, rows_per_group);
		hipLaunchKernelGGL(kernel, dim3(groups), dim3(64 * Cfg::WAVES), Cfg::LDS_BYTES, stream, reinterpret_cast<const uint8_t*>(input),
				reinterpret_cast<const uint8_t*>(weights), pixels, height, width, rows_per_group, ahead, 0u, epilogue);
	}
	/* the epilogue is a FloatEpilogue<half_t, ACT, WITH_C, 1> with D (and C) dense rows of 64 halfs, 16-byte aligned */
	template<typename T, typename Epilogue>
	inline void launch_conv_window(hipStream_t stream, const void *input, const void *weights, int pixels, int height, int width, const Epilogue &epilogue)
	{
		typedef ConvWindowConfig Cfg;
		constexpr bool WITH_RESIDUAL = !Epilogue::no_side_input;
		auto kernel = kernel_conv_window<T, WITH_RESIDUAL, Epilogue>;
		ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), Cfg::LDS_BYTES);
		const int halo = Cfg::PAD * (width + 1);
		const int lead_max = 1 + (2 * halo + 6) / Cfg::BM;
		const int ahead = Cfg::RING_BLOCKS - 1 - lead_max;
		int groups = device_compute_units();
		const int rows_per_group = ceil_div(ceil_div(pixels, groups), 32) * 32;
		groups = ceil_div(pixels, rows_per_group);
		hipLaunchKernelGGL(kernel, dim3(groups), dim3(64 * Cfg::WAVES), Cfg::LDS_BYTES, stream, reinterpret_cast<const uint8_t*>(input),
				reinterpret_cast<const uint8_t*>(weights), pixels, height, width, rows_per_group, ahead, 0u, epilogue);
	}
} /* namespace mlhip */

#endif /* MINML_AMD_CONV_WINDOW_HPP_ */
