/*
 * ceilings.hip — probes of what one MI355X sustains, independent of the backend's kernels: plain read / write / copy streams over a
 * buffer of a given size (HBM when the buffer exceeds the 256 MB last-level cache, that cache or the L2s when it fits) and a pure MFMA
 * loop on operands held in registers. Built as its own small library (libminml_ceilings.so) and used only by
 * `python3 kernel_bench.py --group ceilings` (which also builds it: --build-ceilings); nothing in the backend library depends on it.
 *
 * The entry points take a hipStream_t and raw device pointers and launch one kernel each; the caller times them with events. They are
 * called through ctypes, so no exception may leave them: each returns 0, or -1 after storing a message that ceil_last_error() returns.
 */
#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>
#include <string>

namespace
{
	typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
	typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
	typedef float float16_t __attribute__((ext_vector_type(16)));
	typedef int int16_t_v __attribute__((ext_vector_type(16)));
	typedef int int4_v __attribute__((ext_vector_type(4)));

	void check(hipError_t status, const char *what)
	{
		if (status != hipSuccess)
			throw std::runtime_error(std::string("ceilings: ") + what + ": " + hipGetErrorString(status));
	}

	template<bool NT>
	__device__ __forceinline__ uint4_t load16(const uint4_t *p)
	{
		return NT ? __builtin_nontemporal_load(p) : *p;
	}
	template<bool NT>
	__device__ __forceinline__ void store16(uint4_t *p, uint4_t v)
	{
		if (NT)
			__builtin_nontemporal_store(v, p);
		else
			*p = v;
	}

	/*
	 * MODE 0: read `chunks` 16-byte pieces of src, 1: write them to dst, 2: copy src -> dst. Each workgroup owns a contiguous span;
	 * within a span every instruction of a wavefront touches 1 KB of consecutive addresses, four instructions in flight per lane.
	 */
	template<int MODE, bool NT>
	__global__ __launch_bounds__(256) void kernel_stream(uint4_t *__restrict__ dst, const uint4_t *__restrict__ src, size_t chunks, size_t chunks_per_wg)
	{
		const size_t begin = static_cast<size_t>(blockIdx.x) * chunks_per_wg;
		const size_t end = (begin + chunks_per_wg < chunks) ? begin + chunks_per_wg : chunks;
		uint32_t acc = 0;
		size_t i = begin + threadIdx.x;
		for (; i + 3 * 256 < end; i += 4 * 256)
		{
			uint4_t v[4];
#pragma unroll
			for (int j = 0; j < 4; j++)
			{
				if (MODE != 1)
					v[j] = load16<NT>(src + i + j * 256);
				else
					v[j] = uint4_t { static_cast<uint32_t>(i), 1u, 2u, static_cast<uint32_t>(j) };
			}
#pragma unroll
			for (int j = 0; j < 4; j++)
			{
				if (MODE != 0)
					store16<NT>(dst + i + j * 256, v[j]);
				else
					acc += v[j].x ^ v[j].w;
			}
		}
		for (; i < end; i += 256)
		{
			uint4_t v = uint4_t { static_cast<uint32_t>(i), 1u, 2u, 3u };
			if (MODE != 1)
				v = load16<NT>(src + i);
			if (MODE != 0)
				store16<NT>(dst + i, v);
			else
				acc += v.x ^ v.w;
		}
		if (MODE == 0 && acc == 0x9e3779b9u && dst != nullptr)
			dst[0] = uint4_t { acc, 0u, 0u, 0u };
	}

	/*
	 * Pure matrix-pipe loop: every wavefront keeps 4 + 4 operand fragments in registers and issues 16 independent MFMAs per iteration
	 * (a 128 x 128 sub-tile per k step, as a GEMM inner loop would, minus all memory traffic). RANDOM selects operand bits: all lanes
	 * 1.0 (the pipes toggle little) or pseudo-random halfs / bytes in [-2, 2] (what real data looks like to the multipliers).
	 * out[0..3] of workgroup 0 = shader-clock ticks and 100 MHz real-time ticks spent in the loop, for the clock the loop ran at.
	 */
	/* KIND 0: v_mfma_f32_32x32x16_f16, 1: v_mfma_i32_32x32x32_i8, 2: v_mfma_f32_32x32x2_f32 (one float of each operand per lane) */
	template<int KIND>
	__global__ __launch_bounds__(256, 1) void kernel_mfma_loop(uint64_t *out, int iters, int random)
	{
		const uint32_t lane = threadIdx.x;
		uint4_t a[4], b[4];
		for (int i = 0; i < 4; i++)
			for (int j = 0; j < 4; j++)
			{
				const uint32_t h = (lane * 2654435761u) ^ ((i * 4 + j) * 40503u) ^ (blockIdx.x * 97u);
				uint32_t word;
				constexpr bool INT8 = (KIND == 1);
				if (INT8)
					word = random ? (h * 2246822519u) : 0x01010101u;
				else if (KIND == 2) /* a float with magnitude in [0.5, 1) and a pseudo-random sign, or 1.0 */
					word = random ? ((0x3f000000u | (h & 0x7fffffu)) ^ ((h << 3) & 0x80000000u)) : 0x3f800000u;
				else
				{
					const uint32_t lo = 0x3000u | (h & 0x8fffu), hi = 0x3000u | ((h >> 16) & 0x8fffu);
					word = random ? (lo | (hi << 16)) : 0x3c003c00u;
				}
				a[i][j] = word;
				b[i][j] = word ^ (random ? 0x00010001u * (j + 1) : 0u);
			}
		float16_t accf[16];
		int16_t_v acci[16];
		for (int i = 0; i < 16; i++)
			for (int r = 0; r < 16; r++)
			{
				accf[i][r] = 0.0f;
				acci[i][r] = 0;
			}
		const uint64_t c0 = clock64();
		const uint64_t w0 = wall_clock64();
		for (int it = 0; it < iters; it++)
		{
#pragma unroll
			for (int i = 0; i < 4; i++)
#pragma unroll
				for (int j = 0; j < 4; j++)
				{
					if (KIND == 2)
						accf[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, b[j][0]), __builtin_bit_cast(float, a[i][0]),
								accf[i * 4 + j], 0, 0, 0);
					else if (KIND == 1)
						acci[i * 4 + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(int4_v, b[j]), __builtin_bit_cast(int4_v, a[i]), acci[i * 4 + j],
								0, 0, 0);
					else
						accf[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, b[j]), __builtin_bit_cast(half8_t, a[i]),
								accf[i * 4 + j], 0, 0, 0);
				}
		}
		const uint64_t c1 = clock64();
		const uint64_t w1 = wall_clock64();
		float s = 0.0f;
		for (int i = 0; i < 16; i++)
			for (int r = 0; r < 16; r++)
				s += accf[i][r] + static_cast<float>(acci[i][r]);
		if (blockIdx.x == 0 && threadIdx.x == 0)
		{
			out[0] = c1 - c0;
			out[1] = w1 - w0;
		}
		if (s == 12345.678f)
			out[2 + threadIdx.x] = static_cast<uint64_t>(s);
	}
}

namespace
{
	typedef __attribute__((address_space(3))) void *lds_ptr_t;
	typedef __attribute__((address_space(1))) const void *global_ptr_t;

	/*
	 * Operand delivery of a hypothetical one-kernel Winograd layer (batched product + output transform inside one workgroup). Such a
	 * workgroup must hold the fp32 accumulators of ALL 36 matrix positions of its tiles: 36 x T x N x 4 bytes within ~300 KB of
	 * registers, i.e. T x N ~ 2048 (T tiles x N output channels). It therefore fetches, per task, the rows of its T tiles (36 x T x 512
	 * bytes at 256 channels in fp16) and the weight slice of its N columns (36 x N x 512 bytes) — the weights again for every group of T
	 * tiles, the tile rows again for every column slice. This kernel moves exactly those operands into LDS with direct-to-LDS loads,
	 * one matrix position per step, two steps in flight, and does nothing else (no MFMA, no LDS read, no store): its duration is a
	 * lower bound for that design. v = [36][tiles][512 bytes], u = [36][columns][512 bytes].
	 */
	/*
	 * FROM_X: the variant in which the workgroup would make its A operand itself, by running the input transform on the pixels of its T
	 * tiles (T / 16 images of 15 x 15 x 256 halfs = T * 7200 bytes per task, fetched here in 36 equal portions, one per step, from x =
	 * [images][225][512 bytes]) instead of fetching their 36 x T transformed rows; the weight slice is fetched as before.
	 */
	template<int T, int N, bool FROM_X>
	__global__ __launch_bounds__(512) void kernel_fused_layer_operand_stream(const uint8_t *v, const uint8_t *u, int tiles, int columns, int tasks)
	{
		extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
		constexpr int PATCH_BYTES = T * 7200;
		constexpr int A_BLOCKS = FROM_X ? (PATCH_BYTES / 36 + 1023) / 1024 : T * 512 / 1024; /* 1 KB per wavefront instruction */
		constexpr int B_BLOCKS = N * 512 / 1024;
		constexpr int BLOCKS = A_BLOCKS + B_BLOCKS;
		constexpr int STEP_BYTES = BLOCKS * 1024;
		constexpr int LOADS = (BLOCKS + 7) / 8;
		const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
		const int slices = columns / N;
		for (int task = blockIdx.x; task < tasks; task += gridDim.x)
		{
			const int group = task / slices, slice = task % slices;
			for (int p = 0; p < 36; p++)
			{
				uint8_t *buffer = lds + (p & 1) * STEP_BYTES;
				const uint8_t *a = FROM_X ? v + static_cast<size_t>(group) * PATCH_BYTES + static_cast<size_t>(p) * (A_BLOCKS * 1024)
						: v + (static_cast<size_t>(p) * tiles + static_cast<size_t>(group) * T) * 512;
				const uint8_t *a_last = v + static_cast<size_t>(group + 1) * PATCH_BYTES - 1024; /* FROM_X: the last portion ends with the patch */
				const uint8_t *b = u + (static_cast<size_t>(p) * columns + static_cast<size_t>(slice) * N) * 512;
#pragma unroll
				for (int l = 0; l < LOADS; l++)
				{
					const int block = wave + 8 * l;
					if (block < BLOCKS)
					{
						const uint8_t *src = (block < A_BLOCKS) ? a + block * 1024 : b + (block - A_BLOCKS) * 1024;
						if (FROM_X && block < A_BLOCKS && src > a_last)
							src = a_last;
						__builtin_amdgcn_global_load_lds((global_ptr_t) (src + lane * 16), (lds_ptr_t) (buffer + block * 1024), 16, 0, 0);
					}
				}
				/* the previous step's loads have landed in every wavefront before its buffer is overwritten by the next step (a wavefront
				 * whose last block index falls beyond BLOCKS has one load less in flight: its wait is merely earlier than needed) */
				__builtin_amdgcn_s_waitcnt(0x0f70 | (LOADS & 15) | ((LOADS >> 4) << 14));
				__builtin_amdgcn_s_barrier();
			}
		}
		__builtin_amdgcn_s_waitcnt(0x0f70);
	}
}

namespace
{
	std::string last_error;
	template<typename F>
	int guarded(F &&body)
	{
		try
		{
			body();
			return 0;
		}
		catch (const std::exception &e)
		{
			last_error = e.what();
		}
		catch (...)
		{
			last_error = "ceilings: unknown failure";
		}
		return -1;
	}
}

extern "C"
{
	/* v: 36 * tiles * 512 bytes (from_x: the pixels instead, tiles / 16 * 115200 bytes), u: 36 * columns * 512 bytes; tile_group x column_slice is
	 * 32 x 64 or 64 x 32; returns the bytes one launch moves into LDS */
	static size_t fused_layer_operand_stream(void *stream, const void *v, const void *u, int tiles, int columns, int tile_group, int column_slice, int workgroups,
			int from_x)
	{
		if (tiles <= 0 || columns <= 0 || tiles % tile_group != 0 || columns % column_slice != 0 || workgroups <= 0)
			throw std::logic_error("ceilings: ceil_fused_layer_operand_stream: bad arguments");
		hipStream_t s = reinterpret_cast<hipStream_t>(stream);
		const int tasks = (tiles / tile_group) * (columns / column_slice);
		const uint8_t *pv = reinterpret_cast<const uint8_t*>(v), *pu = reinterpret_cast<const uint8_t*>(u);
		const int a_blocks = from_x ? (tile_group * 7200 / 36 + 1023) / 1024 : tile_group * 512 / 1024;
		const int blocks = a_blocks + column_slice * 512 / 1024;
		const size_t lds_bytes = 2 * static_cast<size_t>(blocks) * 1024;
#define CEIL_LAUNCH_OPERANDS(T, N, X) \
		do { \
			check(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel_fused_layer_operand_stream<T, N, X>), hipFuncAttributeMaxDynamicSharedMemorySize, \
					static_cast<int>(lds_bytes)), "hipFuncSetAttribute"); \
			hipLaunchKernelGGL((kernel_fused_layer_operand_stream<T, N, X>), dim3(workgroups), dim3(512), lds_bytes, s, pv, pu, tiles, columns, tasks); \
		} while (0)
		if (tile_group == 32 && column_slice == 64 && !from_x)
			CEIL_LAUNCH_OPERANDS(32, 64, false);
		else if (tile_group == 64 && column_slice == 32 && !from_x)
			CEIL_LAUNCH_OPERANDS(64, 32, false);
		else if (tile_group == 32 && column_slice == 64)
			CEIL_LAUNCH_OPERANDS(32, 64, true);
		else if (tile_group == 64 && column_slice == 32)
			CEIL_LAUNCH_OPERANDS(64, 32, true);
		else
			throw std::logic_error("ceilings: ceil_fused_layer_operand_stream: 32 x 64 or 64 x 32 only");
#undef CEIL_LAUNCH_OPERANDS
		check(hipGetLastError(), "launch of kernel_fused_layer_operand_stream");
		return static_cast<size_t>(tasks) * 36 * static_cast<size_t>(blocks) * 1024;
	}

	/* mode 0 read, 1 write, 2 copy; bytes must be a multiple of 16; nt != 0 uses non-temporal accesses */
	static void stream_launch(void *stream, void *dst, const void *src, size_t bytes, int mode, int nt, int workgroups)
	{
		if (bytes % 16 != 0 || workgroups <= 0 || mode < 0 || mode > 2)
			throw std::logic_error("ceilings: ceil_stream: bad arguments");
		const size_t chunks = bytes / 16;
		size_t per_wg = (chunks + workgroups - 1) / workgroups;
		per_wg = (per_wg + 1023) / 1024 * 1024; /* whole 16 KB blocks per workgroup */
		const unsigned int grid = static_cast<unsigned int>((chunks + per_wg - 1) / per_wg);
		hipStream_t s = reinterpret_cast<hipStream_t>(stream);
		uint4_t *d = reinterpret_cast<uint4_t*>(dst);
		const uint4_t *r = reinterpret_cast<const uint4_t*>(src);
#define CEIL_LAUNCH(M, N) hipLaunchKernelGGL((kernel_stream<M, N>), dim3(grid), dim3(256), 0, s, d, r, chunks, per_wg)
		switch (mode * 2 + (nt ? 1 : 0))
		{
			case 0: CEIL_LAUNCH(0, false); break;
			case 1: CEIL_LAUNCH(0, true); break;
			case 2: CEIL_LAUNCH(1, false); break;
			case 3: CEIL_LAUNCH(1, true); break;
			case 4: CEIL_LAUNCH(2, false); break;
			default: CEIL_LAUNCH(2, true); break;
		}
#undef CEIL_LAUNCH
		check(hipGetLastError(), "launch of kernel_stream");
	}
	/* one launch of the MFMA loop on `workgroups` workgroups of 4 wavefronts; `out` = at least 2 + 256 uint64 of device memory */
	static void mfma_launch(void *stream, void *out, int iters, int random, int int8 /* 0 fp16, 1 int8, 2 fp32 */, int workgroups)
	{
		hipStream_t s = reinterpret_cast<hipStream_t>(stream);
		if (int8 == 1)
			hipLaunchKernelGGL(kernel_mfma_loop<1>, dim3(workgroups), dim3(256), 0, s, reinterpret_cast<uint64_t*>(out), iters, random);
		else if (int8 == 2)
			hipLaunchKernelGGL(kernel_mfma_loop<2>, dim3(workgroups), dim3(256), 0, s, reinterpret_cast<uint64_t*>(out), iters, random);
		else
			hipLaunchKernelGGL(kernel_mfma_loop<0>, dim3(workgroups), dim3(256), 0, s, reinterpret_cast<uint64_t*>(out), iters, random);
		check(hipGetLastError(), "launch of kernel_mfma_loop");
	}

	const char* ceil_last_error()
	{
		return last_error.c_str();
	}
	/* *bytes_moved receives the bytes one launch brings into LDS */
	int ceil_fused_layer_operand_stream(void *stream, const void *v, const void *u, int tiles, int columns, int tile_group, int column_slice, int workgroups,
			int from_x, size_t *bytes_moved)
	{
		return guarded([&]() { *bytes_moved = fused_layer_operand_stream(stream, v, u, tiles, columns, tile_group, column_slice, workgroups, from_x); });
	}
	int ceil_stream(void *stream, void *dst, const void *src, size_t bytes, int mode, int nt, int workgroups)
	{
		return guarded([&]() { stream_launch(stream, dst, src, bytes, mode, nt, workgroups); });
	}
	int ceil_mfma(void *stream, void *out, int iters, int random, int int8, int workgroups)
	{
		return guarded([&]() { mfma_launch(stream, out, iters, random, int8, workgroups); });
	}
}
