/*
 * winograd.hip — Winograd F(4x4, 3x3) weight / input / output transforms for gfx950, NHWC, fp16 and fp32 storage, fp32 arithmetic.
 *
 * What they compute follows the reference CPU backend:
 *   tile geometry, zero padding, matrix index order      src/backend/cpu/winograd/winograd_runtime.cpp:47-232
 *   weight transform (columns first, then rows)          src/backend/cpu/winograd/def_winograd_kernels.cpp:165-184,380-424
 *   input / output 1-D transforms incl. FMA placement    src/backend/cpu/winograd/avx2_winograd_kernels.cpp:241-279 (same in avx512f_*:241-279)
 *   output epilogue order: + bias, + ext, ReLU           src/backend/cpu/winograd/avx2_winograd_kernels.cpp:611-622
 *   other activations = separate pass over the stored y  src/backend/cpu/winograd/winograd_runtime.cpp:529-536
 * The floating-point expression trees below are written to be evaluated exactly as the reference evaluates them (explicit fma
 * where it uses one, no contraction elsewhere), so fp32 results and truncated fp16 results agree bit for bit.
 *
 * How they run: the transforms are pure streaming kernels (bound by HBM bandwidth). One thread owns VEC consecutive channels of one
 * tile, so that a wavefront touches 64*VEC consecutive channels with one 4/8/16-byte access per lane; a 6x6 tile of
 * VEC channels lives in registers. Neighbouring tiles of one image are placed on the same XCD so that the two rows / columns of
 * halo they share are served by that XCD's L2.
 */
#include "common.hpp"
#include "device_utils.hpp"
#include "gemm_stream.hpp"

#include <map>
#include <mutex>

#pragma clang fp contract(off)

namespace
{
	using namespace mlhip;

	/* ---------------------------------------------------------------------------------------------------------------------
	 * 1-D transforms on VEC channels at once
	 * ------------------------------------------------------------------------------------------------------------------- */
	template<int VEC>
	struct Line6
	{
			float v[6][VEC];
	};
	template<int VEC>
	struct Line4
	{
			float v[4][VEC];
	};

	/* Bt * d, rows evaluated as  r0=(l0-l2)+c14(l4-l2)  r1=(l1+l2)-c14(l3+l4)  r2=(l2-l1)+c14(l3-l4)
	 *                            r3=(l3-l1)+c12(l4-l2)  r4=(l1-l3)+c12(l4-l2)  r5=(l1-l3)+c14(l5-l3), last step fused */
	template<int VEC>
	__device__ __forceinline__ void input_transform_1d(const float (&l)[6][VEC], float (&r)[6][VEC])
	{
#pragma unroll
		for (int c = 0; c < VEC; c++)
		{
			const float l0 = l[0][c], l1 = l[1][c], l2 = l[2][c], l3 = l[3][c], l4 = l[4][c], l5 = l[5][c];
			r[0][c] = __builtin_fmaf(0.25f, l4 - l2, l0 - l2);
			r[1][c] = __builtin_fmaf(-0.25f, l3 + l4, l1 + l2);
			r[2][c] = __builtin_fmaf(0.25f, l3 - l4, l2 - l1);
			r[3][c] = __builtin_fmaf(0.5f, l4 - l2, l3 - l1);
			r[4][c] = __builtin_fmaf(0.5f, l4 - l2, l1 - l3);
			r[5][c] = __builtin_fmaf(0.25f, l5 - l3, l1 - l3);
		}
	}
	/* At * m:  s=l1+l2 d=l1-l2 p=l3+l4 q=l3-l4;  o0=(l0+s)+c14*p  o1=d+c12*q  o2=s+p  o3=(d+2*l5)+2*q */
	template<int VEC>
	__device__ __forceinline__ void output_transform_1d(const float (&l)[6][VEC], float (&o)[4][VEC])
	{
#pragma unroll
		for (int c = 0; c < VEC; c++)
		{
			const float l0 = l[0][c], l1 = l[1][c], l2 = l[2][c], l3 = l[3][c], l4 = l[4][c], l5 = l[5][c];
			const float s = l1 + l2;
			const float d = l1 - l2;
			const float p = l3 + l4;
			const float q = l3 - l4;
			o[0][c] = __builtin_fmaf(0.25f, p, l0 + s);
			o[1][c] = __builtin_fmaf(0.5f, q, d);
			o[2][c] = s + p;
			o[3][c] = __builtin_fmaf(2.0f, q, __builtin_fmaf(2.0f, l5, d));
		}
	}
	/* G * g with the constants rounded to fp32 and no fused operations */
	__device__ __forceinline__ void weight_transform_1d(const float (&g)[3], float (&w)[6])
	{
		const float c13 = 1.0 / 3.0;
		const float c23 = 2.0 / 3.0;
		const float c43 = 4.0 / 3.0;
		const float c2 = 2.0;
		w[0] = g[0];
		w[1] = c23 * ((g[0] + g[1]) + g[2]);
		w[2] = c23 * ((g[0] - g[1]) + g[2]);
		w[3] = (c13 * g[0] + c23 * g[1]) + c43 * g[2];
		w[4] = (c13 * g[0] - c23 * g[1]) + c43 * g[2];
		w[5] = c2 * g[2];
	}

	/* ---------------------------------------------------------------------------------------------------------------------
	 * kernels
	 * ------------------------------------------------------------------------------------------------------------------- */
	/* weights [Cout][3][3][Cin] -> matrices [36][Cout][Cin]; one thread per (cout, cin) */
	template<typename T>
	__global__ __launch_bounds__(256) void kernel_weight_transform_4x4_3x3(const T *__restrict__ weights, T *__restrict__ matrices,
			int filters_out, int filters_in, bool invert)
	{
		const size_t total = static_cast<size_t>(filters_out) * filters_in;
		const size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
		if (gid >= total)
			return;
		const int out = static_cast<int>(gid / filters_in);
		const int in = static_cast<int>(gid % filters_in);

		float tile[3][3];
#pragma unroll
		for (int i = 0; i < 3; i++)
#pragma unroll
			for (int j = 0; j < 3; j++)
			{
				const int x = invert ? (2 - i) : i;
				const int y = invert ? (2 - j) : j;
				tile[i][j] = Storage<T>::load(weights + ((static_cast<size_t>(out) * 3 + x) * 3 + y) * filters_in + in);
			}

		float tmp[6][3]; /* columns first */
#pragma unroll
		for (int col = 0; col < 3; col++)
		{
			const float g[3] = { tile[0][col], tile[1][col], tile[2][col] };
			float w[6];
			weight_transform_1d(g, w);
#pragma unroll
			for (int row = 0; row < 6; row++)
				tmp[row][col] = w[row];
		}
#pragma unroll
		for (int row = 0; row < 6; row++)
		{
			float w[6];
			weight_transform_1d(tmp[row], w);
#pragma unroll
			for (int col = 0; col < 6; col++)
				Storage<T>::store(matrices + (static_cast<size_t>(row * 6 + col) * filters_out + out) * filters_in + in, w[col]);
		}
	}

	/* VEC storage elements moved by one load instruction and kept unconverted until they are needed */
	template<typename T, int N>
	struct RawVec
	{
			typedef T type __attribute__((ext_vector_type(N)));
			__device__ static __forceinline__ float get(const type &r, int i)
			{
				return static_cast<float>(r[i]);
			}
	};
	template<typename T>
	struct RawVec<T, 1>
	{
			typedef T type;
			__device__ static __forceinline__ float get(const type &r, int)
			{
				return static_cast<float>(r);
			}
	};

	/*
	 * input [B][H][W][C] -> matrices [36][B*tiles_h*tiles_w][C]
	 * All 36 loads of a tile are issued back to back, unconditionally, from coordinates clamped into the image; elements that lie outside
	 * are replaced by zero afterwards. (A load under a bounds test would sit in its own basic block and be waited for on its own, which
	 * leaves one 512-byte request in flight per wavefront.) Offsets are 32-bit element offsets from the tensor base.
	 */
	template<typename T, int VEC>
	__global__ __launch_bounds__(256) void kernel_input_transform_4x4_3x3(const T *__restrict__ input, T *__restrict__ matrices, int batch_size,
			int height, int width, int channels, int tiles_h, int tiles_w)
	{
		typedef typename RawVec<T, VEC>::type raw_t;
		const unsigned int groups = channels / VEC;
		const unsigned int tiles_per_image = tiles_h * tiles_w;
		const unsigned int nb_of_tiles = batch_size * tiles_per_image;
		const unsigned int total = nb_of_tiles * groups;

		const unsigned int block = xcd_contiguous_block_id(blockIdx.x, gridDim.x);
		const unsigned int gid = block * blockDim.x + threadIdx.x;
		if (gid >= total)
			return;
		const unsigned int tile_idx = gid / groups;
		const unsigned int channel = (gid - tile_idx * groups) * VEC;

		const unsigned int batch = tile_idx / tiles_per_image;
		const unsigned int in_image = tile_idx - batch * tiles_per_image;
		const int tile_x = in_image / tiles_w;
		const int x0 = 4 * tile_x - 1;
		const int y0 = 4 * (in_image - tile_x * tiles_w) - 1;

		unsigned int row_offset[6], col_offset[6];
		bool row_valid[6], col_valid[6];
#pragma unroll
		for (int i = 0; i < 6; i++)
		{
			const int x = x0 + i;
			const int y = y0 + i;
			row_valid[i] = (x >= 0) && (x < height);
			col_valid[i] = (y >= 0) && (y < width);
			const int xc = min(max(x, 0), height - 1);
			const int yc = min(max(y, 0), width - 1);
			row_offset[i] = (batch * height + xc) * width * channels;
			col_offset[i] = yc * channels + channel;
		}

		raw_t raw[6][6];
#pragma unroll
		for (int row = 0; row < 6; row++)
#pragma unroll
			for (int col = 0; col < 6; col++)
				raw[row][col] = *reinterpret_cast<const raw_t*>(input + (row_offset[row] + col_offset[col]));

		float tmp[6][6][VEC]; /* [row after the column pass][col] */
#pragma unroll
		for (int col = 0; col < 6; col++)
		{
			float line[6][VEC];
#pragma unroll
			for (int row = 0; row < 6; row++)
			{
				const bool valid = row_valid[row] && col_valid[col];
#pragma unroll
				for (int c = 0; c < VEC; c++)
					line[row][c] = valid ? RawVec<T, VEC>::get(raw[row][col], c) : 0.0f;
			}
			float res[6][VEC];
			input_transform_1d<VEC>(line, res);
#pragma unroll
			for (int row = 0; row < 6; row++)
#pragma unroll
				for (int c = 0; c < VEC; c++)
					tmp[row][col][c] = res[row][c];
		}

		T *dst = matrices + static_cast<size_t>(tile_idx) * channels + channel;
		const size_t matrix_stride = static_cast<size_t>(nb_of_tiles) * channels;
#pragma unroll
		for (int row = 0; row < 6; row++)
		{
			float res[6][VEC];
			input_transform_1d<VEC>(tmp[row], res);
#pragma unroll
			for (int col = 0; col < 6; col++)
			{
				Vec<T, VEC> out;
#pragma unroll
				for (int c = 0; c < VEC; c++)
					out.v[c] = res[col][c];
				/* non-temporal: measured 94.2k against 88.2k positions per second on the 20-block network run as three calls per layer */
				out.store_streaming(dst + static_cast<size_t>(row * 6 + col) * matrix_stride);
			}
		}
	}

	/*
	 * matrices [36][B*tiles_h*tiles_w][C] (+ bias [C], + ext [B][H][W][C]) -> output [B][H][W][C]
	 * ACT: 0 = linear, 1 = ReLU (both fused as the reference fuses them), 2 = any other activation, selected at run time.
	 * The 36 matrix rows and the 16 residual vectors (from clamped coordinates) are requested before any arithmetic.
	 */
	template<typename T, int VEC, int ACT, bool HAS_EXT>
	__global__ __launch_bounds__(256) void kernel_output_transform_4x4_3x3(const T *__restrict__ matrices, T *output, const T *__restrict__ bias,
			const T *ext, int act, int batch_size, int height, int width, int channels, int tiles_h, int tiles_w)
	{
		typedef typename RawVec<T, VEC>::type raw_t;
		const unsigned int groups = channels / VEC;
		const unsigned int tiles_per_image = tiles_h * tiles_w;
		const unsigned int nb_of_tiles = batch_size * tiles_per_image;
		const unsigned int total = nb_of_tiles * groups;

		/* runs of 16 workgroups (64 tiles of 256 channels) per XCD, the runs going round the XCDs: measured 102 -> 92 us for the 20 x 256
		 * network's layer with residual against one contiguous eighth of the tiles per XCD (the input transform is the other way round:
		 * 63 us with contiguous eighths, 64-75 us with runs) */
		const unsigned int block = xcd_run_block_id(blockIdx.x, gridDim.x, 16);
		const unsigned int gid = block * blockDim.x + threadIdx.x;
		if (gid >= total)
			return;
		const unsigned int tile_idx = gid / groups;
		const unsigned int channel = (gid - tile_idx * groups) * VEC;

		const unsigned int batch = tile_idx / tiles_per_image;
		const unsigned int in_image = tile_idx - batch * tiles_per_image;
		const int tile_x = in_image / tiles_w;
		const int x0 = 4 * tile_x;
		const int y0 = 4 * (in_image - tile_x * tiles_w);

		const T *src = matrices + static_cast<size_t>(tile_idx) * channels + channel;
		const size_t matrix_stride = static_cast<size_t>(nb_of_tiles) * channels;
		raw_t raw[6][6];
#pragma unroll
		for (int row = 0; row < 6; row++)
#pragma unroll
			for (int col = 0; col < 6; col++)
				raw[row][col] = __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(src + static_cast<size_t>(row * 6 + col) * matrix_stride));

		unsigned int offset[4][4]; /* element offsets of the 4x4 outputs, clamped into the image */
#pragma unroll
		for (int row = 0; row < 4; row++)
#pragma unroll
			for (int col = 0; col < 4; col++)
			{
				const int xc = min(x0 + row, height - 1);
				const int yc = min(y0 + col, width - 1);
				offset[row][col] = ((batch * height + xc) * width + yc) * channels + channel;
			}
		raw_t residual[4][4];
		if constexpr (HAS_EXT)
		{
#pragma unroll
			for (int row = 0; row < 4; row++)
#pragma unroll
				for (int col = 0; col < 4; col++)
					residual[row][col] = __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(ext + offset[row][col]));
		}
		Vec<T, VEC> b;
		if (bias != nullptr)
			b.load(bias + channel);
		else
			b.zero();

		float tmp[4][6][VEC];
#pragma unroll
		for (int col = 0; col < 6; col++)
		{
			float line[6][VEC];
#pragma unroll
			for (int row = 0; row < 6; row++)
#pragma unroll
				for (int c = 0; c < VEC; c++)
					line[row][c] = RawVec<T, VEC>::get(raw[row][col], c);
			float res[4][VEC];
			output_transform_1d<VEC>(line, res);
#pragma unroll
			for (int row = 0; row < 4; row++)
#pragma unroll
				for (int c = 0; c < VEC; c++)
					tmp[row][col][c] = res[row][c];
		}

#pragma unroll
		for (int row = 0; row < 4; row++)
		{
			float res[4][VEC];
			output_transform_1d<VEC>(tmp[row], res);
#pragma unroll
			for (int col = 0; col < 4; col++)
			{
				Vec<T, VEC> out;
#pragma unroll
				for (int c = 0; c < VEC; c++)
				{
					float t = res[col][c] + b.v[c];
					if constexpr (HAS_EXT)
						t = t + RawVec<T, VEC>::get(residual[row][col], c);
					if constexpr (ACT == 1)
						t = fmaxf(t, 0.0f);
					if constexpr (ACT == 2)
					{ /* the reference stores y and then runs the activation over it: round through the storage type in between */
						if constexpr (sizeof(T) == 2)
							t = half_bits_to_float(half_bits_rtz(t));
						t = activate(act, t);
					}
					out.v[c] = t;
				}
				if ((x0 + row) < height && (y0 + col) < width)
					out.store(output + offset[row][col]); /* cacheable: the next launch usually reads y right away */
			}
		}
	}

	/* one image's share of a fused output -> input transform: where its matrices, pixels and next matrices lie */
	template<typename T>
	struct FusedImage
	{
			const T *matrices; /* position 0, first tile of the image, channel 0 */
			size_t matrix_stride; /* elements between two positions */
			T *output; /* first pixel of the image, channel 0; nullptr: y is not written */
			const T *ext; /* first pixel of the image's residual (only read when HAS_EXT) */
			const T *bias; /* [channels] or nullptr */
			T *next_matrices; /* like `matrices`, for the next layer */
			size_t next_stride;
			int act, height, width, channels, tiles_h, tiles_w;
			int slice; /* which SLICE channels of the image this workgroup owns */
	};

	/* phase 1: output transform of the image's tiles into the LDS image [height * width + 1][SLICE] (and to g.output) */
	template<typename T, int VEC, int SLICE, int ACT, bool HAS_EXT, int THREADS, bool STREAM_OUTPUT = false, bool STREAM_MATRICES = false>
	__device__ __forceinline__ void fused_transform_phase1(const FusedImage<T> &g, uint8_t *lds_bytes)
	{
		typedef typename RawVec<T, VEC>::type raw_t;
		constexpr int CHANNEL_LANES = SLICE / VEC;
		constexpr int TILE_LANES = THREADS / CHANNEL_LANES;
		T *image = reinterpret_cast<T*>(lds_bytes); /* the extra last pixel stays zero */
		const int height = g.height, width = g.width, channels = g.channels;
		const int channel_local = (threadIdx.x % CHANNEL_LANES) * VEC;
		const unsigned int channel = g.slice * SLICE + channel_local;
		const int tile_lane = threadIdx.x / CHANNEL_LANES;
		const unsigned int tiles_per_image = g.tiles_h * g.tiles_w;
		const int tiles_w = g.tiles_w;
		const size_t matrix_stride = g.matrix_stride;
		const int zero_pixel = height * width;

		if (tile_lane == 0)
		{
			Vec<T, VEC> z;
			z.zero();
			z.store(image + zero_pixel * SLICE + channel_local);
		}
		Vec<T, VEC> b;
		if (g.bias != nullptr)
			b.load(g.bias + channel);
		else
			b.zero();

		/*
		 * The residual slice of this image goes straight into the image buffer with direct-to-LDS loads (16 bytes per lane, no staging
		 * registers): phase 1 then adds it from LDS and overwrites it in place with y. Every (pixel, channel) of the buffer is read and
		 * written by the one thread that owns its tile, so no further synchronisation is needed inside phase 1.
		 */
		if constexpr (HAS_EXT)
		{
			typedef __attribute__((address_space(3))) void *lds_ptr_t;
			typedef __attribute__((address_space(1))) const void *global_ptr_t;
			constexpr int CHUNKS_PER_PIXEL = SLICE * static_cast<int>(sizeof(T)) / 16;
			const int total_chunks = zero_pixel * CHUNKS_PER_PIXEL;
			const uint8_t *ext_slice = reinterpret_cast<const uint8_t*>(g.ext + g.slice * SLICE);
			const int lane = threadIdx.x & 63;
			for (int base = (threadIdx.x >> 6) * 64; base < total_chunks; base += THREADS)
			{
				const int chunk = base + lane;
				if (chunk < total_chunks)
				{
					const int px = chunk / CHUNKS_PER_PIXEL;
					const int part = chunk - px * CHUNKS_PER_PIXEL;
					__builtin_amdgcn_global_load_lds((global_ptr_t) (ext_slice + static_cast<size_t>(px) * channels * sizeof(T) + part * 16),
							(lds_ptr_t) (lds_bytes + base * 16), 16, 0, STREAM_OUTPUT ? 2 : 0);
				}
			}
		}

		raw_t raw[6][6];
		auto load_matrices = [&](unsigned int in_image) __attribute__((always_inline))
		{
			const T *src = g.matrices + static_cast<size_t>(in_image) * channels + channel;
#pragma unroll
			for (int row = 0; row < 6; row++)
#pragma unroll
				for (int col = 0; col < 6; col++)
				{
					const raw_t *p = reinterpret_cast<const raw_t*>(src + static_cast<size_t>(row * 6 + col) * matrix_stride);
					if constexpr (STREAM_MATRICES)
						raw[row][col] = __builtin_nontemporal_load(p); /* read once: not worth a place in the caches */
					else
						raw[row][col] = *p;
				}
		};
		unsigned int in_image = tile_lane;
		bool loaded = false;
		if constexpr (HAS_EXT)
		{ /* the first tile's matrices are requested before the wait, so that they fly together with the residual slice */
			if (in_image < tiles_per_image)
			{
				load_matrices(in_image);
				loaded = true;
			}
			__syncthreads(); /* waits for this wavefront's loads, then for everyone's: the residual slice is complete */
		}
#pragma clang loop unroll(disable)
		while (in_image < tiles_per_image)
		{
			if (!loaded)
				load_matrices(in_image);
			loaded = false;
			const int tile_x = in_image / tiles_w;
			const int x0 = 4 * tile_x;
			const int y0 = 4 * (in_image - tile_x * tiles_w);

			int pixel[4][4]; /* pixel index within the image, clamped */
#pragma unroll
			for (int row = 0; row < 4; row++)
#pragma unroll
				for (int col = 0; col < 4; col++)
					pixel[row][col] = min(x0 + row, height - 1) * width + min(y0 + col, width - 1);

			float tmp[4][6][VEC];
#pragma unroll
			for (int col = 0; col < 6; col++)
			{
				float line[6][VEC];
#pragma unroll
				for (int row = 0; row < 6; row++)
#pragma unroll
					for (int c = 0; c < VEC; c++)
						line[row][c] = RawVec<T, VEC>::get(raw[row][col], c);
				float res[4][VEC];
				output_transform_1d<VEC>(line, res);
#pragma unroll
				for (int row = 0; row < 4; row++)
#pragma unroll
					for (int c = 0; c < VEC; c++)
						tmp[row][col][c] = res[row][c];
			}
#pragma unroll
			for (int row = 0; row < 4; row++)
			{
				float res[4][VEC];
				output_transform_1d<VEC>(tmp[row], res);
#pragma unroll
				for (int col = 0; col < 4; col++)
				{
					T *in_lds = image + pixel[row][col] * SLICE + channel_local;
					raw_t residual;
					if constexpr (HAS_EXT)
						residual = *reinterpret_cast<const raw_t*>(in_lds);
					Vec<T, VEC> out;
#pragma unroll
					for (int c = 0; c < VEC; c++)
					{
						float t = res[col][c] + b.v[c];
						if constexpr (HAS_EXT)
							t = t + RawVec<T, VEC>::get(residual, c);
						if constexpr (ACT == 1)
							t = fmaxf(t, 0.0f);
						if constexpr (ACT == 2)
						{ /* the reference stores y and then runs the activation over it: round through the storage type in between */
							if constexpr (sizeof(T) == 2)
								t = half_bits_to_float(half_bits_rtz(t));
							t = activate(g.act, t);
						}
						out.v[c] = t;
					}
					if ((x0 + row) < height && (y0 + col) < width)
					{
						out.store(in_lds);
						if (g.output != nullptr)
						{
							if constexpr (STREAM_OUTPUT)
								out.store_streaming(g.output + static_cast<size_t>(pixel[row][col]) * channels + channel);
							else
								out.store(g.output + static_cast<size_t>(pixel[row][col]) * channels + channel);
						}
					}
				}
			}
			in_image += TILE_LANES;
		}
	}

	/* phase 2: input transform of the next layer out of the LDS image (all of phase 1 must have finished: barrier in between) */
	template<typename T, int VEC, int SLICE, int THREADS, bool STREAM = false>
	__device__ __forceinline__ void fused_transform_phase2(const FusedImage<T> &g, const uint8_t *lds_bytes)
	{
		typedef typename RawVec<T, VEC>::type raw_t;
		constexpr int CHANNEL_LANES = SLICE / VEC;
		constexpr int TILE_LANES = THREADS / CHANNEL_LANES;
		const T *image = reinterpret_cast<const T*>(lds_bytes);
		const int height = g.height, width = g.width, channels = g.channels;
		const int channel_local = (threadIdx.x % CHANNEL_LANES) * VEC;
		const unsigned int channel = g.slice * SLICE + channel_local;
		const int tile_lane = threadIdx.x / CHANNEL_LANES;
		const unsigned int tiles_per_image = g.tiles_h * g.tiles_w;
		const int tiles_w = g.tiles_w;
		const size_t next_stride = g.next_stride;
		const int zero_pixel = height * width;
#pragma clang loop unroll(disable)
		for (unsigned int in_image = tile_lane; in_image < tiles_per_image; in_image += TILE_LANES)
		{
			const int tile_x = in_image / tiles_w;
			const int x0 = 4 * tile_x - 1;
			const int y0 = 4 * (in_image - tile_x * tiles_w) - 1;
			int row_pixel[6], col_pixel[6];
			bool row_valid[6], col_valid[6];
#pragma unroll
			for (int i = 0; i < 6; i++)
			{
				row_valid[i] = (x0 + i >= 0) && (x0 + i < height);
				col_valid[i] = (y0 + i >= 0) && (y0 + i < width);
				row_pixel[i] = min(max(x0 + i, 0), height - 1) * width;
				col_pixel[i] = min(max(y0 + i, 0), width - 1);
			}
			raw_t raw[6][6];
#pragma unroll
			for (int row = 0; row < 6; row++)
#pragma unroll
				for (int col = 0; col < 6; col++)
				{
					const int px = (row_valid[row] && col_valid[col]) ? (row_pixel[row] + col_pixel[col]) : zero_pixel;
					raw[row][col] = *reinterpret_cast<const raw_t*>(image + px * SLICE + channel_local);
				}

			float tmp[6][6][VEC];
#pragma unroll
			for (int col = 0; col < 6; col++)
			{
				float line[6][VEC];
#pragma unroll
				for (int row = 0; row < 6; row++)
#pragma unroll
					for (int c = 0; c < VEC; c++)
						line[row][c] = RawVec<T, VEC>::get(raw[row][col], c);
				float res[6][VEC];
				input_transform_1d<VEC>(line, res);
#pragma unroll
				for (int row = 0; row < 6; row++)
#pragma unroll
					for (int c = 0; c < VEC; c++)
						tmp[row][col][c] = res[row][c];
			}
			T *dst = g.next_matrices + static_cast<size_t>(in_image) * channels + channel;
#pragma unroll
			for (int row = 0; row < 6; row++)
			{
				float res[6][VEC];
				input_transform_1d<VEC>(tmp[row], res);
#pragma unroll
				for (int col = 0; col < 6; col++)
				{
					Vec<T, VEC> out;
#pragma unroll
					for (int c = 0; c < VEC; c++)
						out.v[c] = res[col][c];
					if constexpr (STREAM)
						out.store_streaming(dst + static_cast<size_t>(row * 6 + col) * next_stride);
					else
						out.store(dst + static_cast<size_t>(row * 6 + col) * next_stride);
				}
			}
		}
	}

	/*
	 * Output transform of one layer fused with the input transform of the next 3x3 layer:
	 *   matrices [36][tiles][C] (+ bias, + ext) -> y [B][H][W][C] (written only if `output` is given) -> next_matrices [36][tiles][C]
	 * One workgroup owns one image and a slice of SLICE channels: its THREADS threads are THREADS / (SLICE / VEC) tile lanes x
	 * SLICE / VEC channel lanes. Phase 1 runs the output transform of the image's tiles (same arithmetic and epilogue as the stand-alone
	 * kernel) and leaves y, rounded to the storage type as the stand-alone kernel would store it, in LDS; phase 2 reads the 6x6 windows
	 * back (zero outside the image) and runs the input transform. Results are bit-identical to the two separate calls; what is saved is
	 * the write and re-read of y through HBM (or only the re-read, when y is also needed as a later residual).
	 */
	template<typename T, int VEC, int SLICE, int ACT, bool HAS_EXT, int THREADS>
		__global__ __launch_bounds__(THREADS, ((VEC <= 2) ? 1024 : 512) / THREADS) void kernel_output_input_transform_4x4_3x3(const T *__restrict__ matrices, T *output, const T *__restrict__ bias,
			const T *ext, int act, T *__restrict__ next_matrices, int batch_size, int height, int width, int channels, int tiles_h, int tiles_w)
	{
		extern __shared__ __attribute__((aligned(16))) uint8_t lds_bytes[];
		const unsigned int slices = channels / SLICE;
		/* the slices of one image (at least 4 workgroups) run on one XCD, the images go round the XCDs: neighbouring 128-byte pieces of a
		 * row of the matrices are then fetched and written through the same L2 at about the same time (124-130 -> 117-121 us for the
		 * 20 x 256 network's layer against the hardware's own order, in which consecutive workgroups sit on different XCDs) */
		const unsigned int run = (slices >= 4) ? slices : slices * (4 / slices);
		const unsigned int lin = xcd_run_block_id(blockIdx.x, gridDim.x, run);
		const unsigned int batch = lin / slices;
		const unsigned int tiles_per_image = tiles_h * tiles_w;
		const size_t image_pixels = static_cast<size_t>(batch) * height * width;
		FusedImage<T> g;
		g.matrix_stride = static_cast<size_t>(batch_size) * tiles_per_image * channels;
		g.next_stride = g.matrix_stride;
		g.matrices = matrices + static_cast<size_t>(batch) * tiles_per_image * channels;
		g.next_matrices = next_matrices + static_cast<size_t>(batch) * tiles_per_image * channels;
		g.output = (output != nullptr) ? output + image_pixels * channels : nullptr;
		g.ext = HAS_EXT ? ext + image_pixels * channels : nullptr;
		g.bias = bias;
		g.act = act;
		g.height = height;
		g.width = width;
		g.channels = channels;
		g.tiles_h = tiles_h;
		g.tiles_w = tiles_w;
		g.slice = lin - batch * slices;
		/*
		 * Cache hints, chosen by measurement on the 20-block network: the product matrices, the residual and y are non-temporal (each
		 * is touched once here), the next layer's matrices are written cacheable, because the product that follows walks them from
		 * the end and finds the rows written last still in the last-level cache.
		 */
		fused_transform_phase1<T, VEC, SLICE, ACT, HAS_EXT, THREADS, true, true>(g, lds_bytes);
		__syncthreads();
		fused_transform_phase2<T, VEC, SLICE, THREADS, false>(g, lds_bytes);
	}

	/* ---------------------------------------------------------------------------------------------------------------------
	 * A whole 3x3 layer in one launch (fp16, 256 -> 256 channels, 16 tiles per image):
	 *   V [36][T][256] x U [36][256][256]^T -> M -> output transform (+ bias, + ext, activation) -> y -> input transform -> V' [36][T][256]
	 * The product M never reaches HBM: it lives in the L2 of one XCD between the workgroups that make it and those that transform it.
	 *
	 * 512 workgroups of 256 threads, all resident at once (two per CU), find out which XCD they run on and take a role there:
	 *   36 GEMM workgroups, one per matrix position: the position's B operand (256 x 256) stays in registers for the whole launch
	 *     (4 wavefronts x 64 columns); for every chunk of 64 tiles (4 images) the XCD owns, 32 KB of A come HBM -> LDS by direct-to-LDS
	 *     loads (requested one chunk ahead), 64 MFMAs per wavefront make the 64 x 256 product, and it is stored to a scratch buffer
	 *     that is reused every LAYER_BUFFERS chunks and therefore stays in the XCD's L2;
	 *   28 transform workgroups: each takes (image, 64-channel slice) tasks of a finished chunk in turn and runs the fused
	 *     output -> input transform on them, reading M from the scratch buffer.
	 * Two counters per chunk order them: `produced` (36 arrivals: the chunk's M is complete) and `consumed` (16 arrivals: every task
	 * has read its part, the buffer may be overwritten). Stores are acknowledged by the L2 before a workgroup arrives, and a consumer
	 * drops its L1 lines after the wait, so data passes between CUs of one XCD without any L2 write-back. Every wait is bounded: a
	 * workgroup that gives up counts itself in the error word and leaves, and the others follow, so the grid always drains.
	 * Streaming traffic (A, the residual, y and V') is marked non-temporal so that it evicts as little of M as possible.
	 *
	 * Status (MI355X, batch 1024): results are bit-identical to the separate launches, but the launch takes about 430 us where the
	 * streaming product plus the fused transform take about 290 us. Measured reasons: only 28 of the 64 workgroups of an XCD transform,
	 * and a task is a chain of latencies (about 14 us), so the transform side limits the pipeline; while a chunk of M waits for it, two
	 * chunks' worth of streaming data pass through the 4 MiB L2 and evict about 80 % of M to HBM after all (HBM writes 548 MB per
	 * launch where 302 MB are V'). With a single scratch copy (1.1 MiB resident) M does stay in the L2 (HBM traffic 665 MB per launch
	 * against 1210 MB for the separate launches), but product and transform then alternate and the launch takes 520 us: the 4 MiB L2
	 * cannot hold enough chunks in flight to cover the latency of a transform task. A probe of the mechanism alone shows what is available: data ping-ponged between CUs of one XCD stays
	 * out of HBM (22 MB written for 3.4 GB exchanged), an XCD-wide barrier costs about 0.8 us, dropping the L1 costs little, whereas an
	 * agent-scope acquire fence costs about 8 us.
	 * ------------------------------------------------------------------------------------------------------------------- */
	constexpr int LAYER_CHUNK_TILES = 64; /* rows of one GEMM unit = 4 images of 16 tiles */
	constexpr int LAYER_CHANNELS = 256;
	constexpr int LAYER_BUFFERS = 2; /* scratch copies of a chunk's M per XCD: 2 x 36 x 64 x 256 x 2 bytes = 2.25 MiB of the 4 MiB L2 */
	constexpr int LAYER_GEMM_WORKGROUPS = 36, LAYER_WORKGROUPS_PER_XCD = 64, LAYER_XCDS = 8;
	constexpr int LAYER_TRANSFORM_WORKGROUPS = LAYER_WORKGROUPS_PER_XCD - LAYER_GEMM_WORKGROUPS;
	constexpr int LAYER_TASKS_PER_CHUNK = 16; /* 4 images x 4 slices of 64 channels */
	constexpr int LAYER_MAX_CHUNKS = 128; /* chunks per XCD that the counters cover: batch <= 8 * 128 * 4 images */
	constexpr size_t LAYER_CHUNK_ELEMENTS = static_cast<size_t>(36) * LAYER_CHUNK_TILES * LAYER_CHANNELS;

	struct LayerSync /* one per XCD; every counter on a cache line of its own */
	{
			unsigned int ticket, pad0[15];
			unsigned int produced[LAYER_MAX_CHUNKS][16];
			unsigned int consumed[LAYER_MAX_CHUNKS][16];
	};

	__device__ __forceinline__ int xcc_id()
	{
		return __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 7; /* hardware register XCC_ID, bits 3:0 */
	}
	/* polls until *counter >= target; false after `limit` polls */
	__device__ __forceinline__ bool wait_for_counter(unsigned int *counter, unsigned int target, unsigned int limit)
	{
		unsigned int polls = 0;
		while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target)
		{
			if (++polls >= limit)
				return false;
			__builtin_amdgcn_s_sleep(1);
		}
		return true;
	}

	template<int ACT, bool HAS_EXT>
	__global__ __launch_bounds__(256, 2) void kernel_winograd_layer_f16(const half_t *V, const half_t *U, const half_t *bias, const half_t *ext, half_t *output,
			half_t *next_matrices, half_t *scratch, LayerSync *sync, unsigned int *errors, int batch, int height, int width, int tiles_h, int tiles_w,
			int act, unsigned int spin_limit)
	{
		typedef MfmaTraits<half_t> Traits;
		typedef Traits::acc_vec acc_vec;
		extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
		__shared__ unsigned int s_word;
		const int xcd = xcc_id();
		LayerSync &my = sync[xcd];
		if (threadIdx.x == 0)
			s_word = __hip_atomic_fetch_add(&my.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		__syncthreads();
		const unsigned int role = s_word;
		__syncthreads();
		if (role >= LAYER_WORKGROUPS_PER_XCD)
			return; /* more workgroups on this XCD than roles */

		const int total_chunks = batch / 4;
		const int my_chunks = (total_chunks - xcd + LAYER_XCDS - 1) / LAYER_XCDS; /* chunks xcd, xcd + 8, ... */
		half_t *my_scratch = scratch + static_cast<size_t>(xcd) * LAYER_BUFFERS * LAYER_CHUNK_ELEMENTS;
		const size_t all_tiles = static_cast<size_t>(batch) * 16;
		const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

		if (role < LAYER_GEMM_WORKGROUPS)
		{
			const int p = role;
			const int frag_row = lane & 31, half_sel = lane >> 5;
			uint4_t b_regs[2][16]; /* 2 groups of 32 columns x 16 k steps */
			{
				const uint8_t *b_base = reinterpret_cast<const uint8_t*>(U + static_cast<size_t>(p) * LAYER_CHANNELS * LAYER_CHANNELS);
#pragma unroll
				for (int cg = 0; cg < 2; cg++)
				{
					const uint8_t *row = b_base + static_cast<size_t>(wave * 64 + cg * 32 + frag_row) * 512 + half_sel * 16;
#pragma unroll
					for (int k = 0; k < 16; k++)
						b_regs[cg][k] = *reinterpret_cast<const uint4_t*>(row + k * 32);
				}
			}
			/* a chunk of A: 64 rows x 512 bytes, kept as 4 k stages of 64 rows x 128 bytes; a wavefront moves 8 blocks of 1 KB */
			int source_offset[8];
#pragma unroll
			for (int i = 0; i < 8; i++)
			{
				const int block = wave + 4 * i;
				const int row = (block & 7) * 8 + (lane >> 3);
				source_offset[i] = row * 512 + (block >> 3) * 128 + (((lane & 7) ^ ((row >> 1) & 7)) * 16);
			}
			const uint8_t *a_base = reinterpret_cast<const uint8_t*>(V + static_cast<size_t>(p) * all_tiles * LAYER_CHANNELS);
			auto request_chunk = [&](int ci) __attribute__((always_inline))
			{
				const uint8_t *a = a_base + static_cast<size_t>(xcd + LAYER_XCDS * ci) * LAYER_CHUNK_TILES * 512;
				uint8_t *slot = lds + (ci & 1) * 32768;
#pragma unroll
				for (int i = 0; i < 8; i++)
					__builtin_amdgcn_global_load_lds((global_ptr_t) (a + source_offset[i]), (lds_ptr_t) (slot + (wave + 4 * i) * 1024), 16, 0, 2); /* non-temporal */
			};
			int frag_first[2];
#pragma unroll
			for (int rb = 0; rb < 2; rb++)
			{
				const int row = 32 * rb + frag_row;
				frag_first[rb] = row * 128 + ((half_sel ^ ((row >> 1) & 7)) * 16);
			}
			if (my_chunks > 0)
				request_chunk(0);
			for (int ci = 0; ci < my_chunks; ci++)
			{
				wait_vmcnt<0>(); /* this chunk's A has landed (and the B operand, the first time) */
				barrier_no_fence(); /* ... for every wavefront; nobody reads the other slot any more */
				if (ci + 1 < my_chunks)
					request_chunk(ci + 1);
				const uint8_t *slot = lds + (ci & 1) * 32768;
				acc_vec acc[2][2];
#pragma unroll
				for (int rb = 0; rb < 2; rb++)
#pragma unroll
					for (int cg = 0; cg < 2; cg++)
#pragma unroll
						for (int r = 0; r < 16; r++)
							acc[rb][cg][r] = 0;
				uint4_t frags[2][2];
#pragma unroll
				for (int rb = 0; rb < 2; rb++)
					frags[0][rb] = *reinterpret_cast<const uint4_t*>(slot + frag_first[rb]);
				stream_static_for<16>([&](auto step)
				{
					constexpr int t = decltype(step)::value;
					constexpr int cur = t & 1, nxt = 1 - cur;
					if constexpr (t + 1 < 16)
					{
						constexpr int ks = (t + 1) / 4, kk = (t + 1) % 4;
#pragma unroll
						for (int rb = 0; rb < 2; rb++)
							frags[nxt][rb] = *reinterpret_cast<const uint4_t*>(slot + ks * 8192 + (frag_first[rb] ^ (kk * 32)));
					}
#pragma unroll
					for (int cg = 0; cg < 2; cg++)
#pragma unroll
						for (int rb = 0; rb < 2; rb++)
							Traits::mma(b_regs[cg][t], frags[cur][rb], acc[rb][cg]);
				});
				/* the scratch copy this chunk goes to was last used by chunk ci - LAYER_BUFFERS: all its tasks must have read it */
				if (threadIdx.x == 0)
					s_word = (ci < LAYER_BUFFERS) ? 1u
							: (wait_for_counter(&my.consumed[ci - LAYER_BUFFERS][0], LAYER_TASKS_PER_CHUNK, spin_limit) ? 1u : 0u);
				__syncthreads();
				if (s_word == 0)
				{
					if (threadIdx.x == 0)
						__hip_atomic_fetch_add(errors, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
					return;
				}
				/* lane l, register r of a block: m = 32 rb + l % 32, n = 64 wave + 32 cg + 8 (r / 4) + 4 (l / 32) + r % 4 */
				half_t *dst = my_scratch + (static_cast<size_t>(ci % LAYER_BUFFERS) * 36 + p) * LAYER_CHUNK_TILES * LAYER_CHANNELS;
#pragma unroll
				for (int rb = 0; rb < 2; rb++)
#pragma unroll
					for (int cg = 0; cg < 2; cg++)
#pragma unroll
						for (int q = 0; q < 4; q++)
						{
							uint2_t packed;
							packed[0] = pack_rtz(acc[rb][cg][4 * q], acc[rb][cg][4 * q + 1]);
							packed[1] = pack_rtz(acc[rb][cg][4 * q + 2], acc[rb][cg][4 * q + 3]);
							*reinterpret_cast<uint2_t*>(dst + (32 * rb + frag_row) * LAYER_CHANNELS + wave * 64 + cg * 32 + 8 * q + 4 * half_sel) = packed;
						}
				wait_vmcnt<0>(); /* the L2 has this wavefront's stores */
				__syncthreads(); /* ... and everyone's */
				if (threadIdx.x == 0)
					__hip_atomic_fetch_add(&my.produced[ci][0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
		}
		else
		{
			const int first_task = role - LAYER_GEMM_WORKGROUPS;
			const int tasks = my_chunks * LAYER_TASKS_PER_CHUNK;
			for (int task = first_task; task < tasks; task += LAYER_TRANSFORM_WORKGROUPS)
			{
				const int ci = task / LAYER_TASKS_PER_CHUNK;
				const int sub = task - ci * LAYER_TASKS_PER_CHUNK;
				const int image_in_chunk = sub >> 2;
				__syncthreads(); /* the previous task has left the LDS image */
				if (threadIdx.x == 0)
					s_word = wait_for_counter(&my.produced[ci][0], LAYER_GEMM_WORKGROUPS, spin_limit) ? 1u : 0u;
				__syncthreads();
				if (s_word == 0)
				{
					if (threadIdx.x == 0)
						__hip_atomic_fetch_add(errors, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
					return;
				}
				asm volatile("buffer_inv sc0" ::: "memory"); /* this CU's L1 may hold lines of an earlier chunk at the same addresses */
				wait_vmcnt<0>();
				const size_t image = static_cast<size_t>(xcd + LAYER_XCDS * ci) * 4 + image_in_chunk;
				const size_t image_elements = static_cast<size_t>(height) * width * LAYER_CHANNELS;
				FusedImage<half_t> g;
				g.matrices = my_scratch + static_cast<size_t>(ci % LAYER_BUFFERS) * LAYER_CHUNK_ELEMENTS + image_in_chunk * 16 * LAYER_CHANNELS;
				g.matrix_stride = static_cast<size_t>(LAYER_CHUNK_TILES) * LAYER_CHANNELS;
				g.output = (output != nullptr) ? output + image * image_elements : nullptr;
				g.ext = HAS_EXT ? ext + image * image_elements : nullptr;
				g.bias = bias;
				g.next_matrices = next_matrices + image * 16 * LAYER_CHANNELS;
				g.next_stride = all_tiles * LAYER_CHANNELS;
				g.act = act;
				g.height = height;
				g.width = width;
				g.channels = LAYER_CHANNELS;
				g.tiles_h = tiles_h;
				g.tiles_w = tiles_w;
				g.slice = sub & 3;
				fused_transform_phase1<half_t, 4, 64, ACT, HAS_EXT, 256, true>(g, lds);
				__syncthreads(); /* every thread has taken what it needs from the scratch copy */
				if (threadIdx.x == 0)
					__hip_atomic_fetch_add(&my.consumed[ci][0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				fused_transform_phase2<half_t, 4, 64, 256, true>(g, lds);
			}
		}
	}

	/* ---------------------------------------------------------------------------------------------------------------------
	 * host side
	 * ------------------------------------------------------------------------------------------------------------------- */
	int integer_sqrt(int x)
	{
		int r = 0;
		while ((r + 1) * (r + 1) <= x)
			r++;
		return r;
	}
	/* the kernel size is not an argument: matrices.dim[0] = (tile + kernel - 1)^2 (reference: src/core/math.cpp:107-118) */
	void require_supported(int tile_size, const mlTensor_t &matrices, mlDataType_t dtype)
	{
		MLHIP_REQUIRE(matrices.rank == 3, "Winograd matrices must have rank 3");
		const int transform = integer_sqrt(matrices.dim[0]);
		const int kernel_size = transform + 1 - tile_size;
		const bool ok = (transform * transform == matrices.dim[0]) && tile_size == 4 && kernel_size == 3
				&& (dtype == DTYPE_FLOAT16 || dtype == DTYPE_FLOAT32);
		if (!ok)
			fail_runtime("No suitable Winograd transform runtime");
	}
	int pick_vec(int channels, const void *p0, const void *p1, const void *p2, const void *p3, int elem_size)
	{
		/* widest access is 16 bytes for fp32 (4 channels) and 8 bytes for fp16 (4 channels): 144 live fp32 values per thread */
		int vec = 4;
		while (vec > 1)
		{
			const uintptr_t bytes = static_cast<uintptr_t>(vec) * elem_size;
			const bool aligned = (reinterpret_cast<uintptr_t>(p0) % bytes == 0) && (reinterpret_cast<uintptr_t>(p1) % bytes == 0)
					&& (reinterpret_cast<uintptr_t>(p2) % bytes == 0) && (reinterpret_cast<uintptr_t>(p3) % bytes == 0);
			if (channels % vec == 0 && aligned)
				break;
			vec /= 2;
		}
		return vec;
	}
	unsigned int grid_for(size_t threads)
	{
		const size_t blocks = (threads + 255) / 256;
		MLHIP_REQUIRE(blocks <= 0x7fffffffu, "tensor too large for one launch");
		return static_cast<unsigned int>(blocks);
	}

	template<typename T>
	void launch_input(hipStream_t stream, const mlTensor_t &x, mlTensor_t &matrices)
	{
		const int batch = x.dim[0], height = x.dim[1], width = x.dim[2], channels = x.dim[3];
		const int tiles_h = ceil_div(height, 4), tiles_w = ceil_div(width, 4);
		const size_t tiles = static_cast<size_t>(batch) * tiles_h * tiles_w;
		const int vec = pick_vec(channels, x.data, matrices.data, nullptr, nullptr, sizeof(T));
		const dim3 block(256);
		const dim3 grid(grid_for(tiles * (channels / vec)));
		const T *in = ptr<const T>(x);
		T *out = ptr<T>(matrices);
		switch (vec)
		{
			case 4:
				hipLaunchKernelGGL((kernel_input_transform_4x4_3x3<T, 4>), grid, block, 0, stream, in, out, batch, height, width, channels, tiles_h, tiles_w);
				break;
			case 2:
				hipLaunchKernelGGL((kernel_input_transform_4x4_3x3<T, 2>), grid, block, 0, stream, in, out, batch, height, width, channels, tiles_h, tiles_w);
				break;
			default:
				hipLaunchKernelGGL((kernel_input_transform_4x4_3x3<T, 1>), grid, block, 0, stream, in, out, batch, height, width, channels, tiles_h, tiles_w);
				break;
		}
		MLHIP_CHECK(hipGetLastError());
	}
	template<typename T, int VEC>
	void launch_output_vec(hipStream_t stream, dim3 grid, const T *in, T *out, const T *b, const T *e, int act, int batch, int height, int width,
			int channels, int tiles_h, int tiles_w)
	{
		const dim3 block(256);
		const int mode = (act == ACTIVATION_LINEAR) ? 0 : ((act == ACTIVATION_RELU) ? 1 : 2);
#define MLHIP_LAUNCH_OUTPUT(MODE, EXT) \
		hipLaunchKernelGGL((kernel_output_transform_4x4_3x3<T, VEC, MODE, EXT>), grid, block, 0, stream, in, out, b, e, act, batch, height, width, channels, tiles_h, tiles_w)
		if (e != nullptr)
		{
			if (mode == 0)
				MLHIP_LAUNCH_OUTPUT(0, true);
			else if (mode == 1)
				MLHIP_LAUNCH_OUTPUT(1, true);
			else
				MLHIP_LAUNCH_OUTPUT(2, true);
		}
		else
		{
			if (mode == 0)
				MLHIP_LAUNCH_OUTPUT(0, false);
			else if (mode == 1)
				MLHIP_LAUNCH_OUTPUT(1, false);
			else
				MLHIP_LAUNCH_OUTPUT(2, false);
		}
#undef MLHIP_LAUNCH_OUTPUT
	}
	template<typename T>
	void launch_output(hipStream_t stream, const mlTensor_t &matrices, const mlTensor_t &bias, const mlTensor_t &ext, mlTensor_t &y, mlActivationType_t act)
	{
		const int batch = y.dim[0], height = y.dim[1], width = y.dim[2], channels = y.dim[3];
		const int tiles_h = ceil_div(height, 4), tiles_w = ceil_div(width, 4);
		const size_t tiles = static_cast<size_t>(batch) * tiles_h * tiles_w;
		const int vec = pick_vec(channels, matrices.data, y.data, bias.data, ext.data, sizeof(T));
		const dim3 grid(grid_for(tiles * (channels / vec)));
		const T *in = ptr<const T>(matrices);
		T *out = ptr<T>(y);
		const T *b = ptr<const T>(bias);
		const T *e = ptr<const T>(ext);
		const int a = static_cast<int>(act);
		switch (vec)
		{
			case 4:
				launch_output_vec<T, 4>(stream, grid, in, out, b, e, a, batch, height, width, channels, tiles_h, tiles_w);
				break;
			case 2:
				launch_output_vec<T, 2>(stream, grid, in, out, b, e, a, batch, height, width, channels, tiles_h, tiles_w);
				break;
			default:
				launch_output_vec<T, 1>(stream, grid, in, out, b, e, a, batch, height, width, channels, tiles_h, tiles_w);
				break;
		}
		MLHIP_CHECK(hipGetLastError());
	}
	/* fused output + next input transform: channels must be a multiple of 64 and 4-element accesses aligned */
	template<typename T, int SLICE, int VEC, int THREADS>
	void launch_output_input(hipStream_t stream, const mlTensor_t &matrices, const mlTensor_t &bias, const mlTensor_t &ext, const mlShape_t &shape, void *output,
			mlActivationType_t act, mlTensor_t &next)
	{
		const int batch = shape.dim[0], height = shape.dim[1], width = shape.dim[2], channels = shape.dim[3];
		const int tiles_h = ceil_div(height, 4), tiles_w = ceil_div(width, 4);
		const size_t lds = static_cast<size_t>(height * width + 1) * SLICE * sizeof(T);
		MLHIP_REQUIRE(lds <= 160 * 1024, "Winograd fused transform: image too large for LDS");
		const dim3 grid(static_cast<unsigned int>(batch) * (channels / SLICE)), block(THREADS);
		const T *in = ptr<const T>(matrices);
		T *out = reinterpret_cast<T*>(output);
		const T *b = ptr<const T>(bias);
		const T *e = ptr<const T>(ext);
		T *nxt = ptr<T>(next);
		const int a = static_cast<int>(act);
		const int mode = (act == ACTIVATION_LINEAR) ? 0 : ((act == ACTIVATION_RELU) ? 1 : 2);
#define MLHIP_LAUNCH_FUSED(MODE, EXT) \
		do { \
			auto kernel = kernel_output_input_transform_4x4_3x3<T, VEC, SLICE, MODE, EXT, THREADS>; \
			if (lds > 64 * 1024) \
				ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), static_cast<int>(lds)); \
			hipLaunchKernelGGL(kernel, grid, block, lds, stream, in, out, b, e, a, nxt, batch, height, width, channels, tiles_h, tiles_w); \
		} while (0)
		if (e != nullptr)
		{
			if (mode == 0)
				MLHIP_LAUNCH_FUSED(0, true);
			else if (mode == 1)
				MLHIP_LAUNCH_FUSED(1, true);
			else
				MLHIP_LAUNCH_FUSED(2, true);
		}
		else
		{
			if (mode == 0)
				MLHIP_LAUNCH_FUSED(0, false);
			else if (mode == 1)
				MLHIP_LAUNCH_FUSED(1, false);
			else
				MLHIP_LAUNCH_FUSED(2, false);
		}
#undef MLHIP_LAUNCH_FUSED
		MLHIP_CHECK(hipGetLastError());
	}
}

namespace
{
	/*
	 * Device memory of the whole-layer launch that the library owns for the life of the process, one copy per device: the word that
	 * counts workgroups which gave up waiting, the per-XCD counters and the product scratch (2 chunks of 36 x 64 x 256 halfs per XCD).
	 * hip_winograd_layer_forward keeps counters and scratch in the context's growable workspace; hip_winograd_layer_forward_static, for
	 * callers that must not allocate, keeps them here. The array's name is a host-side handle only: its device address is looked up
	 * once per device with hipGetSymbolAddress and only that pointer is ever handed to kernels.
	 */
	constexpr size_t LAYER_ERROR_BYTES = 256;
	constexpr size_t LAYER_SYNC_BYTES = sizeof(LayerSync) * LAYER_XCDS;
	constexpr size_t LAYER_SCRATCH_BYTES = static_cast<size_t>(LAYER_XCDS) * LAYER_BUFFERS * LAYER_CHUNK_ELEMENTS * sizeof(half_t);
	constexpr size_t LAYER_STATIC_BYTES = LAYER_ERROR_BYTES + (LAYER_SYNC_BYTES + 255) / 256 * 256 + LAYER_SCRATCH_BYTES; /* 18.1 MiB */
	static __device__ __align__(256) uint8_t layer_static_memory[LAYER_STATIC_BYTES];

	uint8_t* layer_static_pointer(int device_index)
	{
		static std::mutex guard;
		static std::map<int, uint8_t*> pointers;
		std::lock_guard<std::mutex> lock(guard);
		auto it = pointers.find(device_index);
		if (it == pointers.end())
		{
			MLHIP_CHECK(hipSetDevice(device_index)); /* every device holds its own copy of the array, at its own address */
			void *address = nullptr;
			MLHIP_CHECK(hipGetSymbolAddress(&address, HIP_SYMBOL(layer_static_memory)));
			MLHIP_REQUIRE(address != nullptr, "Winograd layer: no device address for the library's static memory");
			it = pointers.insert(std::make_pair(device_index, reinterpret_cast<uint8_t*>(address))).first;
		}
		return it->second;
	}
	/* device word that counts workgroups of the whole-layer kernel that gave up waiting (zero when the module is loaded) */
	unsigned int* layer_error_word(int device_index)
	{
		return reinterpret_cast<unsigned int*>(layer_static_pointer(device_index));
	}
	/* clears `words` 32-bit words; a kernel rather than a memset node, so that callers may capture the launch sequence into a graph */
	__global__ void kernel_clear_words(unsigned int *dst, unsigned int words)
	{
		for (unsigned int i = blockIdx.x * blockDim.x + threadIdx.x; i < words; i += gridDim.x * blockDim.x)
			dst[i] = 0u;
	}
	/* the shapes the one-launch kernel is written for, the upper limit of the batch (layer_batch_fits) apart */
	bool layer_kernel_shape(const mlTensor_t &input_matrices, const mlTensor_t &weight_matrices, const mlShape_t &shape, const mlTensor_t &bias,
			const mlTensor_t &ext, const void *output, mlActivationType_t act)
	{
		const auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) % 16) == 0; };
		return input_matrices.dtype == DTYPE_FLOAT16 && shape.dim[3] == LAYER_CHANNELS && input_matrices.dim[2] == LAYER_CHANNELS
				&& weight_matrices.dim[1] == LAYER_CHANNELS && weight_matrices.dim[2] == LAYER_CHANNELS
				&& ceil_div(shape.dim[1], 4) * ceil_div(shape.dim[2], 4) == 16 && shape.dim[0] % 4 == 0 && shape.dim[0] >= 4 * LAYER_XCDS
				&& (act == ACTIVATION_LINEAR || act == ACTIVATION_RELU)
				&& aligned16(input_matrices.data) && aligned16(weight_matrices.data) && aligned16(bias.data) && aligned16(ext.data) && aligned16(output)
				&& device_compute_units() == 256;
	}
	/* the per-XCD counters (in the workspace or in the static array) cover this many images per launch */
	bool layer_batch_fits(const mlShape_t &shape)
	{
		return shape.dim[0] <= 4 * LAYER_XCDS * LAYER_MAX_CHUNKS;
	}
	void launch_layer(mlContext_t context, const mlTensor_t &input_matrices, const mlTensor_t &weight_matrices, const mlTensor_t &bias, const mlTensor_t &ext,
			const mlShape_t &shape, void *output, mlActivationType_t act, mlTensor_t &next, bool static_memory)
	{
		const hipStream_t stream = stream_of(context);
		const int device_index = get(context)->device_index;
		const size_t sync_bytes = (LAYER_SYNC_BYTES + 255) / 256 * 256;
		uint8_t *block = static_memory ? layer_static_pointer(device_index) + LAYER_ERROR_BYTES
				: reinterpret_cast<uint8_t*>(get_workspace(context, sync_bytes + LAYER_SCRATCH_BYTES));
		LayerSync *sync = reinterpret_cast<LayerSync*>(block);
		half_t *scratch = reinterpret_cast<half_t*>(block + sync_bytes);
		unsigned int *errors = layer_error_word(device_index);
		/* the counters start every launch at zero; the scratch needs no clearing (every row is written before it is read) */
		hipLaunchKernelGGL(kernel_clear_words, dim3(32), dim3(256), 0, stream, reinterpret_cast<unsigned int*>(sync),
				static_cast<unsigned int>(LAYER_SYNC_BYTES / sizeof(unsigned int)));
		const int lds = 65536;
		const dim3 grid(LAYER_XCDS * LAYER_WORKGROUPS_PER_XCD), block_dim(256);
		const unsigned int spin_limit = 1u << 17; /* about a tenth of a second per wait before a workgroup gives up */
#define MLHIP_LAUNCH_LAYER(ACT, EXT) \
		do { \
			auto kernel = kernel_winograd_layer_f16<ACT, EXT>; \
			ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), lds); \
			hipLaunchKernelGGL(kernel, grid, block_dim, lds, stream, ptr<const half_t>(input_matrices), ptr<const half_t>(weight_matrices), \
					ptr<const half_t>(bias), ptr<const half_t>(ext), reinterpret_cast<half_t*>(output), ptr<half_t>(next), scratch, sync, errors, shape.dim[0], \
					shape.dim[1], shape.dim[2], ceil_div(shape.dim[1], 4), ceil_div(shape.dim[2], 4), static_cast<int>(act), spin_limit); \
		} while (0)
		const bool relu = (act == ACTIVATION_RELU);
		if (ext.data != nullptr)
		{
			if (relu)
				MLHIP_LAUNCH_LAYER(1, true);
			else
				MLHIP_LAUNCH_LAYER(0, true);
		}
		else
		{
			if (relu)
				MLHIP_LAUNCH_LAYER(1, false);
			else
				MLHIP_LAUNCH_LAYER(0, false);
		}
#undef MLHIP_LAUNCH_LAYER
		MLHIP_CHECK(hipGetLastError());
	}
}

namespace mlhip
{
	void prepare_static_memory(int device_index)
	{
		(void) layer_static_pointer(device_index);
	}
}

extern "C"
{
	using namespace mlhip;

	void hip_winograd_weight_transform(mlContext_t context, int tile_size, const mlTensor_t w, mlTensor_t matrices, bool invert)
	try
	{
		MLHIP_REQUIRE(w.rank == 4 && w.dim[1] == w.dim[2], "Winograd weights must be [Cout, k, k, Cin] with a square kernel");
		require_supported(tile_size, matrices, w.dtype);
		MLHIP_REQUIRE(w.dim[1] == 3, "Winograd weight transform: weight kernel size does not match the matrices");
		MLHIP_REQUIRE(matrices.dtype == w.dtype, "Winograd weight transform: dtype mismatch");
		MLHIP_REQUIRE(matrices.dim[1] == w.dim[0] && matrices.dim[2] == w.dim[3], "Winograd weight transform: matrices must be [36, Cout, Cin]");
		MLHIP_REQUIRE(w.data != nullptr && matrices.data != nullptr, "Winograd weight transform: null tensor");

		const size_t threads = static_cast<size_t>(w.dim[0]) * w.dim[3];
		if (threads == 0)
			return;
		const dim3 block(256);
		const dim3 grid(grid_for(threads));
		if (w.dtype == DTYPE_FLOAT16)
			hipLaunchKernelGGL(kernel_weight_transform_4x4_3x3<half_t>, grid, block, 0, stream_of(context), ptr<const half_t>(w), ptr<half_t>(matrices), w.dim[0],
					w.dim[3], invert);
		else
			hipLaunchKernelGGL(kernel_weight_transform_4x4_3x3<float>, grid, block, 0, stream_of(context), ptr<const float>(w), ptr<float>(matrices), w.dim[0],
					w.dim[3], invert);
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_winograd_input_transform(mlContext_t context, int tile_size, const mlTensor_t x, mlTensor_t matrices)
	try
	{
		MLHIP_REQUIRE(x.rank == 4, "Winograd input transform: input must be [B, H, W, C]");
		require_supported(tile_size, matrices, x.dtype);
		MLHIP_REQUIRE(matrices.dtype == x.dtype, "Winograd input transform: dtype mismatch");
		const size_t tiles = static_cast<size_t>(x.dim[0]) * ceil_div(x.dim[1], 4) * ceil_div(x.dim[2], 4);
		MLHIP_REQUIRE(static_cast<size_t>(matrices.dim[1]) == tiles && matrices.dim[2] == x.dim[3],
				"Winograd input transform: matrices must be [36, B*ceil(H/4)*ceil(W/4), C]");
		if (tiles == 0 || x.dim[3] == 0)
			return;
		MLHIP_REQUIRE(volume(x) <= 0xffffffffu && tiles * x.dim[3] <= 0xffffffffu, "Winograd input transform: tensor too large for 32-bit element offsets");
		MLHIP_REQUIRE(x.data != nullptr && matrices.data != nullptr, "Winograd input transform: null tensor");
		mlTensor_t m = matrices;
		if (x.dtype == DTYPE_FLOAT16)
			launch_input<half_t>(stream_of(context), x, m);
		else
			launch_input<float>(stream_of(context), x, m);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_winograd_output_transform(mlContext_t context, int tile_size, const mlTensor_t matrices, const mlTensor_t bias, const mlTensor_t ext,
			mlTensor_t y, mlActivationType_t act)
	try
	{
		MLHIP_REQUIRE(y.rank == 4, "Winograd output transform: output must be [B, H, W, C]");
		require_supported(tile_size, matrices, y.dtype);
		MLHIP_REQUIRE(matrices.dtype == y.dtype, "Winograd output transform: dtype mismatch");
		const size_t tiles = static_cast<size_t>(y.dim[0]) * ceil_div(y.dim[1], 4) * ceil_div(y.dim[2], 4);
		MLHIP_REQUIRE(static_cast<size_t>(matrices.dim[1]) == tiles && matrices.dim[2] == y.dim[3],
				"Winograd output transform: matrices must be [36, B*ceil(H/4)*ceil(W/4), C]");
		if (bias.data != nullptr)
			MLHIP_REQUIRE(bias.dtype == y.dtype && volume(bias) == static_cast<size_t>(y.dim[3]), "Winograd output transform: bias must be [C] of the output dtype");
		if (ext.data != nullptr)
			MLHIP_REQUIRE(ext.dtype == y.dtype && volume(ext) == volume(y), "Winograd output transform: ext must have the output's shape and dtype");
		if (tiles == 0 || y.dim[3] == 0)
			return;
		MLHIP_REQUIRE(volume(y) <= 0xffffffffu && tiles * y.dim[3] <= 0xffffffffu, "Winograd output transform: tensor too large for 32-bit element offsets");
		MLHIP_REQUIRE(y.data != nullptr && matrices.data != nullptr, "Winograd output transform: null tensor");
		mlTensor_t out = y;
		if (y.dtype == DTYPE_FLOAT16)
			launch_output<half_t>(stream_of(context), matrices, bias, ext, out, act);
		else
			launch_output<float>(stream_of(context), matrices, bias, ext, out, act);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_winograd_output_input_transform(mlContext_t context, int tile_size, const mlTensor_t matrices, const mlTensor_t bias, const mlTensor_t ext,
			mlShape_t output_shape, void *output, mlActivationType_t act, mlTensor_t next_matrices)
	try
	{
		MLHIP_REQUIRE(output_shape.rank == 4, "Winograd fused transform: output shape must be [B, H, W, C]");
		require_supported(tile_size, matrices, matrices.dtype);
		require_supported(tile_size, next_matrices, matrices.dtype);
		MLHIP_REQUIRE(next_matrices.dtype == matrices.dtype, "Winograd fused transform: dtype mismatch");
		const int channels = output_shape.dim[3];
		const size_t tiles = static_cast<size_t>(output_shape.dim[0]) * ceil_div(output_shape.dim[1], 4) * ceil_div(output_shape.dim[2], 4);
		MLHIP_REQUIRE(static_cast<size_t>(matrices.dim[1]) == tiles && matrices.dim[2] == channels && static_cast<size_t>(next_matrices.dim[1]) == tiles
				&& next_matrices.dim[2] == channels, "Winograd fused transform: both sets of matrices must be [36, B*ceil(H/4)*ceil(W/4), C]");
		if (bias.data != nullptr)
			MLHIP_REQUIRE(bias.dtype == matrices.dtype && volume(bias) == static_cast<size_t>(channels), "Winograd fused transform: bias must be [C] of the output dtype");
		if (ext.data != nullptr)
			MLHIP_REQUIRE(ext.dtype == matrices.dtype && volume(ext) == volume(output_shape), "Winograd fused transform: ext must have the output's shape and dtype");
		if (tiles == 0 || channels == 0)
			return;
		MLHIP_REQUIRE(volume(output_shape) <= 0xffffffffu && tiles * channels <= 0xffffffffu, "Winograd fused transform: tensor too large for 32-bit element offsets");
		MLHIP_REQUIRE(matrices.data != nullptr && next_matrices.data != nullptr, "Winograd fused transform: null tensor");
		const int esize = size_of(matrices.dtype);
		const bool fusable = (channels % 64 == 0) && pick_vec(channels, matrices.data, next_matrices.data, bias.data, ext.data, esize) == 4
				&& pick_vec(channels, output, nullptr, nullptr, nullptr, esize) == 4
				&& static_cast<size_t>(output_shape.dim[1] * output_shape.dim[2] + 1) * 64 * esize <= 160 * 1024;
		if (!fusable)
		{ /* shapes the fused kernel does not take: the two stand-alone transforms, which need y in memory */
			MLHIP_REQUIRE(output != nullptr, "Winograd fused transform: this shape needs the output tensor as intermediate storage");
			mlTensor_t y = make_tensor(output, matrices.dtype, output_shape);
			mlhip::NestedEntryCalls nested;
			hip_winograd_output_transform(context, tile_size, matrices, bias, ext, y, act);
			hip_winograd_input_transform(context, tile_size, y, next_matrices);
			return;
		}
		mlTensor_t next = next_matrices;
		/* 64-channel slices, 256 threads, two workgroups per CU. Measured alternatives that were not faster: slices of 128 or 256 channels
		 * (longer contiguous segments) with 512 or 1024 threads, and 2-element vectors at twice the occupancy. */
		if (matrices.dtype == DTYPE_FLOAT16)
			launch_output_input<half_t, 64, 4, 256>(stream_of(context), matrices, bias, ext, output_shape, output, act, next);
		else
			launch_output_input<float, 64, 4, 256>(stream_of(context), matrices, bias, ext, output_shape, output, act, next);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	static void winograd_layer_forward(mlContext_t context, int tile_size, const mlTensor_t &input_matrices, const mlTensor_t &weight_matrices,
			mlTensor_t &output_matrices, const mlTensor_t &bias, const mlTensor_t &ext, const mlShape_t &output_shape, void *output, mlActivationType_t act,
			mlTensor_t &next_matrices, bool static_memory)
	{
		MLHIP_REQUIRE(output_shape.rank == 4, "Winograd layer: output shape must be [B, H, W, C]");
		require_supported(tile_size, input_matrices, input_matrices.dtype);
		require_supported(tile_size, next_matrices, input_matrices.dtype);
		MLHIP_REQUIRE(weight_matrices.rank == 3 && weight_matrices.dim[0] == 36 && weight_matrices.dtype == input_matrices.dtype
				&& next_matrices.dtype == input_matrices.dtype, "Winograd layer: weight matrices must be [36, Cout, Cin] of the input's data type");
		const size_t tiles = static_cast<size_t>(output_shape.dim[0]) * ceil_div(output_shape.dim[1], 4) * ceil_div(output_shape.dim[2], 4);
		MLHIP_REQUIRE(static_cast<size_t>(input_matrices.dim[1]) == tiles && input_matrices.dim[2] == weight_matrices.dim[2]
				&& weight_matrices.dim[1] == output_shape.dim[3] && static_cast<size_t>(next_matrices.dim[1]) == tiles
				&& next_matrices.dim[2] == output_shape.dim[3], "Winograd layer: matrices must be [36, tiles, Cin], [36, Cout, Cin] and [36, tiles, Cout]");
		if (tiles == 0 || output_shape.dim[3] == 0)
			return;
		MLHIP_REQUIRE(input_matrices.data != nullptr && weight_matrices.data != nullptr && next_matrices.data != nullptr, "Winograd layer: null tensor");
		if (bias.data != nullptr)
			MLHIP_REQUIRE(bias.dtype == input_matrices.dtype && volume(bias) == static_cast<size_t>(output_shape.dim[3]), "Winograd layer: bias must be [Cout]");
		if (ext.data != nullptr)
			MLHIP_REQUIRE(ext.dtype == input_matrices.dtype && volume(ext) == volume(output_shape), "Winograd layer: ext must have the output's shape and dtype");
		if (layer_kernel_shape(input_matrices, weight_matrices, output_shape, bias, ext, output, act))
		{
			if (layer_batch_fits(output_shape))
			{
				mlTensor_t next = next_matrices;
				launch_layer(context, input_matrices, weight_matrices, bias, ext, output_shape, output, act, next, static_memory);
				return;
			}
			/* the one shape whose launch uses the library's static memory: a batch beyond what that memory covers is refused, not rerouted */
			MLHIP_REQUIRE(!static_memory, "Winograd layer (static memory): at most 4096 images per call fit the library's static counters; split the batch");
		}
		/* every other shape: the batched product into the caller's matrices, then the fused (or two-step) transform; neither uses
		 * library-side memory, so the static entry point takes these shapes at any batch size */
		MLHIP_REQUIRE(output_matrices.data != nullptr && output_matrices.dtype == input_matrices.dtype && output_matrices.rank == 3
				&& output_matrices.dim[0] == 36 && static_cast<size_t>(output_matrices.dim[1]) == tiles && output_matrices.dim[2] == output_shape.dim[3],
				"Winograd layer: this shape needs output matrices [36, tiles, Cout] as intermediate storage");
		mlhip::NestedEntryCalls nested;
		hip_gemm_batched(context, input_matrices.dtype, shape_of(output_matrices), output_matrices.data, shape_of(input_matrices), input_matrices.data,
				shape_of(weight_matrices), weight_matrices.data, 'n', 't', 1.0f, 0.0f);
		hip_winograd_output_input_transform(context, tile_size, output_matrices, bias, ext, output_shape, output, act, next_matrices);
	}
	void hip_winograd_layer_forward(mlContext_t context, int tile_size, const mlTensor_t input_matrices, const mlTensor_t weight_matrices,
			mlTensor_t output_matrices, const mlTensor_t bias, const mlTensor_t ext, mlShape_t output_shape, void *output, mlActivationType_t act,
			mlTensor_t next_matrices)
	try
	{
		winograd_layer_forward(context, tile_size, input_matrices, weight_matrices, output_matrices, bias, ext, output_shape, output, act, next_matrices,
				false);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_winograd_layer_forward_static(mlContext_t context, int tile_size, const mlTensor_t input_matrices, const mlTensor_t weight_matrices,
			mlTensor_t output_matrices, const mlTensor_t bias, const mlTensor_t ext, mlShape_t output_shape, void *output, mlActivationType_t act,
			mlTensor_t next_matrices)
	try
	{
		winograd_layer_forward(context, tile_size, input_matrices, weight_matrices, output_matrices, bias, ext, output_shape, output, act, next_matrices,
				true);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	int hip_winograd_layer_errors(mlContext_t context)
	try
	{
		MLHIP_CHECK(hipStreamSynchronize(stream_of(context)));
		unsigned int *word = layer_error_word(get(context)->device_index);
		unsigned int count = 0;
		MLHIP_CHECK(hipMemcpy(&count, word, sizeof(count), hipMemcpyDeviceToHost));
		if (count != 0)
			MLHIP_CHECK(hipMemset(word, 0, sizeof(count)));
		return static_cast<int>(count);
	}
	catch (...)
	{
		return mlhip::entry_failed<int>();
	}
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(winograd_weight_transform)
MLHIP_ALSO_AS_CUDA(winograd_input_transform)
MLHIP_ALSO_AS_CUDA(winograd_output_transform)
