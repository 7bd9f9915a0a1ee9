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
				out.store(dst + static_cast<size_t>(row * 6 + col) * matrix_stride);
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

		const unsigned int block = xcd_contiguous_block_id(blockIdx.x, gridDim.x);
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
				raw[row][col] = *reinterpret_cast<const raw_t*>(src + static_cast<size_t>(row * 6 + col) * matrix_stride);

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
					residual[row][col] = *reinterpret_cast<const raw_t*>(ext + offset[row][col]);
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
					out.store(output + offset[row][col]);
			}
		}
	}

	/*
	 * Output transform of one layer fused with the input transform of the next 3x3 layer:
	 *   matrices [36][tiles][C] (+ bias, + ext) -> y [B][H][W][C] (written only if `output` is given) -> next_matrices [36][tiles][C]
	 * One workgroup owns one image and a slice of SLICE channels: its 256 threads are 256 / (SLICE / VEC) tile lanes x SLICE / VEC
	 * channel lanes. Phase 1 runs the output transform of the image's tiles (same arithmetic and epilogue as the stand-alone kernel) and
	 * leaves y, rounded to the storage type as the stand-alone kernel would store it, in LDS; phase 2 reads the 6x6 windows back
	 * (zero outside the image) and runs the input transform. Results are bit-identical to the two separate calls; what is saved is
	 * the write and re-read of y through HBM (or only the re-read, when y is also needed as a later residual).
	 */
	template<typename T, int VEC, int SLICE, int ACT, bool HAS_EXT, int THREADS>
	__global__ __launch_bounds__(THREADS, ((VEC <= 2) ? 1024 : 512) / THREADS) void kernel_output_input_transform_4x4_3x3(const T *__restrict__ matrices, T *output, const T *__restrict__ bias,
			const T *ext, int act, T *__restrict__ next_matrices, int batch_size, int height, int width, int channels, int tiles_h, int tiles_w)
	{
		typedef typename RawVec<T, VEC>::type raw_t;
		constexpr int CHANNEL_LANES = SLICE / VEC;
		constexpr int TILE_LANES = THREADS / CHANNEL_LANES;
		extern __shared__ __attribute__((aligned(16))) uint8_t lds_bytes[];
		T *image = reinterpret_cast<T*>(lds_bytes); /* [height * width + 1][SLICE]; the extra last pixel stays zero */

		const unsigned int slices = channels / SLICE;
		const unsigned int batch = blockIdx.x / slices;
		const unsigned int slice = blockIdx.x - batch * slices;
		const int channel_local = (threadIdx.x % CHANNEL_LANES) * VEC;
		const unsigned int channel = slice * SLICE + channel_local;
		const int tile_lane = threadIdx.x / CHANNEL_LANES;
		const unsigned int tiles_per_image = tiles_h * tiles_w;
		const unsigned int nb_of_tiles = batch_size * tiles_per_image;
		const size_t matrix_stride = static_cast<size_t>(nb_of_tiles) * channels;
		const int zero_pixel = height * width;

		if (tile_lane == 0)
		{
			Vec<T, VEC> z;
			z.zero();
			z.store(image + zero_pixel * SLICE + channel_local);
		}
		Vec<T, VEC> b;
		if (bias != nullptr)
			b.load(bias + channel);
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
			const uint8_t *ext_slice = reinterpret_cast<const uint8_t*>(ext + static_cast<size_t>(batch) * zero_pixel * channels + slice * SLICE);
			const int lane = threadIdx.x & 63;
			for (int base = (threadIdx.x >> 6) * 64; base < total_chunks; base += THREADS)
			{
				const int chunk = base + lane;
				if (chunk < total_chunks)
				{
					const int px = chunk / CHUNKS_PER_PIXEL;
					const int part = chunk - px * CHUNKS_PER_PIXEL;
					__builtin_amdgcn_global_load_lds((global_ptr_t) (ext_slice + static_cast<size_t>(px) * channels * sizeof(T) + part * 16),
							(lds_ptr_t) (lds_bytes + base * 16), 16, 0, 0);
				}
			}
		}

		/* ---- phase 1: output transform into LDS (and to `output`) ---- */
		const unsigned int image_base = batch * height * width;
		raw_t raw[6][6];
		auto load_matrices = [&](unsigned int in_image) __attribute__((always_inline))
		{
			const T *src = matrices + static_cast<size_t>(batch * tiles_per_image + in_image) * channels + channel;
#pragma unroll
			for (int row = 0; row < 6; row++)
#pragma unroll
				for (int col = 0; col < 6; col++)
					raw[row][col] = *reinterpret_cast<const raw_t*>(src + static_cast<size_t>(row * 6 + col) * matrix_stride);
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
						{
							if constexpr (sizeof(T) == 2)
								t = half_bits_to_float(half_bits_rtz(t));
							t = activate(act, t);
						}
						out.v[c] = t;
					}
					if ((x0 + row) < height && (y0 + col) < width)
					{
						out.store(in_lds);
						if (output != nullptr)
							out.store(output + (image_base + pixel[row][col]) * channels + channel);
					}
				}
			}
			in_image += TILE_LANES;
		}
		__syncthreads();

		/* ---- phase 2: input transform of the next layer out of LDS ---- */
#pragma clang loop unroll(disable)
		for (unsigned int in_image = tile_lane; in_image < tiles_per_image; in_image += TILE_LANES)
		{
			const unsigned int tile_idx = batch * tiles_per_image + in_image;
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
			T *dst = next_matrices + static_cast<size_t>(tile_idx) * channels + channel;
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
					out.store(dst + static_cast<size_t>(row * 6 + col) * matrix_stride);
				}
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

extern "C"
{
	using namespace mlhip;

	void hip_winograd_weight_transform(mlContext_t context, int tile_size, const mlTensor_t w, mlTensor_t matrices, bool invert)
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
	void hip_winograd_input_transform(mlContext_t context, int tile_size, const mlTensor_t x, mlTensor_t matrices)
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
	void hip_winograd_output_transform(mlContext_t context, int tile_size, const mlTensor_t matrices, const mlTensor_t bias, const mlTensor_t ext,
			mlTensor_t y, mlActivationType_t act)
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
	void hip_winograd_output_input_transform(mlContext_t context, int tile_size, const mlTensor_t matrices, const mlTensor_t bias, const mlTensor_t ext,
			mlShape_t output_shape, void *output, mlActivationType_t act, mlTensor_t next_matrices)
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
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(winograd_weight_transform)
MLHIP_ALSO_AS_CUDA(winograd_input_transform)
MLHIP_ALSO_AS_CUDA(winograd_output_transform)
