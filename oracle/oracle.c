/*
 * oracle.c — CPU restatement of minml's convolution / GEMM inference arithmetic. TEST INFRASTRUCTURE ONLY (see oracle.h):
 * the HIP backend never calls into this file; tests, the smoke check and the benchmark's CPU-baseline leg do.
 *
 * Built with -ffp-contract=off: a fused multiply-add appears only where it is written as fmaf(), which is where the reference's
 * SIMD kernels use one. Reference file:line citations are relative to the reference checkout.
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;

void oracle_set_num_threads(int threads)
{
	g_threads = (threads < 1) ? 1 : threads;
}

/* ------------------------------------------------------------------------------------------------------------------------
 * fp16 <-> fp32: src/backend/cpu/fp16.hpp:61-78 with the tables of src/backend/cpu/fp16.cpp:32-153 written out as arithmetic.
 * Narrowing keeps the leading mantissa bits (round toward zero); magnitudes >= 2^16 become infinity, < 2^-24 become zero.
 * ---------------------------------------------------------------------------------------------------------------------- */
uint16_t oracle_fp32_to_fp16(float x)
{
	uint32_t bits;
	memcpy(&bits, &x, 4);
	const uint32_t sign = (bits >> 16) & 0x8000u;
	const int e = (int) ((bits >> 23) & 0xffu) - 127;
	const uint32_t mant = bits & 0x007fffffu;
	uint32_t base, shift;
	if (e < -24)
	{
		base = 0;
		shift = 24;
	}
	else if (e < -14)
	{
		base = 0x0400u >> (-e - 14);
		shift = (uint32_t) (-e - 1);
	}
	else if (e <= 15)
	{
		base = (uint32_t) (e + 15) << 10;
		shift = 13;
	}
	else if (e < 128)
	{
		base = 0x7c00u;
		shift = 24;
	}
	else
	{ /* inf / nan */
		base = 0x7c00u;
		shift = 13;
	}
	return (uint16_t) (sign | (base + (mant >> shift)));
}
float oracle_fp16_to_fp32(uint16_t h)
{
	const uint32_t sign = ((uint32_t) h & 0x8000u) << 16;
	const uint32_t exp = (h >> 10) & 0x1fu;
	uint32_t mant = h & 0x03ffu;
	uint32_t bits;
	if (exp == 0)
	{
		if (mant == 0)
			bits = sign;
		else
		{ /* subnormal half: normalise */
			int e = -1;
			do
			{
				e++;
				mant <<= 1;
			} while ((mant & 0x0400u) == 0);
			bits = sign | ((uint32_t) (127 - 15 - e) << 23) | ((mant & 0x03ffu) << 13);
		}
	}
	else if (exp == 31)
		bits = sign | 0x7f800000u | (mant << 13);
	else
		bits = sign | ((exp + 112u) << 23) | (mant << 13);
	float result;
	memcpy(&result, &bits, 4);
	return result;
}
void oracle_convert_fp32_to_fp16(const float *src, uint16_t *dst, size_t elements)
{
	for (size_t i = 0; i < elements; i++)
		dst[i] = oracle_fp32_to_fp16(src[i]);
}
void oracle_convert_fp16_to_fp32(const uint16_t *src, float *dst, size_t elements)
{
	for (size_t i = 0; i < elements; i++)
		dst[i] = oracle_fp16_to_fp32(src[i]);
}

static inline float load_as_float(const void *base, size_t index, int dtype)
{
	if (dtype == ORACLE_FLOAT16)
		return oracle_fp16_to_fp32(((const uint16_t*) base)[index]);
	return ((const float*) base)[index];
}
static inline void store_from_float(void *base, size_t index, int dtype, float x)
{
	if (dtype == ORACLE_FLOAT16)
		((uint16_t*) base)[index] = oracle_fp32_to_fp16(x);
	else
		((float*) base)[index] = x;
}
static inline float round_to_dtype(float x, int dtype)
{
	return (dtype == ORACLE_FLOAT16) ? oracle_fp16_to_fp32(oracle_fp32_to_fp16(x)) : x;
}
static inline size_t dtype_size(int dtype)
{
	return (dtype == ORACLE_FLOAT16) ? 2 : 4;
}

/* src/backend/cpu/common_math.hpp:40-55, def_misc_kernels.cpp:52-72 */
static inline float activation(int act, float x)
{
	switch (act)
	{
		default:
		case 0:
			return x;
		case 1:
			return 1.0f / (1.0f + expf(-x));
		case 2:
			return tanhf(x);
		case 3:
			return (x > 0.0f) ? x : 0.0f;
		case 4:
			return (x > 0.0f) ? x : 0.1f * x;
		case 5:
			return expf(x);
	}
}

/* ------------------------------------------------------------------------------------------------------------------------
 * Winograd F(4x4, 3x3)
 * ---------------------------------------------------------------------------------------------------------------------- */
/* def_winograd_kernels.cpp:165-184 — constants rounded to float, plain multiplies and adds, evaluated left to right */
static void weight_line(const float g[3], float w[6])
{
	const float c13 = (float) (1.0 / 3.0);
	const float c23 = (float) (2.0 / 3.0);
	const float c43 = (float) (4.0 / 3.0);
	const float c2 = 2.0f;
	w[0] = g[0];
	w[1] = c23 * ((g[0] + g[1]) + g[2]);
	w[2] = c23 * ((g[0] - g[1]) + g[2]);
	w[3] = (c13 * g[0] + c23 * g[1]) + c43 * g[2];
	w[4] = (c13 * g[0] - c23 * g[1]) + c43 * g[2];
	w[5] = c2 * g[2];
}
/* avx2_winograd_kernels.cpp:241-264 — two differences / sums, then one fused multiply-add */
static void input_line(const float l[6], float r[6])
{
	r[0] = fmaf(0.25f, l[4] - l[2], l[0] - l[2]);
	r[1] = fmaf(-0.25f, l[3] + l[4], l[1] + l[2]);
	r[2] = fmaf(0.25f, l[3] - l[4], l[2] - l[1]);
	r[3] = fmaf(0.5f, l[4] - l[2], l[3] - l[1]);
	r[4] = fmaf(0.5f, l[4] - l[2], l[1] - l[3]);
	r[5] = fmaf(0.25f, l[5] - l[3], l[1] - l[3]);
}
/* avx2_winograd_kernels.cpp:266-279 */
static void output_line(const float l[6], float o[4])
{
	const float s = l[1] + l[2];
	const float d = l[1] - l[2];
	const float p = l[3] + l[4];
	const float q = l[3] - l[4];
	o[0] = fmaf(0.25f, p, l[0] + s);
	o[1] = fmaf(0.5f, q, d);
	o[2] = s + p;
	o[3] = fmaf(2.0f, q, fmaf(2.0f, l[5], d));
}

void oracle_winograd_weight_transform(int dtype, int filters_out, int filters_in, const void *weights, void *matrices, int invert)
{
	/* winograd_runtime.cpp:78-91: matrix i of output filter `out` at [i][out][:]; invert = 180 degree rotation of the 3x3 kernel */
#pragma omp parallel for num_threads(g_threads)
	for (int out = 0; out < filters_out; out++)
		for (int in = 0; in < filters_in; in++)
		{
			float tile[3][3], tmp[6][3];
			for (int i = 0; i < 3; i++)
				for (int j = 0; j < 3; j++)
				{
					const int x = invert ? (2 - i) : i;
					const int y = invert ? (2 - j) : j;
					tile[i][j] = load_as_float(weights, (((size_t) out * 3 + x) * 3 + y) * filters_in + in, dtype);
				}
			/* def_winograd_kernels.cpp:393-402: columns first ... */
			for (int col = 0; col < 3; col++)
			{
				const float g[3] = { tile[0][col], tile[1][col], tile[2][col] };
				float w[6];
				weight_line(g, w);
				for (int row = 0; row < 6; row++)
					tmp[row][col] = w[row];
			}
			/* ... :404-422 then rows */
			for (int row = 0; row < 6; row++)
			{
				float w[6];
				weight_line(tmp[row], w);
				for (int col = 0; col < 6; col++)
					store_from_float(matrices, ((size_t) (row * 6 + col) * filters_out + out) * filters_in + in, dtype, w[col]);
			}
		}
}

void oracle_winograd_input_transform(int dtype, int batch, int height, int width, int filters, const void *input, void *matrices)
{
	/* winograd_runtime.cpp:103-111: padding 1, tiles = ceil(H/4) x ceil(W/4), tile index = batch-major, then tile row, then tile column */
	const int tiles_h = (height + 3) / 4, tiles_w = (width + 3) / 4;
	const int tiles_per_image = tiles_h * tiles_w;
	const size_t nb_of_tiles = (size_t) batch * tiles_per_image;
#pragma omp parallel for num_threads(g_threads)
	for (size_t tile_idx = 0; tile_idx < nb_of_tiles; tile_idx++)
	{
		const int b = (int) (tile_idx / tiles_per_image);
		const int tile_x = (int) (tile_idx % tiles_per_image) / tiles_w;
		const int tile_y = (int) (tile_idx % tiles_per_image) % tiles_w;
		for (int f = 0; f < filters; f++)
		{
			float tile[6][6], tmp[6][6];
			for (int i = 0; i < 6; i++)
				for (int j = 0; j < 6; j++)
				{ /* :141-150 out-of-image elements read a line of zeros */
					const int x = 4 * tile_x + i - 1, y = 4 * tile_y + j - 1;
					tile[i][j] = (x >= 0 && x < height && y >= 0 && y < width) ?
							load_as_float(input, (((size_t) b * height + x) * width + y) * filters + f, dtype) : 0.0f;
				}
			for (int col = 0; col < 6; col++)
			{
				const float l[6] = { tile[0][col], tile[1][col], tile[2][col], tile[3][col], tile[4][col], tile[5][col] };
				float r[6];
				input_line(l, r);
				for (int row = 0; row < 6; row++)
					tmp[row][col] = r[row];
			}
			for (int row = 0; row < 6; row++)
			{
				float r[6];
				input_line(tmp[row], r);
				for (int col = 0; col < 6; col++)
					store_from_float(matrices, ((size_t) (row * 6 + col) * nb_of_tiles + tile_idx) * filters + f, dtype, r[col]);
			}
		}
	}
}

void oracle_winograd_output_transform(int dtype, int batch, int height, int width, int filters, const void *matrices, void *output, const void *bias,
		const void *ext, int act)
{
	const int tiles_h = (height + 3) / 4, tiles_w = (width + 3) / 4;
	const int tiles_per_image = tiles_h * tiles_w;
	const size_t nb_of_tiles = (size_t) batch * tiles_per_image;
#pragma omp parallel for num_threads(g_threads)
	for (size_t tile_idx = 0; tile_idx < nb_of_tiles; tile_idx++)
	{
		const int b = (int) (tile_idx / tiles_per_image);
		const int tile_x = (int) (tile_idx % tiles_per_image) / tiles_w;
		const int tile_y = (int) (tile_idx % tiles_per_image) % tiles_w;
		for (int f = 0; f < filters; f++)
		{
			float tile[6][6], tmp[4][6];
			for (int i = 0; i < 36; i++)
				tile[i / 6][i % 6] = load_as_float(matrices, ((size_t) i * nb_of_tiles + tile_idx) * filters + f, dtype);
			for (int col = 0; col < 6; col++)
			{
				const float l[6] = { tile[0][col], tile[1][col], tile[2][col], tile[3][col], tile[4][col], tile[5][col] };
				float o[4];
				output_line(l, o);
				for (int row = 0; row < 4; row++)
					tmp[row][col] = o[row];
			}
			const float bias_value = (bias != NULL) ? load_as_float(bias, f, dtype) : 0.0f;
			for (int row = 0; row < 4; row++)
			{
				float o[4];
				output_line(tmp[row], o);
				for (int col = 0; col < 4; col++)
				{
					const int x = 4 * tile_x + row, y = 4 * tile_y + col;
					if (x < height && y < width) /* winograd_runtime.cpp:209-224: outputs outside the image are dropped */
					{
						const size_t offset = (((size_t) b * height + x) * width + y) * filters + f;
						float value = o[col] + bias_value; /* avx2_winograd_kernels.cpp:611-622: + bias, + ext, ReLU */
						if (ext != NULL)
							value = value + load_as_float(ext, offset, dtype);
						if (act == 3)
							value = (value > 0.0f) ? value : 0.0f;
						else if (act != 0) /* winograd_runtime.cpp:532-535: other activations run over the stored tensor */
							value = activation(act, round_to_dtype(value, dtype));
						store_from_float(output, offset, dtype, value);
					}
				}
			}
		}
	}
}

/* ------------------------------------------------------------------------------------------------------------------------
 * GEMM
 * ---------------------------------------------------------------------------------------------------------------------- */
static void gemm_single(int dtype, int ta, int tb, int M, int N, int K, float alpha, const void *A, const void *B, float beta, const void *C,
		void *D, const void *bias, int act, int k_tile)
{
	if (k_tile <= 0 || k_tile > K)
		k_tile = (K > 0) ? K : 1;
	/* operands widened to fp32 once, B as [K][N] so that the inner loop runs over n (gemm_runtime.cpp packs to fp32 fragments: :264-266) */
	float *a = (float*) malloc(sizeof(float) * (size_t) M * K + 4);
	float *b = (float*) malloc(sizeof(float) * (size_t) K * N + 4);
	for (int m = 0; m < M; m++)
		for (int k = 0; k < K; k++)
			a[(size_t) m * K + k] = load_as_float(A, ta ? ((size_t) k * M + m) : ((size_t) m * K + k), dtype);
	for (int k = 0; k < K; k++)
		for (int n = 0; n < N; n++)
			b[(size_t) k * N + n] = load_as_float(B, tb ? ((size_t) n * K + k) : ((size_t) k * N + n), dtype);

#pragma omp parallel num_threads(g_threads)
	{
		float *acc = (float*) malloc(sizeof(float) * (size_t) N + 4);
#pragma omp for
		for (int m = 0; m < M; m++)
		{
			for (int k0 = 0; k0 < K || k0 == 0; k0 += k_tile)
			{
				const int k1 = (k0 + k_tile < K) ? (k0 + k_tile) : K;
				const int first = (k0 == 0), last = (k1 == K);
				for (int n = 0; n < N; n++)
					acc[n] = 0.0f;
				for (int k = k0; k < k1; k++) /* avx512f_kernels.cpp:45-70: one fused multiply-add per k, in order */
				{
					const float av = a[(size_t) m * K + k];
					const float *brow = b + (size_t) k * N;
					for (int n = 0; n < N; n++)
						acc[n] = fmaf(av, brow[n], acc[n]);
				}
				/* gemm_runtime.cpp:196-197: beta applies to C on the first K tile, later tiles add to what is already in D */
				const float tile_beta = first ? beta : 1.0f;
				const void *src = first ? C : D;
				for (int n = 0; n < N; n++)
				{
					float x = acc[n] * alpha; /* avx512f_kernels.cpp:798-806 */
					if (bias != NULL && last) /* :808-813, gemm_runtime.cpp:209 */
						x = x + load_as_float(bias, n, dtype);
					if (tile_beta != 0.0f) /* :815-849 fused multiply-add of beta and C */
						x = fmaf(load_as_float(src, (size_t) m * N + n, dtype), tile_beta, x);
					if (act == 3 && last) /* :851-856 */
						x = (x > 0.0f) ? x : 0.0f;
					store_from_float(D, (size_t) m * N + n, dtype, x);
				}
				if (K == 0)
					break;
			}
		}
		free(acc);
	}
	free(a);
	free(b);
	if (act != 0 && act != 3) /* gemm.cpp:81-82: other activations are a second pass over D */
		for (size_t i = 0; i < (size_t) M * N; i++)
			store_from_float(D, i, dtype, activation(act, load_as_float(D, i, dtype)));
}

void oracle_gemm(int dtype, char opA, char opB, int M, int N, int K, int batch, float alpha, const void *A, size_t stride_a, const void *B,
		size_t stride_b, float beta, const void *C, void *D, size_t stride_c, const void *bias, int act, int k_tile)
{
	const int ta = (opA == 't' || opA == 'T'), tb = (opB == 't' || opB == 'T');
	const size_t es = dtype_size(dtype);
	for (int i = 0; i < batch; i++)
	{
		const void *c = (C != NULL) ? (const void*) ((const uint8_t*) C + es * stride_c * i) : NULL;
		gemm_single(dtype, ta, tb, M, N, K, alpha, (const uint8_t*) A + es * stride_a * i, (const uint8_t*) B + es * stride_b * i, beta, c,
				(uint8_t*) D + es * stride_c * i, bias, act, k_tile);
	}
}

void oracle_int8_gemm_nt(int M, int N, int K, const int8_t *A, const int8_t *B, int32_t *C)
{
#pragma omp parallel for num_threads(g_threads)
	for (int m = 0; m < M; m++)
		for (int n = 0; n < N; n++)
		{
			int32_t acc = 0;
			for (int k = 0; k < K; k++)
				acc += (int32_t) A[(size_t) m * K + k] * (int32_t) B[(size_t) n * K + k];
			C[(size_t) m * N + n] = acc;
		}
}

/* ------------------------------------------------------------------------------------------------------------------------
 * im2row and explicit-GEMM convolution
 * ---------------------------------------------------------------------------------------------------------------------- */
void oracle_im2row(int esize, int batch, int height, int width, int filters, int kernel_size, const void *input, void *output)
{
	/* conv_im2row.cpp:21-59: row (b,h,w) = for i, for j: the channel vector at (h + i - pad, w + j - pad) or zeros */
	const int pad = (kernel_size - 1) / 2;
	const size_t block = (size_t) esize * filters;
	const size_t pixels = (size_t) batch * height * width;
#pragma omp parallel for num_threads(g_threads)
	for (size_t p = 0; p < pixels; p++)
	{
		const int b = (int) (p / ((size_t) height * width));
		const int h = (int) ((p / width) % height);
		const int w = (int) (p % width);
		uint8_t *dst = (uint8_t*) output + p * kernel_size * kernel_size * block;
		for (int i = -pad; i < kernel_size - pad; i++)
			for (int j = -pad; j < kernel_size - pad; j++, dst += block)
				if (h + i >= 0 && h + i < height && w + j >= 0 && w + j < width)
					memcpy(dst, (const uint8_t*) input + ((((size_t) b * height + h + i) * width) + w + j) * block, block);
				else
					memset(dst, 0, block);
	}
}

void oracle_conv2d_forward(int dtype, int batch, int height, int width, int filters_in, int filters_out, int kernel_size, const void *input,
		const void *weights, void *output, const void *bias, const void *add, int act, int k_tile)
{
	/* src/core/math.cpp:1607-1625 */
	const int M = batch * height * width;
	const int K = kernel_size * kernel_size * filters_in;
	const void *matrix = input;
	void *workspace = NULL;
	if (kernel_size != 1)
	{
		workspace = malloc(dtype_size(dtype) * (size_t) M * K + 16);
		oracle_im2row((int) dtype_size(dtype), batch, height, width, filters_in, kernel_size, input, workspace);
		matrix = workspace;
	}
	oracle_gemm(dtype, 'n', 't', M, filters_out, K, 1, 1.0f, matrix, 0, weights, 0, (add != NULL) ? 1.0f : 0.0f, add, output, 0, bias, act, k_tile);
	free(workspace);
}

/* ------------------------------------------------------------------------------------------------------------------------
 * int8 path
 * ---------------------------------------------------------------------------------------------------------------------- */
int32_t oracle_quantize(float x, int bits)
{ /* quantization.cpp:39-43 */
	const float limit = (float) (1 << (bits - 1));
	float r = roundf(x);
	if (r > limit - 1.0f)
		r = limit - 1.0f;
	if (r < -limit)
		r = -limit;
	return (int32_t) r;
}
/* AffineTransform::operator() (quantization.hpp:39-43): float(x) * scale + shift, two roundings */
static inline float affine(float x, float scale, float shift)
{
	const float t = x * scale;
	return t + shift;
}
static inline float int8_tail(int32_t acc, float scale, float bias, const int8_t *ext, size_t offset, float ext_scale, float ext_shift, int act)
{
	/* Conv2D.cpp:284-306 */
	float tmp = (float) acc * scale;
	tmp = tmp + bias;
	if (ext != NULL)
		tmp = tmp + affine((float) ext[offset], ext_scale, ext_shift);
	switch (act)
	{
		case 1:
			tmp = 1.0f / (1.0f + expf(-tmp));
			break;
		case 2:
			tmp = tanhf(tmp);
			break;
		case 3:
			tmp = (tmp > 0.0f) ? tmp : 0.0f;
			break;
		case 5:
			tmp = expf(tmp);
			break;
		default:
			break;
	}
	return tmp;
}
static inline void int8_store(void *output, size_t offset, int output_dtype, float tmp, float inv_scale, float inv_shift)
{
	if (output_dtype == ORACLE_INT8)
		((int8_t*) output)[offset] = (int8_t) oracle_quantize(affine(tmp, inv_scale, inv_shift), 8);
	else if (output_dtype == ORACLE_FLOAT16)
		((uint16_t*) output)[offset] = oracle_fp32_to_fp16(tmp);
	else
		((float*) output)[offset] = tmp;
}

void oracle_int8_conv2d_forward(int batch, int height, int width, int filters_in, int filters_out, int kernel_size, const int8_t *input,
		float input_scale, float input_shift, const int8_t *weights, const float *channel_scales, const float *bias, int output_dtype, void *output,
		float output_scale, float output_shift, const int8_t *ext, float ext_scale, float ext_shift, int act)
{
	const int pad = -(kernel_size - 1) / 2; /* Conv2D.cpp:242-243 */
	/* get_zero<int32_t> (quantization.hpp:57-61) of the inverse transform (1/scale, -shift/scale) (:44-47) */
	const int32_t input_zero = (int32_t) roundf(affine(0.0f, 1.0f / input_scale, -input_shift / input_scale));
	const float inv_scale = 1.0f / output_scale, inv_shift = -output_shift / output_scale;
	const size_t pixels = (size_t) batch * height * width;
#pragma omp parallel for num_threads(g_threads)
	for (size_t p = 0; p < pixels; p++)
	{
		const int b = (int) (p / ((size_t) height * width));
		const int h = (int) ((p / width) % height);
		const int w = (int) (p % width);
		for (int out = 0; out < filters_out; out++)
		{
			int32_t acc = 0;
			for (int i = 0; i < kernel_size; i++)
				for (int j = 0; j < kernel_size; j++)
				{
					const int x = pad + h + i, y = pad + w + j;
					const int8_t *wgt = weights + (((size_t) out * kernel_size + i) * kernel_size + j) * filters_in;
					if (0 <= x && x < height && 0 <= y && y < width)
					{
						const int8_t *src = input + (((size_t) b * height + x) * width + y) * filters_in;
						for (int in = 0; in < filters_in; in++)
							acc += (int32_t) wgt[in] * (int32_t) src[in];
					}
					else
						for (int in = 0; in < filters_in; in++)
							acc += (int32_t) wgt[in] * input_zero;
				}
			const size_t offset = p * filters_out + out;
			const float tmp = int8_tail(acc, channel_scales[out], bias[out], ext, offset, ext_scale, ext_shift, act);
			int8_store(output, offset, output_dtype, tmp, inv_scale, inv_shift);
		}
	}
}

void oracle_quantized_scale_shift_act(int output_dtype, size_t first_dim, int last_dim, void *output, float output_scale, float output_shift,
		const int32_t *input, const float *scales, const float *bias, int act, const int8_t *ext, float ext_scale, float ext_shift)
{
	const float inv_scale = 1.0f / output_scale, inv_shift = -output_shift / output_scale;
#pragma omp parallel for num_threads(g_threads)
	for (size_t i = 0; i < first_dim; i++)
		for (int j = 0; j < last_dim; j++)
		{
			const size_t offset = i * last_dim + j;
			const float tmp = int8_tail(input[offset], scales[j], bias[j], ext, offset, ext_scale, ext_shift, act);
			int8_store(output, offset, output_dtype, tmp, inv_scale, inv_shift);
		}
}

void oracle_quantize_weights(int rows, int cols, const float *weights, const float *bias, float input_scale, float input_shift, int8_t *q_weights,
		float *channel_scales, float *q_bias)
{
	/* quantization.cpp:69-86 */
	for (int i = 0; i < rows; i++)
	{
		float max_abs = 0.0f;
		for (int j = 0; j < cols; j++)
		{
			const float v = fabsf(weights[(size_t) i * cols + j]);
			max_abs = (v > max_abs) ? v : max_abs;
		}
		const float channel_scale = 127.0f / max_abs;
		channel_scales[i] = input_scale / channel_scale;
		int32_t sum_q = 0;
		for (int j = 0; j < cols; j++)
		{
			const int32_t q = oracle_quantize(weights[(size_t) i * cols + j] * channel_scale, 8);
			sum_q += q;
			q_weights[(size_t) i * cols + j] = (int8_t) q;
		}
		const float b = (bias != NULL) ? bias[i] : 0.0f;
		const float t = input_shift / channel_scale * (float) sum_q;
		q_bias[i] = t + b;
	}
}

/* ------------------------------------------------------------------------------------------------------------------------
 * element-wise neighbours
 * ---------------------------------------------------------------------------------------------------------------------- */
void oracle_add_bias_act(int dtype, size_t first_dim, int last_dim, void *output, const void *input, const void *bias, int act)
{
#pragma omp parallel for num_threads(g_threads)
	for (size_t i = 0; i < first_dim; i++)
		for (int j = 0; j < last_dim; j++)
		{
			const size_t offset = i * last_dim + j;
			float x = load_as_float(input, offset, dtype);
			if (bias != NULL)
				x = x + load_as_float(bias, j, dtype);
			store_from_float(output, offset, dtype, activation(act, x));
		}
}
void oracle_add_tensors(int dtype, size_t elements, float a1, const void *x1, float a2, const void *x2, float a3, const void *x3, float beta, void *y)
{
	for (size_t i = 0; i < elements; i++)
	{
		const float v1 = (x1 != NULL && a1 != 0.0f) ? load_as_float(x1, i, dtype) : 0.0f;
		const float v2 = (x2 != NULL && a2 != 0.0f) ? load_as_float(x2, i, dtype) : 0.0f;
		const float v3 = (x3 != NULL && a3 != 0.0f) ? load_as_float(x3, i, dtype) : 0.0f;
		const float vy = (beta != 0.0f) ? load_as_float(y, i, dtype) : 0.0f;
		store_from_float(y, i, dtype, a1 * v1 + a2 * v2 + a3 * v3 + beta * vy);
	}
}
void oracle_unpack_input(int dtype, size_t first_dim, int last_dim, void *dst, const uint32_t *src)
{
	const int stride = (last_dim + 31) / 32;
	for (size_t i = 0; i < first_dim; i++)
		for (int j = 0; j < last_dim; j++)
		{
			const uint32_t bit = (src[i * stride + j / 32] >> (j % 32)) & 1u;
			const size_t offset = i * last_dim + j;
			switch (dtype)
			{
				case ORACLE_FLOAT16:
					((uint16_t*) dst)[offset] = bit ? 0x3c00u : 0x0000u;
					break;
				case ORACLE_FLOAT32:
					((float*) dst)[offset] = bit ? 1.0f : 0.0f;
					break;
				case ORACLE_INT8:
					((int8_t*) dst)[offset] = (int8_t) bit;
					break;
				case ORACLE_INT32:
					((int32_t*) dst)[offset] = (int32_t) bit;
					break;
				default:
					break;
			}
		}
}

/* ------------------------------------------------------------------------------------------------------------------------
 * heads and glue after the convolution trunk
 * ---------------------------------------------------------------------------------------------------------------------- */
/* src/backend/cpu/avx_misc_kernels.cpp:81-112 (kernel_softmax; the 3-column form at :53-79 is the same arithmetic): row maximum,
 * exp(x - max) summed in column order, every exponent multiplied by 1 / sum. */
void oracle_softmax_forward(int dtype, size_t first_dim, int last_dim, void *output, const void *input)
{
	float *row = (float*) malloc(sizeof(float) * (size_t) last_dim);
	for (size_t i = 0; i < first_dim; i++)
	{
		const size_t base = i * (size_t) last_dim;
		for (int j = 0; j < last_dim; j++)
			row[j] = load_as_float(input, base + j, dtype);
		float max_value = row[0];
		for (int j = 0; j < last_dim; j++)
			max_value = fmaxf(max_value, row[j]);
		float sum = 0.0f;
		for (int j = 0; j < last_dim; j++)
		{
			row[j] = expf(row[j] - max_value);
			sum += row[j];
		}
		const float scale = 1.0f / sum;
		for (int j = 0; j < last_dim; j++)
			store_from_float(output, base + j, dtype, row[j] * scale);
	}
	free(row);
}
/* src/backend/cpu/kernels/pooling_and_scaling.cpp:142-180 with the SIMD kernels of avx_kernels.cpp:303-560: per (image, channel) the
 * pixels are summed in row-major order in fp32 and the sum is multiplied by 1.0f / (height * width). alpha and beta follow the
 * device form (src/backend/cuda/kernels/global_pooling.cu:28-70): y = alpha * mean + beta * y; the CPU entry point only accepts 1, 0. */
void oracle_global_average_pooling_forward(int dtype, int batch, int hw, int channels, float alpha, const void *input, float beta, void *output)
{
	const float inv = 1.0f / (float) hw;
	/* pooling_and_scaling.cpp:61-92,156-176 on a host with AVX: the widest vector kernel whose step fits the channel count (64 or 8
	 * columns; 32 or 4 for fp32 through the SSE2 kernels) takes whole steps and multiplies the sum by 1 / hw; what is left goes column
	 * by column through the scalar kernel, which divides the sum by hw (kernels/def_kernels.cpp:40-54). */
	int step = 1;
	if (channels >= 64)
		step = 64;
	else if (channels >= 8)
		step = 8;
	else if (channels >= 4 && dtype == ORACLE_FLOAT32)
		step = 4;
	const int vector_channels = (step > 1) ? (channels / step) * step : 0;
	for (int b = 0; b < batch; b++)
		for (int c = 0; c < channels; c++)
		{
			float acc = 0.0f;
			for (int p = 0; p < hw; p++)
				acc += load_as_float(input, ((size_t) b * hw + p) * channels + c, dtype);
			const size_t o = (size_t) b * channels + c;
			float y = (c < vector_channels) ? acc * inv : acc / (float) hw;
			if (alpha != 1.0f)
				y *= alpha;
			if (beta != 0.0f)
				y += beta * load_as_float(output, o, dtype);
			store_from_float(output, o, dtype, y);
		}
}
/* src/backend/cuda/kernels/batchnorm.cu:57-104: scale = gamma / sqrt(variance + 1e-6), shift = -mean * scale + beta_bn;
 * y = alpha * act(x * scale + shift) + beta * y. avg_var is fp32 [2, last_dim] (means, then variances); gamma / bias have the
 * tensor's type and may be NULL (1 and 0). The CPU dispatch of this entry point is commented out (src/core/math.cpp:722-737). */
void oracle_batchnorm_inference(int dtype, size_t first_dim, int last_dim, float alpha, const void *input, const void *gamma, const void *bias,
		const float *avg_var, float beta, void *output, int act)
{
	for (size_t i = 0; i < first_dim; i++)
		for (int j = 0; j < last_dim; j++)
		{
			const float g = (gamma != NULL) ? load_as_float(gamma, j, dtype) : 1.0f;
			const float b = (bias != NULL) ? load_as_float(bias, j, dtype) : 0.0f;
			const float scale = g / sqrtf(avg_var[last_dim + j] + 1.0e-6f);
			const float mean_scaled = avg_var[j] * scale;
			const float shift = b - mean_scaled;
			const size_t o = i * (size_t) last_dim + j;
			const float xs = load_as_float(input, o, dtype) * scale;
			float y = activation(act, xs + shift) * alpha;
			if (beta != 0.0f)
				y += beta * load_as_float(output, o, dtype);
			store_from_float(output, o, dtype, y);
		}
}
/* src/backend/cpu/normalization.cpp:296-343 (cpu_fold_batchnorm) / src/backend/cuda/kernels/batchnorm.cu:357-394: channel-first
 * weights [channels, last] (channels_last == 0) or depthwise weights [first, channels] (channels_last != 0) are scaled by
 * gamma / sqrt(variance + 1e-6); bias = bias * scale + (-mean * scale + beta_bn). A NULL bn bias counts as 0 (the device form;
 * the CPU form uses 1 there and is never called that way: src/graph/graph_optimizers.cpp:165-172 always passes the tensor). */
void oracle_fold_batchnorm(int dtype, int channels, int other, int channels_last, void *layer_weights, void *layer_bias, const void *bn_weights,
		const void *bn_bias, const float *bn_avg_var)
{
	for (int c = 0; c < channels; c++)
	{
		const float gamma = (bn_weights != NULL) ? load_as_float(bn_weights, c, dtype) : 1.0f;
		const float beta = (bn_bias != NULL) ? load_as_float(bn_bias, c, dtype) : 0.0f;
		const float scale = gamma / sqrtf(bn_avg_var[channels + c] + 1.0e-6f);
		const float neg_mean_scaled = -bn_avg_var[c] * scale;
		const float shift = neg_mean_scaled + beta;
		const float old_bias_scaled = load_as_float(layer_bias, c, dtype) * scale;
		store_from_float(layer_bias, c, dtype, old_bias_scaled + shift);
		for (int k = 0; k < other; k++)
		{
			const size_t o = channels_last ? ((size_t) k * channels + c) : ((size_t) c * other + k);
			store_from_float(layer_weights, o, dtype, load_as_float(layer_weights, o, dtype) * scale);
		}
	}
}

/* ------------------------------------------------------------------------------------------------------------------------
 * Transformer-block pieces: RMS normalisation and multi-head attention with a 2-D relative-position bias
 * ---------------------------------------------------------------------------------------------------------------------- */
/* src/backend/cpu/normalization.cpp:452-486: rms = sqrt(sum x^2 / n) with the sum taken in order, y = (gamma * x) * (1 / (1e-6 + rms)).
 * The reference implements fp32 only; fp16 here widens on load and truncates on store like every other fp16 function. */
void oracle_rmsnorm_forward(int dtype, size_t first_dim, int last_dim, const void *input, void *output, const void *weights)
{
#pragma omp parallel for num_threads(g_threads)
	for (size_t i = 0; i < first_dim; i++)
	{
		float sum_square = 0.0f;
		for (int j = 0; j < last_dim; j++)
		{
			const float x = load_as_float(input, i * last_dim + j, dtype);
			const float sq = x * x;
			sum_square = sum_square + sq;
		}
		const float rms = sqrtf(sum_square / (float) last_dim);
		const float inv_rms = 1.0f / (1.0e-6f + rms);
		for (int j = 0; j < last_dim; j++)
		{
			const float x = load_as_float(input, i * last_dim + j, dtype);
			const float scaled = (weights != NULL) ? load_as_float(weights, j, dtype) * x : x;
			store_from_float(output, i * last_dim + j, dtype, scaled * inv_rms);
		}
	}
}

/* src/backend/cpu/attention.cpp:395-431 (cpu_multi_head_attention_forward) with softmax_forward_in_place :142-214:
 * input [B, H, W, (3 - symmetric) * E] holds per token q (heads x head_dim), k (absent when symmetric: k = q), v; per (b, head):
 *   s[i][j] = (q_i . k_j, one fused multiply-add per element of the head in order) * (1 / sqrt(head_dim))        gemm 'n','t', :415-416
 *   t[i][j] = s[i][j] + table[head][r + clamp(h_j - h_i, -r, r)][r + clamp(w_j - w_i, -r, r)],  r = (table_size - 1) / 2   :165-172
 *   p[i][j] = exp(t[i][j] - max_j t[i][j]) * (1 / sum_j exp(...)), the sum taken in order                         :177-193
 *   y[i][:] = sum_j p[i][j] * v_j, one fused multiply-add per j in order                                         gemm 'n','n', :423-424
 * table is [heads][table_size][round_up(table_size, 4)] in the tensor's type, NULL for no bias. Output [B, H, W, E]. */
void oracle_multi_head_attention_forward(int dtype, int batch, int height, int width, int embedding, int num_heads, int symmetric,
		const void *input, void *output, const void *table, int table_size)
{
	const int tokens = height * width;
	const int head_dim = embedding / num_heads;
	const int parts = symmetric ? 2 : 3;
	const size_t token_stride = (size_t) parts * embedding;
	const float scale = (float) (1.0 / sqrt((double) head_dim)); /* :413 takes the root of an int: evaluated in double, then narrowed */
	const int range = (table_size - 1) / 2;
	const int table_row = (table_size + 3) / 4 * 4;
#pragma omp parallel for collapse(2) num_threads(g_threads)
	for (int b = 0; b < batch; b++)
		for (int h = 0; h < num_heads; h++)
		{
			float *row = (float*) malloc(sizeof(float) * (size_t) tokens + 4);
			float *acc = (float*) malloc(sizeof(float) * (size_t) head_dim + 4);
			const size_t image = (size_t) b * tokens * token_stride;
			const size_t q_off = image + (size_t) h * head_dim;
			const size_t k_off = symmetric ? q_off : q_off + embedding;
			const size_t v_off = q_off + (size_t) (parts - 1) * embedding;
			for (int i = 0; i < tokens; i++)
			{
				const int h1 = i / width, w1 = i % width;
				float max_value = -1.0e+32f;
				for (int j = 0; j < tokens; j++)
				{
					float dot = 0.0f;
					for (int d = 0; d < head_dim; d++)
						dot = fmaf(load_as_float(input, q_off + i * token_stride + d, dtype), load_as_float(input, k_off + j * token_stride + d, dtype), dot);
					float t = dot * scale;
					if (table != NULL)
					{
						int dh = j / width - h1, dw = j % width - w1;
						dh = (dh < -range) ? -range : ((dh > range) ? range : dh);
						dw = (dw < -range) ? -range : ((dw > range) ? range : dw);
						t = t + load_as_float(table, ((size_t) h * table_size + range + dh) * table_row + range + dw, dtype);
					}
					max_value = (t > max_value) ? t : max_value;
					row[j] = t;
				}
				float sum = 0.0f;
				for (int j = 0; j < tokens; j++)
				{
					row[j] = expf(row[j] - max_value);
					sum = sum + row[j];
				}
				const float inv_sum = 1.0f / sum;
				for (int d = 0; d < head_dim; d++)
					acc[d] = 0.0f;
				for (int j = 0; j < tokens; j++)
				{
					const float p = row[j] * inv_sum;
					for (int d = 0; d < head_dim; d++)
						acc[d] = fmaf(p, load_as_float(input, v_off + j * token_stride + d, dtype), acc[d]);
				}
				for (int d = 0; d < head_dim; d++)
					store_from_float(output, ((size_t) b * tokens + i) * embedding + (size_t) h * head_dim + d, dtype, acc[d]);
			}
			free(row);
			free(acc);
		}
}
