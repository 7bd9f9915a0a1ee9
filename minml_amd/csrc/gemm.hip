/*
 * gemm.hip — GEMM entry points of the HIP backend: gemm / gemm_batched (both descriptor styles) and gemm_ex.
 *
 * Semantics follow the reference CPU backend (src/backend/cpu/gemm/gemm.cpp:34-83):
 *   gemm:          C = alpha * op(A) * op(B) + beta * C
 *   gemm_batched:  the same for every leading index; a rank-2 operand is broadcast (batch stride 0, gemm.cpp:18-29)
 *   gemm_ex:       D = act(alpha * op(A) * op(B) + bias + beta * C), one dtype for A, B, C, D and bias, fp32 arithmetic
 *   C.dtype INT32: int8 x int8 -> int32, alpha = 1, beta = 0 (src/backend/cuda/gemms.cpp:119-130)
 * M, N, K are derived from the shapes as in src/backend/cpu/gemm/gemm_runtime.cpp:352-354.
 *
 * The inference path only ever asks for op(A) = 'n', op(B) = 't' (both operands K-contiguous): that case runs on the MFMA tile
 * engine. Everything else (transposed forms used by training, K rows that are not 16-byte multiples, unaligned pointers) goes to
 * a plain one-thread-per-output kernel that is correct for every case and makes no performance claim.
 */
#include "common.hpp"

#include <algorithm>
#include "gemm_core.hpp"
#include "epilogues.hpp"
#include "gemm_launch.hpp"
#include "gemm_stream.hpp"
#include "gemm_dma.hpp"

namespace
{
	using namespace mlhip;

	template<typename T, typename Cfg, typename Epilogue>
	__global__ __launch_bounds__(Cfg::THREADS) void kernel_gemm_nt(const T *A, const T *B, int M, int N, int k_bytes, size_t stride_a,
			size_t stride_b, size_t stride_c, Epilogue epilogue, int tiles_n)
	{
		__shared__ __attribute__((aligned(16))) uint8_t lds[Cfg::LDS_BYTES];

		const unsigned int linear = xcd_contiguous_block_id(blockIdx.x, gridDim.x);
		const int tile_m = linear / tiles_n;
		const int tile_n = linear % tiles_n;
		const size_t batch = blockIdx.y;

		DenseRows<T> a_loader { A + batch * stride_a, M, k_bytes };
		DenseRows<T> b_loader { B + batch * stride_b, N, k_bytes };
		Epilogue local = epilogue;
		local.D += batch * stride_c;
		if constexpr (Epilogue::has_c)
			local.C += batch * stride_c;
		gemm_tile<T, Cfg>(a_loader, b_loader, M, k_bytes, tile_m * Cfg::BM, tile_n * Cfg::BN, lds, local);
	}

	/* Fallback: one thread per output element, any op combination, any alignment. */
	template<typename T, typename AccT, typename Epilogue>
	__global__ __launch_bounds__(256) void kernel_gemm_generic(const T *A, const T *B, int M, int N, int K, size_t a_row, size_t a_col, size_t b_row,
			size_t b_col, size_t stride_a, size_t stride_b, size_t stride_c, Epilogue epilogue, int out_stride)
	{
		const size_t gid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
		if (gid >= static_cast<size_t>(M) * N)
			return;
		const int m = static_cast<int>(gid / N);
		const int n = static_cast<int>(gid % N);
		const size_t batch = blockIdx.y;
		const T *a = A + batch * stride_a + m * a_row;
		const T *b = B + batch * stride_b + n * b_row;
		AccT acc = 0;
		for (int k = 0; k < K; k++)
		{
			if constexpr (sizeof(T) == 1)
				acc += static_cast<int>(a[k * a_col]) * static_cast<int>(b[k * b_col]);
			else
				acc += static_cast<float>(a[k * a_col]) * static_cast<float>(b[k * b_col]);
		}
		Epilogue local = epilogue;
		local.D += batch * stride_c;
		if constexpr (Epilogue::has_c)
			local.C += batch * stride_c;
		local.vectorized = false;
		/* hand the single value over as the first of a group of 4 whose other members lie outside the matrix */
		Epilogue single = local;
		const AccT vals[4] = { acc, 0, 0, 0 };
		single.N = n + 1;
		single.row_stride = out_stride; /* elements between consecutive rows of D and C */
		single(m, n, vals);
	}

	bool aligned_to(const void *p, size_t bytes)
	{
		return p == nullptr || (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
	}

	template<typename T>
	FloatEpilogue<T> make_float_epilogue(const GemmArgs &g, bool vectorized)
	{
		FloatEpilogue<T> ep;
		ep.D = reinterpret_cast<T*>(g.D);
		ep.C = reinterpret_cast<const T*>(g.C);
		ep.bias = reinterpret_cast<const T*>(g.bias);
		ep.N = g.N;
		ep.row_stride = g.N;
		ep.alpha = g.alpha;
		ep.beta = g.beta;
		ep.act = g.act;
		ep.vectorized = vectorized;
		return ep;
	}
	/*
	 * Tall products with very few columns (the 1x1 policy head: [B*H*W, C] x [1, C]^T): a matrix-vector product per column, bound by the
	 * read of A. One row of A is 16 bytes per lane on LANES lanes (K rows of 16 ... 1024 bytes, LANES a power of two), so a wavefront
	 * instruction covers 64 / LANES consecutive rows = 1 KB of consecutive memory; the lanes of a row hold their 16-byte pieces of the
	 * NMAX rows of B in registers, multiply, and meet in a butterfly of cross-lane additions; the row's first lane applies the epilogue.
	 * Four row groups are in flight per wavefront.
	 */
	template<typename T, int NMAX>
	__global__ __launch_bounds__(256) void kernel_gemv_rows(const T *A, const T *B, int M, int N, int lanes, size_t k_elements, FloatEpilogue<T> epilogue)
	{
		constexpr int E = 16 / sizeof(T); /* elements per 16-byte piece */
		constexpr int UNROLL = 4;
		const int lane = threadIdx.x & 63;
		const int piece = lane & (lanes - 1), row_in_group = lane / lanes;
		const int rows_per_group = 64 / lanes;
		float b[NMAX][E];
#pragma unroll
		for (int n = 0; n < NMAX; n++)
		{
			Vec<T, E> tmp;
			if (n < N)
				tmp.load(B + static_cast<size_t>(n) * k_elements + piece * E);
			else
				tmp.zero();
#pragma unroll
			for (int e = 0; e < E; e++)
				b[n][e] = tmp.v[e];
		}
		epilogue.vectorized = false;
		const size_t wave = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
		const size_t waves = (static_cast<size_t>(gridDim.x) * blockDim.x) >> 6;
		const size_t groups = (static_cast<size_t>(M) + rows_per_group - 1) / rows_per_group;
		for (size_t first = wave * UNROLL; first < groups; first += waves * UNROLL)
		{
			Vec<T, E> a[UNROLL];
#pragma unroll
			for (int u = 0; u < UNROLL; u++)
			{
				const size_t m = min((first + u) * rows_per_group + row_in_group, static_cast<size_t>(M) - 1);
				a[u].load(A + m * k_elements + piece * E);
			}
#pragma unroll
			for (int u = 0; u < UNROLL; u++)
			{
				float sum[NMAX];
#pragma unroll
				for (int n = 0; n < NMAX; n++)
				{
					sum[n] = 0.0f;
#pragma unroll
					for (int e = 0; e < E; e++)
						sum[n] = fmaf(a[u].v[e], b[n][e], sum[n]);
				}
				for (int offset = 1; offset < lanes; offset <<= 1)
#pragma unroll
					for (int n = 0; n < NMAX; n++)
						sum[n] += __shfl_xor(sum[n], offset);
				const size_t m = (first + u) * rows_per_group + row_in_group;
				if (piece == 0 && first + u < groups && m < static_cast<size_t>(M))
				{
#pragma unroll
					for (int n = 0; n < NMAX; n++)
						if (n < N)
						{
							FloatEpilogue<T> single = epilogue;
							const float vals[4] = { sum[n], 0.0f, 0.0f, 0.0f };
							single.N = n + 1; /* the other members of the group of 4 lie outside the matrix */
							single(static_cast<int>(m), n, vals);
						}
				}
			}
		}
	}
	template<typename T>
	bool try_launch_gemv(hipStream_t stream, const GemmArgs &g, bool fast, size_t k_bytes)
	{
		const size_t pieces = k_bytes / 16;
		if (!(fast && g.batch == 1 && g.N >= 1 && g.N <= 4 && k_bytes % 16 == 0 && pieces >= 1 && pieces <= 64 && (pieces & (pieces - 1)) == 0))
			return false;
		FloatEpilogue<T> ep = make_float_epilogue<T>(g, false);
		const int rows_per_group = 64 / static_cast<int>(pieces);
		const size_t groups = (static_cast<size_t>(g.M) + rows_per_group - 1) / rows_per_group;
		/* 4 wavefronts per workgroup, 4 row groups per wavefront and round; enough workgroups for 8 wavefronts per SIMD */
		const size_t wanted = (groups + 15) / 16;
		const unsigned int grid = static_cast<unsigned int>(std::min<size_t>(wanted, static_cast<size_t>(device_compute_units()) * 8));
		if (g.N == 1)
			hipLaunchKernelGGL((kernel_gemv_rows<T, 1>), dim3(grid), dim3(256), 0, stream, reinterpret_cast<const T*>(g.A), reinterpret_cast<const T*>(g.B), g.M, g.N,
					static_cast<int>(pieces), static_cast<size_t>(g.K), ep);
		else
			hipLaunchKernelGGL((kernel_gemv_rows<T, 4>), dim3(grid), dim3(256), 0, stream, reinterpret_cast<const T*>(g.A), reinterpret_cast<const T*>(g.B), g.M, g.N,
					static_cast<int>(pieces), static_cast<size_t>(g.K), ep);
		return true;
	}
}

namespace mlhip
{
	void launch_gemm(hipStream_t stream, const GemmArgs &g)
	{
		if (g.M == 0 || g.N == 0 || g.batch == 0)
			return;
		MLHIP_REQUIRE(g.A != nullptr && g.B != nullptr && g.D != nullptr, "gemm: null matrix");
		MLHIP_REQUIRE(g.beta == 0.0f || g.C != nullptr, "gemm: beta != 0 needs a C matrix");
		if (g.batch > 65535)
		{ /* the matrix index rides in the grid's second dimension: longer batches go slice by slice */
			const int esize_in = size_of(g.dtype), esize_out = (g.dtype == DTYPE_INT8) ? 4 : esize_in;
			for (int first = 0; first < g.batch; first += 65535)
			{
				GemmArgs part = g;
				part.batch = std::min(65535, g.batch - first);
				part.A = reinterpret_cast<const uint8_t*>(g.A) + static_cast<size_t>(first) * g.stride_a * esize_in;
				part.B = reinterpret_cast<const uint8_t*>(g.B) + static_cast<size_t>(first) * g.stride_b * esize_in;
				part.D = reinterpret_cast<uint8_t*>(g.D) + static_cast<size_t>(first) * g.stride_c * esize_out;
				if (g.C != nullptr)
					part.C = reinterpret_cast<const uint8_t*>(g.C) + static_cast<size_t>(first) * g.stride_c * esize_out;
				launch_gemm(stream, part);
			}
			return;
		}

		const int esize = size_of(g.dtype);
		const bool nt = !g.transpose_a && g.transpose_b;
		const size_t k_bytes = static_cast<size_t>(g.K) * esize;
		const bool fast = nt && g.K > 0 && (k_bytes % 16 == 0) && aligned_to(g.A, 16) && aligned_to(g.B, 16)
				&& ((g.stride_a * esize) % 16 == 0) && ((g.stride_b * esize) % 16 == 0);

		const int out_size = (g.dtype == DTYPE_INT8) ? 4 : esize;
		const bool vectorized = (g.N % 4 == 0) && aligned_to(g.D, 4 * out_size) && aligned_to(g.C, 4 * out_size) && aligned_to(g.bias, 4 * esize)
				&& ((g.stride_c * out_size) % (4 * out_size) == 0);

		/* products with at most 4 columns (policy heads): one pass over A, no matrix cores; taken at every number of rows, so that a
		 * position's result does not depend on the size of the batch it is part of */
		if ((g.dtype == DTYPE_FLOAT16 && try_launch_gemv<half_t>(stream, g, fast, k_bytes)) || (g.dtype == DTYPE_FLOAT32 && try_launch_gemv<float>(stream, g, fast, k_bytes)))
		{
			MLHIP_CHECK(hipGetLastError());
			return;
		}
		/*
		 * Products with short K rows (128 / 256 / 512 bytes) and many rows are bound by HBM: they take the persistent streaming kernel -
		 * the Winograd products with a plain 16-byte store, everything else (gemm_ex, 1x1 convolutions, the int8 product) with the
		 * fused epilogue on 4 consecutive outputs.
		 */
		const bool plain = (g.alpha == 1.0f) && (g.beta == 0.0f) && (g.bias == nullptr) && (g.act == ACTIVATION_LINEAR) && (g.N * esize) % 16 == 0
				&& aligned_to(g.D, 16) && ((g.stride_c * esize) % 16 == 0) && g.dtype != DTYPE_INT8;
		if (fast && (g.stride_a != 0 || g.batch == 1)
				&& ((plain || g.dtype == DTYPE_FLOAT16) ? stream_gemm_plain_applies(g.M, g.batch, k_bytes, esize) : stream_gemm_applies(g.M, g.batch, k_bytes)))
		{
			const StreamGemmArgs sg { g.A, g.B, g.D, g.M, g.N, static_cast<int>(k_bytes), g.batch, g.stride_a, g.stride_b, g.stride_c };
			bool launched = true;
			if (g.dtype == DTYPE_FLOAT16 && plain)
				launch_stream_gemm<half_t>(stream, sg, PlainStore { });
			else if (g.dtype == DTYPE_FLOAT32 && plain)
				launch_stream_gemm<float>(stream, sg, PlainStore { });
			else if (g.dtype == DTYPE_FLOAT16 && vectorized)
				specialise_epilogue(make_float_epilogue<half_t>(g, true), [&](const auto &ep)
				{
					launch_stream_gemm<half_t>(stream, sg, ep);
				});
			else if (g.dtype == DTYPE_FLOAT32 && vectorized)
				launch_stream_gemm<float>(stream, sg, make_float_epilogue<float>(g, true));
			else if (g.dtype == DTYPE_INT8 && vectorized && g.bias == nullptr && g.act == ACTIVATION_LINEAR)
			{
				Int32Epilogue ep;
				ep.D = reinterpret_cast<int32_t*>(g.D);
				ep.N = g.N;
				ep.row_stride = g.N;
				ep.vectorized = true;
				launch_stream_gemm<int8_t>(stream, sg, ep);
			}
			else
				launched = false;
			if (launched)
			{
				MLHIP_CHECK(hipGetLastError());
				return;
			}
		}


		/* strides of op(A)[m][k] and op(B)^T[n][k] in elements, for the generic kernel */
		const size_t a_row = g.transpose_a ? 1 : g.K, a_col = g.transpose_a ? g.M : 1;
		const size_t b_row = g.transpose_b ? g.K : 1, b_col = g.transpose_b ? 1 : g.N;

		/* K rows that are whole 128-byte chunks take the direct-to-LDS engine */
		const bool dma = fast && (k_bytes % 128 == 0) && k_bytes <= 0x7fffffffu;
		const DenseDmaRows dma_a { reinterpret_cast<const uint8_t*>(g.A), g.M, static_cast<int>(k_bytes) };
		const DenseDmaRows dma_b { reinterpret_cast<const uint8_t*>(g.B), g.N, static_cast<int>(k_bytes) };

		typedef TileConfig<128, 128, 64, 2, 2> Cfg;
		const int tiles_m = ceil_div(g.M, Cfg::BM), tiles_n = ceil_div(g.N, Cfg::BN);
		const dim3 fast_grid(static_cast<unsigned int>(tiles_m) * tiles_n, g.batch);
		const size_t outputs = static_cast<size_t>(g.M) * g.N;
		MLHIP_REQUIRE((outputs + 255) / 256 <= 0x7fffffffu, "gemm: matrix too large");
		const dim3 slow_grid(static_cast<unsigned int>((outputs + 255) / 256), g.batch);

		switch (g.dtype)
		{
			case DTYPE_FLOAT16:
			{
				FloatEpilogue<half_t> ep;
				ep.D = reinterpret_cast<half_t*>(g.D);
				ep.C = reinterpret_cast<const half_t*>(g.C);
				ep.bias = reinterpret_cast<const half_t*>(g.bias);
				ep.N = g.N;
				ep.row_stride = g.N;
				ep.alpha = g.alpha;
				ep.beta = g.beta;
				ep.act = g.act;
				ep.vectorized = vectorized;
				if (dma)
					launch_gemm_dma<half_t>(stream, dma_a, dma_b, g.M, g.N, static_cast<int>(k_bytes), g.batch, g.stride_a * esize, g.stride_b * esize,
							g.stride_c, ep);
				else if (fast)
					specialise_epilogue(ep, [&](const auto &fixed)
					{
						typedef typename std::decay<decltype(fixed)>::type Fixed;
						hipLaunchKernelGGL((kernel_gemm_nt<half_t, Cfg, Fixed>), fast_grid, dim3(Cfg::THREADS), 0, stream,
								reinterpret_cast<const half_t*>(g.A), reinterpret_cast<const half_t*>(g.B), g.M, g.N, static_cast<int>(k_bytes), g.stride_a,
								g.stride_b, g.stride_c, fixed, tiles_n);
					});
				else
					hipLaunchKernelGGL((kernel_gemm_generic<half_t, float, FloatEpilogue<half_t>>), slow_grid, dim3(256), 0, stream,
							reinterpret_cast<const half_t*>(g.A), reinterpret_cast<const half_t*>(g.B), g.M, g.N, g.K, a_row, a_col, b_row, b_col, g.stride_a,
							g.stride_b, g.stride_c, ep, g.N);
				break;
			}
			case DTYPE_FLOAT32:
			{
				FloatEpilogue<float> ep;
				ep.D = reinterpret_cast<float*>(g.D);
				ep.C = reinterpret_cast<const float*>(g.C);
				ep.bias = reinterpret_cast<const float*>(g.bias);
				ep.N = g.N;
				ep.row_stride = g.N;
				ep.alpha = g.alpha;
				ep.beta = g.beta;
				ep.act = g.act;
				ep.vectorized = vectorized;
				if (dma)
					launch_gemm_dma<float>(stream, dma_a, dma_b, g.M, g.N, static_cast<int>(k_bytes), g.batch, g.stride_a * esize, g.stride_b * esize,
							g.stride_c, ep);
				else if (fast)
					hipLaunchKernelGGL((kernel_gemm_nt<float, Cfg, FloatEpilogue<float>>), fast_grid, dim3(Cfg::THREADS), 0, stream,
							reinterpret_cast<const float*>(g.A), reinterpret_cast<const float*>(g.B), g.M, g.N, static_cast<int>(k_bytes), g.stride_a,
							g.stride_b, g.stride_c, ep, tiles_n);
				else
					hipLaunchKernelGGL((kernel_gemm_generic<float, float, FloatEpilogue<float>>), slow_grid, dim3(256), 0, stream,
							reinterpret_cast<const float*>(g.A), reinterpret_cast<const float*>(g.B), g.M, g.N, g.K, a_row, a_col, b_row, b_col, g.stride_a,
							g.stride_b, g.stride_c, ep, g.N);
				break;
			}
			case DTYPE_INT8:
			{
				MLHIP_REQUIRE(g.bias == nullptr && g.act == ACTIVATION_LINEAR, "gemm: the int8 product has no fused epilogue");
				Int32Epilogue ep;
				ep.D = reinterpret_cast<int32_t*>(g.D);
				ep.N = g.N;
				ep.row_stride = g.N;
				ep.vectorized = vectorized;
				if (dma)
					launch_gemm_dma<int8_t>(stream, dma_a, dma_b, g.M, g.N, static_cast<int>(k_bytes), g.batch, g.stride_a * esize, g.stride_b * esize,
							g.stride_c, ep);
				else if (fast)
					hipLaunchKernelGGL((kernel_gemm_nt<int8_t, Cfg, Int32Epilogue>), fast_grid, dim3(Cfg::THREADS), 0, stream,
							reinterpret_cast<const int8_t*>(g.A), reinterpret_cast<const int8_t*>(g.B), g.M, g.N, static_cast<int>(k_bytes), g.stride_a,
							g.stride_b, g.stride_c, ep, tiles_n);
				else
					hipLaunchKernelGGL((kernel_gemm_generic<int8_t, int, Int32Epilogue>), slow_grid, dim3(256), 0, stream,
							reinterpret_cast<const int8_t*>(g.A), reinterpret_cast<const int8_t*>(g.B), g.M, g.N, g.K, a_row, a_col, b_row, b_col, g.stride_a,
							g.stride_b, g.stride_c, ep, g.N);
				break;
			}
			default:
				fail_logic("HIP backend: gemm: unsupported data type");
		}
		MLHIP_CHECK(hipGetLastError());
	}

	GemmArgs make_gemm_args(mlDataType_t dtype, char opA, char opB, const mlShape_t &shape_A, const mlShape_t &shape_B, const mlShape_t &shape_D,
			bool batched)
	{
		GemmArgs g;
		g.dtype = dtype;
		g.transpose_a = is_transpose(opA);
		g.transpose_b = is_transpose(opB);
		MLHIP_REQUIRE(shape_A.rank == 2 || shape_A.rank == 3, "gemm: A must have rank 2 or 3");
		MLHIP_REQUIRE(shape_B.rank == 2 || shape_B.rank == 3, "gemm: B must have rank 2 or 3");
		const int ar = shape_A.dim[shape_A.rank - 2], ac = shape_A.dim[shape_A.rank - 1];
		const int br = shape_B.dim[shape_B.rank - 2], bc = shape_B.dim[shape_B.rank - 1];
		g.M = g.transpose_a ? ac : ar;
		g.K = g.transpose_a ? ar : ac;
		g.N = g.transpose_b ? br : bc;
		const int kb = g.transpose_b ? bc : br;
		MLHIP_REQUIRE(kb == g.K, "gemm: inner dimensions of A and B differ");
		if (batched)
		{
			MLHIP_REQUIRE(shape_D.rank == 3, "gemm_batched: C must have rank 3");
			MLHIP_REQUIRE(shape_A.rank == 3 || shape_B.rank == 3, "gemm_batched: at least one of A, B must have rank 3");
			g.batch = shape_D.dim[0];
			if (shape_A.rank == 3)
				MLHIP_REQUIRE(shape_A.dim[0] == g.batch, "gemm_batched: batch size of A differs from C");
			if (shape_B.rank == 3)
				MLHIP_REQUIRE(shape_B.dim[0] == g.batch, "gemm_batched: batch size of B differs from C");
			g.stride_a = (shape_A.rank == 3) ? static_cast<size_t>(ar) * ac : 0;
			g.stride_b = (shape_B.rank == 3) ? static_cast<size_t>(br) * bc : 0;
			g.stride_c = static_cast<size_t>(shape_D.dim[1]) * shape_D.dim[2];
			MLHIP_REQUIRE(shape_D.dim[1] == g.M && shape_D.dim[2] == g.N, "gemm_batched: shape of C does not match op(A) * op(B)");
		}
		else
		{
			MLHIP_REQUIRE(shape_A.rank == 2 && shape_B.rank == 2 && shape_D.rank == 2, "gemm: matrices must have rank 2");
			g.batch = 1;
			MLHIP_REQUIRE(shape_D.dim[0] == g.M && shape_D.dim[1] == g.N, "gemm: shape of the output does not match op(A) * op(B)");
		}
		return g;
	}
}

namespace
{
	void run_gemm(mlContext_t context, const mlhip::GemmArgs &g)
	{
		if (g.M == 0 || g.N == 0 || g.batch == 0)
			return; /* nothing to compute: no context needed */
		mlhip::launch_gemm(mlhip::stream_of(context), g);
	}
}

extern "C"
{
	using namespace mlhip;

	void hip_gemm(mlContext_t context, mlDataType_t dtype, mlShape_t shape_C, void *C, mlShape_t shape_A, const void *A, mlShape_t shape_B,
			const void *B, char opA, char opB, float alpha, float beta)
	try
	{
		GemmArgs g = make_gemm_args(dtype, opA, opB, shape_A, shape_B, shape_C, false);
		g.A = A;
		g.B = B;
		g.C = C;
		g.D = C;
		g.alpha = alpha;
		g.beta = beta;
		run_gemm(context, g);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_gemm_batched(mlContext_t context, mlDataType_t dtype, mlShape_t shape_C, void *C, mlShape_t shape_A, const void *A, mlShape_t shape_B,
			const void *B, char opA, char opB, float alpha, float beta)
	try
	{
		GemmArgs g = make_gemm_args(dtype, opA, opB, shape_A, shape_B, shape_C, true);
		g.A = A;
		g.B = B;
		g.C = C;
		g.D = C;
		g.alpha = alpha;
		g.beta = beta;
		run_gemm(context, g);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_group_gemm(mlContext_t context, char opA, char opB, float alpha, const mlTensor_t A, const mlTensor_t B, float beta, mlTensor_t C, int groups)
	try
	{
		MLHIP_REQUIRE(A.rank == 2 && B.rank == 2 && C.rank == 2, "group_gemm: A, B and C must be matrices");
		MLHIP_REQUIRE(groups > 0 && A.dim[1] % groups == 0 && B.dim[1] % groups == 0 && C.dim[1] % groups == 0,
				"group_gemm: the last dimension of every matrix must be a multiple of the number of groups");
		MLHIP_REQUIRE(A.dtype == C.dtype && B.dtype == C.dtype && (C.dtype == DTYPE_FLOAT16 || C.dtype == DTYPE_FLOAT32), "group_gemm: fp16 or fp32 matrices of one type");
		const bool ta = is_transpose(opA), tb = is_transpose(opB);
		const int lda = A.dim[1], ldb = B.dim[1], ldc = C.dim[1];
		const int part_a = lda / groups, part_b = ldb / groups, part_c = ldc / groups; /* columns of one group in each matrix */
		const int M = ta ? part_a : A.dim[0], K = ta ? A.dim[0] : part_a, N = tb ? B.dim[0] : part_b;
		MLHIP_REQUIRE((tb ? part_b : B.dim[0]) == K && C.dim[0] == M && part_c == N, "group_gemm: shapes do not agree");
		if (M == 0 || N == 0)
			return;
		MLHIP_REQUIRE(A.data != nullptr && B.data != nullptr && C.data != nullptr && groups <= 65535, "group_gemm: null matrix or too many groups");
		const hipStream_t stream = stream_of(context);
		const int esize = size_of(C.dtype);
		const size_t k_bytes = static_cast<size_t>(K) * esize;
		const auto launch = [&](auto zero)
		{
			typedef decltype(zero) T;
			FloatEpilogue<T> ep;
			ep.D = reinterpret_cast<T*>(C.data);
			ep.C = reinterpret_cast<const T*>(C.data);
			ep.bias = nullptr;
			ep.N = N;
			ep.row_stride = ldc;
			ep.alpha = alpha;
			ep.beta = beta;
			ep.act = ACTIVATION_LINEAR;
			ep.vectorized = N % 4 == 0 && aligned_to(C.data, 4 * esize) && (static_cast<size_t>(ldc) * esize) % (4 * esize) == 0;
			const bool dma = !ta && tb && K > 0 && k_bytes % 128 == 0 && aligned_to(A.data, 16) && aligned_to(B.data, 16)
					&& static_cast<size_t>(lda) * esize <= 0x7fffffffu && static_cast<size_t>(ldb) * esize <= 0x7fffffffu;
			if (dma)
			{
				/* the forward form of a grouped 1x1 convolution: the groups are the matrices of one launch of the tile engine, whose operand
				 * rows may lie any distance apart; group i starts i * K elements into the rows of A and B and i * N elements into those of C */
				DenseDmaRows a_loader { reinterpret_cast<const uint8_t*>(A.data), M, static_cast<int>(k_bytes) };
				a_loader.row_stride_bytes = static_cast<int>(static_cast<size_t>(lda) * esize);
				DenseDmaRows b_loader { reinterpret_cast<const uint8_t*>(B.data), N, static_cast<int>(k_bytes) };
				b_loader.row_stride_bytes = static_cast<int>(static_cast<size_t>(ldb) * esize);
				launch_gemm_dma<T>(stream, a_loader, b_loader, M, N, static_cast<int>(k_bytes), groups, k_bytes, k_bytes, static_cast<size_t>(N), ep);
			}
			else
			{
				const size_t a_row = ta ? 1 : lda, a_col = ta ? lda : 1, b_row = tb ? ldb : 1, b_col = tb ? 1 : ldb;
				const size_t outputs = static_cast<size_t>(M) * N;
				MLHIP_REQUIRE((outputs + 255) / 256 <= 0x7fffffffu, "group_gemm: too large");
				hipLaunchKernelGGL((kernel_gemm_generic<T, float, FloatEpilogue<T>>), dim3(static_cast<unsigned int>((outputs + 255) / 256), groups), dim3(256), 0,
						stream, reinterpret_cast<const T*>(A.data), reinterpret_cast<const T*>(B.data), M, N, K, a_row, a_col, b_row, b_col,
						static_cast<size_t>(part_a), static_cast<size_t>(part_b), static_cast<size_t>(part_c), ep, ldc);
			}
		};
		if (C.dtype == DTYPE_FLOAT16)
			launch(half_t(0));
		else
			launch(0.0f);
		MLHIP_CHECK(hipGetLastError());
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_gemm_v2(mlContext_t context, char opA, char opB, float alpha, const mlTensor_t A, const mlTensor_t B, float beta, mlTensor_t C)
	try
	{
		mlDataType_t dtype = C.dtype;
		if (C.dtype == DTYPE_INT32)
		{
			MLHIP_REQUIRE(A.dtype == DTYPE_INT8 && B.dtype == DTYPE_INT8, "gemm: an INT32 result needs INT8 operands");
			MLHIP_REQUIRE(alpha == 1.0f && beta == 0.0f, "gemm: the int8 product supports alpha = 1, beta = 0 only");
			dtype = DTYPE_INT8;
		}
		else
			MLHIP_REQUIRE(A.dtype == C.dtype && B.dtype == C.dtype, "gemm: A, B and C must have one data type");
		mlhip::NestedEntryCalls nested;
		hip_gemm(context, dtype, shape_of(C), C.data, shape_of(A), A.data, shape_of(B), B.data, opA, opB, alpha, beta);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_gemm_batched_v2(mlContext_t context, char opA, char opB, float alpha, const mlTensor_t A, const mlTensor_t B, float beta, mlTensor_t C)
	try
	{
		MLHIP_REQUIRE(A.dtype == C.dtype && B.dtype == C.dtype, "gemm_batched: A, B and C must have one data type");
		MLHIP_REQUIRE(C.dtype == DTYPE_FLOAT16 || C.dtype == DTYPE_FLOAT32, "gemm_batched: unsupported data type");
		mlhip::NestedEntryCalls nested;
		hip_gemm_batched(context, C.dtype, shape_of(C), C.data, shape_of(A), A.data, shape_of(B), B.data, opA, opB, alpha, beta);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
	void hip_gemm_ex(mlContext_t context, mlDataType_t dtype, mlShape_t shape_D, void *D, float alpha, char opA, mlShape_t shape_A, const void *A,
			char opB, mlShape_t shape_B, const void *B, float beta, mlShape_t shape_C, const void *C, const void *bias, mlActivationType_t act)
	try
	{
		MLHIP_REQUIRE(dtype == DTYPE_FLOAT16 || dtype == DTYPE_FLOAT32, "gemm_ex: unsupported data type");
		GemmArgs g = make_gemm_args(dtype, opA, opB, shape_A, shape_B, shape_D, false);
		if (beta != 0.0f)
			MLHIP_REQUIRE(shape_C.rank == 2 && shape_C.dim[0] == g.M && shape_C.dim[1] == g.N, "gemm_ex: C must have the shape of D");
		g.A = A;
		g.B = B;
		g.C = C;
		g.D = D;
		g.alpha = alpha;
		g.beta = beta;
		g.bias = bias;
		g.act = act;
		run_gemm(context, g);
	}
	catch (...)
	{
		return mlhip::entry_failed<void>();
	}
} /* extern "C" */

MLHIP_ALSO_AS_CUDA(gemm)
MLHIP_ALSO_AS_CUDA(gemm_batched)
MLHIP_ALSO_AS_CUDA(gemm_v2)
MLHIP_ALSO_AS_CUDA(gemm_batched_v2)
MLHIP_ALSO_AS_CUDA(gemm_ex)
MLHIP_ALSO_AS_CUDA(group_gemm)
