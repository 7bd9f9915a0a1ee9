/*
 * gemm_launch.hpp — host-side description of one (batched) GEMM with the reference's fused tail, shared by the GEMM entry
 * points and by the convolution entry points that reduce to a GEMM (1x1 convolution = gemm_ex on the [B*H*W, Cin] view,
 * reference src/core/math.cpp:1595-1626).
 */
#ifndef MINML_AMD_GEMM_LAUNCH_HPP_
#define MINML_AMD_GEMM_LAUNCH_HPP_

#include "common.hpp"

namespace mlhip
{
	struct GemmArgs
	{
			mlDataType_t dtype = DTYPE_UNKNOWN; /* operand type; DTYPE_INT8 => int32 output */
			bool transpose_a = false, transpose_b = false;
			int M = 0, N = 0, K = 0;
			int batch = 1;
			size_t stride_a = 0, stride_b = 0, stride_c = 0; /* elements between consecutive matrices, 0 = broadcast */
			const void *A = nullptr;
			const void *B = nullptr;
			const void *C = nullptr; /* read only when beta != 0 */
			void *D = nullptr;
			const void *bias = nullptr;
			float alpha = 1.0f, beta = 0.0f;
			mlActivationType_t act = ACTIVATION_LINEAR;
	};

	GemmArgs make_gemm_args(mlDataType_t dtype, char opA, char opB, const mlShape_t &shape_A, const mlShape_t &shape_B, const mlShape_t &shape_D,
			bool batched);
	void launch_gemm(hipStream_t stream, const GemmArgs &args);
}

#endif /* MINML_AMD_GEMM_LAUNCH_HPP_ */
