/*
 * oracle.h — CPU restatement of the arithmetic of minml's convolution / GEMM inference path.
 *
 * TEST INFRASTRUCTURE ONLY. This library is the checker that the HIP backend is compared against (tests, smoke check, the
 * CPU-baseline leg of the benchmark). Nothing in the product path may call it.
 *
 * Every function restates, in plain C, what the reference CPU backend computes, citing the reference file:line it follows
 * (paths relative to the reference checkout). dtype arguments use the reference's mlDataType_t numbering
 * (2 = FLOAT16, 3 = FLOAT32, 6 = INT8, 8 = INT32), activations its mlActivationType_t numbering
 * (0 LINEAR, 1 SIGMOID, 2 TANH, 3 RELU, 4 LEAKY_RELU, 5 EXP). fp16 values are raw uint16_t bit patterns.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   winograd_*            golden vectors of test/backend/test_winograd.cpp:218-323; closed form At[(G g Gt) o (Bt d B)]A = conv3x3;
 *                         bit-exact agreement with the compiled reference CPU backend (oracle/_ref) on awkward shapes
 *   gemm / gemm_batched   numpy matmul in float64; bit-exact agreement with oracle/_ref (fp32) for K <= 1024
 *   im2row                brute-force gather; exact agreement with oracle/_ref
 *   conv2d_forward        direct convolution in float64 (baseline_conv2D_forward, test/backend/test_conv2D.cpp:22-59)
 *   int8_conv2d_forward   integer part against numpy int64; float tail against an independent numpy float32 evaluation and the
 *                         closed-form cases scale=1/shift=0; quantize() against the cases of test/backend/test_quantization.cpp:33-36
 *   fp16 conversion       exhaustive over all 65536 halfs (round trip) and against numpy with explicit truncation
 *   rmsnorm_forward       float64 closed form, scale invariance, unit-norm rows; bit-exact agreement with oracle/_ref (fp32). The fp16 form
 *                         has no counterpart in the reference CPU backend (normalization.cpp:460 has an fp32 branch only): closed form only.
 *   multi_head_attention_forward   float64 closed form; uniform attention for equal keys (output = mean of v); a table that forbids all
 *                         but one offset (output = the v of that neighbour); bit-exact agreement with oracle/_ref (fp32). The fp16 form
 *                         (fp16 in, fp32 arithmetic, truncated fp16 out) has no counterpart in the reference CPU backend, whose softmax
 *                         reads the score matrix as fp32 whatever the tensor type (attention.cpp:420-426): it is pinned by the closed
 *                         form only.
 */
#ifndef MINML_ORACLE_H_
#define MINML_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

	enum
	{
		ORACLE_FLOAT16 = 2, ORACLE_FLOAT32 = 3, ORACLE_INT8 = 6, ORACLE_INT32 = 8
	};

	void oracle_set_num_threads(int threads); /* OpenMP threads used by the loops below; per-element arithmetic order never depends on it */

	/* src/backend/cpu/fp16.hpp:61-78, fp16.cpp:12-153 — truncating narrowing, exact widening */
	uint16_t oracle_fp32_to_fp16(float x);
	float oracle_fp16_to_fp32(uint16_t x);
	void oracle_convert_fp32_to_fp16(const float *src, uint16_t *dst, size_t elements);
	void oracle_convert_fp16_to_fp32(const uint16_t *src, float *dst, size_t elements);

	/* src/backend/cpu/winograd/winograd_runtime.cpp:47-93 + def_winograd_kernels.cpp:165-184,380-424; weights [Cout,3,3,Cin] -> [36,Cout,Cin] */
	void oracle_winograd_weight_transform(int dtype, int filters_out, int filters_in, const void *weights, void *matrices, int invert);
	/* winograd_runtime.cpp:94-155 + avx2_winograd_kernels.cpp:241-264; input [B,H,W,C] -> [36, B*ceil(H/4)*ceil(W/4), C] */
	void oracle_winograd_input_transform(int dtype, int batch, int height, int width, int filters, const void *input, void *matrices);
	/* winograd_runtime.cpp:156-232,529-536 + avx2_winograd_kernels.cpp:266-279,611-622; matrices -> output [B,H,W,C], + bias, + ext, activation */
	void oracle_winograd_output_transform(int dtype, int batch, int height, int width, int filters, const void *matrices, void *output,
			const void *bias, const void *ext, int act);

	/*
	 * D = act(alpha * op(A) * op(B) + bias + beta * C) for `batch` matrices (src/backend/cpu/gemm/gemm.cpp:34-83, gemm_runtime.cpp:185-236,
	 * avx512f_kernels.cpp:45-70,790-870). stride_* are elements between consecutive matrices (0 = broadcast).
	 * k_tile restates the reference's split of K (inner_tile.K = 1024 for its AVX2 / AVX-512 kernels, gemm_runtime.cpp:103-143): each K
	 * tile is accumulated from zero, scaled by alpha and added to the value already stored in D (rounded to dtype in between);
	 * k_tile <= 0 accumulates the whole K extent in one pass.
	 */
	void oracle_gemm(int dtype, char opA, char opB, int M, int N, int K, int batch, float alpha, const void *A, size_t stride_a, const void *B,
			size_t stride_b, float beta, const void *C, void *D, size_t stride_c, const void *bias, int act, int k_tile);
	/* int8 x int8 -> int32, A [M,K], B [N,K] (src/backend/cuda/gemms.cpp:119-130 as called from src/layers/Conv2D.cpp:230) */
	void oracle_int8_gemm_nt(int M, int N, int K, const int8_t *A, const int8_t *B, int32_t *C);

	/* src/backend/cpu/conv_im2row.cpp:21-84; input [B,H,W,C] of element size esize -> [B*H*W, k*k*C], zeros outside */
	void oracle_im2row(int esize, int batch, int height, int width, int filters, int kernel_size, const void *input, void *output);
	/*
	 * explicit_gemm_forward (src/core/math.cpp:1595-1626): im2row + gemm_ex('n','t', beta = 1 on add) == act(conv(x,w) + bias + add),
	 * pad (k-1)/2, weights [Cout,k,k,Cin]. k_tile as in oracle_gemm.
	 */
	void oracle_conv2d_forward(int dtype, int batch, int height, int width, int filters_in, int filters_out, int kernel_size, const void *input,
			const void *weights, void *output, const void *bias, const void *add, int act, int k_tile);

	/* src/layers/quantization.cpp:39-43 — clamp(round_half_away(x)) to `bits` bits */
	int32_t oracle_quantize(float x, int bits);
	/* src/layers/Conv2D.cpp:240-308 (== test/backend/test_quantization.cpp:56-117); output_dtype INT8 or FLOAT32; ext may be NULL */
	void oracle_int8_conv2d_forward(int batch, int height, int width, int filters_in, int filters_out, int kernel_size, const int8_t *input,
			float input_scale, float input_shift, const int8_t *weights, const float *channel_scales, const float *bias, int output_dtype,
			void *output, float output_scale, float output_shift, const int8_t *ext, float ext_scale, float ext_shift, int act);
	/* the float tail of the above applied to given int32 accumulators [first_dim, last_dim] (output_dtype INT8, FLOAT32 or FLOAT16) */
	void oracle_quantized_scale_shift_act(int output_dtype, size_t first_dim, int last_dim, void *output, float output_scale, float output_shift,
			const int32_t *input, const float *scales, const float *bias, int act, const int8_t *ext, float ext_scale, float ext_shift);
	/* src/layers/quantization.cpp:55-93 with mode "per_first_dim", bits = 8: weights [rows, cols] fp32 -> int8 + channel_scales + folded bias */
	void oracle_quantize_weights(int rows, int cols, const float *weights, const float *bias, float input_scale, float input_shift,
			int8_t *q_weights, float *channel_scales, float *q_bias);

	/* src/backend/cpu/dispatcher.cpp:267-311 + def_misc_kernels.cpp:52-72: y = act(x + bias); bias may be NULL */
	void oracle_add_bias_act(int dtype, size_t first_dim, int last_dim, void *output, const void *input, const void *bias, int act);
	/* src/backend/cuda/kernels/tensor_op.cu:289-312: y = a1*x1 + a2*x2 + a3*x3 + beta*y (NULL inputs skipped) */
	void oracle_add_tensors(int dtype, size_t elements, float a1, const void *x1, float a2, const void *x2, float a3, const void *x3, float beta, void *y);
	/* src/backend/cpu/dispatcher.cpp:112-123,143-174: bit j of word (i, j/32) -> 1 / 0 */
	void oracle_unpack_input(int dtype, size_t first_dim, int last_dim, void *dst, const uint32_t *src);

	/* src/backend/cpu/avx_misc_kernels.cpp:53-112: row-wise softmax over [first_dim, last_dim] */
	void oracle_softmax_forward(int dtype, size_t first_dim, int last_dim, void *output, const void *input);
	/* src/backend/cpu/kernels/pooling_and_scaling.cpp:142-180: [batch, hw, channels] -> [batch, channels], y = alpha * mean + beta * y */
	void oracle_global_average_pooling_forward(int dtype, int batch, int hw, int channels, float alpha, const void *input, float beta,
			void *output);
	/* src/backend/cuda/kernels/batchnorm.cu:57-104: y = alpha * act(x * scale + shift) + beta * y with folded statistics */
	void oracle_batchnorm_inference(int dtype, size_t first_dim, int last_dim, float alpha, const void *input, const void *gamma,
			const void *bias, const float *avg_var, float beta, void *output, int act);
	/* src/backend/cpu/normalization.cpp:296-343: batch normalisation folded into the preceding layer's weights and bias, in place */
	void oracle_fold_batchnorm(int dtype, int channels, int other, int channels_last, void *layer_weights, void *layer_bias,
			const void *bn_weights, const void *bn_bias, const float *bn_avg_var);

	/* src/backend/cpu/normalization.cpp:452-486: y = (gamma * x) / (1e-6 + sqrt(mean x^2)) per row of [first_dim, last_dim]; gamma may be NULL */
	void oracle_rmsnorm_forward(int dtype, size_t first_dim, int last_dim, const void *input, void *output, const void *weights);
	/* src/backend/cpu/attention.cpp:142-214,395-431: softmax(q k^T / sqrt(head_dim) + relative-position bias) v per image and head;
	 * input [B, H, W, (3 - symmetric) * E] (q, k, v per token; k = q when symmetric), output [B, H, W, E],
	 * table [heads][table_size][round_up(table_size, 4)] or NULL */
	void oracle_multi_head_attention_forward(int dtype, int batch, int height, int width, int embedding, int num_heads, int symmetric,
			const void *input, void *output, const void *table, int table_size);

#ifdef __cplusplus
}
#endif

#endif /* MINML_ORACLE_H_ */
