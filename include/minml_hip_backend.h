/*
 * minml_hip_backend.h — C-ABI of the MI355X (gfx950) HIP backend for minml's convolution / GEMM inference path.
 *
 * Every entry point mirrors, argument for argument, the device-backend entry point that minml's core dispatcher
 * (reference: src/core/math.cpp, src/core/ml_memory.cpp, src/core/Context.cpp, src/core/Event.cpp) calls in its
 * DeviceType::CUDA branch, declared in the reference at include/minml/backend/cuda_backend.h. The library exports
 * each function twice: under the hip_* name declared here and under the cuda_* name of the reference, so that the
 * unmodified dispatcher links against it in place of src/backend/cuda_dummy_backend.cpp.
 *
 * Conventions (same as the reference backends):
 *   - descriptors are passed by value; all tensors are dense, row-major, NHWC for images;
 *   - an absent optional tensor is signalled by data == NULL (reference: include/minml/backend/backend_utils.hpp:138-141);
 *   - every call is asynchronous on the context's stream; hip_synchronize_with_context is the only barrier;
 *   - failures are C++ exceptions crossing the C boundary (std::runtime_error / std::logic_error), never return codes
 *     (reference: src/backend/cuda_dummy_backend.cpp:25-27, src/backend/cpu/winograd/winograd_runtime.cpp:516).
 */
#ifndef MINML_HIP_BACKEND_H_
#define MINML_HIP_BACKEND_H_

#include <stddef.h>
#include <stdbool.h>

#ifdef __cplusplus
extern "C"
{
#endif

/* ---- descriptor types: binary-compatible with reference include/minml/backend/backend_types.h:28-73 ---- */
#ifndef MINML_BACKEND_BACKEND_TYPES_H_
	typedef struct
	{
		int rank;
		int dim[6];
	} mlShape_t;

	typedef struct
	{
		float scale;
		float shift;
	} mlQuantizationData_t;

	typedef enum
	{
		DTYPE_UNKNOWN, DTYPE_FLOAT8, DTYPE_FLOAT16, DTYPE_FLOAT32, DTYPE_FLOAT64, DTYPE_UINT8, DTYPE_INT8, DTYPE_INT16, DTYPE_INT32
	} mlDataType_t;

	typedef enum
	{
		ACTIVATION_LINEAR, ACTIVATION_SIGMOID, ACTIVATION_TANH, ACTIVATION_RELU, ACTIVATION_LEAKY_RELU, ACTIVATION_EXP
	} mlActivationType_t;

	typedef struct
	{
		void *data;
		mlDataType_t dtype;
		int rank;
		int dim[6];
	} mlTensor_t;

	typedef void *mlContext_t;
	typedef void *mlEvent_t;
#endif

	/* ---- device identity (reference: cuda_backend.h:49-57, src/backend/cuda/cuda_properties.cpp) ---- */
	int hip_get_number_of_devices(void);
	int hip_get_memory(int index); /* in MB */
	bool hip_supports_type(int index, mlDataType_t dtype); /* FLOAT16, FLOAT32, INT32, INT8 (cuda_properties.cpp:222-244) */
	const char* hip_get_device_info(int index);
	const char* hip_get_device_features(int index);
	void hip_enable_tf32(mlContext_t context, bool b); /* accepted and ignored: fp32 GEMMs run in full fp32 */

	/* ---- context = one stream (reference: cuda_backend.h:59-63, src/backend/cuda/cuda_context.cpp) ---- */
	mlContext_t hip_create_context(int device_index);
	void hip_synchronize_with_context(mlContext_t context);
	bool hip_is_context_ready(mlContext_t context);
	void hip_destroy_context(mlContext_t context);

	/* ---- events (reference: cuda_backend.h:65-70, src/backend/cuda/cuda_event.cpp) ---- */
	mlEvent_t hip_create_event(mlContext_t context); /* records on the context's stream */
	double hip_get_time_between_events(mlEvent_t start, mlEvent_t end); /* seconds */
	void hip_wait_for_event(mlEvent_t event);
	bool hip_is_event_ready(mlEvent_t event);
	void hip_destroy_event(mlEvent_t event);

	/* ---- memory (reference: cuda_backend.h:72-83, src/backend/cuda/cuda_memory.cu:133-276); context == NULL => synchronous ---- */
	void* hip_malloc(int device_index, size_t count);
	void hip_page_lock(void *ptr, size_t count); /* no-op: registering existing host memory is not available on the target hosts */
	void hip_page_unlock(void *ptr);
	void hip_free(void *ptr);
	void* hip_create_view(void *src, size_t offset, size_t count); /* src + offset, non-owning */
	void hip_destroy_view(void *ptr);
	void hip_memset(mlContext_t context, void *dst, size_t dst_offset, size_t dst_count, const void *src, size_t src_count); /* pattern of 0,1,2,4,8 bytes */
	void hip_memcpy_within_device(mlContext_t context, void *dst, size_t dst_offset, const void *src, size_t src_offset, size_t count);
	void hip_memcpy_from_host(mlContext_t context, void *dst, size_t dst_offset, const void *src, size_t count);
	void hip_memcpy_to_host(mlContext_t context, void *dst, const void *src, size_t src_offset, size_t count);

	/* ---- step before the path (reference: cuda_backend.h:85-88, src/backend/cpu/dispatcher.cpp:112-188) ---- */
	void hip_unpack_input(mlContext_t context, mlShape_t shape, mlDataType_t dst_dtype, void *dst, const void *src);
	void hip_convert_type(mlContext_t context, void *dst, mlDataType_t dst_dtype, const void *src, mlDataType_t src_dtype, int elements);

	/* ---- Winograd F(4x4,3x3) transforms (reference: cuda_backend.h:96-100; arithmetic follows the CPU backend,
	 *      src/backend/cpu/winograd/winograd_runtime.cpp:47-232,519-536). The kernel size is derived from
	 *      matrices.dim[0] = (tile + k - 1)^2; any (tile, kernel, dtype) other than (4, 3, fp16|fp32) throws
	 *      std::runtime_error("No suitable Winograd transform runtime"). ---- */
	void hip_winograd_weight_transform(mlContext_t context, int tile_size, const mlTensor_t w, mlTensor_t matrices, bool invert);
	void hip_winograd_input_transform(mlContext_t context, int tile_size, const mlTensor_t x, mlTensor_t matrices);
	void hip_winograd_output_transform(mlContext_t context, int tile_size, const mlTensor_t matrices, const mlTensor_t bias, const mlTensor_t ext,
			mlTensor_t y, mlActivationType_t act);
	/*
	 * hip_winograd_output_input_transform: hip_winograd_output_transform of one layer followed by hip_winograd_input_transform of the
	 * next 3x3 layer on the result, in one launch; bit-identical to the two calls. `output` may be NULL when y is not needed in
	 * memory (for channel counts that are multiples of 64; other shapes run the two transforms through `output`, which must then be
	 * given). No counterpart in the reference, whose layers call the two transforms separately (src/layers/Conv2D.cpp:365-378): it
	 * removes one write and one read of the activation tensor per layer from the Winograd path.
	 */
	void hip_winograd_output_input_transform(mlContext_t context, int tile_size, const mlTensor_t matrices, const mlTensor_t bias, const mlTensor_t ext,
			mlShape_t output_shape, void *output, mlActivationType_t act, mlTensor_t next_matrices);

	/*
	 * hip_winograd_layer_forward: one whole 3x3 layer between two sets of Winograd matrices, in one launch:
	 *   input_matrices [36, tiles, Cin] x weight_matrices [36, Cout, Cin]^T -> output transform (+ bias, + ext, act) -> y (`output`, may be
	 *   NULL) -> input transform -> next_matrices [36, tiles, Cout]
	 * i.e. hip_gemm_batched followed by hip_winograd_output_input_transform, with identical results. For fp16, 256 -> 256 channels,
	 * boards of 16 tiles (13x13 .. 16x16), batches that are multiples of 4 (at least 32) and linear / ReLU activation the product never
	 * leaves the L2 cache; every other case runs the two calls through `output_matrices` [36, tiles, Cout], which must then be given.
	 * No counterpart in the reference (src/layers/Conv2D.cpp:365-378 calls the three steps one by one).
	 * EXPERIMENTAL, opt-in: the one-launch form assumes that the device places its 512 workgroups 64 to an XCD, all resident at once,
	 * i.e. that nothing else runs on the GPU; it measures slower than the two calls, which remain the recommended sequence. A caller
	 * that uses it must check hip_winograd_layer_errors after the pass.
	 * hip_winograd_layer_errors waits for the context's stream and returns how many workgroups of such launches gave up waiting for
	 * one another since the last call (0 unless the device was shared with other work; results are then invalid).
	 */
	void hip_winograd_layer_forward(mlContext_t context, int tile_size, const mlTensor_t input_matrices, const mlTensor_t weight_matrices,
			mlTensor_t output_matrices, const mlTensor_t bias, const mlTensor_t ext, mlShape_t output_shape, void *output, mlActivationType_t act,
			mlTensor_t next_matrices);
	int hip_winograd_layer_errors(mlContext_t context);
	/*
	 * hip_winograd_layer_forward_static: hip_winograd_layer_forward with identical arguments and results that allocates nothing, neither
	 * on the first call nor later. No counterpart in the reference; it is for callers that cannot allocate device memory: code under
	 * HIP graph capture, serving loops and harnesses that forbid hipMalloc. hip_winograd_layer_forward keeps the counters and the
	 * product scratch of its one-launch form in the context's growable workspace (hipMalloc on first use); this entry point keeps them in
	 * a static device array of the library (18.1 MiB per GPU, held until the process ends) and clears its counters with a kernel. Limit:
	 * at most 4096 images per call at the shape that uses the array (256 -> 256 channels, 16 tiles per image, fp16, 256 CUs; larger
	 * batches of it are rejected with std::logic_error: split them); every other shape runs as the batched product followed by the fused
	 * transform, which use no library-side memory at all and take any batch. All calls on one GPU share that
	 * array: calls that overlap on one GPU (two contexts, two threads) race; calls on one context run in stream order and are safe.
	 */
	void hip_winograd_layer_forward_static(mlContext_t context, int tile_size, const mlTensor_t input_matrices, const mlTensor_t weight_matrices,
			mlTensor_t output_matrices, const mlTensor_t bias, const mlTensor_t ext, mlShape_t output_shape, void *output, mlActivationType_t act,
			mlTensor_t next_matrices);

	/* ---- GEMMs (reference: cuda_backend.h:147-154; semantics of src/backend/cpu/gemm/gemm.cpp:34-83).
	 *      C.dtype == INT32 selects the int8 x int8 -> int32 product (src/backend/cuda/gemms.cpp:119-130). ---- */
	void hip_gemm_v2(mlContext_t context, char opA, char opB, float alpha, const mlTensor_t A, const mlTensor_t B, float beta, mlTensor_t C);
	/* grouped product (reference: cuda_backend.h:239-240, src/backend/cuda/kernels/group_conv.cu:120-203; reached from the grouped 1x1
	 * convolution, src/layers/Conv2D.cpp:341-349 via src/core/math.cpp:1079-1093): the last dimension of A, B and C is split into `groups`
	 * equal column ranges and group i computes C[:, i-th range] = alpha * op(A[:, i-th range]) * op(B[:, i-th range]) + beta * C[:, i-th range].
	 * The reference has no CPU implementation of it; it is checked against the definition (one plain product per group). */
	void hip_group_gemm(mlContext_t context, char opA, char opB, float alpha, const mlTensor_t A, const mlTensor_t B, float beta, mlTensor_t C, int groups);
	void hip_gemm_batched_v2(mlContext_t context, char opA, char opB, float alpha, const mlTensor_t A, const mlTensor_t B, float beta, mlTensor_t C);
	void hip_gemm(mlContext_t context, mlDataType_t dtype, mlShape_t shape_C, void *C, mlShape_t shape_A, const void *A, mlShape_t shape_B,
			const void *B, char opA, char opB, float alpha, float beta);
	void hip_gemm_batched(mlContext_t context, mlDataType_t dtype, mlShape_t shape_C, void *C, mlShape_t shape_A, const void *A, mlShape_t shape_B,
			const void *B, char opA, char opB, float alpha, float beta);
	/* D = act(alpha * op_A(A) * op_B(B) + bias + beta * C)  (reference: cuda_backend.h:160-162, src/backend/cpu/gemm/gemm.cpp:66-83) */
	void hip_gemm_ex(mlContext_t context, mlDataType_t dtype, mlShape_t shape_D, void *D, float alpha, char opA, mlShape_t shape_A, const void *A,
			char opB, mlShape_t shape_B, const void *B, float beta, mlShape_t shape_C, const void *C, const void *bias, mlActivationType_t act);

	/* ---- fused convolution y = act(conv(x, w) + bias + add), stride 1, pad (k-1)/2, weights [Cout,k,k,Cin]
	 *      (reference: cuda_backend.h:103-106, src/core/math.cpp:399-416; oracle = explicit_gemm_forward,
	 *      src/core/math.cpp:1595-1626). dtype INT8 is not part of this entry point (see hip_quantized_conv_forward). ---- */
	void hip_convolution_implicit_gemm_forward(mlContext_t context, mlDataType_t dtype, mlShape_t input_shape, mlShape_t weights_shape,
			const void *input, const void *weights, void *output, const void *bias, const void *add, mlActivationType_t act);
	void hip_im2row(mlContext_t context, mlDataType_t dtype, mlShape_t input_shape, void *output, const void *input, int kernel_size, bool invert,
			const void *padding); /* reference: cuda_backend.h:326-327; `padding` = pointer to one host element or NULL for zeros */

	/* ---- int8 epilogue (reference: cuda_backend.h:323-325; arithmetic of the CPU path, src/layers/Conv2D.cpp:284-306) ---- */
	void hip_quantized_scale_shift_act(mlContext_t context, mlDataType_t dtype, mlShape_t shape, void *output, mlQuantizationData_t output_qd,
			const void *input, const void *scales, const void *bias, mlActivationType_t act, const void *ext, mlQuantizationData_t ext_qd);

	/* ---- non-fused fallbacks (reference: cuda_backend.h:172-173,222-223,296-297) ---- */
	void hip_add_bias_act(mlContext_t context, float alpha, const mlTensor_t x, const mlTensor_t b, float beta, mlTensor_t y, mlActivationType_t act);
	void hip_activation_forward(mlContext_t context, float alpha, const mlTensor_t x, float beta, mlTensor_t y, mlActivationType_t act);
	void hip_add_tensors(mlContext_t context, float alpha1, const mlTensor_t x1, float alpha2, const mlTensor_t x2, float alpha3, const mlTensor_t x3,
			float beta, mlTensor_t y);
	void hip_scale_tensor(mlContext_t context, float alpha, mlTensor_t x); /* x *= alpha (reference: cuda_backend.h:295) */

	/* ---- steps after the path: policy softmax, pooling before a value head, batch normalisation in inference mode and its folding
	 *      into the preceding layer (reference: cuda_backend.h:127,177-178,185-186,230; arithmetic of the CPU backend where it has one:
	 *      src/backend/cpu/avx_misc_kernels.cpp:53-112, src/backend/cpu/kernels/pooling_and_scaling.cpp:142-180,
	 *      src/backend/cpu/normalization.cpp:296-343; batchnorm_inference follows src/backend/cuda/kernels/batchnorm.cu:57-104,
	 *      its CPU dispatch being commented out in src/core/math.cpp:722-737). fp16 and fp32. ---- */
	void hip_softmax_forward(mlContext_t context, mlDataType_t dtype, mlShape_t shape, void *output, const void *input); /* rows of the last dim; in place allowed */
	void hip_global_average_pooling_forward(mlContext_t context, float alpha, const mlTensor_t x, float beta, mlTensor_t y); /* [B,H,W,C] -> [B,C] */
	void hip_batchnorm_inference(mlContext_t context, float alpha, const mlTensor_t x, const mlTensor_t w, const mlTensor_t b, const mlTensor_t avg_var,
			float beta, mlTensor_t y, mlActivationType_t act); /* avg_var fp32 [2, C]: means, variances; w / b may be empty */
	void hip_fold_batchnorm(mlContext_t context, mlTensor_t layer_weights, mlTensor_t layer_bias, const mlTensor_t bn_weights, const mlTensor_t bn_bias,
			const mlTensor_t bn_avg_var); /* in place; rank-3 weights are depthwise (channels last), others channels first */

	/* ---- transformer-block pieces of the hybrid networks: RMS normalisation and multi-head self-attention over the board's tokens with a
	 *      2-D relative-position bias (reference: cuda_backend.h:199-200,207-210; arithmetic of the CPU backend:
	 *      src/backend/cpu/normalization.cpp:452-486, src/backend/cpu/attention.cpp:142-214,395-431). fp16 and fp32, inference only. ---- */
	void hip_rmsnorm_forward(mlContext_t context, mlShape_t shape, mlDataType_t dtype, const void *input, void *output,
			const void *weights); /* rows of the last dim; weights (gamma) may be NULL */
	int hip_multi_head_attention_get_workspace_size(mlShape_t input_shape, mlShape_t weights_shape, int num_heads,
			bool training); /* elements; 0 for inference: the attention matrix never leaves the chip */
	void hip_multi_head_attention_forward(mlContext_t context, mlShape_t input_shape, mlShape_t weights_shape, mlShape_t bias_shape, mlDataType_t dtype,
			const void *input, void *output, const void *weights, const void *bias, void *workspace, void *backward_data, int num_heads,
			bool symmetric); /* input [B,H,W,(3 - symmetric) E] = q,k,v per token; weights = position table [heads, 2r-1, round_up(2r-1, 4)] or NULL;
			                    bias and workspace unused; backward_data must be NULL */

	/* ---- mixture of experts: the feed-forward half of the hybrid networks' transformer blocks (reference: cuda_backend.h:245-265,
	 *      src/backend/cuda/kernels/moe.cu, callers src/layers/{Router,GatherTokens,MixtureOfExperts,ScatterTokens}.cpp). The reference
	 *      implements these for its CUDA backend only (src/core/math.cpp:1328-1491 does nothing on the CPU). fp16 and fp32, inference only.
	 *      x = router scores [B, H, W, E]; indices_and_values [B, 2, E, K] in the tensors' type: plane 0 = token index held by slot k of
	 *      expert e (-1 = empty), plane 1 = its gate. Equal scores are ordered by ascending token index. ---- */
	void hip_expert_choice_routing_forward(mlContext_t context, const mlTensor_t x,
			mlTensor_t indices_and_values); /* every expert takes its K best tokens of each image, best first; gate = sigmoid(score) (moe.cu:438-479) */
	void hip_token_choice_routing_forward(mlContext_t context, const mlTensor_t x, const mlTensor_t bias,
			mlTensor_t indices_and_values); /* every token takes the expert with the largest score + bias[E]; gate = its softmax; K best per expert (moe.cu:191-350) */
	void hip_hash_routing(mlContext_t context, const mlTensor_t x, mlTensor_t indices_and_values); /* token k * E + e -> slot k of expert e, gate 1 (moe.cu:167-189) */
	void hip_gather_tokens_forward(mlContext_t context, const mlTensor_t x, const mlTensor_t indices_and_values, float beta,
			mlTensor_t y); /* x [B, H, W, C] -> y [B, K, E, C] = x[token] + beta * y; empty slots: beta * y (0 when beta = 0) (moe.cu:505-532) */
	void hip_moe_forward(mlContext_t context, const mlTensor_t x, const mlTensor_t w, const mlTensor_t b, float beta, mlTensor_t y,
			mlActivationType_t act); /* y [B, K, E, N] = act(x [B, K, E, C] . w[e] [N, C]^T + b [E, N] + beta * y), one dense layer per expert (moe.cu:1395-1432) */
	void hip_scatter_tokens_forward(mlContext_t context, const mlTensor_t x, const mlTensor_t indices_and_values, float beta,
			mlTensor_t y); /* y [B, H, W, C] = beta * y + sum over the slots holding each token of gate * x [B, K, E, C], in fp32, experts ascending (moe.cu:559-582).
			                * A token may hold at most one slot per expert, as every router of this library and of the reference writes its table; of
			                * duplicates in a hand-made table only the lowest slot counts, where the reference's atomic additions would add them all. */

	/* ---- additions with no counterpart in the reference ABI ----
	 * hip_quantized_conv_forward: the whole int8 convolution of reference src/layers/Conv2D.cpp:240-308 (int8 implicit GEMM with
	 * zero-point padding, int32 accumulation, per-channel scale + bias, optional int8 residual, activation, requantisation)
	 * in one launch, so that neither the im2row matrix nor the int32 accumulators touch HBM. output dtype INT8 or FLOAT32. */
	void hip_quantized_conv_forward(mlContext_t context, mlShape_t input_shape, mlShape_t weights_shape, const void *input,
			mlQuantizationData_t input_qd, const void *weights, const void *scales, const void *bias, mlDataType_t output_dtype, void *output,
			mlQuantizationData_t output_qd, const void *ext, mlQuantizationData_t ext_qd, mlActivationType_t act);
	/* hip_get_stream: the hipStream_t of a context, for callers that time or capture work on it. */
	void* hip_get_stream(mlContext_t context);
	/*
	 * Recording a pass as a HIP graph (no counterpart in the reference, whose layers launch kernel by kernel). Between
	 * hip_graph_begin_capture and hip_graph_end_capture the calls made on the context are recorded instead of executed;
	 * hip_graph_launch replays them, in order, on the context's stream with one submission. For passes made of many short dependent
	 * launches (small batches) the host's cost per launch bounds the pass, and the replay removes it. Buffers are recorded by address:
	 * the replay reads and writes the same tensors. Record only after one ordinary pass (first-use work such as weight transforms and
	 * workspace growth synchronises or allocates, which a recording cannot hold), and never hip_winograd_layer_errors, copies to or
	 * from pageable host memory, or context-less (NULL) memory calls.
	 */
	typedef void *mlGraph_t;
	void hip_graph_begin_capture(mlContext_t context);
	mlGraph_t hip_graph_end_capture(mlContext_t context);
	void hip_graph_launch(mlContext_t context, mlGraph_t graph);
	void hip_graph_destroy(mlGraph_t graph);

	/*
	 * Error capture for hosts that cannot catch C++ exceptions (no counterpart in the reference, whose only callers are C++). Every entry
	 * point above reports errors by throwing std::logic_error / std::runtime_error, as the reference's backends do. After
	 * hip_set_error_capture(1) an entry point that fails records the exception instead, returns normally (zero / null where it returns
	 * a value) and has done none of its work; hip_take_last_error copies the message of the first failure since its last call into
	 * `buffer` (at most size - 1 characters), clears it and returns 0 (no failure), 1 (std::logic_error: a bad argument), 2
	 * (std::runtime_error: the device or the runtime refused) or 3 (anything else). hip_error_flag_address returns the address of the
	 * int that holds that code (non-zero while a failure waits to be taken), for hosts that want to test it without a call.
	 * Process-wide; off by default.
	 */
	void hip_set_error_capture(int enabled);
	int hip_take_last_error(char *buffer, int size);
	const int* hip_error_flag_address(void);

#ifdef __cplusplus
}
#endif

#endif /* MINML_HIP_BACKEND_H_ */
