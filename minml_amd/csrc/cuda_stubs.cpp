/*
 * cuda_stubs.cpp — link-completeness for the drop-in: minml's core dispatcher (reference: the .cpp files of src/core) references every cuda_*
 * symbol of include/minml/backend/cuda_backend.h, whether a model uses it or not. The entry points of the convolution / GEMM
 * inference path are real (each hip_* function is also exported under its cuda_* name next to its definition); every other symbol of
 * that header is defined here and throws, which is how the reference itself fills a backend that is not built
 * (src/backend/cuda_dummy_backend.cpp:25-27 throws NotImplemented from every function).
 *
 * The symbols have C linkage, so only their names matter to the linker; a stub never reads its arguments and never returns.
 */
#include <stdexcept>
#include <string>

namespace
{
	[[noreturn]] void not_implemented(const char *name)
	{
		throw std::logic_error(std::string("function '") + name + "' is not implemented by the HIP backend (outside the convolution / GEMM inference path)");
	}
}

#define MLHIP_STUB(name) extern "C" void name() { not_implemented(#name); }

/* layout changes */
MLHIP_STUB(cuda_transpose_021)
MLHIP_STUB(cuda_space_to_depth)
MLHIP_STUB(cuda_depth_to_space)
MLHIP_STUB(cuda_transpose)
MLHIP_STUB(cuda_window_partitioning)
MLHIP_STUB(cuda_window_merging)
MLHIP_STUB(cuda_channel_shuffle)
/* training halves of the Winograd path */
MLHIP_STUB(cuda_winograd_gradient_transform)
MLHIP_STUB(cuda_winograd_update_transform)
/* depthwise convolution */
MLHIP_STUB(cuda_depthwise_conv_forward)
MLHIP_STUB(cuda_depthwise_conv_backward)
MLHIP_STUB(cuda_depthwise_conv_update)
MLHIP_STUB(cudnn_depthwise_conv_forward)
MLHIP_STUB(cudnn_depthwise_conv_backward)
MLHIP_STUB(cudnn_depthwise_conv_update)
MLHIP_STUB(cuda_quantized_depthwise_conv_forward)
/* pooling and scaling */
MLHIP_STUB(cuda_average_pooling_forward)
MLHIP_STUB(cuda_average_pooling_backward)
MLHIP_STUB(cuda_global_average_pooling_backward)
MLHIP_STUB(cuda_channel_scaling_forward)
MLHIP_STUB(cuda_channel_scaling_backward)
MLHIP_STUB(cuda_channel_average_pooling_forward)
MLHIP_STUB(cuda_channel_average_pooling_backward)
MLHIP_STUB(cuda_spatial_scaling_forward)
MLHIP_STUB(cuda_spatial_scaling_backward)
MLHIP_STUB(cuda_learnable_scaling_forward)
MLHIP_STUB(cuda_learnable_scaling_backward)
/* normalisation */
MLHIP_STUB(cuda_batchnorm_forward)
MLHIP_STUB(cuda_batchnorm_backward)
MLHIP_STUB(cuda_batchnorm_update)
MLHIP_STUB(cuda_layernorm_forward)
MLHIP_STUB(cuda_layernorm_backward)
MLHIP_STUB(cuda_rmsnorm_backward)
/* attention, mixture of experts */
MLHIP_STUB(cuda_multi_head_attention_backward)
MLHIP_STUB(cuda_token_choice_routing_backward)
MLHIP_STUB(cuda_expert_choice_routing_backward)
MLHIP_STUB(cuda_select_top_k)
MLHIP_STUB(cuda_gather_tokens_backward)
MLHIP_STUB(cuda_scatter_tokens_backward)
MLHIP_STUB(cuda_moe_backward)
/* backward passes, softmax, tensor helpers */
MLHIP_STUB(cuda_activation_backward)
MLHIP_STUB(cuda_softmax_backward)
MLHIP_STUB(cuda_fused_act_bias_copy_backward)
MLHIP_STUB(cuda_emulate_low_precision)
MLHIP_STUB(cuda_multiply_tensors)
MLHIP_STUB(cuda_sum_over_first_dim)
MLHIP_STUB(cuda_dequantize)
/* losses and optimisers */
MLHIP_STUB(cuda_l2_norm)
MLHIP_STUB(cuda_mean_squared_loss)
MLHIP_STUB(cuda_cross_entropy_loss)
MLHIP_STUB(cuda_mean_squared_gradient)
MLHIP_STUB(cuda_cross_entropy_gradient)
MLHIP_STUB(cuda_fused_radam_optimize)
MLHIP_STUB(cuda_fused_lion_optimize)
MLHIP_STUB(cuda_fused_is_nan_or_inf)
MLHIP_STUB(cuda_fused_l2_regularization)
MLHIP_STUB(cuda_combined_loss)
