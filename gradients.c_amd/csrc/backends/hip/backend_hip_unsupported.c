/*
 * Entry points of the reference's backend boundary (src/core/backend.h, src/core/backend_generated.h)
 * that are not on the inference decode path: training kernels (backward passes, losses, optimizer,
 * AMP, dropout), unary/binary operators the decoder does not call, batched matmuls, reductions,
 * permute/split, the backward pass of the MiniMax-M3 sparse attention.  The reference's core references all of them, so a
 * drop-in backend has to define them; like the reference's null backend
 * (src/backends/null/backend_null.c, src/backends/null/backend_generated.c) each one reports
 * GD_ERR_UNSUPPORTED and touches nothing.
 *
 * The definitions take no named parameters (the arguments the caller passes are ignored), which keeps
 * this file independent of the argument structs of operators this backend does not implement.
 */
#include "gd_backend_hip.h"

#pragma GCC visibility push(default)

#define GD_UNSUPPORTED_ENTRY(name) \
    gd_status name();              \
    gd_status name() { return GD_ERR_UNSUPPORTED; }

GD_UNSUPPORTED_ENTRY(gd_backend_accumulate)
GD_UNSUPPORTED_ENTRY(gd_backend_adamw_batch)
GD_UNSUPPORTED_ENTRY(gd_backend_amp_begin_step)
GD_UNSUPPORTED_ENTRY(gd_backend_amp_fill_scale)
GD_UNSUPPORTED_ENTRY(gd_backend_amp_finish_step)
GD_UNSUPPORTED_ENTRY(gd_backend_amp_scale)
GD_UNSUPPORTED_ENTRY(gd_backend_amp_unscale_batch)
GD_UNSUPPORTED_ENTRY(gd_backend_batched_matmul)
GD_UNSUPPORTED_ENTRY(gd_backend_batched_matmul_nt)
GD_UNSUPPORTED_ENTRY(gd_backend_batched_matmul_tn)
GD_UNSUPPORTED_ENTRY(gd_backend_broadcast_axis)
GD_UNSUPPORTED_ENTRY(gd_backend_broadcast_scalar)
GD_UNSUPPORTED_ENTRY(gd_backend_concat_from_full)
GD_UNSUPPORTED_ENTRY(gd_backend_cross_entropy_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_cross_entropy_backward_stats)
GD_UNSUPPORTED_ENTRY(gd_backend_cross_entropy_loss)
GD_UNSUPPORTED_ENTRY(gd_backend_cross_entropy_loss_stats)
GD_UNSUPPORTED_ENTRY(gd_backend_dropout_add_forward)
GD_UNSUPPORTED_ENTRY(gd_backend_dropout_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_dropout_backward_mask)
GD_UNSUPPORTED_ENTRY(gd_backend_dropout_forward)
GD_UNSUPPORTED_ENTRY(gd_backend_embedding_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_grad_clip_scale)
GD_UNSUPPORTED_ENTRY(gd_backend_huber_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_huber_forward)
GD_UNSUPPORTED_ENTRY(gd_backend_lm_cross_entropy_backward_chunk)
GD_UNSUPPORTED_ENTRY(gd_backend_lm_cross_entropy_finalize)
GD_UNSUPPORTED_ENTRY(gd_backend_lm_cross_entropy_online_update)
GD_UNSUPPORTED_ENTRY(gd_backend_lm_cross_entropy_reduce_normalize)
GD_UNSUPPORTED_ENTRY(gd_backend_matmul_tn)
GD_UNSUPPORTED_ENTRY(gd_backend_minimax_m3_sparse_attention_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_mse_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_mse_forward)
GD_UNSUPPORTED_ENTRY(gd_backend_mul)
GD_UNSUPPORTED_ENTRY(gd_backend_mul_backward_direct)
GD_UNSUPPORTED_ENTRY(gd_backend_mul_reduce_suffix)
GD_UNSUPPORTED_ENTRY(gd_backend_permute)
GD_UNSUPPORTED_ENTRY(gd_backend_powlu_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_powlu_forward)
GD_UNSUPPORTED_ENTRY(gd_backend_powlu_split_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_powlu_split_forward)
GD_UNSUPPORTED_ENTRY(gd_backend_qkv_split_rope_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_reduce_axis)
GD_UNSUPPORTED_ENTRY(gd_backend_reduce_broadcast)
GD_UNSUPPORTED_ENTRY(gd_backend_reduce_contiguous)
GD_UNSUPPORTED_ENTRY(gd_backend_reduce_rows)
GD_UNSUPPORTED_ENTRY(gd_backend_relu)
GD_UNSUPPORTED_ENTRY(gd_backend_relu_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_rms_norm_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_rms_norm_backward_stats)
GD_UNSUPPORTED_ENTRY(gd_backend_rms_norm_forward_stats)
GD_UNSUPPORTED_ENTRY(gd_backend_rms_norm_inv)
GD_UNSUPPORTED_ENTRY(gd_backend_rms_norm_weight_backward_stats)
GD_UNSUPPORTED_ENTRY(gd_backend_rope)
GD_UNSUPPORTED_ENTRY(gd_backend_rope_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_scale)
GD_UNSUPPORTED_ENTRY(gd_backend_sdpa_varlen_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_sigmoid)
GD_UNSUPPORTED_ENTRY(gd_backend_sigmoid_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_sigmoid_backward_from_output)
GD_UNSUPPORTED_ENTRY(gd_backend_split_from_full)
GD_UNSUPPORTED_ENTRY(gd_backend_split_to_full)
GD_UNSUPPORTED_ENTRY(gd_backend_sub)
GD_UNSUPPORTED_ENTRY(gd_backend_swiglu_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_swiglu_forward)
GD_UNSUPPORTED_ENTRY(gd_backend_swiglu_split_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_tanh)
GD_UNSUPPORTED_ENTRY(gd_backend_tanh_backward)
GD_UNSUPPORTED_ENTRY(gd_backend_tanh_backward_from_output)

#pragma GCC visibility pop
