/*
 * gd_minimax_m3_index_topk (forward): front end restating the rules of the reference's
 * src/ops/minimax_m3_index_topk/core_minimax_m3_index_topk.c:9-140: F16 index_q / index_k [N,H,Dh], I32 cu_seqlens
 * [B+1], result I32 topk_idx [Hkv,N,topk].  Kernels: ops/minimax_m3/hip.
 */
#include "../minimax_m3/minimax_m3_common.h"

gd_status gd_minimax_m3_index_topk(gd_context *ctx, const gd_tensor *index_q, const gd_tensor *index_k,
                                   const gd_tensor *cu_seqlens, const gd_minimax_m3_sparse_config *config,
                                   gd_tensor *topk_idx)
{
    gd_backend_minimax_m3_sparse_args args;
    gd_backend_tensor_view qv, kv, cv, tv;
    gd_tensor out;
    int64_t shape[3];
    if (topk_idx != NULL) memset(topk_idx, 0, sizeof(*topk_idx));
    if (ctx == NULL || index_q == NULL || index_k == NULL || cu_seqlens == NULL || topk_idx == NULL)
        return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, index_q));
    GD_TRY(gd_tensor_validate(ctx, index_k));
    GD_TRY(gd_tensor_validate(ctx, cu_seqlens));
    if (index_q->dtype != GD_DTYPE_F16 || index_k->dtype != GD_DTYPE_F16)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "minimax_m3 indexer requires f16 q/k");
    if (cu_seqlens->dtype != GD_DTYPE_I32) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "minimax_m3 indexer cu_seqlens must be i32");
    if (index_q->rank != 3U || index_k->rank != 3U || cu_seqlens->rank != 1U || cu_seqlens->shape[0] < 2 ||
        index_q->shape[0] <= 0 || index_q->shape[1] <= 0 || index_q->shape[2] <= 0 || index_k->shape[0] != index_q->shape[0] ||
        index_k->shape[1] != index_q->shape[1] || index_k->shape[2] != index_q->shape[2])
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "minimax_m3 indexer expects q/k [N,H,D] and cu [B+1]");
    if (index_q->shape[2] > M3_DH_MAX || index_q->shape[0] > (int64_t)INT_MAX)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "minimax_m3 indexer dimensions exceed kernel limits");
    if (!gd_tensor_is_contiguous(index_q) || !gd_tensor_is_contiguous(index_k) || !gd_tensor_is_contiguous(cu_seqlens))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "minimax_m3 indexer requires contiguous tensors");
    GD_TRY(gd_minimax_m3_resolve(ctx, index_q, config, &args));
    shape[0] = index_k->shape[1];
    shape[1] = index_q->shape[0];
    shape[2] = (int64_t)args.topk;
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_I32, 3U, shape, &out));
    if (!gd_op_tensor_view(index_q, &qv) || !gd_op_tensor_view(index_k, &kv) || !gd_op_tensor_view(cu_seqlens, &cv) ||
        !gd_op_tensor_view(&out, &tv))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "minimax_m3 indexer view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_minimax_m3_index_topk(gd_context_backend(ctx), &qv, &kv, &cv, &tv, &args),
                                "backend minimax_m3_index_topk failed"));
    *topk_idx = out;
    return GD_OK;
}
