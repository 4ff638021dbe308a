/*
 * gd_minimax_m3_sparse_attention (forward): front end restating the rules of the reference's
 * src/ops/minimax_m3_sparse_attention/core_minimax_m3_sparse_attention.c:14-130: F16 q / k / v [N,H,Dh], I32
 * cu_seqlens [B+1] and topk_idx [Hkv,N,topk].  Kernels: ops/minimax_m3/hip.
 */
#include "../minimax_m3/minimax_m3_common.h"

gd_status gd_minimax_m3_sparse_attention(gd_context *ctx, const gd_tensor *q, const gd_tensor *k, const gd_tensor *v,
                                         const gd_tensor *cu_seqlens, const gd_tensor *topk_idx,
                                         const gd_minimax_m3_sparse_config *config, gd_tensor *out)
{
    gd_backend_minimax_m3_sparse_args args;
    gd_backend_tensor_view qv, kv, vv, cv, tv, ov;
    gd_tensor o;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || q == NULL || k == NULL || v == NULL || cu_seqlens == NULL || topk_idx == NULL || out == NULL)
        return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, q));
    GD_TRY(gd_tensor_validate(ctx, k));
    GD_TRY(gd_tensor_validate(ctx, v));
    GD_TRY(gd_tensor_validate(ctx, cu_seqlens));
    GD_TRY(gd_tensor_validate(ctx, topk_idx));
    if (q->dtype != GD_DTYPE_F16 || k->dtype != q->dtype || v->dtype != q->dtype)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "minimax_m3 sparse attention requires f16 q/k/v");
    if (cu_seqlens->dtype != GD_DTYPE_I32 || topk_idx->dtype != GD_DTYPE_I32)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "minimax_m3 sparse attention metadata must be i32");
    if (q->rank != 3U || k->rank != 3U || v->rank != 3U || cu_seqlens->rank != 1U || topk_idx->rank != 3U ||
        cu_seqlens->shape[0] < 2 || q->shape[0] <= 0 || q->shape[1] <= 0 || q->shape[2] <= 0 || k->shape[0] != q->shape[0] ||
        v->shape[0] != q->shape[0] || k->shape[1] <= 0 || v->shape[1] != k->shape[1] || k->shape[2] != q->shape[2] ||
        v->shape[2] != q->shape[2] || (q->shape[1] % k->shape[1]) != 0 || topk_idx->shape[0] != k->shape[1] ||
        topk_idx->shape[1] != q->shape[0])
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "minimax_m3 sparse attention shape mismatch");
    if (q->shape[2] > M3_DH_MAX || q->shape[0] > (int64_t)INT_MAX)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "minimax_m3 sparse attention dimensions exceed kernel limits");
    if (!gd_tensor_is_contiguous(q) || !gd_tensor_is_contiguous(k) || !gd_tensor_is_contiguous(v) ||
        !gd_tensor_is_contiguous(cu_seqlens) || !gd_tensor_is_contiguous(topk_idx))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "minimax_m3 sparse attention requires contiguous tensors");
    GD_TRY(gd_minimax_m3_resolve(ctx, q, config, &args));
    if (topk_idx->shape[2] != (int64_t)args.topk) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "minimax_m3 topk shape/config mismatch");
    GD_TRY(gd_tensor_alloc_like_shape(ctx, q->dtype, 3U, q->shape, &o));
    if (!gd_op_tensor_view(q, &qv) || !gd_op_tensor_view(k, &kv) || !gd_op_tensor_view(v, &vv) ||
        !gd_op_tensor_view(cu_seqlens, &cv) || !gd_op_tensor_view(topk_idx, &tv) || !gd_op_tensor_view(&o, &ov))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "minimax_m3 sparse attention view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_minimax_m3_sparse_attention(gd_context_backend(ctx), &qv, &kv, &vv, &cv, &tv,
                                                                              &ov, &args),
                                "backend minimax_m3_sparse_attention failed"));
    *out = o;
    return GD_OK;
}
