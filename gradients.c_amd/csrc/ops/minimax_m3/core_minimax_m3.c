/*
 * gd_minimax_m3_index_topk and gd_minimax_m3_sparse_attention (forward): front ends restating the rules of the
 * reference's src/ops/minimax_m3_index_topk/core_minimax_m3_index_topk.c:9-140 and
 * src/ops/minimax_m3_sparse_attention/core_minimax_m3_sparse_attention.c:14-130: F16 [N,H,Dh] tensors, I32
 * cu_seqlens [B+1] and topk_idx [Hkv,N,topk], head size <= 64, block size <= 128 (default 128), topk <= 16
 * (default 4), init / local blocks default 1 without a configuration, scale <= 0 selects 1 / sqrt(Dh).
 */
#include "../op_common.h"

#define M3_BLOCK_DEFAULT 128
#define M3_BLOCK_MAX 128
#define M3_TOPK_MAX 16
#define M3_DH_MAX 64

static gd_status resolve(gd_context *ctx, const gd_tensor *q, const gd_minimax_m3_sparse_config *c,
                         gd_backend_minimax_m3_sparse_args *a)
{
    const int32_t block = c != NULL && c->block_size > 0 ? c->block_size : M3_BLOCK_DEFAULT;
    const int32_t topk = c != NULL && c->topk > 0 ? c->topk : 4;
    const int32_t init_blocks = c != NULL ? c->init_blocks : 1, local_blocks = c != NULL ? c->local_blocks : 1;
    const int64_t max_seqlen = c != NULL && c->max_seqlen > 0 ? c->max_seqlen : q->shape[0];
    const double scale = c != NULL && c->scale > 0.0f ? (double)c->scale : 1.0 / sqrt((double)q->shape[2]);
    if (block > M3_BLOCK_MAX || topk > M3_TOPK_MAX || init_blocks < 0 || local_blocks < 0 || max_seqlen <= 0)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "minimax_m3 sparse config out of range");
    if (!isfinite(scale) || scale <= 0.0) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "minimax_m3 sparse scale must be finite");
    memset(a, 0, sizeof(*a));
    a->scale = (float)scale;
    a->block_size = (uint32_t)block;
    a->topk = (uint32_t)topk;
    a->init_blocks = (uint32_t)init_blocks;
    a->local_blocks = (uint32_t)local_blocks;
    a->max_seqlen = (uint32_t)(max_seqlen > (int64_t)UINT32_MAX ? UINT32_MAX : max_seqlen);
    return GD_OK;
}

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
    GD_TRY(resolve(ctx, index_q, config, &args));
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
    GD_TRY(resolve(ctx, q, config, &args));
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
