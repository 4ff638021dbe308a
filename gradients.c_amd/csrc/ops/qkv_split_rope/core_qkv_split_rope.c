/*
 * gd_qkv_split_rope (forward): front end restating the rules of the reference's
 * src/ops/qkv_split_rope/core_qkv_split_rope.c:28-102,199-300: qkv F16 [N, 3*H*D], pos I32 [N];
 * theta <= 0 -> 10000, n_dims <= 0 -> D; odd or oversized n_dims is invalid; partial rotation
 * (n_dims != D) is unsupported by this fused form.
 */
#include "../op_common.h"

gd_status gd_qkv_split_rope(gd_context *ctx, const gd_tensor *qkv, const gd_tensor *pos_ids, int32_t n_heads,
                            int32_t head_dim, const gd_rope_config *config, gd_tensor *q, gd_tensor *k, gd_tensor *v)
{
    gd_backend_tensor_view qkvv, pv, qv, kv, vv;
    gd_backend_rope_args args;
    gd_tensor tq, tk, tv;
    int64_t shape[3];
    int32_t n_dims;
    if (q != NULL) memset(q, 0, sizeof(*q));
    if (k != NULL) memset(k, 0, sizeof(*k));
    if (v != NULL) memset(v, 0, sizeof(*v));
    if (ctx == NULL || qkv == NULL || pos_ids == NULL || q == NULL || k == NULL || v == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, qkv));
    GD_TRY(gd_tensor_validate(ctx, pos_ids));
    if (qkv->dtype != GD_DTYPE_F16 || pos_ids->dtype != GD_DTYPE_I32)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "qkv_split_rope requires f16 qkv and i32 positions");
    if (n_heads <= 0 || head_dim <= 0 || qkv->rank != 2U || pos_ids->rank != 1U || pos_ids->shape[0] != qkv->shape[0] ||
        qkv->shape[1] != (int64_t)3 * n_heads * head_dim)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "qkv_split_rope expects qkv [N, 3*H*Dh] and positions [N]");
    if (!gd_tensor_is_contiguous(qkv) || !gd_tensor_is_contiguous(pos_ids))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "qkv_split_rope requires contiguous tensors");
    args.theta = (config != NULL && config->theta > 0.0f) ? config->theta : 10000.0f;
    n_dims = (config != NULL && config->n_dims > 0) ? config->n_dims : head_dim;
    if ((n_dims & 1) != 0 || n_dims > head_dim) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "qkv_split_rope n_dims must be even and <= head_dim");
    if (n_dims != head_dim) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "qkv_split_rope fast path requires full-head RoPE");
    args.n_dims = (uint32_t)n_dims;
    args.interleaved = (config != NULL && config->interleaved) ? 1U : 0U;
    shape[0] = qkv->shape[0];
    shape[1] = n_heads;
    shape[2] = head_dim;
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F16, 3U, shape, &tq));
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F16, 3U, shape, &tk));
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F16, 3U, shape, &tv));
    if (!gd_op_tensor_view(qkv, &qkvv) || !gd_op_tensor_view(pos_ids, &pv) || !gd_op_tensor_view(&tq, &qv) ||
        !gd_op_tensor_view(&tk, &kv) || !gd_op_tensor_view(&tv, &vv))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "qkv_split_rope view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_qkv_split_rope_forward(gd_context_backend(ctx), &qkvv, &pv, &qv, &kv, &vv,
                                                                       (uint32_t)n_heads, (uint32_t)head_dim, &args),
                                "backend qkv_split_rope failed"));
    *q = tq;
    *k = tk;
    *v = tv;
    return GD_OK;
}
