/*
 * gd_sdpa_varlen (forward): front end restating the rules of the reference's
 * src/ops/sdpa_varlen/core_sdpa_varlen.c:12-270; head-size limit 256 instead of 64;
 * max_seqlen == 0 means "number of packed rows".
 */
#include "../op_common.h"

gd_status gd_sdpa_varlen(gd_context *ctx, const gd_tensor *q, const gd_tensor *k, const gd_tensor *v,
                         const gd_tensor *cu_seqlens, const gd_sdpa_varlen_config *config, gd_tensor *out)
{
    gd_backend_tensor_view qv, kv, vv, cv, ov;
    gd_backend_sdpa_varlen_args args;
    gd_tensor o;
    uint32_t i;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || q == NULL || k == NULL || v == NULL || cu_seqlens == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, q));
    GD_TRY(gd_tensor_validate(ctx, k));
    GD_TRY(gd_tensor_validate(ctx, v));
    GD_TRY(gd_tensor_validate(ctx, cu_seqlens));
    if ((q->dtype != GD_DTYPE_F16 && q->dtype != GD_DTYPE_F32) || k->dtype != q->dtype || v->dtype != q->dtype ||
        cu_seqlens->dtype != GD_DTYPE_I32)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "sdpa_varlen requires matching f16/f32 q/k/v and i32 cu_seqlens");
    if (q->rank != 3U || k->rank != 3U || v->rank != 3U || cu_seqlens->rank != 1U || cu_seqlens->shape[0] < 2)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_varlen expects q/k/v [N,H,Dh] and cu_seqlens [B+1]");
    for (i = 0U; i < 3U; ++i) {
        if (k->shape[i] != v->shape[i]) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_varlen k/v shapes must match");
    }
    if (q->shape[0] != k->shape[0] || q->shape[2] != k->shape[2] || (q->shape[1] % k->shape[1]) != 0)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_varlen shape mismatch");
    if (q->shape[2] > 256 || q->shape[0] > (int64_t)INT_MAX)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "sdpa_varlen dimensions exceed kernel limits");
    if (!gd_tensor_is_contiguous(q) || !gd_tensor_is_contiguous(k) || !gd_tensor_is_contiguous(v) ||
        !gd_tensor_is_contiguous(cu_seqlens))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "sdpa_varlen requires contiguous tensors");
    memset(&args, 0, sizeof(args));
    args.scale = config != NULL ? config->scale : 0.0f;
    args.causal = config != NULL ? (config->causal ? 1U : 0U) : 1U;
    if (config != NULL && (config->sliding_window < 0 || config->prefix_len < 0 || config->max_seqlen < 0))
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_varlen window/prefix/max_seqlen must be non-negative");
    args.sliding_window = (uint32_t)(config != NULL ? config->sliding_window : 0);
    args.prefix_len = (uint32_t)(config != NULL ? config->prefix_len : 0);
    args.max_seqlen = (uint32_t)(config != NULL ? config->max_seqlen : 0);
    if (args.prefix_len > 0U && args.causal == 0U) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_varlen prefix requires causal");
    if (args.max_seqlen == 0U) args.max_seqlen = (uint32_t)q->shape[0];
    if (args.prefix_len > args.max_seqlen) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_varlen prefix exceeds max_seqlen");
    if (args.scale != args.scale) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_varlen scale must be finite");
    if (args.scale <= 0.0f) args.scale = (float)(1.0 / sqrt((double)q->shape[2]));
    else if (!isfinite(args.scale)) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_varlen scale must be finite");
    GD_TRY(gd_tensor_alloc_like_shape(ctx, q->dtype, 3U, q->shape, &o));
    if (!gd_op_tensor_view(q, &qv) || !gd_op_tensor_view(k, &kv) || !gd_op_tensor_view(v, &vv) ||
        !gd_op_tensor_view(cu_seqlens, &cv) || !gd_op_tensor_view(&o, &ov))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "sdpa_varlen view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_sdpa_varlen(gd_context_backend(ctx), &qv, &kv, &vv, &cv, &ov, NULL, &args),
                                "backend sdpa_varlen failed"));
    *out = o;
    return GD_OK;
}
