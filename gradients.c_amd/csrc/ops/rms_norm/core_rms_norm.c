/*
 * gd_rms_norm (forward): front end restating the rules of the reference's
 * src/ops/rms_norm/core_rms_norm.c:43-96,326-404 (no-stats inference branch).
 */
#include "../op_common.h"

gd_status gd_rms_norm(gd_context *ctx, const gd_tensor *x, const gd_tensor *weight, float eps, gd_tensor *out)
{
    gd_backend_tensor_view xv, wv, ov;
    gd_backend_rms_norm_args args;
    gd_tensor o;
    int64_t n;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || x == NULL || weight == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (!(eps > 0.0f)) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "rms_norm eps must be positive");
    GD_TRY(gd_tensor_validate(ctx, x));
    GD_TRY(gd_tensor_validate(ctx, weight));
    if ((x->dtype != GD_DTYPE_F16 && x->dtype != GD_DTYPE_F32) || weight->dtype != x->dtype)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "rms_norm requires matching f16/f32 x and weight");
    if (x->rank < 1U || weight->rank != 1U || weight->shape[0] != x->shape[x->rank - 1U])
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "rms_norm weight must be [last dim of x]");
    if (!gd_tensor_is_contiguous(x) || !gd_tensor_is_contiguous(weight))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "rms_norm requires contiguous tensors");
    if (gd_tensor_numel(x, &n) != GD_OK) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "rms_norm invalid shape");
    GD_TRY(gd_tensor_alloc_like_shape(ctx, x->dtype, x->rank, x->shape, &o));
    memset(&args, 0, sizeof(args));
    args.cols = (uint64_t)x->shape[x->rank - 1U];
    args.rows = (uint64_t)n / args.cols;
    args.eps = eps;
    if (!gd_op_tensor_view(x, &xv) || !gd_op_tensor_view(weight, &wv) || !gd_op_tensor_view(&o, &ov))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "rms_norm view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_rms_norm_forward(gd_context_backend(ctx), &xv, &wv, &ov, &args),
                                "backend rms_norm failed"));
    *out = o;
    return GD_OK;
}
