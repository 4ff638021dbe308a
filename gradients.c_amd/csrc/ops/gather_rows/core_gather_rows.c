/*
 * gd_gather_rows: out[i,:] = x[rows[i],:].  Stands in for the per-sequence gd_tensor_slice +
 * gd_concat the reference uses to pick the last prompt row of every packed sequence
 * (examples/gpt_lm/gpt_lm_shared.c:1117-1169).
 */
#include "../op_common.h"

gd_status gd_gather_rows(gd_context *ctx, const gd_tensor *x, const gd_tensor *rows, gd_tensor *out)
{
    gd_backend_tensor_view xv, rv, ov;
    gd_tensor o;
    int64_t shape[2];
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || x == NULL || rows == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, x));
    GD_TRY(gd_tensor_validate(ctx, rows));
    if ((x->dtype != GD_DTYPE_F16 && x->dtype != GD_DTYPE_F32) || rows->dtype != GD_DTYPE_I32)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "gather_rows requires f16/f32 x and i32 rows");
    if (x->rank != 2U || rows->rank != 1U) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "gather_rows expects x [N, D] and rows [B]");
    if (!gd_tensor_is_contiguous(x) || !gd_tensor_is_contiguous(rows)) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "gather_rows requires contiguous tensors");
    shape[0] = rows->shape[0];
    shape[1] = x->shape[1];
    GD_TRY(gd_tensor_alloc_like_shape(ctx, x->dtype, 2U, shape, &o));
    if (!gd_op_tensor_view(x, &xv) || !gd_op_tensor_view(rows, &rv) || !gd_op_tensor_view(&o, &ov))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "gather_rows view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_gather_rows(gd_context_backend(ctx), &xv, &rv, &ov), "backend gather_rows failed"));
    *out = o;
    return GD_OK;
}
