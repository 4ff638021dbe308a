/*
 * gd_linear (forward): x [..., K] @ w [K, N] (+ bias), one F16 rounding.  Front end restating
 * the reference's src/ops/linear/core_linear.c:7-74: gd_backend_linear with a bias,
 * gd_backend_matmul without.
 */
#include "linear_impl.h"

gd_status gd_linear(gd_context *ctx, const gd_tensor *x, const gd_tensor *w, const gd_tensor *bias, gd_tensor *out)
{
    gd_linear_shape_info info;
    gd_backend_matrix_view xm, wm, ym;
    gd_backend_vector_view bv;
    gd_tensor o;
    gd_status st;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_linear_validate(ctx, x, w, bias, false, 1, "linear", &info));
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F16, info.rank, info.out_shape, &o));
    if (!gd_op_rows_matrix_view(x, &xm) || !gd_op_matrix_view(w, &wm) || !gd_op_rows_matrix_view(&o, &ym) ||
        (bias != NULL && !gd_op_vector_view(bias, &bv)))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "linear view construction failed");
    st = bias != NULL ? gd_backend_linear(gd_context_backend(ctx), &xm, &wm, &bv, &ym)
                      : gd_backend_matmul(gd_context_backend(ctx), &xm, &wm, &ym);
    GD_TRY(gd_op_backend_result(ctx, st, "backend linear failed"));
    *out = o;
    return GD_OK;
}
