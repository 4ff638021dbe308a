/*
 * gd_linear_transposed_weight (forward): x [..., K] @ w[N, K]^T (+ bias).  The reference runs
 * gd_backend_matmul_nt and then gd_backend_add for the bias, i.e. two F16 roundings
 * (src/ops/linear_transposed_weight/core_linear_transposed_weight.c:7-103); this front end issues
 * the same arithmetic as one launch (gd_backend_linear_nt).
 */
#include "../linear/linear_impl.h"

gd_status gd_linear_transposed_weight(gd_context *ctx, const gd_tensor *x, const gd_tensor *w,
                                      const gd_tensor *bias, gd_tensor *out)
{
    gd_linear_shape_info info;
    gd_backend_matrix_view xm, wm, ym;
    gd_backend_vector_view bv;
    gd_tensor o;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_linear_validate(ctx, x, w, bias, true, 1, "linear_transposed_weight", &info));
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F16, info.rank, info.out_shape, &o));
    if (!gd_op_rows_matrix_view(x, &xm) || !gd_op_matrix_view(w, &wm) || !gd_op_rows_matrix_view(&o, &ym) ||
        (bias != NULL && !gd_op_vector_view(bias, &bv)))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "linear_transposed_weight view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_linear_nt(gd_context_backend(ctx), &xm, &wm, bias != NULL ? &bv : NULL, &ym),
                                "backend linear_transposed_weight failed"));
    *out = o;
    return GD_OK;
}
