/*
 * gd_swiglu_split_linear (forward): y = linear(swiglu_split(x12), w [H, N], bias).  The reference
 * composes gd_swiglu_split and gd_linear and frees the activation span in inference
 * (src/ops/swiglu_split_linear/core_swiglu_split_linear.c:22-121,226-301).  For the few rows of a decode
 * step the activation is formed inside the projection kernel (gd_backend_swiglu_split_linear), keeping
 * its F16 rounding, so no intermediate tensor exists.  For many rows (prefill) the reference's two-kernel
 * form is faster: the activation goes to a scratch span that is released as soon as the projection is
 * enqueued, and the projection then stages both operands straight into LDS.  Same arithmetic either way.
 */
#include "../linear/linear_impl.h"

#define GD_SWIGLU_UNFUSED_MIN_ROWS 128u

gd_status gd_swiglu_split_linear(gd_context *ctx, const gd_tensor *x12, const gd_tensor *w, const gd_tensor *bias,
                                 gd_tensor *out)
{
    gd_linear_shape_info info;
    gd_backend_matrix_view xm, wm, ym;
    gd_backend_vector_view bv;
    gd_tensor o;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || x12 == NULL || w == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, x12));
    if (x12->dtype != GD_DTYPE_F16) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "swiglu_split_linear supports f16 tensors only");
    if (x12->rank < 1U || x12->shape[x12->rank - 1U] <= 0 || (x12->shape[x12->rank - 1U] & 1) != 0)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "swiglu_split_linear expects an even last dimension");
    if (!gd_tensor_is_contiguous(x12)) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "swiglu_split_linear requires contiguous x12");
    GD_TRY(gd_linear_validate(ctx, x12, w, bias, false, 2, "swiglu_split_linear", &info));
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F16, info.rank, info.out_shape, &o));
    if (!gd_op_rows_matrix_view(x12, &xm) || !gd_op_matrix_view(w, &wm) || !gd_op_rows_matrix_view(&o, &ym) ||
        (bias != NULL && !gd_op_vector_view(bias, &bv)))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "swiglu_split_linear view construction failed");
    if (ym.rows >= GD_SWIGLU_UNFUSED_MIN_ROWS) {
        gd_tensor act;
        gd_backend_tensor_view x12v, actv;
        gd_backend_matrix_view am;
        int64_t act_shape[2];
        gd_status st;
        act_shape[0] = (int64_t)ym.rows;
        act_shape[1] = x12->shape[x12->rank - 1U] / 2;
        GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F16, 2U, act_shape, &act)); /* top of the scratch stack */
        if (!gd_op_tensor_view(x12, &x12v) || !gd_op_tensor_view(&act, &actv) || !gd_op_matrix_view(&act, &am))
            GD_FAIL(ctx, GD_ERR_INTERNAL, "swiglu_split_linear view construction failed");
        st = gd_backend_swiglu_split_forward(gd_context_backend(ctx), &x12v, &actv);
        if (st == GD_OK) {
            st = bias != NULL ? gd_backend_linear(gd_context_backend(ctx), &am, &wm, &bv, &ym)
                              : gd_backend_matmul(gd_context_backend(ctx), &am, &wm, &ym);
        }
        gd_context_release_scratch(ctx, &act.storage); /* later kernels run after these two on the same stream */
        GD_TRY(gd_op_backend_result(ctx, st, "backend swiglu_split_linear failed"));
    } else {
        GD_TRY(gd_op_backend_result(ctx, gd_backend_swiglu_split_linear(gd_context_backend(ctx), &xm, &wm, bias != NULL ? &bv : NULL, &ym),
                                    "backend swiglu_split_linear failed"));
    }
    *out = o;
    return GD_OK;
}
