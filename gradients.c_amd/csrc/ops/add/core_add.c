/*
 * gd_add (forward): F16 elementwise add with NumPy right-aligned broadcasting.  Front end
 * restating the reference's src/ops/add/core_add.c:7-32 and src/ops/_shared/binary/
 * binary_core.h:67-131: F16 x (else UNSUPPORTED), same dtype, contiguous operands, incompatible
 * shapes -> INVALID_ARGUMENT "not broadcast-compatible".
 */
#include "../op_common.h"

gd_status gd_add(gd_context *ctx, const gd_tensor *x, const gd_tensor *y, gd_tensor *out)
{
    gd_backend_tensor_view xv, yv, ov;
    gd_tensor o;
    int64_t shape[GD_MAX_DIMS];
    uint32_t rank, d;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || x == NULL || y == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, x));
    GD_TRY(gd_tensor_validate(ctx, y));
    if (x->dtype != GD_DTYPE_F16 || y->dtype != x->dtype) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "add supports matching f16 tensors");
    if (!gd_tensor_is_contiguous(x) || !gd_tensor_is_contiguous(y)) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "add requires contiguous tensors");
    rank = x->rank > y->rank ? x->rank : y->rank;
    for (d = 0U; d < rank; ++d) {
        const int64_t xd = d < x->rank ? x->shape[x->rank - 1U - d] : 1;
        const int64_t yd = d < y->rank ? y->shape[y->rank - 1U - d] : 1;
        if (xd != yd && xd != 1 && yd != 1) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "add operands are not broadcast-compatible");
        shape[rank - 1U - d] = xd > yd ? xd : yd;
    }
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F16, rank, shape, &o));
    if (!gd_op_tensor_view(x, &xv) || !gd_op_tensor_view(y, &yv) || !gd_op_tensor_view(&o, &ov))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "add view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_add(gd_context_backend(ctx), &xv, &yv, &ov), "backend add failed"));
    *out = o;
    return GD_OK;
}
