/*
 * gd_swiglu_split (forward): x12 [..., 2H] -> [..., H].  Front end restating the reference's
 * src/ops/swiglu/core_swiglu.c:154-202,340-392: F16 only, even last dim, contiguous input.
 */
#include "../op_common.h"

gd_status gd_swiglu_split(gd_context *ctx, const gd_tensor *x12, gd_tensor *out)
{
    gd_backend_tensor_view xv, ov;
    gd_tensor o;
    int64_t shape[GD_MAX_DIMS];
    uint32_t i;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || x12 == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, x12));
    if (x12->dtype != GD_DTYPE_F16) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "swiglu_split supports f16 tensors only");
    if (x12->rank < 1U || x12->shape[x12->rank - 1U] <= 0 || (x12->shape[x12->rank - 1U] & 1) != 0)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "swiglu_split expects an even last dimension");
    if (!gd_tensor_is_contiguous(x12)) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "swiglu_split requires contiguous input");
    for (i = 0U; i < x12->rank; ++i) shape[i] = x12->shape[i];
    shape[x12->rank - 1U] /= 2;
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F16, x12->rank, shape, &o));
    if (!gd_op_tensor_view(x12, &xv) || !gd_op_tensor_view(&o, &ov)) GD_FAIL(ctx, GD_ERR_INTERNAL, "swiglu_split view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_swiglu_split_forward(gd_context_backend(ctx), &xv, &ov), "backend swiglu_split failed"));
    *out = o;
    return GD_OK;
}
