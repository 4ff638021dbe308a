/*
 * gd_reshape: metadata-only view of a contiguous tensor with a new shape of the same element
 * count (reference src/ops/reshape/core_reshape.c:185; one dimension may be -1 and is inferred).
 */
#include "../op_common.h"

gd_status gd_reshape(gd_context *ctx, const gd_tensor *x, gd_shape shape, gd_tensor *out)
{
    gd_tensor v;
    int64_t n, known = 1;
    int infer = -1;
    uint32_t i;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || x == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, x));
    if (shape.rank > GD_MAX_DIMS) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "reshape rank too large");
    if (!gd_tensor_is_contiguous(x)) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "reshape requires a contiguous tensor");
    if (gd_tensor_numel(x, &n) != GD_OK) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "reshape invalid input shape");
    for (i = 0U; i < shape.rank; ++i) {
        if (shape.dims[i] == -1 && infer < 0) infer = (int)i;
        else if (shape.dims[i] <= 0) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "reshape dimensions must be positive");
        else known *= shape.dims[i];
    }
    if (infer >= 0) {
        if (known == 0 || n % known != 0) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "reshape cannot infer dimension");
        shape.dims[infer] = n / known;
        known = n;
    }
    if (known != n) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "reshape element count mismatch");
    v = *x;
    v.id = gd_context_next_tensor_id(ctx);
    v.rank = shape.rank;
    memset(v.shape, 0, sizeof(v.shape));
    memset(v.strides, 0, sizeof(v.strides));
    for (i = 0U; i < shape.rank; ++i) v.shape[i] = shape.dims[i];
    gd_tensor_set_contiguous_strides(&v);
    v.is_view = true;
    v.is_leaf = false;
    *out = v;
    return GD_OK;
}
