/*
 * Shape and layout rules shared by gd_linear, gd_linear_transposed_weight and
 * gd_swiglu_split_linear.  Restated from the reference's src/ops/linear/linear_impl.h:33-241:
 * F16 only (else UNSUPPORTED); x rank >= 1, w rank 2, bias rank 1; K and N must agree (else
 * INVALID_ARGUMENT); K, N and the flattened row count must fit 32 bits (else OUT_OF_MEMORY);
 * unit last stride, row-strided w, rank-2 x may be row-strided, rank-N x must be contiguous
 * (else UNSUPPORTED); the output shape is x.shape[:-1] + [N].
 */
#ifndef GD_OPS_LINEAR_IMPL_H
#define GD_OPS_LINEAR_IMPL_H

#include "../op_common.h"

typedef struct gd_linear_shape_info {
    uint32_t rank;
    int64_t rows, k, n;
    int64_t out_shape[GD_MAX_DIMS];
} gd_linear_shape_info;

/* x_cols_per_k: 1 for plain projections, 2 when x carries [value | gate] halves (swiglu) */
static inline gd_status gd_linear_validate(gd_context *ctx, const gd_tensor *x, const gd_tensor *w,
                                           const gd_tensor *bias, bool w_is_nk, int x_cols_per_k,
                                           const char *what, gd_linear_shape_info *info)
{
    uint32_t axis;
    int64_t rows = 1, wk, wn;
    (void)what;
    if (ctx == NULL || x == NULL || w == NULL || info == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, x));
    GD_TRY(gd_tensor_validate(ctx, w));
    if (bias != NULL) GD_TRY(gd_tensor_validate(ctx, bias));
    memset(info, 0, sizeof(*info));
    if (x->dtype != GD_DTYPE_F16 || w->dtype != GD_DTYPE_F16 || (bias != NULL && bias->dtype != GD_DTYPE_F16))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "linear currently supports f16 tensors only");
    if (x->rank < 1U || w->rank != 2U || (bias != NULL && bias->rank != 1U))
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "linear expects x [..., K], w rank 2, bias [N]");
    wk = w_is_nk ? w->shape[1] : w->shape[0];
    wn = w_is_nk ? w->shape[0] : w->shape[1];
    info->rank = x->rank;
    if (x->shape[x->rank - 1U] <= 0 || (x->shape[x->rank - 1U] % x_cols_per_k) != 0)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "linear shape mismatch");
    info->k = x->shape[x->rank - 1U] / x_cols_per_k;
    info->n = wn;
    if (info->k <= 0 || info->n <= 0 || info->k != wk || (bias != NULL && bias->shape[0] != info->n))
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "linear shape mismatch");
    if (info->k > (int64_t)UINT32_MAX / 2 || info->n > (int64_t)UINT32_MAX)
        GD_FAIL(ctx, GD_ERR_OUT_OF_MEMORY, "linear matrix dimension overflow");
    for (axis = 0U; axis + 1U < x->rank; ++axis) {
        if (x->shape[axis] <= 0 || rows > INT64_MAX / x->shape[axis])
            GD_FAIL(ctx, GD_ERR_OUT_OF_MEMORY, "linear flattened row count overflow");
        rows *= x->shape[axis];
        info->out_shape[axis] = x->shape[axis];
    }
    if (rows > (int64_t)UINT32_MAX) GD_FAIL(ctx, GD_ERR_OUT_OF_MEMORY, "linear flattened row count overflow");
    info->out_shape[x->rank - 1U] = info->n;
    info->rows = rows;
    if (x->strides[x->rank - 1U] != 1 || w->strides[1] != 1 || w->strides[0] <= 0 ||
        (bias != NULL && bias->strides[0] != 1))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "linear requires row-strided inputs");
    if (x->rank == 2U) {
        if (x->strides[0] <= 0) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "linear requires row-strided inputs");
    } else if (!gd_tensor_is_contiguous(x)) {
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "linear rank-N input must be contiguous");
    }
    return GD_OK;
}

#endif
