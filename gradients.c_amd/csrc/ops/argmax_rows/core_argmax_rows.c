/*
 * gd_argmax_rows: greedy next token per logits row on the device.  No counterpart in the
 * reference, whose generator downloads the logits and scans them on the host
 * (examples/gpt_lm/gpt_lm_shared.c:1388-1400, 1658-1661); the selection rule is the same.
 */
#include "../op_common.h"

gd_status gd_argmax_rows(gd_context *ctx, const gd_tensor *logits, gd_tensor *ids, gd_tensor *gap)
{
    gd_backend_tensor_view lv, iv, gv;
    gd_tensor ti, tg;
    int64_t rows;
    if (ids != NULL) memset(ids, 0, sizeof(*ids));
    if (gap != NULL) memset(gap, 0, sizeof(*gap));
    if (ctx == NULL || logits == NULL || ids == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, logits));
    if (logits->dtype != GD_DTYPE_F16 && logits->dtype != GD_DTYPE_F32) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "argmax_rows supports f16/f32 logits");
    if (logits->rank != 2U) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "argmax_rows expects logits [rows, vocab]");
    if (!gd_tensor_is_contiguous(logits)) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "argmax_rows requires contiguous logits");
    rows = logits->shape[0];
    GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_I32, 1U, &rows, &ti));
    if (gap != NULL) GD_TRY(gd_tensor_alloc_like_shape(ctx, GD_DTYPE_F32, 1U, &rows, &tg));
    if (!gd_op_tensor_view(logits, &lv) || !gd_op_tensor_view(&ti, &iv) || (gap != NULL && !gd_op_tensor_view(&tg, &gv)))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "argmax_rows view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_argmax_rows(gd_context_backend(ctx), &lv, &iv, gap != NULL ? &gv : NULL), "backend argmax_rows failed"));
    *ids = ti;
    if (gap != NULL) *gap = tg;
    return GD_OK;
}
