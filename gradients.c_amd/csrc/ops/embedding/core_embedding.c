/*
 * gd_embedding (forward): out[..., :] = table[ids[...], :].  Front end restating the reference's
 * src/ops/embedding/core_embedding.c:31-137,201-268: table F16/F32 rank 2 contiguous, ids I32
 * rank >= 1 contiguous and non-empty; out shape = ids.shape + [dim].  The 32-bit element-count
 * limit of the reference (a Metal grid limit) does not apply here.
 */
#include "../op_common.h"

gd_status gd_embedding(gd_context *ctx, const gd_tensor *table, const gd_tensor *ids, gd_tensor *out)
{
    gd_backend_tensor_view tv, iv, ov;
    gd_backend_embedding_args args;
    gd_tensor o;
    int64_t shape[GD_MAX_DIMS], n;
    uint32_t i;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || table == NULL || ids == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, table));
    GD_TRY(gd_tensor_validate(ctx, ids));
    if ((table->dtype != GD_DTYPE_F16 && table->dtype != GD_DTYPE_F32) || ids->dtype != GD_DTYPE_I32)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "embedding requires an f16/f32 table and i32 ids");
    if (table->rank != 2U || ids->rank < 1U || ids->rank + 1U > GD_MAX_DIMS)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "embedding expects table [vocab, dim] and ids of rank >= 1");
    if (!gd_tensor_is_contiguous(table) || !gd_tensor_is_contiguous(ids))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "embedding requires contiguous tensors");
    if (gd_tensor_numel(ids, &n) != GD_OK || n <= 0) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "embedding ids must be non-empty");
    for (i = 0U; i < ids->rank; ++i) shape[i] = ids->shape[i];
    shape[ids->rank] = table->shape[1];
    GD_TRY(gd_tensor_alloc_like_shape(ctx, table->dtype, ids->rank + 1U, shape, &o));
    args.ids_count = (uint64_t)n;
    args.vocab = (uint64_t)table->shape[0];
    args.dim = (uint64_t)table->shape[1];
    if (!gd_op_tensor_view(table, &tv) || !gd_op_tensor_view(ids, &iv) || !gd_op_tensor_view(&o, &ov))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "embedding view construction failed");
    GD_TRY(gd_op_backend_result(ctx, gd_backend_embedding_forward(gd_context_backend(ctx), &tv, &iv, &ov, &args), "backend embedding failed"));
    *out = o;
    return GD_OK;
}
