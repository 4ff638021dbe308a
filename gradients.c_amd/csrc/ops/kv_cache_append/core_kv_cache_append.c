/*
 * gd_kv_cache_append_{at,positions,packed}: front ends restating the rules of the reference's
 * src/ops/kv_cache_append/core_kv_cache_append.c:13-351.  In-place on the state arena, inference
 * and eval scopes only; per-row range errors of the tensor-position forms are left to the device,
 * which skips such rows.  A successful call bumps the version of both caches.
 */
#include "../op_common.h"

static gd_status validate(gd_context *ctx, gd_tensor *kc, gd_tensor *vc, const gd_tensor *kn, const gd_tensor *vn,
                          uint32_t new_rank)
{
    uint32_t i;
    if (ctx == NULL || kc == NULL || vc == NULL || kn == NULL || vn == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, kc));
    GD_TRY(gd_tensor_validate(ctx, vc));
    GD_TRY(gd_tensor_validate(ctx, kn));
    GD_TRY(gd_tensor_validate(ctx, vn));
    if (gd_context_scope_mode(ctx) == GD_SCOPE_TRAIN || kc->requires_grad || vc->requires_grad ||
        kn->requires_grad || vn->requires_grad)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "kv_cache_append is inference/eval only");
    if ((kc->dtype != GD_DTYPE_F16 && kc->dtype != GD_DTYPE_F32) || vc->dtype != kc->dtype ||
        kn->dtype != kc->dtype || vn->dtype != kc->dtype)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "kv_cache_append requires matching f16/f32 tensors");
    if (kc->rank != 4U || vc->rank != 4U || kn->rank != new_rank || vn->rank != new_rank)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "kv_cache_append expects caches [B,Tmax,H,Dh]");
    for (i = 0U; i < 4U; ++i) {
        if (kc->shape[i] != vc->shape[i]) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "kv_cache_append k/v cache shapes must match");
    }
    for (i = 0U; i < new_rank; ++i) {
        if (kn->shape[i] != vn->shape[i]) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "kv_cache_append k/v new shapes must match");
    }
    if (new_rank == 4U) {
        if (kn->shape[0] != kc->shape[0] || kn->shape[2] != kc->shape[2] || kn->shape[3] != kc->shape[3] ||
            kn->shape[1] > kc->shape[1])
            GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "kv_cache_append shape mismatch");
    } else if (kn->shape[1] != kc->shape[2] || kn->shape[2] != kc->shape[3]) {
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "kv_cache_append shape mismatch");
    }
    for (i = 0U; i < 4U; ++i) {
        if (kc->shape[i] > (int64_t)INT_MAX) GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "kv_cache_append dimensions exceed kernel limits");
    }
    if (!gd_tensor_is_contiguous(kc) || !gd_tensor_is_contiguous(vc) || !gd_tensor_is_contiguous(kn) ||
        !gd_tensor_is_contiguous(vn))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "kv_cache_append requires contiguous tensors");
    return GD_OK;
}

static gd_status validate_i32_vector(gd_context *ctx, const gd_tensor *t, int64_t len, const char *msg)
{
    if (t == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, t));
    if (t->dtype != GD_DTYPE_I32 || t->rank != 1U || t->shape[0] != len || !gd_tensor_is_contiguous(t))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, msg);
    return GD_OK;
}

gd_status gd_kv_cache_append_at(gd_context *ctx, gd_tensor *k_cache, gd_tensor *v_cache, int32_t cache_pos,
                                const gd_tensor *k_new, const gd_tensor *v_new)
{
    gd_backend_tensor_view kc, vc, kn, vn;
    gd_backend_kv_cache_append_args args;
    GD_TRY(validate(ctx, k_cache, v_cache, k_new, v_new, 4U));
    if (cache_pos < 0 || (int64_t)cache_pos > k_cache->shape[1] || k_new->shape[1] > k_cache->shape[1] - (int64_t)cache_pos)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "kv_cache_append cache_pos out of range");
    if (!gd_op_tensor_view(k_cache, &kc) || !gd_op_tensor_view(v_cache, &vc) || !gd_op_tensor_view(k_new, &kn) ||
        !gd_op_tensor_view(v_new, &vn))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "kv_cache_append view construction failed");
    args.cache_pos = cache_pos;
    GD_TRY(gd_op_backend_result(ctx, gd_backend_kv_cache_append_at(gd_context_backend(ctx), &kc, &vc, &kn, &vn, &args),
                                "backend kv_cache_append failed"));
    gd_op_bump_version(k_cache);
    gd_op_bump_version(v_cache);
    return GD_OK;
}

gd_status gd_kv_cache_append_positions(gd_context *ctx, gd_tensor *k_cache, gd_tensor *v_cache,
                                       const gd_tensor *cache_pos, const gd_tensor *k_new, const gd_tensor *v_new)
{
    gd_backend_tensor_view kc, vc, kn, vn, pos;
    gd_backend_kv_cache_append_args args;
    GD_TRY(validate(ctx, k_cache, v_cache, k_new, v_new, 4U));
    GD_TRY(validate_i32_vector(ctx, cache_pos, k_cache->shape[0], "kv_cache_append cache_pos must be i32 [B]"));
    if (!gd_op_tensor_view(k_cache, &kc) || !gd_op_tensor_view(v_cache, &vc) || !gd_op_tensor_view(k_new, &kn) ||
        !gd_op_tensor_view(v_new, &vn) || !gd_op_tensor_view(cache_pos, &pos))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "kv_cache_append view construction failed");
    args.cache_pos = 0;
    GD_TRY(gd_op_backend_result(ctx, gd_backend_kv_cache_append_positions(gd_context_backend(ctx), &kc, &vc, &pos, &kn, &vn, &args),
                                "backend kv_cache_append failed"));
    gd_op_bump_version(k_cache);
    gd_op_bump_version(v_cache);
    return GD_OK;
}

gd_status gd_kv_cache_append_packed(gd_context *ctx, gd_tensor *k_cache, gd_tensor *v_cache,
                                    const gd_tensor *cache_pos, const gd_tensor *cu_seqlens,
                                    const gd_tensor *k_new, const gd_tensor *v_new)
{
    gd_backend_tensor_view kc, vc, kn, vn, pos, cu;
    gd_backend_kv_cache_append_args args;
    GD_TRY(validate(ctx, k_cache, v_cache, k_new, v_new, 3U));
    GD_TRY(validate_i32_vector(ctx, cache_pos, k_cache->shape[0], "kv_cache_append cache_pos must be i32 [B]"));
    GD_TRY(validate_i32_vector(ctx, cu_seqlens, k_cache->shape[0] + 1, "kv_cache_append cu_seqlens must be i32 [B+1]"));
    if (!gd_op_tensor_view(k_cache, &kc) || !gd_op_tensor_view(v_cache, &vc) || !gd_op_tensor_view(k_new, &kn) ||
        !gd_op_tensor_view(v_new, &vn) || !gd_op_tensor_view(cache_pos, &pos) || !gd_op_tensor_view(cu_seqlens, &cu))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "kv_cache_append view construction failed");
    args.cache_pos = 0;
    GD_TRY(gd_op_backend_result(ctx, gd_backend_kv_cache_append_packed(gd_context_backend(ctx), &kc, &vc, &pos, &cu, &kn, &vn, &args),
                                "backend kv_cache_append failed"));
    gd_op_bump_version(k_cache);
    gd_op_bump_version(v_cache);
    return GD_OK;
}
