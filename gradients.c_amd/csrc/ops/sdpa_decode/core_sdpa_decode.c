/*
 * gd_sdpa_decode{,_at,_positions}: front ends restating the rules of the reference's
 * src/ops/sdpa_decode/core_sdpa_decode.c:11-321; the head-size limit is 256 instead of 64.
 * scale <= 0 selects 1/sqrt(Dh) computed in double; out is allocated in scratch with q's shape.
 */
#include "../op_common.h"

#define GD_SDPA_DECODE_MAX_HEAD_DIM 256

static gd_status validate_common(gd_context *ctx, const gd_tensor *q, const gd_tensor *kc, const gd_tensor *vc,
                                 const gd_sdpa_decode_config *config, gd_backend_sdpa_decode_args *args)
{
    uint32_t i;
    if (ctx == NULL || q == NULL || kc == NULL || vc == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(gd_tensor_validate(ctx, q));
    GD_TRY(gd_tensor_validate(ctx, kc));
    GD_TRY(gd_tensor_validate(ctx, vc));
    if ((q->dtype != GD_DTYPE_F16 && q->dtype != GD_DTYPE_F32) || kc->dtype != q->dtype || vc->dtype != q->dtype)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "sdpa_decode requires matching f16/f32 q/k/v");
    if (q->rank != 4U || kc->rank != 4U || vc->rank != 4U)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_decode expects q/cache tensors [B,T,H,Dh]");
    for (i = 0U; i < 4U; ++i) {
        if (kc->shape[i] != vc->shape[i]) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_decode k/v cache shapes must match");
    }
    if (q->shape[0] != kc->shape[0] || q->shape[3] != kc->shape[3] || (q->shape[2] % kc->shape[2]) != 0)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_decode shape mismatch");
    if (q->shape[0] > (int64_t)INT_MAX || q->shape[1] > (int64_t)INT_MAX || kc->shape[1] > (int64_t)INT_MAX ||
        q->shape[2] > (int64_t)INT_MAX || q->shape[3] > GD_SDPA_DECODE_MAX_HEAD_DIM)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "sdpa_decode dimensions exceed kernel limits");
    if (!gd_tensor_is_contiguous(q) || !gd_tensor_is_contiguous(kc) || !gd_tensor_is_contiguous(vc))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "sdpa_decode requires contiguous tensors");
    if (config != NULL && (config->sliding_window < 0 || config->prefix_len < 0 || config->prefix_len > kc->shape[1]))
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_decode window/prefix must be non-negative and in range");
    memset(args, 0, sizeof(*args));
    args->scale = config != NULL ? config->scale : 0.0f;
    args->sliding_window = (uint32_t)(config != NULL ? config->sliding_window : 0);
    args->prefix_len = (uint32_t)(config != NULL ? config->prefix_len : 0);
    if (args->scale != args->scale) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_decode scale must be finite");
    if (args->scale <= 0.0f) args->scale = (float)(1.0 / sqrt((double)q->shape[3]));
    else if (!isfinite(args->scale)) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_decode scale must be finite");
    return GD_OK;
}

static gd_status run(gd_context *ctx, const gd_tensor *q, const gd_tensor *kc, const gd_tensor *vc,
                     const gd_tensor *pos, gd_backend_sdpa_decode_args *args, int form, gd_tensor *out)
{
    gd_backend_tensor_view qv, kv, vv, pv, ov;
    gd_tensor o;
    gd_status st;
    GD_TRY(gd_tensor_alloc_like_shape(ctx, q->dtype, 4U, q->shape, &o));
    if (!gd_op_tensor_view(q, &qv) || !gd_op_tensor_view(kc, &kv) || !gd_op_tensor_view(vc, &vv) ||
        !gd_op_tensor_view(&o, &ov) || (pos != NULL && !gd_op_tensor_view(pos, &pv)))
        GD_FAIL(ctx, GD_ERR_INTERNAL, "sdpa_decode view construction failed");
    if (form == 0) st = gd_backend_sdpa_decode(gd_context_backend(ctx), &qv, &kv, &vv, &pv, &ov, args);
    else if (form == 1) st = gd_backend_sdpa_decode_at(gd_context_backend(ctx), &qv, &kv, &vv, &ov, args);
    else st = gd_backend_sdpa_decode_positions(gd_context_backend(ctx), &qv, &kv, &vv, &pv, &ov, args);
    GD_TRY(gd_op_backend_result(ctx, st, "backend sdpa_decode failed"));
    *out = o;
    return GD_OK;
}

gd_status gd_sdpa_decode(gd_context *ctx, const gd_tensor *q, const gd_tensor *k_cache, const gd_tensor *v_cache,
                         const gd_tensor *cache_pos, const gd_sdpa_decode_config *config, gd_tensor *out)
{
    gd_backend_sdpa_decode_args args;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || cache_pos == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(validate_common(ctx, q, k_cache, v_cache, config, &args));
    GD_TRY(gd_tensor_validate(ctx, cache_pos));
    if (cache_pos->dtype != GD_DTYPE_I32 || cache_pos->rank != 0U)
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "sdpa_decode cache_pos must be an i32 scalar");
    return run(ctx, q, k_cache, v_cache, cache_pos, &args, 0, out);
}

gd_status gd_sdpa_decode_at(gd_context *ctx, const gd_tensor *q, const gd_tensor *k_cache, const gd_tensor *v_cache,
                            int32_t cache_pos, const gd_sdpa_decode_config *config, gd_tensor *out)
{
    gd_backend_sdpa_decode_args args;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(validate_common(ctx, q, k_cache, v_cache, config, &args));
    if (cache_pos < 0 || (int64_t)cache_pos > k_cache->shape[1] || q->shape[1] > k_cache->shape[1] - (int64_t)cache_pos)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "sdpa_decode cache_pos out of range");
    args.cache_pos = cache_pos;
    return run(ctx, q, k_cache, v_cache, NULL, &args, 1, out);
}

gd_status gd_sdpa_decode_positions(gd_context *ctx, const gd_tensor *q, const gd_tensor *k_cache,
                                   const gd_tensor *v_cache, const gd_tensor *cache_pos,
                                   const gd_sdpa_decode_config *config, gd_tensor *out)
{
    gd_backend_sdpa_decode_args args;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || cache_pos == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    GD_TRY(validate_common(ctx, q, k_cache, v_cache, config, &args));
    GD_TRY(gd_tensor_validate(ctx, cache_pos));
    if (cache_pos->dtype != GD_DTYPE_I32 || cache_pos->rank != 1U || cache_pos->shape[0] != q->shape[0] ||
        !gd_tensor_is_contiguous(cache_pos))
        GD_FAIL(ctx, GD_ERR_UNSUPPORTED, "sdpa_decode cache_pos must be i32 [B]");
    return run(ctx, q, k_cache, v_cache, cache_pos, &args, 2, out);
}
