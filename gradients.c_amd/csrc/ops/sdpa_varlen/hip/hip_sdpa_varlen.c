/*
 * Host dispatch of gd_backend_sdpa_varlen (reference src/core/backend.h:671-698; checks of
 * src/ops/sdpa_varlen/core_sdpa_varlen.c:12-122 that concern the backend: shapes, dtype,
 * head-size limit raised from 64 to 256, prefix needs causal).  The stats output of the
 * training path is not produced: a non-NULL stats view is refused.
 */
#include <math.h>

#include "../../../backends/hip/backend_hip_internal.h"

int gd_hip_launch_sdpa_varlen(hipStream_t stream, const void *q, const void *k, const void *v, const int32_t *cu,
                              void *out, uint32_t n_rows, uint32_t batch, uint32_t hq, uint32_t hkv, uint32_t dh,
                              uint32_t causal, uint32_t window, uint32_t prefix_len, uint32_t max_seqlen, float scale,
                              int is_f16);
int gd_hip_launch_sdpa_varlen_mfma(hipStream_t stream, const void *q, const void *k, const void *v, const int32_t *cu,
                                   void *out, uint32_t n_rows, uint32_t batch, uint32_t hq, uint32_t hkv, uint32_t dh,
                                   uint32_t causal, uint32_t window, uint32_t prefix_len, uint32_t max_seqlen,
                                   float scale, uint32_t kv_tmax);

gd_status gd_backend_sdpa_varlen(gd_backend *backend, const gd_backend_tensor_view *q,
                                 const gd_backend_tensor_view *k, const gd_backend_tensor_view *v,
                                 const gd_backend_tensor_view *cu_seqlens, const gd_backend_tensor_view *out,
                                 const gd_backend_tensor_view *stats, const gd_backend_sdpa_varlen_args *args)
{
    uint32_t i;
    if (backend == NULL || args == NULL || !gd_hip_view_ok(q) || !gd_hip_view_ok(k) || !gd_hip_view_ok(v) ||
        !gd_hip_view_ok(cu_seqlens) || !gd_hip_view_ok(out))
        return GD_ERR_INVALID_ARGUMENT;
    if (stats != NULL || args->use_forward_stats != 0u) return GD_ERR_UNSUPPORTED;
    if ((q->dtype != GD_BACKEND_DTYPE_F16 && q->dtype != GD_BACKEND_DTYPE_F32) || k->dtype != q->dtype ||
        v->dtype != q->dtype || out->dtype != q->dtype || cu_seqlens->dtype != GD_BACKEND_DTYPE_I32)
        return GD_ERR_UNSUPPORTED;
    if (q->rank != 3u || k->rank != 3u || v->rank != 3u || out->rank != 3u || cu_seqlens->rank != 1u ||
        cu_seqlens->shape[0] < 2 || (cu_seqlens->offset & 3u) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    for (i = 0u; i < 3u; ++i) {
        if (k->shape[i] != v->shape[i] || out->shape[i] != q->shape[i]) return GD_ERR_INVALID_ARGUMENT;
    }
    if (q->shape[0] != k->shape[0] || q->shape[2] != k->shape[2] || (q->shape[1] % k->shape[1]) != 0 ||
        q->shape[2] > 256 || q->shape[1] > 65535 || (uint64_t)q->shape[0] * (uint64_t)q->shape[1] > 0x7fffffffu ||
        cu_seqlens->shape[0] - 1 > (int64_t)INT32_MAX)
        return GD_ERR_INVALID_ARGUMENT;
    if (!(args->scale > 0.0f) || !isfinite(args->scale) || (args->prefix_len > 0u && args->causal == 0u) ||
        (args->max_seqlen > 0u && args->prefix_len > args->max_seqlen))
        return GD_ERR_INVALID_ARGUMENT;
    /* matrix-core kernel: F16, head size 64 or 128, 16-byte aligned rows, 32-bit byte offsets into K and V */
    if (q->dtype == GD_BACKEND_DTYPE_F16 && (q->shape[2] == 64 || q->shape[2] == 128) &&
        ((q->offset | k->offset | v->offset | out->offset) & 15u) == 0u &&
        (uint64_t)k->shape[0] * (uint64_t)k->shape[1] * (uint64_t)k->shape[2] * 2u < 0xffffffffull &&
        args->sliding_window <= (uint32_t)INT32_MAX && args->prefix_len <= (uint32_t)INT32_MAX)
        return gd_hip_finish_op(backend, gd_hip_launch_sdpa_varlen_mfma(
            backend->stream, gd_hip_view_ptr(q), gd_hip_view_ptr(k), gd_hip_view_ptr(v),
            (const int32_t *)gd_hip_view_ptr(cu_seqlens), gd_hip_view_ptr(out), (uint32_t)q->shape[0],
            (uint32_t)(cu_seqlens->shape[0] - 1), (uint32_t)q->shape[1], (uint32_t)k->shape[1], (uint32_t)q->shape[2],
            args->causal, args->sliding_window, args->prefix_len, args->max_seqlen, args->scale, 0u));
    return gd_hip_finish_op(backend, gd_hip_launch_sdpa_varlen(
        backend->stream, gd_hip_view_ptr(q), gd_hip_view_ptr(k), gd_hip_view_ptr(v),
        (const int32_t *)gd_hip_view_ptr(cu_seqlens), gd_hip_view_ptr(out), (uint32_t)q->shape[0],
        (uint32_t)(cu_seqlens->shape[0] - 1), (uint32_t)q->shape[1], (uint32_t)k->shape[1], (uint32_t)q->shape[2],
        args->causal, args->sliding_window, args->prefix_len, args->max_seqlen, args->scale,
        q->dtype == GD_BACKEND_DTYPE_F16));
}

/* Packed attention whose keys and values are read where the prefill has just appended them: the caches
 * [B, Tmax, Hkv, D], token t of segment b in cache row t of sequence b (see the header).  Matrix-core kernel only. */
gd_status gd_backend_sdpa_varlen_cached(gd_backend *backend, const gd_backend_tensor_view *q,
                                        const gd_backend_tensor_view *k_cache, const gd_backend_tensor_view *v_cache,
                                        const gd_backend_tensor_view *cu_seqlens, const gd_backend_tensor_view *out,
                                        const gd_backend_sdpa_varlen_args *args)
{
    uint32_t i;
    if (backend == NULL || args == NULL || !gd_hip_view_ok(q) || !gd_hip_view_ok(k_cache) || !gd_hip_view_ok(v_cache) ||
        !gd_hip_view_ok(cu_seqlens) || !gd_hip_view_ok(out))
        return GD_ERR_INVALID_ARGUMENT;
    if (args->use_forward_stats != 0u) return GD_ERR_UNSUPPORTED;
    if (q->rank != 3u || out->rank != 3u || k_cache->rank != 4u || v_cache->rank != 4u || cu_seqlens->rank != 1u ||
        cu_seqlens->shape[0] < 2 || (cu_seqlens->offset & 3u) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    for (i = 0u; i < 4u; ++i) {
        if (k_cache->shape[i] != v_cache->shape[i]) return GD_ERR_INVALID_ARGUMENT;
    }
    for (i = 0u; i < 3u; ++i) {
        if (out->shape[i] != q->shape[i]) return GD_ERR_INVALID_ARGUMENT;
    }
    if (k_cache->shape[0] != cu_seqlens->shape[0] - 1 || k_cache->shape[0] > (int64_t)INT32_MAX ||
        k_cache->shape[1] <= 0 || k_cache->shape[1] > (int64_t)INT32_MAX || k_cache->shape[2] <= 0 ||
        q->shape[2] != k_cache->shape[3] || (q->shape[1] % k_cache->shape[2]) != 0 || q->shape[1] > 65535 ||
        (uint64_t)q->shape[0] * (uint64_t)q->shape[1] > 0x7fffffffu)
        return GD_ERR_INVALID_ARGUMENT;
    if (!(args->scale > 0.0f) || !isfinite(args->scale) || (args->prefix_len > 0u && args->causal == 0u) ||
        (args->max_seqlen > 0u && args->prefix_len > args->max_seqlen))
        return GD_ERR_INVALID_ARGUMENT;
    if (q->dtype != GD_BACKEND_DTYPE_F16 || k_cache->dtype != GD_BACKEND_DTYPE_F16 ||
        v_cache->dtype != GD_BACKEND_DTYPE_F16 || out->dtype != GD_BACKEND_DTYPE_F16 ||
        cu_seqlens->dtype != GD_BACKEND_DTYPE_I32 || (q->shape[2] != 64 && q->shape[2] != 128) ||
        ((q->offset | k_cache->offset | v_cache->offset | out->offset) & 15u) != 0u ||
        (uint64_t)k_cache->count * 2u >= 0xffffffffull || args->sliding_window > (uint32_t)INT32_MAX ||
        args->prefix_len > (uint32_t)INT32_MAX)
        return GD_ERR_UNSUPPORTED;
    return gd_hip_finish_op(backend, gd_hip_launch_sdpa_varlen_mfma(
        backend->stream, gd_hip_view_ptr(q), gd_hip_view_ptr(k_cache), gd_hip_view_ptr(v_cache),
        (const int32_t *)gd_hip_view_ptr(cu_seqlens), gd_hip_view_ptr(out), (uint32_t)q->shape[0],
        (uint32_t)(cu_seqlens->shape[0] - 1), (uint32_t)q->shape[1], (uint32_t)k_cache->shape[2], (uint32_t)q->shape[2],
        args->causal, args->sliding_window, args->prefix_len, args->max_seqlen, args->scale,
        (uint32_t)k_cache->shape[1]));
}
