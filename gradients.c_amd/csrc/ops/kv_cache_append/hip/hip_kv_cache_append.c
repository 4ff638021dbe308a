/*
 * Host dispatch of gd_backend_kv_cache_append_{at,positions,packed}.
 * Validation restates the reference dispatch src/ops/kv_cache_append/
 * metal_kv_cache_append.m (shape/dtype checks, copy-unit choice :183-198).
 */
#include "../../../backends/hip/backend_hip_internal.h"
#include "hip_kv_cache_append_types.h"

int gd_hip_launch_kv_cache_append(hipStream_t stream, void *k_cache, void *v_cache, const void *k_new,
                                  const void *v_new, const int32_t *pos, const int32_t *cu,
                                  const gd_hip_kv_append_params *params);

static bool caches_ok(const gd_backend_tensor_view *kc, const gd_backend_tensor_view *vc)
{
    uint32_t i;
    if (!gd_hip_view_ok(kc) || !gd_hip_view_ok(vc) || kc->rank != 4u || vc->rank != 4u) return false;
    if ((kc->dtype != GD_BACKEND_DTYPE_F16 && kc->dtype != GD_BACKEND_DTYPE_F32) || vc->dtype != kc->dtype) return false;
    for (i = 0u; i < 4u; ++i) {
        if (kc->shape[i] != vc->shape[i] || kc->shape[i] > (int64_t)INT32_MAX) return false;
    }
    return true;
}

static bool i32_vector_ok(const gd_backend_tensor_view *v, int64_t len)
{
    return gd_hip_view_ok(v) && v->dtype == GD_BACKEND_DTYPE_I32 && v->rank == 1u && v->shape[0] == len &&
           (v->offset & 3u) == 0u;
}

static uint32_t pick_unit(uint64_t row_bytes, const gd_backend_tensor_view *a, const gd_backend_tensor_view *b,
                          const gd_backend_tensor_view *c, const gd_backend_tensor_view *d)
{
    const uint64_t all = row_bytes | a->offset | b->offset | c->offset | d->offset;
    if ((all & 15u) == 0u) return 16u;
    if ((all & 3u) == 0u) return 4u;
    return 1u;
}

static gd_status append_batched(gd_backend *backend, const gd_backend_tensor_view *kc,
                                const gd_backend_tensor_view *vc, const gd_backend_tensor_view *pos,
                                const gd_backend_tensor_view *kn, const gd_backend_tensor_view *vn,
                                int32_t scalar_pos)
{
    gd_hip_kv_append_params p;
    uint32_t i;
    size_t es;
    if (backend == NULL || !caches_ok(kc, vc) || !gd_hip_view_ok(kn) || !gd_hip_view_ok(vn) ||
        kn->rank != 4u || vn->rank != 4u || kn->dtype != kc->dtype || vn->dtype != kc->dtype)
        return GD_ERR_INVALID_ARGUMENT;
    for (i = 0u; i < 4u; ++i) {
        if (kn->shape[i] != vn->shape[i]) return GD_ERR_INVALID_ARGUMENT;
    }
    if (kn->shape[0] != kc->shape[0] || kn->shape[2] != kc->shape[2] || kn->shape[3] != kc->shape[3] ||
        kn->shape[1] > kc->shape[1])
        return GD_ERR_INVALID_ARGUMENT;
    if (pos != NULL && !i32_vector_ok(pos, kc->shape[0])) return GD_ERR_INVALID_ARGUMENT;
    if (pos == NULL && (scalar_pos < 0 || (int64_t)scalar_pos > kc->shape[1] ||
                        kn->shape[1] > kc->shape[1] - (int64_t)scalar_pos))
        return GD_ERR_INVALID_ARGUMENT;
    es = gd_hip_dtype_size(kc->dtype);
    p.row_bytes = (uint64_t)kc->shape[2] * (uint64_t)kc->shape[3] * es;
    p.tnew = (uint64_t)kn->shape[1];
    p.tmax = (uint64_t)kc->shape[1];
    p.batch = (uint64_t)kc->shape[0];
    p.cache_pos = scalar_pos;
    p.copy_unit = pick_unit(p.row_bytes, kc, vc, kn, vn);
    p.total_units = p.batch * p.tnew * p.row_bytes;
    return gd_hip_finish_op(backend, gd_hip_launch_kv_cache_append(
        backend->stream, gd_hip_view_ptr(kc), gd_hip_view_ptr(vc), gd_hip_view_ptr(kn), gd_hip_view_ptr(vn),
        pos != NULL ? (const int32_t *)gd_hip_view_ptr(pos) : NULL, NULL, &p));
}

gd_status gd_backend_kv_cache_append_at(gd_backend *backend, const gd_backend_tensor_view *k_cache,
                                        const gd_backend_tensor_view *v_cache,
                                        const gd_backend_tensor_view *k_new,
                                        const gd_backend_tensor_view *v_new,
                                        const gd_backend_kv_cache_append_args *args)
{
    if (args == NULL) return GD_ERR_INVALID_ARGUMENT;
    return append_batched(backend, k_cache, v_cache, NULL, k_new, v_new, args->cache_pos);
}

gd_status gd_backend_kv_cache_append_positions(gd_backend *backend, const gd_backend_tensor_view *k_cache,
                                               const gd_backend_tensor_view *v_cache,
                                               const gd_backend_tensor_view *cache_pos,
                                               const gd_backend_tensor_view *k_new,
                                               const gd_backend_tensor_view *v_new,
                                               const gd_backend_kv_cache_append_args *args)
{
    (void)args;
    if (cache_pos == NULL) return GD_ERR_INVALID_ARGUMENT;
    return append_batched(backend, k_cache, v_cache, cache_pos, k_new, v_new, 0);
}

gd_status gd_backend_kv_cache_append_packed(gd_backend *backend, const gd_backend_tensor_view *k_cache,
                                            const gd_backend_tensor_view *v_cache,
                                            const gd_backend_tensor_view *cache_pos,
                                            const gd_backend_tensor_view *cu_seqlens,
                                            const gd_backend_tensor_view *k_new,
                                            const gd_backend_tensor_view *v_new,
                                            const gd_backend_kv_cache_append_args *args)
{
    gd_hip_kv_append_params p;
    uint32_t i;
    size_t es;
    const gd_backend_tensor_view *kc = k_cache, *vc = v_cache, *kn = k_new, *vn = v_new;
    (void)args;
    if (backend == NULL || !caches_ok(kc, vc) || !gd_hip_view_ok(kn) || !gd_hip_view_ok(vn) ||
        kn->rank != 3u || vn->rank != 3u || kn->dtype != kc->dtype || vn->dtype != kc->dtype)
        return GD_ERR_INVALID_ARGUMENT;
    for (i = 0u; i < 3u; ++i) {
        if (kn->shape[i] != vn->shape[i]) return GD_ERR_INVALID_ARGUMENT;
    }
    if (kn->shape[1] != kc->shape[2] || kn->shape[2] != kc->shape[3] || kn->shape[0] > (int64_t)INT32_MAX ||
        !i32_vector_ok(cache_pos, kc->shape[0]) || !i32_vector_ok(cu_seqlens, kc->shape[0] + 1))
        return GD_ERR_INVALID_ARGUMENT;
    es = gd_hip_dtype_size(kc->dtype);
    p.row_bytes = (uint64_t)kc->shape[2] * (uint64_t)kc->shape[3] * es;
    p.tnew = 0u;
    p.tmax = (uint64_t)kc->shape[1];
    p.batch = (uint64_t)kc->shape[0];
    p.cache_pos = 0;
    p.copy_unit = pick_unit(p.row_bytes, kc, vc, kn, vn);
    p.total_units = (uint64_t)kn->shape[0] * p.row_bytes;
    return gd_hip_finish_op(backend, gd_hip_launch_kv_cache_append(
        backend->stream, gd_hip_view_ptr(kc), gd_hip_view_ptr(vc), gd_hip_view_ptr(kn), gd_hip_view_ptr(vn),
        (const int32_t *)gd_hip_view_ptr(cache_pos), (const int32_t *)gd_hip_view_ptr(cu_seqlens), &p));
}
