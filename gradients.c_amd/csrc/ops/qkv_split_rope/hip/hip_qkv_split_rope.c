/*
 * Host dispatch of gd_backend_qkv_split_rope_forward.  Checks restate the reference
 * src/ops/qkv_split_rope/metal_qkv_split_rope.m:195-216 (shapes, even head size, full-head
 * rotation only).
 */
#include "../../../backends/hip/backend_hip_internal.h"

int gd_hip_launch_qkv_split_rope(hipStream_t stream, const void *qkv, const int32_t *pos, void *q, void *k,
                                 void *v, uint64_t tokens, uint32_t heads, uint32_t head_dim, float theta,
                                 uint32_t interleaved, int aligned16);

static bool out_ok(const gd_backend_tensor_view *t, int64_t tokens, uint32_t heads, uint32_t head_dim)
{
    return gd_hip_view_ok(t) && t->dtype == GD_BACKEND_DTYPE_F16 && t->rank == 3u && t->shape[0] == tokens &&
           t->shape[1] == (int64_t)heads && t->shape[2] == (int64_t)head_dim;
}

gd_status gd_backend_qkv_split_rope_forward(gd_backend *backend, const gd_backend_tensor_view *qkv,
                                            const gd_backend_tensor_view *pos_ids,
                                            const gd_backend_tensor_view *q, const gd_backend_tensor_view *k,
                                            const gd_backend_tensor_view *v, uint32_t n_heads, uint32_t head_dim,
                                            const gd_backend_rope_args *args)
{
    int64_t tokens;
    uint64_t area;
    if (backend == NULL || args == NULL || !gd_hip_view_ok(qkv) || !gd_hip_view_ok(pos_ids) || n_heads == 0u ||
        head_dim == 0u || qkv->rank != 2u || qkv->dtype != GD_BACKEND_DTYPE_F16 ||
        pos_ids->dtype != GD_BACKEND_DTYPE_I32 || pos_ids->rank != 1u || (pos_ids->offset & 3u) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    tokens = qkv->shape[0];
    area = (uint64_t)n_heads * head_dim;
    if (tokens <= 0 || pos_ids->shape[0] != tokens || (uint64_t)qkv->shape[1] != area * 3u ||
        !out_ok(q, tokens, n_heads, head_dim) || !out_ok(k, tokens, n_heads, head_dim) ||
        !out_ok(v, tokens, n_heads, head_dim) || (head_dim & 1u) != 0u || !(args->theta > 0.0f) ||
        args->n_dims != head_dim || (uint64_t)tokens * area / 2u > 0x7fffffffull * 256u)
        return GD_ERR_INVALID_ARGUMENT;
    return gd_hip_finish_op(backend, gd_hip_launch_qkv_split_rope(
        backend->stream, gd_hip_view_ptr(qkv), (const int32_t *)gd_hip_view_ptr(pos_ids), gd_hip_view_ptr(q),
        gd_hip_view_ptr(k), gd_hip_view_ptr(v), (uint64_t)tokens, n_heads, head_dim, args->theta,
        args->interleaved, ((qkv->offset | q->offset | k->offset | v->offset) & 15u) == 0u));
}

int gd_hip_launch_qkv_rope_append(hipStream_t stream, const void *qkv, const int32_t *rope_pos, const int32_t *cache_pos,
                                  void *q, void *k_cache, void *v_cache, uint64_t tokens, uint32_t heads,
                                  uint32_t head_dim, uint32_t tmax, float theta);

gd_status gd_backend_qkv_rope_append(gd_backend *backend, const gd_backend_tensor_view *qkv,
                                     const gd_backend_tensor_view *pos_ids, const gd_backend_tensor_view *cache_pos,
                                     const gd_backend_tensor_view *q, const gd_backend_tensor_view *k_cache,
                                     const gd_backend_tensor_view *v_cache, uint32_t n_heads, uint32_t head_dim,
                                     const gd_backend_rope_args *args)
{
    int64_t tokens;
    uint32_t i;
    if (backend == NULL || args == NULL || !gd_hip_view_ok(qkv) || !gd_hip_view_ok(pos_ids) || !gd_hip_view_ok(cache_pos) ||
        !gd_hip_view_ok(k_cache) || !gd_hip_view_ok(v_cache) || n_heads == 0u || head_dim == 0u || qkv->rank != 2u ||
        pos_ids->rank != 1u || cache_pos->rank != 1u || k_cache->rank != 4u || v_cache->rank != 4u)
        return GD_ERR_INVALID_ARGUMENT;
    if (qkv->dtype != GD_BACKEND_DTYPE_F16 || k_cache->dtype != GD_BACKEND_DTYPE_F16 ||
        v_cache->dtype != GD_BACKEND_DTYPE_F16 || pos_ids->dtype != GD_BACKEND_DTYPE_I32 ||
        cache_pos->dtype != GD_BACKEND_DTYPE_I32)
        return GD_ERR_UNSUPPORTED;
    tokens = qkv->shape[0];
    for (i = 0u; i < 4u; ++i) {
        if (k_cache->shape[i] != v_cache->shape[i]) return GD_ERR_INVALID_ARGUMENT;
    }
    if (tokens <= 0 || pos_ids->shape[0] != tokens || cache_pos->shape[0] != tokens || k_cache->shape[0] != tokens ||
        k_cache->shape[2] != (int64_t)n_heads || k_cache->shape[3] != (int64_t)head_dim ||
        (uint64_t)qkv->shape[1] != (uint64_t)n_heads * head_dim * 3u || !out_ok(q, tokens, n_heads, head_dim) ||
        k_cache->shape[1] > (int64_t)INT32_MAX || !(args->theta > 0.0f) || args->n_dims != head_dim ||
        ((pos_ids->offset | cache_pos->offset) & 3u) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    /* vector kernel only: NeoX pairing, head size a multiple of 16, 16-byte aligned tensors */
    if (args->interleaved != 0u || (head_dim % 16u) != 0u ||
        ((qkv->offset | q->offset | k_cache->offset | v_cache->offset) & 15u) != 0u)
        return GD_ERR_UNSUPPORTED;
    return gd_hip_finish_op(backend, gd_hip_launch_qkv_rope_append(
        backend->stream, gd_hip_view_ptr(qkv), (const int32_t *)gd_hip_view_ptr(pos_ids),
        (const int32_t *)gd_hip_view_ptr(cache_pos), gd_hip_view_ptr(q), gd_hip_view_ptr(k_cache), gd_hip_view_ptr(v_cache),
        (uint64_t)tokens, n_heads, head_dim, (uint32_t)k_cache->shape[1], args->theta));
}

int gd_hip_launch_qkv_rope_append_packed(hipStream_t stream, const void *qkv, const int32_t *rope_pos,
                                         const int32_t *seq_pos, const int32_t *cu, uint32_t batch, void *q, void *k,
                                         void *v, void *k_cache, void *v_cache, uint64_t tokens, uint32_t heads,
                                         uint32_t head_dim, uint32_t tmax, float theta);

/* Packed-prefill form of qkv_split_rope + kv_cache_append_packed in one launch (see the header). */
gd_status gd_backend_qkv_rope_append_packed(gd_backend *backend, const gd_backend_tensor_view *qkv,
                                            const gd_backend_tensor_view *pos_ids,
                                            const gd_backend_tensor_view *cache_pos, const gd_backend_tensor_view *cu_seqlens,
                                            const gd_backend_tensor_view *q, const gd_backend_tensor_view *k,
                                            const gd_backend_tensor_view *v, const gd_backend_tensor_view *k_cache,
                                            const gd_backend_tensor_view *v_cache, uint32_t n_heads, uint32_t head_dim,
                                            const gd_backend_rope_args *args)
{
    int64_t tokens, batch;
    uint32_t i;
    if (backend == NULL || args == NULL || !gd_hip_view_ok(qkv) || !gd_hip_view_ok(pos_ids) || !gd_hip_view_ok(cache_pos) ||
        !gd_hip_view_ok(cu_seqlens) || !gd_hip_view_ok(k_cache) || !gd_hip_view_ok(v_cache) || n_heads == 0u ||
        head_dim == 0u || qkv->rank != 2u || pos_ids->rank != 1u || cache_pos->rank != 1u || cu_seqlens->rank != 1u ||
        k_cache->rank != 4u || v_cache->rank != 4u)
        return GD_ERR_INVALID_ARGUMENT;
    if (qkv->dtype != GD_BACKEND_DTYPE_F16 || k_cache->dtype != GD_BACKEND_DTYPE_F16 ||
        v_cache->dtype != GD_BACKEND_DTYPE_F16 || pos_ids->dtype != GD_BACKEND_DTYPE_I32 ||
        cache_pos->dtype != GD_BACKEND_DTYPE_I32 || cu_seqlens->dtype != GD_BACKEND_DTYPE_I32)
        return GD_ERR_UNSUPPORTED;
    tokens = qkv->shape[0];
    batch = k_cache->shape[0];
    for (i = 0u; i < 4u; ++i) {
        if (k_cache->shape[i] != v_cache->shape[i]) return GD_ERR_INVALID_ARGUMENT;
    }
    if (tokens <= 0 || batch <= 0 || batch > (int64_t)INT32_MAX || pos_ids->shape[0] != tokens ||
        cache_pos->shape[0] != batch || cu_seqlens->shape[0] != batch + 1 || k_cache->shape[2] != (int64_t)n_heads ||
        k_cache->shape[3] != (int64_t)head_dim || (uint64_t)qkv->shape[1] != (uint64_t)n_heads * head_dim * 3u ||
        !out_ok(q, tokens, n_heads, head_dim) || (k == NULL) != (v == NULL) ||
        (k != NULL && (!out_ok(k, tokens, n_heads, head_dim) || !out_ok(v, tokens, n_heads, head_dim))) ||
        k_cache->shape[1] > (int64_t)INT32_MAX || !(args->theta > 0.0f) ||
        args->n_dims != head_dim || ((pos_ids->offset | cache_pos->offset | cu_seqlens->offset) & 3u) != 0u ||
        (uint64_t)tokens * n_heads * head_dim / 2u > 0x7fffffffull * 256u)
        return GD_ERR_INVALID_ARGUMENT;
    /* vector kernel only: NeoX pairing, head size a multiple of 16, 16-byte aligned tensors */
    if (args->interleaved != 0u || (head_dim % 16u) != 0u ||
        ((qkv->offset | q->offset | (k != NULL ? k->offset | v->offset : 0u) | k_cache->offset | v_cache->offset) & 15u) != 0u)
        return GD_ERR_UNSUPPORTED;
    return gd_hip_finish_op(backend, gd_hip_launch_qkv_rope_append_packed(
        backend->stream, gd_hip_view_ptr(qkv), (const int32_t *)gd_hip_view_ptr(pos_ids),
        (const int32_t *)gd_hip_view_ptr(cache_pos), (const int32_t *)gd_hip_view_ptr(cu_seqlens), (uint32_t)batch,
        gd_hip_view_ptr(q), k != NULL ? gd_hip_view_ptr(k) : NULL, v != NULL ? gd_hip_view_ptr(v) : NULL,
        gd_hip_view_ptr(k_cache), gd_hip_view_ptr(v_cache), (uint64_t)tokens, n_heads, head_dim,
        (uint32_t)k_cache->shape[1], args->theta));
}

int gd_hip_launch_rope_table_packed(hipStream_t stream, const int32_t *pos, const int32_t *cu, const int32_t *seq_pos,
                                    uint32_t batch, float *cos_rows, float *sin_rows, int32_t *cache_row, uint64_t tokens,
                                    uint32_t head_dim, uint32_t tmax, float theta);

/* Angles and cache rows of the packed prompt rows, once per prefill (see the header). */
gd_status gd_backend_rope_table_packed(gd_backend *backend, const gd_backend_tensor_view *pos_ids,
                                       const gd_backend_tensor_view *cache_pos, const gd_backend_tensor_view *cu_seqlens,
                                       const gd_backend_tensor_view *cos_rows, const gd_backend_tensor_view *sin_rows,
                                       const gd_backend_tensor_view *cache_rows, uint32_t head_dim, uint32_t tmax,
                                       const gd_backend_rope_args *args)
{
    int64_t tokens, batch;
    if (backend == NULL || args == NULL || !gd_hip_view_ok(pos_ids) || !gd_hip_view_ok(cache_pos) ||
        !gd_hip_view_ok(cu_seqlens) || !gd_hip_view_ok(cos_rows) || !gd_hip_view_ok(sin_rows) ||
        !gd_hip_view_ok(cache_rows) || pos_ids->rank != 1u || cache_pos->rank != 1u || cu_seqlens->rank != 1u ||
        cos_rows->rank != 2u || sin_rows->rank != 2u || cache_rows->rank != 1u || head_dim == 0u || tmax == 0u)
        return GD_ERR_INVALID_ARGUMENT;
    if (pos_ids->dtype != GD_BACKEND_DTYPE_I32 || cache_pos->dtype != GD_BACKEND_DTYPE_I32 ||
        cu_seqlens->dtype != GD_BACKEND_DTYPE_I32 || cache_rows->dtype != GD_BACKEND_DTYPE_I32 ||
        cos_rows->dtype != GD_BACKEND_DTYPE_F32 || sin_rows->dtype != GD_BACKEND_DTYPE_F32)
        return GD_ERR_UNSUPPORTED;
    tokens = pos_ids->shape[0];
    batch = cache_pos->shape[0];
    if (tokens <= 0 || batch <= 0 || cu_seqlens->shape[0] != batch + 1 || cache_rows->shape[0] != tokens ||
        cos_rows->shape[0] != (tokens + 31) / 32 * 32 || sin_rows->shape[0] != cos_rows->shape[0] || (head_dim % 16u) != 0u ||
        cos_rows->shape[1] != (int64_t)(head_dim / 2u) || sin_rows->shape[1] != (int64_t)(head_dim / 2u) ||
        (uint64_t)batch * (uint64_t)tmax > (uint64_t)INT32_MAX || !(args->theta > 0.0f) || args->n_dims != head_dim ||
        ((pos_ids->offset | cache_pos->offset | cu_seqlens->offset | cache_rows->offset | cos_rows->offset |
          sin_rows->offset) & 3u) != 0u ||
        ((cos_rows->offset | sin_rows->offset) & 15u) != 0u || (uint64_t)cos_rows->shape[0] * (head_dim / 2u) > 0x7fffffffull)
        return GD_ERR_INVALID_ARGUMENT;
    if (args->interleaved != 0u) return GD_ERR_UNSUPPORTED;
    return gd_hip_finish_op(backend, gd_hip_launch_rope_table_packed(
        backend->stream, (const int32_t *)gd_hip_view_ptr(pos_ids), (const int32_t *)gd_hip_view_ptr(cu_seqlens),
        (const int32_t *)gd_hip_view_ptr(cache_pos), (uint32_t)batch, (float *)gd_hip_view_ptr(cos_rows),
        (float *)gd_hip_view_ptr(sin_rows), (int32_t *)gd_hip_view_ptr(cache_rows), (uint64_t)tokens, head_dim, tmax,
        args->theta));
}
