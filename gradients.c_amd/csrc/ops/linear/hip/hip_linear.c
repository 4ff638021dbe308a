/*
 * Host dispatch of the projection entry points: gd_backend_matmul, gd_backend_matmul_nt,
 * gd_backend_linear (reference src/core/backend.h:187-195, 215-219) and the fused
 * gd_backend_linear_nt / gd_backend_swiglu_split_linear.
 */
#include "../../../backends/hip/backend_hip_internal.h"
#include "hip_linear_types.h"

int gd_hip_launch_linear(hipStream_t stream, const void *x, const void *w, const void *bias, const void *residual,
                         const void *norm_w, void *y, const gd_hip_linear_params *params, int vector_ok,
                         int kn_vector_ok, int store_vector_ok, int min_workgroups, const gd_hip_rope_epilogue *rope,
                         int wide_mode, int *family);

static gd_status project_full(gd_backend *backend, const gd_backend_matrix_view *x, const gd_backend_matrix_view *w,
                              const gd_backend_vector_view *bias, const gd_backend_matrix_view *residual,
                              const gd_backend_vector_view *norm_w, float eps, const gd_backend_matrix_view *y,
                              uint32_t w_is_nk, uint32_t epilogue, uint32_t prologue, uint32_t gated)
{
    gd_hip_linear_params p;
    uint32_t K;
    int vec, kn_vec, store_vec;
    if (backend == NULL || !gd_hip_matrix_ok(x) || !gd_hip_matrix_ok(w) || !gd_hip_matrix_ok(y) ||
        (bias != NULL && !gd_hip_vector_ok(bias)) || (residual != NULL && !gd_hip_matrix_ok(residual)) ||
        (norm_w != NULL && !gd_hip_vector_ok(norm_w)))
        return GD_ERR_INVALID_ARGUMENT;
    if (x->dtype != GD_BACKEND_DTYPE_F16 || w->dtype != GD_BACKEND_DTYPE_F16 || y->dtype != GD_BACKEND_DTYPE_F16 ||
        (bias != NULL && bias->dtype != GD_BACKEND_DTYPE_F16) ||
        (residual != NULL && residual->dtype != GD_BACKEND_DTYPE_F16) ||
        (norm_w != NULL && norm_w->dtype != GD_BACKEND_DTYPE_F16))
        return GD_ERR_UNSUPPORTED;
    if (prologue == GD_HIP_PRO_SWIGLU) {
        if ((x->cols & 1u) != 0u) return GD_ERR_INVALID_ARGUMENT;
        K = x->cols / 2u;
    } else {
        K = x->cols;
    }
    if (gated) {
        /* swiglu epilogue: w [2H,K], bias [2H], y [M,H] */
        if (!w_is_nk || residual != NULL) return GD_ERR_UNSUPPORTED;
        if (w->cols != K || (w->rows & 1u) != 0u || w->rows / 2u != y->cols || (bias != NULL && bias->length != w->rows))
            return GD_ERR_INVALID_ARGUMENT;
    } else if (w_is_nk ? (w->cols != K || w->rows != y->cols) : (w->rows != K || w->cols != y->cols)) {
        return GD_ERR_INVALID_ARGUMENT;
    }
    if (x->rows != y->rows || (!gated && bias != NULL && bias->length != y->cols) ||
        (residual != NULL && (residual->rows != y->rows || residual->cols != y->cols)) ||
        ((prologue == GD_HIP_PRO_RMS_NORM) != (norm_w != NULL)) || (norm_w != NULL && (norm_w->length != K || !(eps > 0.0f))))
        return GD_ERR_INVALID_ARGUMENT;
    if ((uint64_t)y->rows * y->cols > 0x7fffffffull * 256u || (y->cols + 15u) / 16u > 0x7fffffffu ||
        (y->rows + 15u) / 16u > 65535u)
        return GD_ERR_UNSUPPORTED;
    p.M = y->rows;
    p.N = y->cols;
    p.K = K;
    p.ldx = (uint32_t)(x->row_bytes / 2u);
    p.ldw = (uint32_t)(w->row_bytes / 2u);
    p.ldy = (uint32_t)(y->row_bytes / 2u);
    p.epilogue = bias != NULL ? epilogue : GD_HIP_EPI_NONE;
    p.w_is_nk = w_is_nk;
    p.prologue = prologue;
    p.has_residual = residual != NULL ? 1u : 0u;
    p.ldr = residual != NULL ? (uint32_t)(residual->row_bytes / 2u) : 0u;
    p.eps = eps;
    p.swiglu_cols = gated ? y->cols : 0u;
    p.rope_heads = p.rope_head_dim = p.rope_tmax = 0u;
    p.rope_freq_scale = 0.0f;
    p.force_tiles = (uint16_t)backend->linear_tiles;
    p.force_waves = (uint16_t)backend->linear_waves;
    p.no_lds_stream = (uint32_t)backend->linear_no_lds_stream;
    /* 16-byte fragment loads: x rows always, w rows when K-contiguous, the norm weight */
    vec = (K % 8u) == 0u && ((x->offset | x->row_bytes) & 15u) == 0u &&
          (!w_is_nk || ((w->offset | w->row_bytes) & 15u) == 0u) && (norm_w == NULL || (norm_w->offset & 15u) == 0u);
    kn_vec = !w_is_nk && (p.N % 8u) == 0u && ((w->offset | w->row_bytes) & 15u) == 0u;
    store_vec = ((y->offset | y->row_bytes) & 15u) == 0u &&
                (residual == NULL || ((residual->offset | residual->row_bytes) & 15u) == 0u);
    if (gated && !vec) return GD_ERR_UNSUPPORTED;
    return gd_hip_finish_op(backend, gd_hip_launch_linear(
        backend->stream, gd_hip_matrix_ptr(x), gd_hip_matrix_ptr(w), bias != NULL ? gd_hip_vector_ptr(bias) : NULL,
        residual != NULL ? gd_hip_matrix_ptr(residual) : NULL, norm_w != NULL ? gd_hip_vector_ptr(norm_w) : NULL,
        gd_hip_matrix_ptr(y), &p, vec, kn_vec, store_vec, 2 * backend->compute_units, NULL, backend->linear_wide,
        &backend->last_linear_family));
}

static gd_status project(gd_backend *backend, const gd_backend_matrix_view *x, const gd_backend_matrix_view *w,
                         const gd_backend_vector_view *bias, const gd_backend_matrix_view *y, uint32_t w_is_nk,
                         uint32_t epilogue, uint32_t swiglu)
{
    return project_full(backend, x, w, bias, NULL, NULL, 0.0f, y, w_is_nk, epilogue,
                        swiglu ? GD_HIP_PRO_SWIGLU : GD_HIP_PRO_NONE, 0u);
}

gd_status gd_backend_matmul(gd_backend *backend, const gd_backend_matrix_view *x, const gd_backend_matrix_view *w,
                            const gd_backend_matrix_view *y)
{
    return project(backend, x, w, NULL, y, 0u, GD_HIP_EPI_NONE, 0u);
}

gd_status gd_backend_matmul_nt(gd_backend *backend, const gd_backend_matrix_view *x,
                               const gd_backend_matrix_view *w, const gd_backend_matrix_view *y)
{
    return project(backend, x, w, NULL, y, 1u, GD_HIP_EPI_NONE, 0u);
}

gd_status gd_backend_linear(gd_backend *backend, const gd_backend_matrix_view *x, const gd_backend_matrix_view *w,
                            const gd_backend_vector_view *bias, const gd_backend_matrix_view *y)
{
    if (bias == NULL) return GD_ERR_INVALID_ARGUMENT;
    return project(backend, x, w, bias, y, 0u, GD_HIP_EPI_BIAS_F32, 0u);
}

gd_status gd_backend_linear_nt(gd_backend *backend, const gd_backend_matrix_view *x,
                               const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                               const gd_backend_matrix_view *y)
{
    return project(backend, x, w, bias, y, 1u, GD_HIP_EPI_BIAS_F16, 0u);
}

gd_status gd_backend_swiglu_split_linear(gd_backend *backend, const gd_backend_matrix_view *x12,
                                         const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                                         const gd_backend_matrix_view *y)
{
    return project(backend, x12, w, bias, y, 0u, GD_HIP_EPI_BIAS_F32, 1u);
}

gd_status gd_backend_fused_linear(gd_backend *backend, const gd_backend_matrix_view *x,
                                  const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                                  const gd_backend_matrix_view *residual, const gd_backend_vector_view *norm_weight,
                                  const gd_backend_matrix_view *y, const gd_backend_fused_linear_args *args)
{
    if (args == NULL || args->bias_mode > 2u || args->prologue > 2u || args->epilogue > 1u ||
        (args->bias_mode != 0u) != (bias != NULL))
        return GD_ERR_INVALID_ARGUMENT;
    return project_full(backend, x, w, bias, residual, norm_weight, args->eps, y, args->w_is_nk != 0u, args->bias_mode,
                        args->prologue, args->epilogue);
}

#include <math.h>
#include <stdio.h>

/* qkv projection of a decode step with the rotation and the cache append in its epilogue */
gd_status gd_backend_fused_qkv_rope_append(gd_backend *backend, const gd_backend_matrix_view *x,
                                           const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                                           const gd_backend_vector_view *norm_weight,
                                           const gd_backend_tensor_view *pos_ids, const gd_backend_tensor_view *cache_pos,
                                           const gd_backend_tensor_view *q, const gd_backend_tensor_view *k_cache,
                                           const gd_backend_tensor_view *v_cache, uint32_t n_heads, uint32_t head_dim,
                                           const gd_backend_rope_args *rope_args,
                                           const gd_backend_fused_linear_args *args)
{
    gd_hip_linear_params p;
    gd_hip_rope_epilogue r;
    uint64_t area;
    uint32_t i;
    if (backend == NULL || args == NULL || rope_args == NULL || !gd_hip_matrix_ok(x) || !gd_hip_matrix_ok(w) ||
        (bias != NULL && !gd_hip_vector_ok(bias)) || (norm_weight != NULL && !gd_hip_vector_ok(norm_weight)) ||
        !gd_hip_view_ok(pos_ids) || !gd_hip_view_ok(cache_pos) || !gd_hip_view_ok(q) || !gd_hip_view_ok(k_cache) ||
        !gd_hip_view_ok(v_cache) || n_heads == 0u || head_dim == 0u || pos_ids->rank != 1u || cache_pos->rank != 1u ||
        q->rank != 3u || k_cache->rank != 4u || v_cache->rank != 4u || args->bias_mode > 2u || args->epilogue != 0u ||
        (args->prologue != GD_HIP_PRO_NONE && args->prologue != GD_HIP_PRO_RMS_NORM) ||
        (args->bias_mode != 0u) != (bias != NULL) || (args->prologue == GD_HIP_PRO_RMS_NORM) != (norm_weight != NULL))
        return GD_ERR_INVALID_ARGUMENT;
    if (x->dtype != GD_BACKEND_DTYPE_F16 || w->dtype != GD_BACKEND_DTYPE_F16 || q->dtype != GD_BACKEND_DTYPE_F16 ||
        k_cache->dtype != GD_BACKEND_DTYPE_F16 || v_cache->dtype != GD_BACKEND_DTYPE_F16 ||
        (bias != NULL && bias->dtype != GD_BACKEND_DTYPE_F16) ||
        (norm_weight != NULL && norm_weight->dtype != GD_BACKEND_DTYPE_F16) ||
        pos_ids->dtype != GD_BACKEND_DTYPE_I32 || cache_pos->dtype != GD_BACKEND_DTYPE_I32)
        return GD_ERR_UNSUPPORTED;
    area = (uint64_t)n_heads * head_dim;
    for (i = 0u; i < 4u; ++i) {
        if (k_cache->shape[i] != v_cache->shape[i]) return GD_ERR_INVALID_ARGUMENT;
    }
    if (area * 3u > 0xffffffffu || w->rows != (uint32_t)(area * 3u) || w->cols != x->cols ||
        (bias != NULL && bias->length != w->rows) || (norm_weight != NULL && (norm_weight->length != x->cols || !(args->eps > 0.0f))) ||
        pos_ids->shape[0] != (int64_t)x->rows || cache_pos->shape[0] != (int64_t)x->rows ||
        q->shape[0] != (int64_t)x->rows || q->shape[1] != (int64_t)n_heads || q->shape[2] != (int64_t)head_dim ||
        k_cache->shape[0] != (int64_t)x->rows || k_cache->shape[2] != (int64_t)n_heads ||
        k_cache->shape[3] != (int64_t)head_dim || k_cache->shape[1] > (int64_t)INT32_MAX || !(rope_args->theta > 0.0f) ||
        rope_args->n_dims != head_dim || ((pos_ids->offset | cache_pos->offset) & 3u) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    /* the few-row kernel with column pairs (c, c + head_dim/2) in one workgroup: [N,K] weight, NeoX pairing,
     * head size a multiple of 32, fewer than 128 rows, 16-byte aligned operand rows */
    if (args->w_is_nk == 0u || rope_args->interleaved != 0u || (head_dim % 32u) != 0u || x->rows >= 128u ||
        (x->cols % 8u) != 0u || ((x->offset | x->row_bytes | w->offset | w->row_bytes) & 15u) != 0u ||
        (norm_weight != NULL && (norm_weight->offset & 15u) != 0u) ||
        ((q->offset | k_cache->offset | v_cache->offset) & 1u) != 0u)
        return GD_ERR_UNSUPPORTED;
    p.M = x->rows;
    p.N = w->rows;
    p.K = x->cols;
    p.ldx = (uint32_t)(x->row_bytes / 2u);
    p.ldw = (uint32_t)(w->row_bytes / 2u);
    p.ldy = 0u;
    p.epilogue = bias != NULL ? args->bias_mode : GD_HIP_EPI_NONE;
    p.w_is_nk = 1u;
    p.prologue = args->prologue;
    p.has_residual = 0u;
    p.ldr = 0u;
    p.eps = args->eps;
    p.swiglu_cols = 0u;
    p.rope_heads = n_heads;
    p.rope_head_dim = head_dim;
    p.rope_tmax = (uint32_t)k_cache->shape[1];
    p.rope_freq_scale = -2.0f * log2f(rope_args->theta) / (float)head_dim;
    p.force_tiles = (uint16_t)backend->linear_tiles;
    p.force_waves = (uint16_t)backend->linear_waves;
    p.no_lds_stream = (uint32_t)backend->linear_no_lds_stream;
    r.rope_pos = (const int32_t *)gd_hip_view_ptr(pos_ids);
    r.cache_pos = (const int32_t *)gd_hip_view_ptr(cache_pos);
    r.q = gd_hip_view_ptr(q);
    r.k_cache = gd_hip_view_ptr(k_cache);
    r.v_cache = gd_hip_view_ptr(v_cache);
    return gd_hip_finish_op(backend, gd_hip_launch_linear(
        backend->stream, gd_hip_matrix_ptr(x), gd_hip_matrix_ptr(w), bias != NULL ? gd_hip_vector_ptr(bias) : NULL, NULL,
        norm_weight != NULL ? gd_hip_vector_ptr(norm_weight) : NULL, NULL, &p, 1, 0, 0, 2 * backend->compute_units, &r,
        backend->linear_wide, &backend->last_linear_family));
}

int gd_hip_launch_linear_tile_rope(hipStream_t stream, const void *x, const void *w, const void *bias,
                                   const gd_hip_linear_params *params, const float *cos_rows, const float *sin_rows,
                                   const int32_t *cache_row, void *q, void *k_cache, void *v_cache, uint32_t hd,
                                   uint32_t half_d, int compute_units);
uint32_t gd_hip_linear_tile_rope_head_rows(uint32_t M, uint32_t N, int compute_units);
int gd_hip_launch_qkv_rope_rows(hipStream_t stream, const void *qkv, const float *cos_rows, const float *sin_rows,
                                const int32_t *cache_row, void *q, void *k_cache, void *v_cache, uint64_t row0,
                                uint64_t rows, uint32_t heads, uint32_t head_dim);

/* qkv projection of a packed prefill with rotation, split and cache append in the projection's epilogue (see the
 * header): the row tiles that fill whole rounds of 256 x 256 tiles go through the tile kernel's rotation epilogue;
 * the rest goes through the plain projection into `work` and the table-driven rotation kernel. */
gd_status gd_backend_linear_qkv_rope_packed(gd_backend *backend, const gd_backend_matrix_view *x,
                                            const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                                            const gd_backend_tensor_view *cos_rows, const gd_backend_tensor_view *sin_rows,
                                            const gd_backend_tensor_view *cache_rows, const gd_backend_tensor_view *q,
                                            const gd_backend_tensor_view *k_cache, const gd_backend_tensor_view *v_cache,
                                            const gd_backend_matrix_view *work, uint32_t n_heads, uint32_t head_dim,
                                            uint32_t bias_mode)
{
    gd_hip_linear_params p;
    uint64_t area;
    uint32_t i, head_rows;
    int e;
    if (backend == NULL || !gd_hip_matrix_ok(x) || !gd_hip_matrix_ok(w) || !gd_hip_matrix_ok(work) ||
        (bias != NULL && !gd_hip_vector_ok(bias)) || !gd_hip_view_ok(cos_rows) || !gd_hip_view_ok(sin_rows) ||
        !gd_hip_view_ok(cache_rows) || !gd_hip_view_ok(q) || !gd_hip_view_ok(k_cache) || !gd_hip_view_ok(v_cache) ||
        n_heads == 0u || head_dim == 0u || cos_rows->rank != 2u || sin_rows->rank != 2u || cache_rows->rank != 1u ||
        q->rank != 3u || k_cache->rank != 4u || v_cache->rank != 4u || bias_mode > 2u || (bias_mode != 0u) != (bias != NULL))
        return GD_ERR_INVALID_ARGUMENT;
    if (x->dtype != GD_BACKEND_DTYPE_F16 || w->dtype != GD_BACKEND_DTYPE_F16 || work->dtype != GD_BACKEND_DTYPE_F16 ||
        q->dtype != GD_BACKEND_DTYPE_F16 || k_cache->dtype != GD_BACKEND_DTYPE_F16 ||
        v_cache->dtype != GD_BACKEND_DTYPE_F16 || (bias != NULL && bias->dtype != GD_BACKEND_DTYPE_F16) ||
        cos_rows->dtype != GD_BACKEND_DTYPE_F32 || sin_rows->dtype != GD_BACKEND_DTYPE_F32 ||
        cache_rows->dtype != GD_BACKEND_DTYPE_I32)
        return GD_ERR_UNSUPPORTED;
    area = (uint64_t)n_heads * head_dim;
    for (i = 0u; i < 4u; ++i) {
        if (k_cache->shape[i] != v_cache->shape[i]) return GD_ERR_INVALID_ARGUMENT;
    }
    if (area * 3u > 0xffffffffu || w->rows != (uint32_t)(area * 3u) || w->cols != x->cols || x->rows == 0u ||
        (bias != NULL && bias->length != w->rows) || work->rows != x->rows || work->cols != w->rows ||
        q->shape[0] != (int64_t)x->rows || q->shape[1] != (int64_t)n_heads || q->shape[2] != (int64_t)head_dim ||
        k_cache->shape[2] != (int64_t)n_heads || k_cache->shape[3] != (int64_t)head_dim ||
        cache_rows->shape[0] != (int64_t)x->rows || cos_rows->shape[0] != ((int64_t)x->rows + 31) / 32 * 32 ||
        sin_rows->shape[0] != cos_rows->shape[0] || cos_rows->shape[1] != (int64_t)(head_dim / 2u) ||
        (uint64_t)cos_rows->shape[0] * (head_dim / 2u) > 0x7fffffffull ||
        sin_rows->shape[1] != (int64_t)(head_dim / 2u) || (cache_rows->offset & 3u) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    if (backend->no_prefill_rope_epilogue) return GD_ERR_UNSUPPORTED; /* tunable "prefill_rope_epilogue" = 0 */
    /* the tile kernel's rotation epilogue: head size 64 or 128, heads * head_dim a multiple of 256 (every 128-column
     * block of a wavefront inside q, k or v), K a multiple of 64, 16-byte aligned rows everywhere, caches whose rows a
     * 31-bit row number reaches */
    if ((head_dim != 64u && head_dim != 128u) || (area % 256u) != 0u || (x->cols % 64u) != 0u || x->cols < 128u ||
        ((x->offset | x->row_bytes | w->offset | w->row_bytes | work->offset | work->row_bytes | q->offset |
          k_cache->offset | v_cache->offset | cos_rows->offset | sin_rows->offset) & 15u) != 0u ||
        (uint64_t)k_cache->shape[0] * (uint64_t)k_cache->shape[1] > (uint64_t)INT32_MAX ||
        work->row_bytes != (size_t)w->rows * 2u) /* the row kernel reads packed rows */
        return GD_ERR_UNSUPPORTED;
    p.M = x->rows;
    p.N = w->rows;
    p.K = x->cols;
    p.ldx = (uint32_t)(x->row_bytes / 2u);
    p.ldw = (uint32_t)(w->row_bytes / 2u);
    p.ldy = (uint32_t)(work->row_bytes / 2u);
    p.epilogue = bias != NULL ? bias_mode : GD_HIP_EPI_NONE;
    p.w_is_nk = 1u;
    p.prologue = GD_HIP_PRO_NONE;
    p.has_residual = 0u;
    p.ldr = 0u;
    p.eps = 0.0f;
    p.swiglu_cols = 0u;
    p.rope_heads = p.rope_head_dim = p.rope_tmax = 0u;
    p.rope_freq_scale = 0.0f;
    p.force_tiles = (uint16_t)backend->linear_tiles;
    p.force_waves = (uint16_t)backend->linear_waves;
    p.no_lds_stream = (uint32_t)backend->linear_no_lds_stream;
    head_rows = gd_hip_linear_tile_rope_head_rows(p.M, p.N, backend->compute_units);
    if (head_rows != 0u) {
        gd_hip_linear_params head = p;
        head.M = head_rows;
        e = gd_hip_launch_linear_tile_rope(backend->stream, gd_hip_matrix_ptr(x), gd_hip_matrix_ptr(w),
                                           bias != NULL ? gd_hip_vector_ptr(bias) : NULL, &head,
                                           (const float *)gd_hip_view_ptr(cos_rows), (const float *)gd_hip_view_ptr(sin_rows),
                                           (const int32_t *)gd_hip_view_ptr(cache_rows), gd_hip_view_ptr(q),
                                           gd_hip_view_ptr(k_cache), gd_hip_view_ptr(v_cache), (uint32_t)area,
                                           head_dim / 2u, backend->compute_units);
        if (e != 0) return gd_hip_finish_op(backend, e);
        backend->last_linear_family = GD_HIP_LINEAR_FAMILY_TILE;
    }
    if (head_rows < p.M) {
        gd_hip_linear_params tail = p;
        char *work_rows = (char *)gd_hip_matrix_ptr(work) + (size_t)head_rows * work->row_bytes;
        /* the projection of the tail rows in whole 128-row tiles: it starts up to 127 rows early (rows of `work`
         * nobody reads), so that no ragged row tile leaves the tile kernel's direct staging path */
        const uint32_t tail_rows = p.M - head_rows;
        const uint32_t up = (tail_rows + 127u) / 128u * 128u;
        const uint32_t first = tail_rows >= 128u && up <= p.M ? p.M - up : head_rows;
        tail.M = p.M - first;
        e = gd_hip_launch_linear(backend->stream, (const char *)gd_hip_matrix_ptr(x) + (size_t)first * x->row_bytes,
                                 gd_hip_matrix_ptr(w), bias != NULL ? gd_hip_vector_ptr(bias) : NULL, NULL, NULL,
                                 (char *)gd_hip_matrix_ptr(work) + (size_t)first * work->row_bytes, &tail, 1, 0, 1,
                                 2 * backend->compute_units, NULL, backend->linear_wide, &backend->last_linear_family);
        if (e != 0) return gd_hip_finish_op(backend, e);
        tail.M = tail_rows;
        e = gd_hip_launch_qkv_rope_rows(backend->stream, work_rows, (const float *)gd_hip_view_ptr(cos_rows),
                                        (const float *)gd_hip_view_ptr(sin_rows),
                                        (const int32_t *)gd_hip_view_ptr(cache_rows), gd_hip_view_ptr(q),
                                        gd_hip_view_ptr(k_cache), gd_hip_view_ptr(v_cache), head_rows, tail.M, n_heads,
                                        head_dim);
        if (e != 0) return gd_hip_finish_op(backend, e);
    }
    return gd_hip_finish_op(backend, 0);
}

/* Which kernel family the last projection call on this backend took: "stream", "wide", "tile" or "scalar". */
gd_status gd_backend_linear_last_kernel(gd_backend *backend, char *out, size_t capacity)
{
    static const char *const names[] = {NULL, "stream", "wide", "tile", "scalar"};
    if (backend == NULL || out == NULL || capacity == 0u) return GD_ERR_INVALID_ARGUMENT;
    if (backend->last_linear_family < 1 || backend->last_linear_family > 4) return GD_ERR_BAD_STATE;
    snprintf(out, capacity, "%s", names[backend->last_linear_family]);
    return GD_OK;
}
