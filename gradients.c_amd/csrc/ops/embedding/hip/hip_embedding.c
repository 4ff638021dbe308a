/*
 * Host dispatch of gd_backend_embedding_forward (reference src/core/backend.h:301-312),
 * gd_backend_gather_rows and gd_backend_add_scalar_i32.
 */
#include "../../../backends/hip/backend_hip_internal.h"

int gd_hip_launch_gather_rows(hipStream_t stream, const void *table, const int32_t *ids, void *out,
                              uint64_t n_ids, uint64_t vocab, uint64_t row_bytes, uint32_t elem_size,
                              int aligned16, int nan_on_invalid);
int gd_hip_launch_add_scalar_i32(hipStream_t stream, const int32_t *src, int32_t *dst, uint64_t n, int32_t delta);
int gd_hip_launch_decode_advance(hipStream_t stream, const int32_t *next_ids, const float *gaps, int32_t *ids,
                                 int32_t *positions, int32_t *step_counter, int32_t *out_ids, float *out_gaps,
                                 uint32_t batch, uint32_t max_steps, int32_t pos_delta);

static gd_status gather(gd_backend *backend, const gd_backend_tensor_view *table, const gd_backend_tensor_view *ids,
                        const gd_backend_tensor_view *out, uint64_t n_ids, uint64_t vocab, uint64_t dim, int nan)
{
    size_t es;
    if (table->dtype != GD_BACKEND_DTYPE_F16 && table->dtype != GD_BACKEND_DTYPE_F32) return GD_ERR_UNSUPPORTED;
    if (out->dtype != table->dtype || ids->dtype != GD_BACKEND_DTYPE_I32) return GD_ERR_UNSUPPORTED;
    if (n_ids == 0u || vocab == 0u || dim == 0u || vocab > SIZE_MAX / dim || n_ids > SIZE_MAX / dim ||
        table->count != (size_t)(vocab * dim) || ids->count != (size_t)n_ids || out->count != (size_t)(n_ids * dim) ||
        (ids->offset & 3u) != 0u || vocab > 0x7fffffffu || n_ids * dim > 0x7fffffffull * 256u)
        return GD_ERR_INVALID_ARGUMENT;
    es = gd_hip_dtype_size(table->dtype);
    return gd_hip_finish_op(backend, gd_hip_launch_gather_rows(
        backend->stream, gd_hip_view_ptr(table), (const int32_t *)gd_hip_view_ptr(ids), gd_hip_view_ptr(out),
        n_ids, vocab, dim * es, (uint32_t)es, ((table->offset | out->offset) & 15u) == 0u, nan));
}

gd_status gd_backend_embedding_forward(gd_backend *backend, const gd_backend_tensor_view *table,
                                       const gd_backend_tensor_view *ids, const gd_backend_tensor_view *out,
                                       const gd_backend_embedding_args *args)
{
    if (backend == NULL || args == NULL || !gd_hip_view_ok(table) || !gd_hip_view_ok(ids) || !gd_hip_view_ok(out))
        return GD_ERR_INVALID_ARGUMENT;
    return gather(backend, table, ids, out, args->ids_count, args->vocab, args->dim, 1);
}

gd_status gd_backend_gather_rows(gd_backend *backend, const gd_backend_tensor_view *src,
                                 const gd_backend_tensor_view *rows, const gd_backend_tensor_view *out)
{
    if (backend == NULL || !gd_hip_view_ok(src) || !gd_hip_view_ok(rows) || !gd_hip_view_ok(out) ||
        src->rank != 2u || out->rank != 2u || rows->rank != 1u || out->shape[0] != rows->shape[0] ||
        out->shape[1] != src->shape[1])
        return GD_ERR_INVALID_ARGUMENT;
    return gather(backend, src, rows, out, (uint64_t)rows->shape[0], (uint64_t)src->shape[0],
                  (uint64_t)src->shape[1], 0);
}

gd_status gd_backend_add_scalar_i32(gd_backend *backend, const gd_backend_tensor_view *src,
                                    const gd_backend_tensor_view *dst, int32_t delta)
{
    if (backend == NULL || !gd_hip_view_ok(src) || !gd_hip_view_ok(dst) || src->dtype != GD_BACKEND_DTYPE_I32 ||
        dst->dtype != GD_BACKEND_DTYPE_I32 || src->count != dst->count || ((src->offset | dst->offset) & 3u) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    return gd_hip_finish_op(backend, gd_hip_launch_add_scalar_i32(
        backend->stream, (const int32_t *)gd_hip_view_ptr(src), (int32_t *)gd_hip_view_ptr(dst), src->count, delta));
}

static bool i32_ok(const gd_backend_tensor_view *v)
{
    return gd_hip_view_ok(v) && v->dtype == GD_BACKEND_DTYPE_I32 && (v->offset & 3u) == 0u;
}

gd_status gd_backend_decode_advance(gd_backend *backend, const gd_backend_tensor_view *next_ids,
                                    const gd_backend_tensor_view *gaps, const gd_backend_tensor_view *ids,
                                    const gd_backend_tensor_view *positions, const gd_backend_tensor_view *step_counter,
                                    const gd_backend_tensor_view *out_ids, const gd_backend_tensor_view *out_gaps,
                                    int32_t pos_delta)
{
    size_t batch;
    if (backend == NULL || !i32_ok(next_ids) || !i32_ok(ids) || !i32_ok(positions) || !i32_ok(step_counter) ||
        !i32_ok(out_ids) || (gaps == NULL) != (out_gaps == NULL))
        return GD_ERR_INVALID_ARGUMENT;
    batch = next_ids->count;
    if (batch == 0u || batch > 0x7fffffffu || ids->count != batch || positions->count != batch ||
        step_counter->count != 1u || out_ids->count < batch || (out_ids->count % batch) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    if (gaps != NULL && (!gd_hip_view_ok(gaps) || !gd_hip_view_ok(out_gaps) || gaps->dtype != GD_BACKEND_DTYPE_F32 ||
                         out_gaps->dtype != GD_BACKEND_DTYPE_F32 || gaps->count != batch ||
                         out_gaps->count != out_ids->count || ((gaps->offset | out_gaps->offset) & 3u) != 0u))
        return GD_ERR_INVALID_ARGUMENT;
    return gd_hip_finish_op(backend, gd_hip_launch_decode_advance(
        backend->stream, (const int32_t *)gd_hip_view_ptr(next_ids), gaps != NULL ? (const float *)gd_hip_view_ptr(gaps) : NULL,
        (int32_t *)gd_hip_view_ptr(ids), (int32_t *)gd_hip_view_ptr(positions), (int32_t *)gd_hip_view_ptr(step_counter),
        (int32_t *)gd_hip_view_ptr(out_ids), out_gaps != NULL ? (float *)gd_hip_view_ptr(out_gaps) : NULL,
        (uint32_t)batch, (uint32_t)(out_ids->count / batch), pos_delta));
}
