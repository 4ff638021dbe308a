/* Host dispatch of gd_backend_argmax_rows and gd_backend_argmax_advance (no counterpart in the reference's backend). */
#include "../../../backends/hip/backend_hip_internal.h"

int gd_hip_launch_argmax_rows(hipStream_t stream, const void *logits, int32_t *ids, float *gap, uint64_t rows,
                              uint64_t cols, int is_f16);

gd_status gd_backend_argmax_rows(gd_backend *backend, const gd_backend_tensor_view *logits,
                                 const gd_backend_tensor_view *ids, const gd_backend_tensor_view *gap)
{
    uint64_t rows, cols;
    if (backend == NULL || !gd_hip_view_ok(logits) || !gd_hip_view_ok(ids) || logits->rank != 2u ||
        (gap != NULL && !gd_hip_view_ok(gap)))
        return GD_ERR_INVALID_ARGUMENT;
    if ((logits->dtype != GD_BACKEND_DTYPE_F16 && logits->dtype != GD_BACKEND_DTYPE_F32) ||
        ids->dtype != GD_BACKEND_DTYPE_I32 || (gap != NULL && gap->dtype != GD_BACKEND_DTYPE_F32))
        return GD_ERR_UNSUPPORTED;
    rows = (uint64_t)logits->shape[0];
    cols = (uint64_t)logits->shape[1];
    if (ids->count != (size_t)rows || (gap != NULL && gap->count != (size_t)rows) || rows > 0x7fffffffu ||
        cols > 0x7fffffffu || (ids->offset & 3u) != 0u || (gap != NULL && (gap->offset & 3u) != 0u))
        return GD_ERR_INVALID_ARGUMENT;
    return gd_hip_finish_op(backend, gd_hip_launch_argmax_rows(
        backend->stream, gd_hip_view_ptr(logits), (int32_t *)gd_hip_view_ptr(ids),
        gap != NULL ? (float *)gd_hip_view_ptr(gap) : NULL, rows, cols, logits->dtype == GD_BACKEND_DTYPE_F16));
}

int gd_hip_launch_argmax_advance(hipStream_t stream, const void *logits, int32_t *ids, uint64_t rows, uint64_t cols,
                                 int is_f16, int32_t *positions, int32_t *step_counters, int32_t *out_ids,
                                 float *out_gaps, uint32_t max_steps, int32_t pos_delta, const void *table, void *next_x,
                                 uint32_t row_bytes);

static int i32_rows(const gd_backend_tensor_view *v, uint64_t rows)
{
    return gd_hip_view_ok(v) && v->dtype == GD_BACKEND_DTYPE_I32 && v->count == (size_t)rows && (v->offset & 3u) == 0u;
}

gd_status gd_backend_argmax_advance(gd_backend *backend, const gd_backend_tensor_view *logits,
                                    const gd_backend_tensor_view *ids, const gd_backend_tensor_view *positions,
                                    const gd_backend_tensor_view *step_counters,
                                    const gd_backend_tensor_view *out_ids, const gd_backend_tensor_view *out_gaps,
                                    int32_t pos_delta, const gd_backend_tensor_view *table,
                                    const gd_backend_tensor_view *next_x)
{
    uint64_t rows, cols, max_steps, row_bytes = 0u;
    if (backend == NULL || !gd_hip_view_ok(logits) || logits->rank != 2u || !gd_hip_view_ok(out_ids) ||
        (out_gaps != NULL && !gd_hip_view_ok(out_gaps)))
        return GD_ERR_INVALID_ARGUMENT;
    if ((logits->dtype != GD_BACKEND_DTYPE_F16 && logits->dtype != GD_BACKEND_DTYPE_F32) ||
        out_ids->dtype != GD_BACKEND_DTYPE_I32 || (out_gaps != NULL && out_gaps->dtype != GD_BACKEND_DTYPE_F32))
        return GD_ERR_UNSUPPORTED;
    rows = (uint64_t)logits->shape[0];
    cols = (uint64_t)logits->shape[1];
    if (rows == 0u || rows > 0x7fffffffu || cols > 0x7fffffffu || !i32_rows(ids, rows) || !i32_rows(positions, rows) ||
        !i32_rows(step_counters, rows) || (out_ids->count % rows) != 0u || (out_ids->offset & 3u) != 0u ||
        (out_gaps != NULL && (out_gaps->count != out_ids->count || (out_gaps->offset & 3u) != 0u)))
        return GD_ERR_INVALID_ARGUMENT;
    max_steps = out_ids->count / rows;
    if (max_steps > 0xffffffffu || (table == NULL) != (next_x == NULL)) return GD_ERR_INVALID_ARGUMENT;
    if (table != NULL) {
        if (!gd_hip_view_ok(table) || !gd_hip_view_ok(next_x) || table->rank != 2u || next_x->rank != 2u ||
            (uint64_t)table->shape[0] != cols || (uint64_t)next_x->shape[0] != rows || next_x->shape[1] != table->shape[1])
            return GD_ERR_INVALID_ARGUMENT;
        if (table->dtype != next_x->dtype || gd_hip_dtype_size(table->dtype) == 0u) return GD_ERR_UNSUPPORTED;
        row_bytes = (uint64_t)table->shape[1] * gd_hip_dtype_size(table->dtype);
        if ((row_bytes & 15u) != 0u || row_bytes > 0xffffffffu || ((table->offset | next_x->offset) & 15u) != 0u)
            return GD_ERR_UNSUPPORTED;
    }
    return gd_hip_finish_op(backend, gd_hip_launch_argmax_advance(
        backend->stream, gd_hip_view_ptr(logits), (int32_t *)gd_hip_view_ptr(ids), rows, cols,
        logits->dtype == GD_BACKEND_DTYPE_F16, (int32_t *)gd_hip_view_ptr(positions),
        (int32_t *)gd_hip_view_ptr(step_counters), (int32_t *)gd_hip_view_ptr(out_ids),
        out_gaps != NULL ? (float *)gd_hip_view_ptr(out_gaps) : NULL, (uint32_t)max_steps, pos_delta,
        table != NULL ? gd_hip_view_ptr(table) : NULL, next_x != NULL ? gd_hip_view_ptr(next_x) : NULL, (uint32_t)row_bytes));
}
