/* Host dispatch of gd_backend_argmax_rows (no counterpart in the reference's backend). */
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
