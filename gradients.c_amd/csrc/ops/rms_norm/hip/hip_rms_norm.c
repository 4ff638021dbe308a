/* Host dispatch of gd_backend_rms_norm_forward (reference src/core/backend.h:540-544). */
#include "../../../backends/hip/backend_hip_internal.h"

int gd_hip_launch_rms_norm(hipStream_t stream, const void *x, const void *w, void *y, uint64_t rows,
                           uint64_t cols, float eps, int is_f16, int aligned16);

gd_status gd_backend_rms_norm_forward(gd_backend *backend, const gd_backend_tensor_view *x,
                                      const gd_backend_tensor_view *weight, const gd_backend_tensor_view *out,
                                      const gd_backend_rms_norm_args *args)
{
    if (backend == NULL || args == NULL || !gd_hip_view_ok(x) || !gd_hip_view_ok(weight) || !gd_hip_view_ok(out))
        return GD_ERR_INVALID_ARGUMENT;
    if (x->dtype != GD_BACKEND_DTYPE_F16 && x->dtype != GD_BACKEND_DTYPE_F32) return GD_ERR_UNSUPPORTED;
    if (weight->dtype != x->dtype || out->dtype != x->dtype) return GD_ERR_UNSUPPORTED;
    if (args->rows == 0u || args->cols == 0u || !(args->eps > 0.0f) || args->rows > 0x7fffffffu ||
        args->rows > SIZE_MAX / args->cols || x->count != (size_t)(args->rows * args->cols) ||
        out->count != x->count || weight->count != (size_t)args->cols)
        return GD_ERR_INVALID_ARGUMENT;
    return gd_hip_finish_op(backend, gd_hip_launch_rms_norm(
        backend->stream, gd_hip_view_ptr(x), gd_hip_view_ptr(weight), gd_hip_view_ptr(out), args->rows,
        args->cols, args->eps, x->dtype == GD_BACKEND_DTYPE_F16,
        ((x->offset | weight->offset | out->offset) & 15u) == 0u));
}
