/* Host dispatch of gd_backend_concat_to_full (reference src/core/backend.h:579-591). */
#include "../../../backends/hip/backend_hip_internal.h"

int gd_hip_launch_concat_to_full(hipStream_t stream, const void *src, void *dst, uint64_t count, uint64_t inner,
                                 uint64_t slice_axis, uint64_t full_axis, uint64_t axis_offset, uint32_t elem_size);

gd_status gd_backend_concat_to_full(gd_backend *backend, const gd_backend_tensor_view *src,
                                    const gd_backend_tensor_view *dst, const gd_backend_concat_args *args)
{
    uint64_t outer;
    if (backend == NULL || args == NULL || !gd_hip_view_ok(src) || !gd_hip_view_ok(dst)) return GD_ERR_INVALID_ARGUMENT;
    if (src->dtype != dst->dtype || gd_hip_dtype_size(src->dtype) == 0u) return GD_ERR_UNSUPPORTED;
    if (args->inner == 0u || args->slice_axis == 0u || args->full_axis == 0u || args->count != (uint64_t)src->count ||
        args->axis_offset > args->full_axis || args->slice_axis > args->full_axis - args->axis_offset ||
        args->count % (args->slice_axis * args->inner) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    outer = args->count / (args->slice_axis * args->inner);
    if (outer * args->full_axis * args->inner != (uint64_t)dst->count || args->count > 0x7fffffffull * 256u)
        return GD_ERR_INVALID_ARGUMENT;
    return gd_hip_finish_op(backend, gd_hip_launch_concat_to_full(
        backend->stream, gd_hip_view_ptr(src), gd_hip_view_ptr(dst), args->count, args->inner, args->slice_axis,
        args->full_axis, args->axis_offset, (uint32_t)gd_hip_dtype_size(src->dtype)));
}
