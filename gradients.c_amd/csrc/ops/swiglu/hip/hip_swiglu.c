/* Host dispatch of gd_backend_swiglu_split_forward (reference src/core/backend.h:520-522). */
#include "../../../backends/hip/backend_hip_internal.h"

int gd_hip_launch_swiglu_split(hipStream_t stream, const void *x12, void *out, uint64_t rows, uint64_t H,
                               int aligned16);

gd_status gd_backend_swiglu_split_forward(gd_backend *backend, const gd_backend_tensor_view *x12,
                                          const gd_backend_tensor_view *out)
{
    uint64_t width, H, rows;
    uint32_t d;
    if (backend == NULL || !gd_hip_view_ok(x12) || !gd_hip_view_ok(out) || x12->rank == 0u || out->rank != x12->rank)
        return GD_ERR_INVALID_ARGUMENT;
    if (x12->dtype != GD_BACKEND_DTYPE_F16 || out->dtype != GD_BACKEND_DTYPE_F16) return GD_ERR_UNSUPPORTED;
    width = (uint64_t)x12->shape[x12->rank - 1u];
    if ((width & 1u) != 0u) return GD_ERR_INVALID_ARGUMENT;
    H = width / 2u;
    for (d = 0u; d + 1u < x12->rank; ++d) {
        if (out->shape[d] != x12->shape[d]) return GD_ERR_INVALID_ARGUMENT;
    }
    if ((uint64_t)out->shape[out->rank - 1u] != H) return GD_ERR_INVALID_ARGUMENT;
    rows = x12->count / width;
    if (out->count > 0x7fffffffull * 256u) return GD_ERR_UNSUPPORTED;
    return gd_hip_finish_op(backend, gd_hip_launch_swiglu_split(backend->stream, gd_hip_view_ptr(x12),
                                                                gd_hip_view_ptr(out), rows, H,
                                                                ((x12->offset | out->offset) & 15u) == 0u));
}
