/*
 * Host dispatch of the projection entry points: gd_backend_matmul, gd_backend_matmul_nt,
 * gd_backend_linear (reference src/core/backend.h:187-195, 215-219) and the fused
 * gd_backend_linear_nt / gd_backend_swiglu_split_linear.
 */
#include "../../../backends/hip/backend_hip_internal.h"
#include "hip_linear_types.h"

int gd_hip_launch_linear(hipStream_t stream, const void *x, const void *w, const void *bias, const void *residual,
                         void *y, const gd_hip_linear_params *params, int vector_ok);

static gd_status project(gd_backend *backend, const gd_backend_matrix_view *x, const gd_backend_matrix_view *w,
                         const gd_backend_vector_view *bias, const gd_backend_matrix_view *y, uint32_t w_is_nk,
                         uint32_t epilogue, uint32_t swiglu)
{
    gd_hip_linear_params p;
    uint32_t K;
    int vec;
    if (backend == NULL || !gd_hip_matrix_ok(x) || !gd_hip_matrix_ok(w) || !gd_hip_matrix_ok(y) ||
        (bias != NULL && !gd_hip_vector_ok(bias)))
        return GD_ERR_INVALID_ARGUMENT;
    if (x->dtype != GD_BACKEND_DTYPE_F16 || w->dtype != GD_BACKEND_DTYPE_F16 || y->dtype != GD_BACKEND_DTYPE_F16 ||
        (bias != NULL && bias->dtype != GD_BACKEND_DTYPE_F16))
        return GD_ERR_UNSUPPORTED;
    if (swiglu) {
        if ((x->cols & 1u) != 0u) return GD_ERR_INVALID_ARGUMENT;
        K = x->cols / 2u;
    } else {
        K = x->cols;
    }
    if (w_is_nk ? (w->cols != K || w->rows != y->cols) : (w->rows != K || w->cols != y->cols))
        return GD_ERR_INVALID_ARGUMENT;
    if (x->rows != y->rows || (bias != NULL && bias->length != y->cols)) return GD_ERR_INVALID_ARGUMENT;
    if ((uint64_t)y->rows * y->cols > 0x7fffffffull * 256u || (y->cols + 15u) / 16u > 0x7fffffffu ||
        (y->rows + 15u) / 16u > 65535u * 4u)
        return GD_ERR_UNSUPPORTED;
    p.M = y->rows;
    p.N = y->cols;
    p.K = K;
    p.ldx = (uint32_t)(x->row_bytes / 2u);
    p.ldw = (uint32_t)(w->row_bytes / 2u);
    p.ldy = (uint32_t)(y->row_bytes / 2u);
    p.epilogue = bias != NULL ? epilogue : GD_HIP_EPI_NONE;
    p.w_is_nk = w_is_nk;
    p.swiglu = swiglu;
    p.has_residual = 0u;
    p.ldr = 0u;
    /* 16-byte fragment loads: x rows always, w rows when K-contiguous */
    vec = (K % 8u) == 0u && ((x->offset | x->row_bytes) & 15u) == 0u &&
          (!w_is_nk || ((w->offset | w->row_bytes) & 15u) == 0u);
    return gd_hip_finish_op(backend, gd_hip_launch_linear(
        backend->stream, gd_hip_matrix_ptr(x), gd_hip_matrix_ptr(w), bias != NULL ? gd_hip_vector_ptr(bias) : NULL,
        NULL, gd_hip_matrix_ptr(y), &p, vec));
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
