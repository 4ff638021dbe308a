/*
 * Host dispatch of gd_backend_add (reference src/core/backend_generated.h:14-17; broadcast
 * rule src/ops/_shared/binary/binary_core.h:67-131: right-aligned, a dim broadcasts when it is 1
 * or missing, out has the broadcast shape).
 */
#include "../../../backends/hip/backend_hip_internal.h"

int gd_hip_launch_add_vec(hipStream_t stream, const void *x, const void *y, void *out, uint64_t count,
                          uint64_t y_count);
int gd_hip_launch_add_bcast(hipStream_t stream, const void *x, const void *y, void *out, uint64_t count,
                            uint32_t rank, const int64_t *shape, const int64_t *xs, const int64_t *ys);

/* y's shape equals the trailing dims of x (after dropping y's leading 1s) */
static bool is_suffix_of(const gd_backend_tensor_view *y, const gd_backend_tensor_view *x)
{
    uint32_t lead = 0u, i, n;
    while (lead < y->rank && y->shape[lead] == 1) ++lead;
    n = y->rank - lead;
    if (n > x->rank) return false;
    for (i = 0u; i < n; ++i) {
        if (y->shape[lead + i] != x->shape[x->rank - n + i]) return false;
    }
    return true;
}

gd_status gd_backend_add(gd_backend *backend, const gd_backend_tensor_view *x, const gd_backend_tensor_view *y,
                         const gd_backend_tensor_view *out)
{
    int64_t xs[8], ys[8];
    uint32_t d;
    if (backend == NULL || !gd_hip_view_ok(x) || !gd_hip_view_ok(y) || !gd_hip_view_ok(out))
        return GD_ERR_INVALID_ARGUMENT;
    if (x->dtype != GD_BACKEND_DTYPE_F16 || y->dtype != GD_BACKEND_DTYPE_F16 || out->dtype != GD_BACKEND_DTYPE_F16)
        return GD_ERR_UNSUPPORTED;
    if (out->rank < x->rank || out->rank < y->rank) return GD_ERR_INVALID_ARGUMENT;
    for (d = 0u; d < out->rank; ++d) {
        const int64_t od = out->shape[out->rank - 1u - d];
        const int64_t xd = d < x->rank ? x->shape[x->rank - 1u - d] : 1;
        const int64_t yd = d < y->rank ? y->shape[y->rank - 1u - d] : 1;
        if ((xd != od && xd != 1) || (yd != od && yd != 1) || (xd == 1 && yd == 1 && od != 1))
            return GD_ERR_INVALID_ARGUMENT;
        xs[out->rank - 1u - d] = (d < x->rank && xd != 1) ? x->strides[x->rank - 1u - d] : 0;
        ys[out->rank - 1u - d] = (d < y->rank && yd != 1) ? y->strides[y->rank - 1u - d] : 0;
    }
    if (((x->offset | y->offset | out->offset) & 15u) == 0u && (out->count % 8u) == 0u) {
        if (x->count == out->count && y->count == out->count)
            return gd_hip_finish_op(backend, gd_hip_launch_add_vec(backend->stream, gd_hip_view_ptr(x),
                                                                   gd_hip_view_ptr(y), gd_hip_view_ptr(out),
                                                                   out->count, out->count));
        if (x->count == out->count && (y->count % 8u) == 0u && is_suffix_of(y, x))
            return gd_hip_finish_op(backend, gd_hip_launch_add_vec(backend->stream, gd_hip_view_ptr(x),
                                                                   gd_hip_view_ptr(y), gd_hip_view_ptr(out),
                                                                   out->count, y->count));
        if (y->count == out->count && (x->count % 8u) == 0u && is_suffix_of(x, y))
            return gd_hip_finish_op(backend, gd_hip_launch_add_vec(backend->stream, gd_hip_view_ptr(y),
                                                                   gd_hip_view_ptr(x), gd_hip_view_ptr(out),
                                                                   out->count, x->count));
    }
    if (out->count > 0x7fffffffull * 256u) return GD_ERR_UNSUPPORTED;
    return gd_hip_finish_op(backend, gd_hip_launch_add_bcast(backend->stream, gd_hip_view_ptr(x), gd_hip_view_ptr(y),
                                                             gd_hip_view_ptr(out), out->count, out->rank,
                                                             out->shape, xs, ys));
}
