/*
 * F16 add for gfx950: out = half(x + y) with NumPy-style broadcasting.  HBM-bound.
 * Same-shape operands (residual adds) and a trailing-suffix operand (bias rows) take a
 * vector path with 16-byte loads; anything else walks the broadcast strides.
 * Arithmetic follows the reference kernel src/ops/add/metal_add.metal:37-59 (half + half:
 * the exact sum rounded once).
 */
#include "../../_shared/hip_device.h"

struct gd_add_bcast {
    uint32_t rank;
    int64_t shape[8];
    int64_t xs[8], ys[8]; /* element strides, 0 on broadcast dims */
};

__global__ void __launch_bounds__(256)
gd_add_vec_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ y, gd_half *__restrict__ out,
                  uint64_t nvec, uint64_t y_vecs)
{
    /* x has nvec vectors of 8 halfs; y repeats every y_vecs vectors (y_vecs == nvec: same shape) */
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec) return;
    const gd_half8 a = reinterpret_cast<const gd_half8 *>(x)[i];
    const gd_half8 b = reinterpret_cast<const gd_half8 *>(y)[y_vecs == nvec ? i : i % y_vecs];
    reinterpret_cast<gd_half8 *>(out)[i] = a + b; /* native F16 adds: exact sum, one rounding */
}

__global__ void __launch_bounds__(256)
gd_add_bcast_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ y, gd_half *__restrict__ out,
                    uint64_t count, gd_add_bcast bc)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    uint64_t rem = i;
    int64_t xi = 0, yi = 0;
    for (int d = (int)bc.rank - 1; d >= 0; --d) {
        const int64_t idx = (int64_t)(rem % (uint64_t)bc.shape[d]);
        rem /= (uint64_t)bc.shape[d];
        xi += idx * bc.xs[d];
        yi += idx * bc.ys[d];
    }
    out[i] = x[xi] + y[yi];
}

extern "C" int gd_hip_launch_add_vec(hipStream_t stream, const void *x, const void *y, void *out, uint64_t count,
                                     uint64_t y_count)
{
    const uint64_t nvec = count / 8u;
    if (nvec == 0) return (int)hipSuccess;
    gd_add_vec_kernel<<<(unsigned)((nvec + 255) / 256), 256, 0, stream>>>(
        (const gd_half *)x, (const gd_half *)y, (gd_half *)out, nvec, y_count / 8u);
    return (int)hipGetLastError();
}

extern "C" int gd_hip_launch_add_bcast(hipStream_t stream, const void *x, const void *y, void *out, uint64_t count,
                                       uint32_t rank, const int64_t *shape, const int64_t *xs, const int64_t *ys)
{
    gd_add_bcast bc;
    if (count == 0) return (int)hipSuccess;
    bc.rank = rank;
    for (uint32_t d = 0; d < 8; ++d) {
        bc.shape[d] = d < rank ? shape[d] : 1;
        bc.xs[d] = d < rank ? xs[d] : 0;
        bc.ys[d] = d < rank ? ys[d] : 0;
    }
    gd_add_bcast_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(
        (const gd_half *)x, (const gd_half *)y, (gd_half *)out, count, bc);
    return (int)hipGetLastError();
}
