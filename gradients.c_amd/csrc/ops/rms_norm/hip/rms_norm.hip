/*
 * rms_norm forward for gfx950: y = x * w * rsqrt(mean(x^2) + eps), one workgroup per row.
 * HBM-bound (reads x and w once, writes y once).  The row is read with 16-byte loads into
 * registers when it fits (cols <= 8 * 256 * 4 halfs), so x is fetched from memory once.
 * Arithmetic follows the reference kernel src/ops/rms_norm/metal_rms_norm.metal:29-67:
 * F32 sum of squares, inv = rsqrt(ss / cols + eps), one rounding of x * w * inv.
 */
#include "../../_shared/hip_device.h"

#define GD_RMS_THREADS 256

__global__ void __launch_bounds__(GD_RMS_THREADS)
gd_rms_norm_f16_vec_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w, gd_half *__restrict__ y,
                           uint64_t rows, uint32_t cols, float eps)
{
    /* cols % 8 == 0 and cols <= 8 * 256 * 4 */
    __shared__ float red[GD_RMS_THREADS / 64];
    const uint64_t row = blockIdx.x;
    if (row >= rows) return;
    const gd_half *xr = x + row * cols;
    gd_half *yr = y + row * cols;
    const uint32_t nvec = cols / 8u;
    gd_half8 xv[4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t v = threadIdx.x + i * GD_RMS_THREADS;
        if (v < nvec) {
            xv[i] = *reinterpret_cast<const gd_half8 *>(xr + v * 8u);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float f = (float)xv[i][e];
                ss = fmaf(f, f, ss);
            }
        }
    }
    ss = gd_block_sum<GD_RMS_THREADS / 64>(ss, red);
    const float inv = rsqrtf(ss / (float)cols + eps);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t v = threadIdx.x + i * GD_RMS_THREADS;
        if (v < nvec) {
            const gd_half8 wv = *reinterpret_cast<const gd_half8 *>(w + v * 8u);
            gd_half8 o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (gd_half)((float)xv[i][e] * (float)wv[e] * inv);
            *reinterpret_cast<gd_half8 *>(yr + v * 8u) = o;
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(GD_RMS_THREADS)
gd_rms_norm_scalar_kernel(const T *__restrict__ x, const T *__restrict__ w, T *__restrict__ y, uint64_t rows,
                          uint64_t cols, float eps)
{
    __shared__ float red[GD_RMS_THREADS / 64];
    const uint64_t row = blockIdx.x;
    if (row >= rows) return;
    const T *xr = x + row * cols;
    T *yr = y + row * cols;
    float ss = 0.f;
    for (uint64_t c = threadIdx.x; c < cols; c += GD_RMS_THREADS) {
        const float f = (float)xr[c];
        ss = fmaf(f, f, ss);
    }
    ss = gd_block_sum<GD_RMS_THREADS / 64>(ss, red);
    const float inv = rsqrtf(ss / (float)cols + eps);
    for (uint64_t c = threadIdx.x; c < cols; c += GD_RMS_THREADS) yr[c] = (T)((float)xr[c] * (float)w[c] * inv);
}

extern "C" int gd_hip_launch_rms_norm(hipStream_t stream, const void *x, const void *w, void *y, uint64_t rows,
                                      uint64_t cols, float eps, int is_f16, int aligned16)
{
    if (rows == 0 || cols == 0) return (int)hipSuccess;
    if (is_f16 && aligned16 && (cols % 8u) == 0u && cols <= 8u * GD_RMS_THREADS * 4u)
        gd_rms_norm_f16_vec_kernel<<<(unsigned)rows, GD_RMS_THREADS, 0, stream>>>(
            (const gd_half *)x, (const gd_half *)w, (gd_half *)y, rows, (uint32_t)cols, eps);
    else if (is_f16)
        gd_rms_norm_scalar_kernel<gd_half><<<(unsigned)rows, GD_RMS_THREADS, 0, stream>>>(
            (const gd_half *)x, (const gd_half *)w, (gd_half *)y, rows, cols, eps);
    else
        gd_rms_norm_scalar_kernel<float><<<(unsigned)rows, GD_RMS_THREADS, 0, stream>>>(
            (const float *)x, (const float *)w, (float *)y, rows, cols, eps);
    return (int)hipGetLastError();
}
