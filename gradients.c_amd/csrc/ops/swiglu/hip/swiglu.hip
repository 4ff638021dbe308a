/*
 * swiglu_split forward for gfx950: out[r,c] = half(x12[r,c] * silu(x12[r,H+c])).  HBM-bound
 * elementwise work (3*H halfs of traffic per row).  Arithmetic follows the reference kernel
 * src/ops/swiglu/metal_swiglu.metal:6-24,94-118: sigmoid through exp(-|z|), gate = z * sigmoid(z),
 * one rounding of x1 * gate.
 */
#include "../../_shared/hip_device.h"

__device__ __forceinline__ float gd_silu(float z)
{
    const float e = __expf(-fabsf(z));
    const float inv = 1.0f / (1.0f + e);
    return z * (z >= 0.0f ? inv : e * inv);
}

__global__ void __launch_bounds__(256)
gd_swiglu_split_vec_kernel(const gd_half *__restrict__ x12, gd_half *__restrict__ out, uint64_t rows, uint64_t hvec)
{
    /* hvec = H / 8 */
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= rows * hvec) return;
    const uint64_t r = gid / hvec, cv = gid - r * hvec;
    const gd_half8 a = reinterpret_cast<const gd_half8 *>(x12 + r * hvec * 16u)[cv];
    const gd_half8 z = reinterpret_cast<const gd_half8 *>(x12 + r * hvec * 16u + hvec * 8u)[cv];
    gd_half8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (gd_half)((float)a[e] * gd_silu((float)z[e]));
    reinterpret_cast<gd_half8 *>(out + r * hvec * 8u)[cv] = o;
}

__global__ void __launch_bounds__(256)
gd_swiglu_split_scalar_kernel(const gd_half *__restrict__ x12, gd_half *__restrict__ out, uint64_t rows, uint64_t H)
{
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= rows * H) return;
    const uint64_t r = gid / H, c = gid - r * H;
    out[gid] = (gd_half)((float)x12[r * 2u * H + c] * gd_silu((float)x12[r * 2u * H + H + c]));
}

extern "C" int gd_hip_launch_swiglu_split(hipStream_t stream, const void *x12, void *out, uint64_t rows, uint64_t H,
                                          int aligned16)
{
    if (rows == 0 || H == 0) return (int)hipSuccess;
    if (aligned16 && (H % 8u) == 0u) {
        const uint64_t total = rows * (H / 8u);
        gd_swiglu_split_vec_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
            (const gd_half *)x12, (gd_half *)out, rows, H / 8u);
    } else {
        const uint64_t total = rows * H;
        gd_swiglu_split_scalar_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
            (const gd_half *)x12, (gd_half *)out, rows, H);
    }
    return (int)hipGetLastError();
}
