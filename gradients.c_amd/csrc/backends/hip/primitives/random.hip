/*
 * Backend primitive: counter-based uniform fill.  Replaces the reference's gd_backend_rand_uniform
 * (src/core/backend.h:178-185; kernel src/backends/metal/primitives/random/metal_random.metal:8-30):
 * element i takes the top 24 bits below bit 64 of splitmix64(seed + i) as u in [0,1) and stores
 * low + (high - low) * u (a fused multiply-add), rounded once more to the element type.  One 64-bit hash per element, one store.
 */
#include "../../../ops/_shared/hip_device.h"

__device__ __forceinline__ uint64_t gd_splitmix64(uint64_t x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

__device__ __forceinline__ float gd_uniform_value(uint64_t seed, uint64_t i, float low, float span)
{
    const uint32_t mant = (uint32_t)((gd_splitmix64(seed + i) >> 40) & 0xffffffu);
    const float u = __fmul_rn((float)mant, 1.0f / 16777216.0f); /* exact: mant < 2^24 */
    return __fmaf_rn(span, u, low); /* one rounding: what a contracting shader compiler emits for low + span*u */
}

template <int DT>
__global__ void __launch_bounds__(256)
gd_rand_uniform_kernel(void *__restrict__ dst, uint64_t count, uint64_t seed, float low, float span)
{
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
        const float v = gd_uniform_value(seed, i, low, span);
        if (DT == 1) ((gd_half *)dst)[i] = (gd_half)v;
        else if (DT == 2) { /* bf16, round to nearest even */
            uint32_t b = __float_as_uint(v);
            b += 0x7fffu + ((b >> 16) & 1u);
            ((uint16_t *)dst)[i] = (uint16_t)(b >> 16);
        } else ((float *)dst)[i] = v;
    }
}

extern "C" int gd_hip_launch_rand_uniform(hipStream_t stream, void *dst, uint64_t count, uint32_t dtype,
                                          uint64_t seed, float low, float high)
{
    uint64_t blocks = (count + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    const float span = high - low;
    if (dtype == 1u) gd_rand_uniform_kernel<1><<<(unsigned)blocks, 256, 0, stream>>>(dst, count, seed, low, span);
    else if (dtype == 2u) gd_rand_uniform_kernel<2><<<(unsigned)blocks, 256, 0, stream>>>(dst, count, seed, low, span);
    else gd_rand_uniform_kernel<3><<<(unsigned)blocks, 256, 0, stream>>>(dst, count, seed, low, span);
    return (int)hipGetLastError();
}
