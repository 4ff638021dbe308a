/*
 * Device-side helpers shared by the operator kernels (gfx950, wave64).
 */
#ifndef GD_OPS_SHARED_HIP_DEVICE_H
#define GD_OPS_SHARED_HIP_DEVICE_H

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#define GD_WAVE 64

typedef _Float16 gd_half;
typedef _Float16 gd_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 gd_half4 __attribute__((ext_vector_type(4)));
typedef _Float16 gd_half2 __attribute__((ext_vector_type(2)));
typedef float gd_float4 __attribute__((ext_vector_type(4)));
typedef float gd_float16 __attribute__((ext_vector_type(16)));

/* 16-byte vector of raw bits for copies */
struct __attribute__((aligned(16))) gd_u128 { uint32_t x, y, z, w; };

__device__ __forceinline__ float gd_wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, GD_WAVE);
    return v;
}

__device__ __forceinline__ float gd_wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, GD_WAVE));
    return v;
}

/* Sum over a block of NW waves; every thread receives the total.  `smem` holds NW floats. */
template <int NW>
__device__ __forceinline__ float gd_block_sum(float v, float *smem)
{
    v = gd_wave_sum(v);
    if (NW == 1) return v;
    const int lane = threadIdx.x & (GD_WAVE - 1), wave = threadIdx.x / GD_WAVE;
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += smem[w];
    return t;
}

/* IEEE round-to-nearest-even float -> half (v_cvt_f16_f32) */
__device__ __forceinline__ gd_half gd_f2h(float v) { return (gd_half)v; }
__device__ __forceinline__ float gd_h2f(gd_half v) { return (float)v; }

#endif
