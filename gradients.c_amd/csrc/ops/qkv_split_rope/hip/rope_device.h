/*
 * RoPE arithmetic shared by the kernels that rotate q and k (qkv_split_rope.hip and the projection epilogue in
 * ops/linear/hip/linear.hip).  Explicitly rounded steps so that every kernel produces the same bits for the same
 * input.  Follows src/ops/qkv_split_rope/metal_qkv_split_rope.metal:6-36: angle = float(pos) * exp2(pair * freq_scale),
 * freq_scale = -2*log2(theta)/n_dims, rotation in F32, one rounding to F16 per output.
 */
#ifndef GD_ROPE_DEVICE_H
#define GD_ROPE_DEVICE_H
#include "../../_shared/hip_device.h"

__device__ __forceinline__ void gd_rope_cos_sin(float fpos, uint32_t pair, float freq_scale, float *c, float *s)
{
    sincosf(__fmul_rn(fpos, exp2f(__fmul_rn((float)pair, freq_scale))), s, c);
}

__device__ __forceinline__ void gd_rope_rotate(float x0, float x1, float c, float s, gd_half *o0, gd_half *o1)
{
    *o0 = (gd_half)__fmaf_rn(x0, c, -__fmul_rn(x1, s));
    *o1 = (gd_half)__fmaf_rn(x0, s, __fmul_rn(x1, c));
}

#endif
