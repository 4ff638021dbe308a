/*
 * Device helpers shared by the sdpa_decode kernels (sdpa_decode.hip): the reference's
 * visibility mask, the position lookup, and the lane-group reductions of the split-KV kernels.
 */
#ifndef GD_SDPA_DECODE_DEVICE_H
#define GD_SDPA_DECODE_DEVICE_H
#include "../../_shared/hip_device.h"
#include "hip_sdpa_decode_types.h"

#define GD_NEG_INF (-__builtin_inff())

__device__ __forceinline__ bool gd_attn_allowed(int qpos, int j, int window, int prefix_len)
{
    if (prefix_len > 0) {
        if (qpos < prefix_len) {
            if (j >= prefix_len) return false;
        } else if (j > qpos) {
            return false;
        }
    } else if (j > qpos) {
        return false;
    }
    if (window > 0) {
        if (prefix_len > 0) {
            if (qpos >= prefix_len && j >= prefix_len && (qpos - j) >= window) return false;
        } else if ((qpos - j) >= window) {
            return false;
        }
    }
    return true;
}

__device__ __forceinline__ int gd_decode_pos(const int32_t *pos, const gd_hip_sdpa_decode_params &p, int b)
{
    if (p.pos_mode == GD_HIP_SDPA_POS_SCALAR) return p.cache_pos;
    return pos[p.pos_mode == GD_HIP_SDPA_POS_VECTOR ? b : 0];
}

/* Device-scope relaxed store / load: the store is written through this XCD's L2, the load is served from behind
 * it, so workgroups on different XCDs (whose L2s do not snoop each other) can hand data over without writing
 * back or invalidating whole caches.  Ordering against other accesses is the caller's business. */
__device__ __forceinline__ void gd_agent_store(float *p, float v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float gd_agent_load(const float *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* ---- split-KV kernel ----------------------------------------------------------- */

/* Sum over aligned groups of N (8 or 16) consecutive lanes; every lane of a group receives the total.
 * Data-parallel-primitive adds (lane swaps inside a row of 16 lanes) instead of LDS shuffles:
 * swap neighbours, swap pairs, mirror the 8-lane half row, and for 16 lanes mirror the row. */
template <int CTRL>
__device__ __forceinline__ float gd_dpp_add(float x)
{
    return x + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}

template <int N>
__device__ __forceinline__ float gd_row_group_sum(float x)
{
    x = gd_dpp_add<0xB1>(x);  /* quad_perm [1,0,3,2] */
    x = gd_dpp_add<0x4E>(x);  /* quad_perm [2,3,0,1] */
    x = gd_dpp_add<0x141>(x); /* row_half_mirror */
    if (N == 16) x = gd_dpp_add<0x140>(x); /* row_mirror */
    return x;
}

/* Reductions over the 64 / N row slots of a wavefront: lanes i, i + N, i + 2N, ... (N = 8 or 16) are combined
 * and every lane receives the result.  Distance 8: rotation by 8 inside the 16-lane row (DPP).  Distances 16
 * and 32: v_permlane16_swap / v_permlane32_swap on two copies of the value, which leave one copy holding the
 * even (lower) partner's value in both places and the other the odd (upper) partner's. */
template <int N, typename OP>
__device__ __forceinline__ float gd_slot_reduce(float x, OP op)
{
    typedef unsigned gd_uint2 __attribute__((ext_vector_type(2)));
    if (N == 8) x = op(x, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x128, 0xf, 0xf, false)));
    gd_uint2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = op(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return op(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

/* Reduction over the 64 lanes of a wavefront, every lane receives the result: swaps inside the 16-lane row, then
 * the row and half swaps. */
template <typename OP>
__device__ __forceinline__ int gd_wave_reduce_i32(int x, OP op)
{
    typedef unsigned gd_uint2 __attribute__((ext_vector_type(2)));
    x = op(x, __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xf, 0xf, false));  /* quad_perm [1,0,3,2] */
    x = op(x, __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xf, 0xf, false));  /* quad_perm [2,3,0,1] */
    x = op(x, __builtin_amdgcn_update_dpp(0, x, 0x141, 0xf, 0xf, false)); /* row_half_mirror */
    x = op(x, __builtin_amdgcn_update_dpp(0, x, 0x140, 0xf, 0xf, false)); /* row_mirror */
    gd_uint2 r = __builtin_amdgcn_permlane16_swap((unsigned)x, (unsigned)x, false, false);
    x = op((int)r[0], (int)r[1]);
    r = __builtin_amdgcn_permlane32_swap((unsigned)x, (unsigned)x, false, false);
    return op((int)r[0], (int)r[1]);
}

template <int N>
__device__ __forceinline__ float gd_slot_sum(float x)
{
    return gd_slot_reduce<N>(x, [](float a, float b) { return a + b; });
}

template <int N>
__device__ __forceinline__ float gd_slot_max(float x)
{
    return gd_slot_reduce<N>(x, [](float a, float b) { return fmaxf(a, b); });
}

#endif
