/*
 * qkv_split_rope forward for gfx950: qkv [N, 3*H*D] -> q, k rotated, v copied, each [N,H,D].
 * HBM-bound elementwise work (reads 3*H*D halfs, writes 3*H*D halfs per token).
 * Arithmetic follows the reference kernel src/ops/qkv_split_rope/metal_qkv_split_rope.metal:6-36,
 * 57-104 and metal_qkv_split_rope.m:228: angle = float(pos) * exp2(pair * freq_scale),
 * freq_scale = -2*log2(theta)/n_dims, NeoX pairs (p, p + D/2) or interleaved (2p, 2p+1),
 * rotation in F32, v moved bit for bit.  sincosf does full range reduction (positions reach 4095).
 *
 * NeoX layout, D % 16 == 0: one thread owns 8 consecutive pairs of one (token, head): two 16-byte
 * loads per tensor (low half and high half of the head), two 16-byte stores.
 */
#include "../../_shared/hip_device.h"

__global__ void __launch_bounds__(256)
gd_qkv_split_rope_neox_vec_kernel(const gd_half *__restrict__ qkv, const int32_t *__restrict__ pos,
                                  gd_half *__restrict__ q, gd_half *__restrict__ k, gd_half *__restrict__ v,
                                  uint64_t tokens, uint32_t heads, uint32_t head_dim, float freq_scale)
{
    const uint32_t half_d = head_dim / 2u, groups = half_d / 8u; /* 8-pair groups per head */
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t total = tokens * heads * groups;
    if (gid >= total) return;
    const uint32_t grp = (uint32_t)(gid % groups);
    const uint32_t h = (uint32_t)((gid / groups) % heads);
    const uint64_t n = gid / ((uint64_t)groups * heads);
    const uint64_t area = (uint64_t)heads * head_dim;
    const gd_half *src = qkv + n * 3u * area + (uint64_t)h * head_dim + grp * 8u;
    const uint64_t dst = n * area + (uint64_t)h * head_dim + grp * 8u;
    const float fpos = (float)pos[n];
    float c[8], s[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float angle = fpos * exp2f((float)(grp * 8u + e) * freq_scale);
        sincosf(angle, &s[e], &c[e]);
    }
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const gd_half8 lo = *reinterpret_cast<const gd_half8 *>(src + which * area);
        const gd_half8 hi = *reinterpret_cast<const gd_half8 *>(src + which * area + half_d);
        gd_half8 olo, ohi;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x0 = (float)lo[e], x1 = (float)hi[e];
            olo[e] = (gd_half)(x0 * c[e] - x1 * s[e]);
            ohi[e] = (gd_half)(x0 * s[e] + x1 * c[e]);
        }
        gd_half *o = which == 0 ? q : k;
        *reinterpret_cast<gd_half8 *>(o + dst) = olo;
        *reinterpret_cast<gd_half8 *>(o + dst + half_d) = ohi;
    }
    *reinterpret_cast<gd_u128 *>(v + dst) = *reinterpret_cast<const gd_u128 *>(src + 2u * area);
    *reinterpret_cast<gd_u128 *>(v + dst + half_d) = *reinterpret_cast<const gd_u128 *>(src + 2u * area + half_d);
}

/* any even head size, either pairing: one thread per (token, head, pair) */
__global__ void __launch_bounds__(256)
gd_qkv_split_rope_scalar_kernel(const gd_half *__restrict__ qkv, const int32_t *__restrict__ pos,
                                gd_half *__restrict__ q, gd_half *__restrict__ k, gd_half *__restrict__ v,
                                uint64_t tokens, uint32_t heads, uint32_t head_dim, float freq_scale,
                                uint32_t interleaved)
{
    const uint32_t half_d = head_dim / 2u;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= tokens * heads * half_d) return;
    const uint32_t pair = (uint32_t)(gid % half_d);
    const uint32_t h = (uint32_t)((gid / half_d) % heads);
    const uint64_t n = gid / ((uint64_t)half_d * heads);
    const uint32_t a = interleaved ? pair * 2u : pair;
    const uint32_t b = interleaved ? pair * 2u + 1u : pair + half_d;
    const uint64_t area = (uint64_t)heads * head_dim;
    const gd_half *src = qkv + n * 3u * area + (uint64_t)h * head_dim;
    const uint64_t dst = n * area + (uint64_t)h * head_dim;
    float s, c;
    sincosf((float)pos[n] * exp2f((float)pair * freq_scale), &s, &c);
    const float q0 = (float)src[a], q1 = (float)src[b];
    const float k0 = (float)src[area + a], k1 = (float)src[area + b];
    q[dst + a] = (gd_half)(q0 * c - q1 * s);
    q[dst + b] = (gd_half)(q0 * s + q1 * c);
    k[dst + a] = (gd_half)(k0 * c - k1 * s);
    k[dst + b] = (gd_half)(k0 * s + k1 * c);
    v[dst + a] = src[2u * area + a];
    v[dst + b] = src[2u * area + b];
}

extern "C" int gd_hip_launch_qkv_split_rope(hipStream_t stream, const void *qkv, const int32_t *pos, void *q,
                                            void *k, void *v, uint64_t tokens, uint32_t heads, uint32_t head_dim,
                                            float theta, uint32_t interleaved, int aligned16)
{
    const float freq_scale = -2.0f * log2f(theta) / (float)head_dim;
    if (tokens == 0) return (int)hipSuccess;
    if (!interleaved && aligned16 && (head_dim % 16u) == 0u) {
        const uint64_t total = tokens * heads * (head_dim / 16u);
        gd_qkv_split_rope_neox_vec_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
            (const gd_half *)qkv, pos, (gd_half *)q, (gd_half *)k, (gd_half *)v, tokens, heads, head_dim, freq_scale);
    } else {
        const uint64_t total = tokens * heads * (head_dim / 2u);
        gd_qkv_split_rope_scalar_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
            (const gd_half *)qkv, pos, (gd_half *)q, (gd_half *)k, (gd_half *)v, tokens, heads, head_dim,
            freq_scale, interleaved);
    }
    return (int)hipGetLastError();
}
