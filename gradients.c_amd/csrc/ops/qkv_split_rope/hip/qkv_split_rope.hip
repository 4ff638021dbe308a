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
#include "rope_device.h"

/* destinations of the packed prefill form: besides k / v [N,H,D] the rows also go into the sequences' caches
 * [B,Tmax,H,D], token t of sequence b (rows cu[b] .. cu[b+1]) into cache row seq_pos[b] + t */
struct gd_rope_packed_caches {
    gd_half *k_cache, *v_cache;
    const int32_t *cu, *seq_pos;
    uint32_t batch;
};

/* cache_pos == nullptr: k and v go to row n of [N,H,D] tensors (split form).  Otherwise they go to
 * row cache_pos[n] of sequence n in [N,Tmax,H,D] caches (decode form, one new token per sequence);
 * a sequence whose position is negative or >= tmax keeps its caches untouched, like the append
 * kernel.  PACKED: the split form that also appends the rows to the caches of their sequences, with the rules of the
 * packed append kernel (gd_kv_append_packed_kernel: nothing is appended unless cu starts at 0, a sequence whose rows
 * do not fit behind its position is skipped).  One kernel serves all forms so that they produce the same bits. */
template <bool PACKED>
__global__ void __launch_bounds__(256)
gd_qkv_split_rope_neox_vec_kernel(const gd_half *__restrict__ qkv, const int32_t *__restrict__ pos,
                                  const int32_t *__restrict__ cache_pos, gd_half *__restrict__ q,
                                  gd_half *__restrict__ k, gd_half *__restrict__ v, uint64_t tokens, uint32_t heads,
                                  uint32_t head_dim, uint32_t tmax, float freq_scale, gd_rope_packed_caches pc)
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
    const uint64_t within = (uint64_t)h * head_dim + grp * 8u;
    const uint64_t qdst = n * area + within;
    bool store_kv = true;
    uint64_t kvdst = qdst;
    if (cache_pos != nullptr) {
        const int32_t cp = cache_pos[n];
        store_kv = cp >= 0 && (uint32_t)cp < tmax;
        kvdst = (n * tmax + (uint64_t)(store_kv ? cp : 0)) * area + within;
    }
    bool store_cache = false;
    uint64_t cdst = 0;
    if (PACKED) {
        if (pc.cu[0] == 0 && (int64_t)n < (int64_t)pc.cu[pc.batch]) {
            uint32_t lo = 0u, hi = pc.batch; /* largest b with cu[b] <= n */
            while (lo + 1u < hi) {
                const uint32_t mid = (lo + hi) >> 1;
                if ((uint64_t)pc.cu[mid] <= n) lo = mid; else hi = mid;
            }
            const int32_t seq_start = pc.cu[lo], seq_end = pc.cu[lo + 1u];
            const int32_t t = (int32_t)n - seq_start, at = pc.seq_pos[lo];
            store_cache = seq_start >= 0 && seq_end >= seq_start && t >= 0 && at >= 0 &&
                          (int64_t)at + (int64_t)(seq_end - seq_start) <= (int64_t)tmax;
            cdst = ((uint64_t)lo * tmax + (uint64_t)(store_cache ? at + t : 0)) * area + within;
        }
    }
    const float fpos = (float)pos[n];
    float c[8], s[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) gd_rope_cos_sin(fpos, grp * 8u + e, freq_scale, &c[e], &s[e]);
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const gd_half8 lo = *reinterpret_cast<const gd_half8 *>(src + which * area);
        const gd_half8 hi = *reinterpret_cast<const gd_half8 *>(src + which * area + half_d);
        gd_half8 olo, ohi;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            gd_half a, b;
            gd_rope_rotate((float)lo[e], (float)hi[e], c[e], s[e], &a, &b);
            olo[e] = a;
            ohi[e] = b;
        }
        if (which == 0) {
            *reinterpret_cast<gd_half8 *>(q + qdst) = olo;
            *reinterpret_cast<gd_half8 *>(q + qdst + half_d) = ohi;
        } else {
            if (store_kv) {
                *reinterpret_cast<gd_half8 *>(k + kvdst) = olo;
                *reinterpret_cast<gd_half8 *>(k + kvdst + half_d) = ohi;
            }
            if (PACKED && store_cache) {
                *reinterpret_cast<gd_half8 *>(pc.k_cache + cdst) = olo;
                *reinterpret_cast<gd_half8 *>(pc.k_cache + cdst + half_d) = ohi;
            }
        }
    }
    const gd_u128 vlo = *reinterpret_cast<const gd_u128 *>(src + 2u * area);
    const gd_u128 vhi = *reinterpret_cast<const gd_u128 *>(src + 2u * area + half_d);
    if (store_kv) {
        *reinterpret_cast<gd_u128 *>(v + kvdst) = vlo;
        *reinterpret_cast<gd_u128 *>(v + kvdst + half_d) = vhi;
    }
    if (PACKED && store_cache) {
        *reinterpret_cast<gd_u128 *>(pc.v_cache + cdst) = vlo;
        *reinterpret_cast<gd_u128 *>(pc.v_cache + cdst + half_d) = vhi;
    }
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
    gd_rope_cos_sin((float)pos[n], pair, freq_scale, &c, &s);
    gd_rope_rotate((float)src[a], (float)src[b], c, s, &q[dst + a], &q[dst + b]);
    gd_rope_rotate((float)src[area + a], (float)src[area + b], c, s, &k[dst + a], &k[dst + b]);
    v[dst + a] = src[2u * area + a];
    v[dst + b] = src[2u * area + b];
}

extern "C" int gd_hip_launch_qkv_rope_append(hipStream_t stream, const void *qkv, const int32_t *rope_pos,
                                             const int32_t *cache_pos, void *q, void *k_cache, void *v_cache,
                                             uint64_t tokens, uint32_t heads, uint32_t head_dim, uint32_t tmax,
                                             float theta)
{
    const float freq_scale = -2.0f * log2f(theta) / (float)head_dim;
    const uint64_t total = tokens * heads * (head_dim / 16u);
    if (total == 0) return (int)hipSuccess;
    gd_qkv_split_rope_neox_vec_kernel<false><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
        (const gd_half *)qkv, rope_pos, cache_pos, (gd_half *)q, (gd_half *)k_cache, (gd_half *)v_cache, tokens, heads,
        head_dim, tmax, freq_scale, gd_rope_packed_caches{nullptr, nullptr, nullptr, nullptr, 0u});
    return (int)hipGetLastError();
}

extern "C" int gd_hip_launch_qkv_split_rope(hipStream_t stream, const void *qkv, const int32_t *pos, void *q,
                                            void *k, void *v, uint64_t tokens, uint32_t heads, uint32_t head_dim,
                                            float theta, uint32_t interleaved, int aligned16)
{
    const float freq_scale = -2.0f * log2f(theta) / (float)head_dim;
    if (tokens == 0) return (int)hipSuccess;
    if (!interleaved && aligned16 && (head_dim % 16u) == 0u) {
        const uint64_t total = tokens * heads * (head_dim / 16u);
        gd_qkv_split_rope_neox_vec_kernel<false><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
            (const gd_half *)qkv, pos, nullptr, (gd_half *)q, (gd_half *)k, (gd_half *)v, tokens, heads, head_dim, 0u,
            freq_scale, gd_rope_packed_caches{nullptr, nullptr, nullptr, nullptr, 0u});
    } else {
        const uint64_t total = tokens * heads * (head_dim / 2u);
        gd_qkv_split_rope_scalar_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
            (const gd_half *)qkv, pos, (gd_half *)q, (gd_half *)k, (gd_half *)v, tokens, heads, head_dim,
            freq_scale, interleaved);
    }
    return (int)hipGetLastError();
}

/* packed prefill: qkv [N, 3*H*D] -> q, k, v [N,H,D], and k / v also into the caches of their sequences */
extern "C" int gd_hip_launch_qkv_rope_append_packed(hipStream_t stream, const void *qkv, const int32_t *rope_pos,
                                                    const int32_t *seq_pos, const int32_t *cu, uint32_t batch, void *q,
                                                    void *k, void *v, void *k_cache, void *v_cache, uint64_t tokens,
                                                    uint32_t heads, uint32_t head_dim, uint32_t tmax, float theta)
{
    const float freq_scale = -2.0f * log2f(theta) / (float)head_dim;
    const uint64_t total = tokens * heads * (head_dim / 16u);
    if (total == 0) return (int)hipSuccess;
    gd_qkv_split_rope_neox_vec_kernel<true><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
        (const gd_half *)qkv, rope_pos, nullptr, (gd_half *)q, (gd_half *)k, (gd_half *)v, tokens, heads, head_dim, tmax,
        freq_scale, gd_rope_packed_caches{(gd_half *)k_cache, (gd_half *)v_cache, cu, seq_pos, batch});
    return (int)hipGetLastError();
}
