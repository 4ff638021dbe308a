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
        if (k == nullptr) store_kv = false; /* the caller reads the rows from the caches */
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

/* Where the angle of pair `pair` of row n sits in the angle tables.  The tile kernel's rotation epilogue reads, per
 * instruction, 4 consecutive pairs of 32 consecutive rows in each half wavefront: the tables are laid out so that
 * such a read is 1 KB of consecutive memory: blocks of 32 rows; inside a block groups of 8 pairs; inside a group the
 * low 4 pairs of all 32 rows, then the high 4 pairs of all 32 rows.  Tables hold ceil(N / 32) * 32 rows. */
__host__ __device__ __forceinline__ uint64_t gd_rope_table_at(uint64_t n, uint32_t pair, uint32_t half_d)
{
    return (((n >> 5) * (half_d >> 3) + (pair >> 3)) * 2u + ((pair >> 2) & 1u)) * 128u + (n & 31u) * 4u + (pair & 3u);
}

/* Angles and cache rows of the N packed prompt rows, computed once per prefill and used by every layer's qkv
 * projection (the rotation epilogue of the tile kernel in ops/linear/hip/linear_tile.hip and the row kernel below):
 * cos_rows / sin_rows F32 (laid out by gd_rope_table_at) with the same arithmetic as the rotation kernels above, cache_row [N] = sequence *
 * tmax + seq_pos[sequence] + token under the rules of the packed append (nothing unless cu starts at 0; a sequence with
 * a negative position or whose rows do not fit behind it is skipped), -1 for a row that is not appended. */
__global__ void __launch_bounds__(256)
gd_rope_table_packed_kernel(const int32_t *__restrict__ pos, const int32_t *__restrict__ cu,
                            const int32_t *__restrict__ seq_pos, uint32_t batch, float *__restrict__ cos_rows,
                            float *__restrict__ sin_rows, int32_t *__restrict__ cache_row, uint64_t tokens,
                            uint32_t half_d, uint32_t tmax, float freq_scale)
{
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= tokens * half_d) return;
    const uint64_t n = gid / half_d;
    const uint32_t pair = (uint32_t)(gid % half_d);
    float c, s;
    gd_rope_cos_sin((float)pos[n], pair, freq_scale, &c, &s);
    const uint64_t at = gd_rope_table_at(n, pair, half_d);
    cos_rows[at] = c;
    sin_rows[at] = s;
    if (pair != 0u) return;
    int32_t row = -1;
    if (cu[0] == 0 && (int64_t)n < (int64_t)cu[batch]) {
        uint32_t lo = 0u, hi = batch; /* largest b with cu[b] <= n */
        while (lo + 1u < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if ((uint64_t)cu[mid] <= n) lo = mid; else hi = mid;
        }
        const int32_t seq_start = cu[lo], seq_end = cu[lo + 1u];
        const int32_t t = (int32_t)n - seq_start, at = seq_pos[lo];
        if (seq_start >= 0 && seq_end >= seq_start && t >= 0 && t < seq_end - seq_start && at >= 0 &&
            (int64_t)at + (int64_t)(seq_end - seq_start) <= (int64_t)tmax)
            row = (int32_t)(lo * tmax + (uint32_t)(at + t));
    }
    cache_row[n] = row;
}

/* Rows row0 .. row0 + rows of a packed prefill whose projection lies in qkv [rows, 3*H*D] (local row 0 = row0):
 * rotated q to row n of q [N,H,D], rotated k and copied v to row cache_row[n] of the caches; angles from the table.
 * The same rounding points as gd_qkv_split_rope_neox_vec_kernel.  For the rows the tile kernel's rotation epilogue
 * does not take (the last, partly filled round of tiles). */
__global__ void __launch_bounds__(256)
gd_qkv_rope_rows_kernel(const gd_half *__restrict__ qkv, const float *__restrict__ cos_rows,
                        const float *__restrict__ sin_rows, const int32_t *__restrict__ cache_row,
                        gd_half *__restrict__ q, gd_half *__restrict__ k_cache, gd_half *__restrict__ v_cache,
                        uint64_t row0, uint64_t rows, uint32_t heads, uint32_t head_dim)
{
    const uint32_t half_d = head_dim / 2u, groups = half_d / 8u;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= rows * heads * groups) return;
    const uint32_t grp = (uint32_t)(gid % groups);
    const uint32_t h = (uint32_t)((gid / groups) % heads);
    const uint64_t local = gid / ((uint64_t)groups * heads), n = row0 + local;
    const uint64_t area = (uint64_t)heads * head_dim, within = (uint64_t)h * head_dim + grp * 8u;
    const gd_half *src = qkv + local * 3u * area + within;
    const int32_t crow = cache_row[n];
    typedef float gd_float4v __attribute__((ext_vector_type(4)));
    const gd_float4v c0 = *reinterpret_cast<const gd_float4v *>(cos_rows + gd_rope_table_at(n, grp * 8u, half_d));
    const gd_float4v c1 = *reinterpret_cast<const gd_float4v *>(cos_rows + gd_rope_table_at(n, grp * 8u + 4u, half_d));
    const gd_float4v s0 = *reinterpret_cast<const gd_float4v *>(sin_rows + gd_rope_table_at(n, grp * 8u, half_d));
    const gd_float4v s1 = *reinterpret_cast<const gd_float4v *>(sin_rows + gd_rope_table_at(n, grp * 8u + 4u, half_d));
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const gd_half8 lo = *reinterpret_cast<const gd_half8 *>(src + which * area);
        const gd_half8 hi = *reinterpret_cast<const gd_half8 *>(src + which * area + half_d);
        gd_half8 olo, ohi;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            gd_half a, b;
            gd_rope_rotate((float)lo[e], (float)hi[e], e < 4 ? c0[e & 3] : c1[e & 3], e < 4 ? s0[e & 3] : s1[e & 3], &a, &b);
            olo[e] = a;
            ohi[e] = b;
        }
        if (which == 0) {
            *reinterpret_cast<gd_half8 *>(q + n * area + within) = olo;
            *reinterpret_cast<gd_half8 *>(q + n * area + within + half_d) = ohi;
        } else if (crow >= 0) {
            *reinterpret_cast<gd_half8 *>(k_cache + (uint64_t)crow * area + within) = olo;
            *reinterpret_cast<gd_half8 *>(k_cache + (uint64_t)crow * area + within + half_d) = ohi;
        }
    }
    if (crow >= 0) {
        *reinterpret_cast<gd_u128 *>(v_cache + (uint64_t)crow * area + within) =
            *reinterpret_cast<const gd_u128 *>(src + 2u * area);
        *reinterpret_cast<gd_u128 *>(v_cache + (uint64_t)crow * area + within + half_d) =
            *reinterpret_cast<const gd_u128 *>(src + 2u * area + half_d);
    }
}

extern "C" int gd_hip_launch_rope_table_packed(hipStream_t stream, const int32_t *pos, const int32_t *cu,
                                               const int32_t *seq_pos, uint32_t batch, float *cos_rows, float *sin_rows,
                                               int32_t *cache_row, uint64_t tokens, uint32_t head_dim, uint32_t tmax,
                                               float theta)
{
    const float freq_scale = -2.0f * log2f(theta) / (float)head_dim;
    const uint64_t total = tokens * (head_dim / 2u);
    if (total == 0) return (int)hipSuccess;
    gd_rope_table_packed_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
        pos, cu, seq_pos, batch, cos_rows, sin_rows, cache_row, tokens, head_dim / 2u, tmax, freq_scale);
    return (int)hipGetLastError();
}

extern "C" int gd_hip_launch_qkv_rope_rows(hipStream_t stream, const void *qkv, const float *cos_rows,
                                           const float *sin_rows, const int32_t *cache_row, void *q, void *k_cache,
                                           void *v_cache, uint64_t row0, uint64_t rows, uint32_t heads, uint32_t head_dim)
{
    const uint64_t total = rows * heads * (head_dim / 16u);
    if (total == 0) return (int)hipSuccess;
    gd_qkv_rope_rows_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
        (const gd_half *)qkv, cos_rows, sin_rows, cache_row, (gd_half *)q, (gd_half *)k_cache, (gd_half *)v_cache, row0,
        rows, heads, head_dim);
    return (int)hipGetLastError();
}
