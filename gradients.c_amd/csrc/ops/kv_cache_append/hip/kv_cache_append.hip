/*
 * K/V cache append for gfx950: cache[b, pos_b + t, :] = fresh[b, t, :] for K and V.
 *
 * Pure byte movement, HBM-bound (reads 2 rows, writes 2 rows per appended token).
 * One thread moves one 16-byte unit of K and of V when every offset and the row
 * size allow it (4- or 1-byte units otherwise), so a wavefront covers 1 KiB of
 * contiguous row bytes per instruction.  Semantics follow the reference kernels
 * src/ops/kv_cache_append/metal_kv_cache_append.metal:30-63 (batched) and
 * :80-122 (packed): rows whose position is negative or whose span passes Tmax
 * are skipped, never trapped.
 */
#include "../../_shared/hip_device.h"
#include "hip_kv_cache_append_types.h"

template <typename U>
__global__ void __launch_bounds__(256)
gd_kv_append_kernel(uint8_t *__restrict__ k_cache, uint8_t *__restrict__ v_cache,
                    const uint8_t *__restrict__ k_new, const uint8_t *__restrict__ v_new,
                    const int32_t *__restrict__ pos_vec, gd_hip_kv_append_params p)
{
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= p.total_units) return;
    const uint64_t src_byte = gid * sizeof(U);
    const uint64_t row = src_byte / p.row_bytes;
    const uint64_t within = src_byte - row * p.row_bytes;
    const uint64_t b = row / p.tnew;
    const uint64_t t = row - b * p.tnew;
    const int64_t pos = pos_vec != nullptr ? (int64_t)pos_vec[b] : (int64_t)p.cache_pos;
    if (pos < 0 || pos + (int64_t)p.tnew > (int64_t)p.tmax) return;
    const uint64_t dst_byte = ((b * p.tmax + (uint64_t)pos + t) * p.row_bytes) + within;
    *reinterpret_cast<U *>(k_cache + dst_byte) = *reinterpret_cast<const U *>(k_new + src_byte);
    *reinterpret_cast<U *>(v_cache + dst_byte) = *reinterpret_cast<const U *>(v_new + src_byte);
}

template <typename U>
__global__ void __launch_bounds__(256)
gd_kv_append_packed_kernel(uint8_t *__restrict__ k_cache, uint8_t *__restrict__ v_cache,
                           const uint8_t *__restrict__ k_new, const uint8_t *__restrict__ v_new,
                           const int32_t *__restrict__ pos_vec, const int32_t *__restrict__ cu,
                           gd_hip_kv_append_params p)
{
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= p.total_units) return;
    const uint32_t units_per_row = (uint32_t)(p.row_bytes / sizeof(U));
    const uint32_t row = (uint32_t)(gid / units_per_row);
    const uint64_t within = (gid - (uint64_t)row * units_per_row) * sizeof(U);
    if (cu[0] != 0 || (int32_t)row >= cu[p.batch]) return;
    /* largest b in [0, batch) with cu[b] <= row */
    uint32_t lo = 0u, hi = (uint32_t)p.batch;
    while (lo + 1u < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if ((uint32_t)cu[mid] <= row) lo = mid; else hi = mid;
    }
    const int32_t seq_start = cu[lo], seq_end = cu[lo + 1u];
    const int32_t t = (int32_t)row - seq_start;
    const int32_t pos = pos_vec[lo];
    if (seq_start < 0 || seq_end < seq_start || t < 0 || pos < 0 ||
        (int64_t)pos + (int64_t)(seq_end - seq_start) > (int64_t)p.tmax) return;
    const uint64_t src_byte = (uint64_t)row * p.row_bytes + within;
    const uint64_t dst_byte = (((uint64_t)lo * p.tmax + (uint64_t)(pos + t)) * p.row_bytes) + within;
    *reinterpret_cast<U *>(k_cache + dst_byte) = *reinterpret_cast<const U *>(k_new + src_byte);
    *reinterpret_cast<U *>(v_cache + dst_byte) = *reinterpret_cast<const U *>(v_new + src_byte);
}

extern "C" int gd_hip_launch_kv_cache_append(hipStream_t stream, void *k_cache, void *v_cache,
                                             const void *k_new, const void *v_new, const int32_t *pos,
                                             const int32_t *cu, const gd_hip_kv_append_params *params)
{
    gd_hip_kv_append_params p = *params;
    const uint64_t total_bytes = p.total_units; /* passed in as bytes, converted below */
    const int block = 256;
    if (total_bytes == 0) return (int)hipSuccess;
#define GD_LAUNCH(U)                                                                               \
    do {                                                                                           \
        p.total_units = total_bytes / sizeof(U);                                                   \
        const uint64_t blocks = (p.total_units + block - 1) / block;                               \
        if (cu != nullptr)                                                                         \
            gd_kv_append_packed_kernel<U><<<(unsigned)blocks, block, 0, stream>>>(                 \
                (uint8_t *)k_cache, (uint8_t *)v_cache, (const uint8_t *)k_new,                    \
                (const uint8_t *)v_new, pos, cu, p);                                               \
        else                                                                                       \
            gd_kv_append_kernel<U><<<(unsigned)blocks, block, 0, stream>>>(                        \
                (uint8_t *)k_cache, (uint8_t *)v_cache, (const uint8_t *)k_new,                    \
                (const uint8_t *)v_new, pos, p);                                                   \
    } while (0)
    if (p.copy_unit == 16u) GD_LAUNCH(gd_u128);
    else if (p.copy_unit == 4u) GD_LAUNCH(uint32_t);
    else GD_LAUNCH(uint8_t);
#undef GD_LAUNCH
    return (int)hipGetLastError();
}
