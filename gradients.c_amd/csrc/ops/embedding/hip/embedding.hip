/*
 * Row gathers for gfx950: embedding lookup and last-row selection.  Pure copies (bit-exact),
 * HBM-bound; 16-byte units when the row size and every offset allow it.
 * Embedding semantics follow the reference kernel src/ops/embedding/metal_embedding.metal:11-33:
 * an id outside [0, vocab) yields a NaN row (F16 0x7e00, F32 0x7fc00000).
 */
#include "../../_shared/hip_device.h"

template <typename U>
__global__ void __launch_bounds__(256)
gd_gather_rows_kernel(const uint8_t *__restrict__ table, const int32_t *__restrict__ ids, uint8_t *__restrict__ out,
                      uint64_t n_ids, uint64_t vocab, uint64_t row_bytes, U nan_unit, int nan_on_invalid)
{
    const uint64_t units_per_row = row_bytes / sizeof(U);
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= n_ids * units_per_row) return;
    const uint64_t row = gid / units_per_row, u = gid - row * units_per_row;
    const int32_t id = ids[row];
    U *dst = reinterpret_cast<U *>(out + row * row_bytes) + u;
    if (id < 0 || (uint64_t)id >= vocab) {
        if (nan_on_invalid) *dst = nan_unit;
        return;
    }
    *dst = reinterpret_cast<const U *>(table + (uint64_t)id * row_bytes)[u];
}

extern "C" int gd_hip_launch_gather_rows(hipStream_t stream, const void *table, const int32_t *ids, void *out,
                                         uint64_t n_ids, uint64_t vocab, uint64_t row_bytes, uint32_t elem_size,
                                         int aligned16, int nan_on_invalid)
{
    if (n_ids == 0 || row_bytes == 0) return (int)hipSuccess;
    if (aligned16 && (row_bytes % 16u) == 0u) {
        gd_u128 nanv;
        nanv.x = nanv.y = nanv.z = nanv.w = elem_size == 2u ? 0x7e007e00u : 0x7fc00000u;
        const uint64_t total = n_ids * (row_bytes / 16u);
        gd_gather_rows_kernel<gd_u128><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
            (const uint8_t *)table, ids, (uint8_t *)out, n_ids, vocab, row_bytes, nanv, nan_on_invalid);
    } else if (elem_size == 2u) {
        const uint64_t total = n_ids * (row_bytes / 2u);
        gd_gather_rows_kernel<uint16_t><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
            (const uint8_t *)table, ids, (uint8_t *)out, n_ids, vocab, row_bytes, (uint16_t)0x7e00u, nan_on_invalid);
    } else {
        const uint64_t total = n_ids * (row_bytes / 4u);
        gd_gather_rows_kernel<uint32_t><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
            (const uint8_t *)table, ids, (uint8_t *)out, n_ids, vocab, row_bytes, 0x7fc00000u, nan_on_invalid);
    }
    return (int)hipGetLastError();
}

__global__ void gd_add_scalar_i32_kernel(const int32_t *__restrict__ src, int32_t *__restrict__ dst, uint64_t n,
                                         int32_t delta)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i] + delta;
}

extern "C" int gd_hip_launch_add_scalar_i32(hipStream_t stream, const int32_t *src, int32_t *dst, uint64_t n,
                                            int32_t delta)
{
    if (n == 0) return (int)hipSuccess;
    gd_add_scalar_i32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(src, dst, n, delta);
    return (int)hipGetLastError();
}

__global__ void __launch_bounds__(256)
gd_decode_advance_kernel(const int32_t *__restrict__ next_ids, const float *__restrict__ gaps, int32_t *__restrict__ ids,
                         int32_t *__restrict__ positions, int32_t *__restrict__ step_counter,
                         int32_t *__restrict__ out_ids, float *__restrict__ out_gaps, uint32_t batch, uint32_t max_steps,
                         int32_t pos_delta)
{
    /* one workgroup: every thread reads the counter before thread 0 advances it */
    const int32_t s = *step_counter;
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < batch; b += blockDim.x) {
        const int32_t t = next_ids[b];
        ids[b] = t;
        positions[b] += pos_delta;
        if (s >= 0 && (uint32_t)s < max_steps) {
            out_ids[(size_t)s * batch + b] = t;
            if (out_gaps != nullptr) out_gaps[(size_t)s * batch + b] = gaps[b];
        }
    }
    if (threadIdx.x == 0) *step_counter = s + 1;
}

extern "C" int gd_hip_launch_decode_advance(hipStream_t stream, const int32_t *next_ids, const float *gaps, int32_t *ids,
                                            int32_t *positions, int32_t *step_counter, int32_t *out_ids,
                                            float *out_gaps, uint32_t batch, uint32_t max_steps, int32_t pos_delta)
{
    gd_decode_advance_kernel<<<1, 256, 0, stream>>>(next_ids, gaps, ids, positions, step_counter, out_ids, out_gaps,
                                                     batch, max_steps, pos_delta);
    return (int)hipGetLastError();
}
