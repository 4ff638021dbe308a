/*
 * Copy of a contiguous slice into its place inside a contiguous concatenated tensor: the device half
 * of the reference's gd_concat (src/core/backend.h:579-591), which its generator uses to collect the
 * last prompt row of every sequence (examples/gpt_lm/gpt_lm_shared.c:1117-1169).  HBM-bound byte copy.
 */
#include "../../_shared/hip_device.h"

template <typename T>
__global__ void __launch_bounds__(256)
gd_concat_to_full_kernel(const T *__restrict__ src, T *__restrict__ dst, uint64_t count, uint64_t inner,
                         uint64_t slice_axis, uint64_t full_axis, uint64_t axis_offset)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const uint64_t slab = slice_axis * inner;
    const uint64_t outer = i / slab, rem = i - outer * slab;
    dst[outer * full_axis * inner + axis_offset * inner + rem] = src[i];
}

extern "C" int gd_hip_launch_concat_to_full(hipStream_t stream, const void *src, void *dst, uint64_t count,
                                            uint64_t inner, uint64_t slice_axis, uint64_t full_axis,
                                            uint64_t axis_offset, uint32_t elem_size)
{
    if (count == 0) return (int)hipSuccess;
    const unsigned blocks = (unsigned)((count + 255) / 256);
    if (elem_size == 2u)
        gd_concat_to_full_kernel<uint16_t><<<blocks, 256, 0, stream>>>((const uint16_t *)src, (uint16_t *)dst, count, inner, slice_axis, full_axis, axis_offset);
    else if (elem_size == 4u)
        gd_concat_to_full_kernel<uint32_t><<<blocks, 256, 0, stream>>>((const uint32_t *)src, (uint32_t *)dst, count, inner, slice_axis, full_axis, axis_offset);
    else
        gd_concat_to_full_kernel<uint8_t><<<blocks, 256, 0, stream>>>((const uint8_t *)src, (uint8_t *)dst, count, inner, slice_axis, full_axis, axis_offset);
    return (int)hipGetLastError();
}
