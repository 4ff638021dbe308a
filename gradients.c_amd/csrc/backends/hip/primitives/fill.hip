/*
 * Backend primitive: pattern fill of 1/2/4-byte elements.  Replaces the
 * reference's gd_backend_fill (src/core/backend.h:172-177); also the safe way to
 * clear memory inside a captured graph (no memset nodes).
 */
#include "../../../ops/_shared/hip_device.h"

template <typename T>
__global__ void gd_fill_kernel(T *__restrict__ dst, size_t count, T value)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) dst[i] = value;
}

extern "C" int gd_hip_launch_fill(hipStream_t stream, void *dst, size_t count, size_t elem_size, uint32_t pattern)
{
    const int block = 256;
    size_t blocks = (count + block - 1) / block;
    if (blocks > 65536) blocks = 65536;
    /* widen to 4-byte stores when the run is aligned and the pattern repeats */
    if (elem_size == 1 && ((uintptr_t)dst & 3u) == 0 && (count & 3u) == 0) {
        const uint32_t b = pattern & 0xffu;
        return gd_hip_launch_fill(stream, dst, count / 4, 4, b | (b << 8) | (b << 16) | (b << 24));
    }
    if (elem_size == 2 && ((uintptr_t)dst & 3u) == 0 && (count & 1u) == 0) {
        const uint32_t h = pattern & 0xffffu;
        return gd_hip_launch_fill(stream, dst, count / 2, 4, h | (h << 16));
    }
    if (elem_size == 1) gd_fill_kernel<uint8_t><<<(unsigned)blocks, block, 0, stream>>>((uint8_t *)dst, count, (uint8_t)pattern);
    else if (elem_size == 2) gd_fill_kernel<uint16_t><<<(unsigned)blocks, block, 0, stream>>>((uint16_t *)dst, count, (uint16_t)pattern);
    else gd_fill_kernel<uint32_t><<<(unsigned)blocks, block, 0, stream>>>((uint32_t *)dst, count, pattern);
    return (int)hipGetLastError();
}
