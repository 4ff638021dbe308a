/*
 * The one form of the few-row projection kernel whose weight stream goes through LDS: [N,K] weights behind an
 * rms_norm, 64 columns and 8 wavefronts per workgroup, the activation slice of a wavefront resident in registers
 * (K up to 2048): the up/gate and LM-head projections of the wide decoders.  The kernel is the template of
 * linear_stream_kernel.h; it lives in a translation unit of its own so that the code object of linear.hip, whose
 * kernels carry the decode step of the small configuration, is laid out exactly as without it.
 */
#include "linear_stream_kernel.h"

extern "C" void gd_hip_launch_linear_lds(hipStream_t stream, const void *x, const void *w, const void *bias,
                                         const void *residual, const void *norm_w, void *y,
                                         const gd_hip_linear_params *p, uint32_t n_tiles,
                                         const gd_hip_rope_epilogue *rope, uint32_t grid_x, uint32_t grid_y)
{
    gd_linear_stream_kernel<4, 8, true, GD_HIP_PRO_RMS_NORM, true, true><<<dim3(grid_x, grid_y), 8 * 64, 0, stream>>>(
        (const gd_half *)x, (const gd_half *)w, (const gd_half *)bias, (const gd_half *)residual,
        (const gd_half *)norm_w, (gd_half *)y, *p, n_tiles, *rope);
}
