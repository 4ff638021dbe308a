#ifndef GD_HIP_LINEAR_TYPES_H
#define GD_HIP_LINEAR_TYPES_H
#include <stdint.h>

/* epilogue of the projection kernels */
#define GD_HIP_EPI_NONE 0u        /* y = half(acc) */
#define GD_HIP_EPI_BIAS_F32 1u    /* y = half(acc + bias)            (gd_backend_linear) */
#define GD_HIP_EPI_BIAS_F16 2u    /* y = half(half(acc) + bias)      (matmul_nt then add) */

typedef struct gd_hip_linear_params {
    uint32_t M, N, K;
    uint32_t ldx, ldw, ldy; /* row pitch in elements */
    uint32_t epilogue;
    uint32_t w_is_nk;       /* 1: w stored [N,K] (x w^T); 0: w stored [K,N] */
    uint32_t swiglu;        /* 1: A operand = half(x[:, :K] * silu(x[:, K:2K])) */
    uint32_t has_residual;  /* 1: y = half(epilogue(acc) + residual) with residual [M,N] pitch ldr */
    uint32_t ldr;
} gd_hip_linear_params;

#endif
