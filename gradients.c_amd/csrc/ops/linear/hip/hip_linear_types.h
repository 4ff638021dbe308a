#ifndef GD_HIP_LINEAR_TYPES_H
#define GD_HIP_LINEAR_TYPES_H
#include <stdint.h>

/* epilogue of the projection kernels */
#define GD_HIP_EPI_NONE 0u        /* y = half(acc) */
#define GD_HIP_EPI_BIAS_F32 1u    /* y = half(acc + bias)            (gd_backend_linear) */
#define GD_HIP_EPI_BIAS_F16 2u    /* y = half(half(acc) + bias)      (matmul_nt then add) */

/* prologue applied to the activation operand before it enters the MFMA, rounded to F16 */
#define GD_HIP_PRO_NONE 0u
#define GD_HIP_PRO_SWIGLU 1u      /* a = half(x[:, k] * silu(x[:, K + k])), x has 2K columns */
#define GD_HIP_PRO_RMS_NORM 2u    /* a = half(x[:, k] * norm_w[k] * rsqrt(mean(x^2) + eps)) */

typedef struct gd_hip_linear_params {
    uint32_t M, N, K;
    uint32_t ldx, ldw, ldy; /* row pitch in elements */
    uint32_t epilogue;
    uint32_t w_is_nk;       /* 1: w stored [N,K] (x w^T); 0: w stored [K,N] */
    uint32_t prologue;
    uint32_t has_residual;  /* 1: y = half(epilogue(acc)) + residual, residual [M,N] pitch ldr */
    uint32_t ldr;
    float eps;              /* rms_norm prologue */
    uint32_t swiglu_cols;   /* 0, or H: w has 2H rows ([N,K] only); y [M,H] = half(u[:, :H] * silu(u[:, H:])) where u is
                             * the projection after the bias epilogue, rounded to F16 like a stored intermediate */
    /* rope + cache append epilogue (rope_head_dim != 0): the projection is the qkv projection of a decode step,
     * N = 3 * heads * head_dim; see gd_hip_rope_epilogue */
    uint32_t rope_heads, rope_head_dim, rope_tmax;
    float rope_freq_scale;
    /* The few-row kernel reads its arguments in one batch at entry: six pointers, this structure and the tile count
     * behind it fill exactly one 128-byte line of the argument segment.  Keep the structure at 76 bytes: with the
     * tile count on a second line every projection launch of a decode step took 0.06 us longer. */
    uint16_t force_tiles, force_waves; /* tunables: 0 = automatic */
    uint32_t no_lds_stream;            /* tunable: 1 = weights always go straight to registers */
} gd_hip_linear_params;
#ifdef __cplusplus
static_assert(sizeof(gd_hip_linear_params) == 76, "the few-row kernel's arguments must stay within one 128-byte line");
#else
_Static_assert(sizeof(gd_hip_linear_params) == 76, "the few-row kernel's arguments must stay within one 128-byte line");
#endif

/* kernel family that took a projection call */
#define GD_HIP_LINEAR_FAMILY_STREAM 1 /* few rows, MFMA fragments from global memory (linear_stream_kernel.h) */
#define GD_HIP_LINEAR_FAMILY_WIDE 2   /* few rows, whole-line weight stream through an LDS ring (linear_wide_kernel.h) */
#define GD_HIP_LINEAR_FAMILY_TILE 3   /* 128 rows and more, LDS-tiled MFMA kernel (linear_tile.hip) */
#define GD_HIP_LINEAR_FAMILY_SCALAR 4 /* unaligned operands */

/* destinations of the rope + append epilogue: q [M,H,D]; caches [M,Tmax,H,D]; positions I32 [M] */
typedef struct gd_hip_rope_epilogue {
    const int32_t *rope_pos, *cache_pos;
    void *q, *k_cache, *v_cache;
} gd_hip_rope_epilogue;

#endif
