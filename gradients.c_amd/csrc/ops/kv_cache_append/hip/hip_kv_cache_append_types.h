#ifndef GD_HIP_KV_CACHE_APPEND_TYPES_H
#define GD_HIP_KV_CACHE_APPEND_TYPES_H
#include <stdint.h>

/* Kernel parameters (passed by value). */
typedef struct gd_hip_kv_append_params {
    uint64_t total_units; /* host passes total source BYTES; the launcher divides by the unit */
    uint64_t row_bytes;   /* Hkv * Dh * elem */
    uint64_t tnew;        /* rows per batch entry (batched form) */
    uint64_t tmax;
    uint64_t batch;
    int32_t cache_pos;    /* scalar position (batched form without a position vector) */
    uint32_t copy_unit;   /* 16, 4 or 1 */
} gd_hip_kv_append_params;

#endif
