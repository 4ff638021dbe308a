#ifndef GD_HIP_SDPA_DECODE_TYPES_H
#define GD_HIP_SDPA_DECODE_TYPES_H
#include <stdint.h>

#define GD_HIP_SDPA_POS_SCALAR 0u  /* params.cache_pos */
#define GD_HIP_SDPA_POS_TENSOR0 1u /* pos[0] for every batch row */
#define GD_HIP_SDPA_POS_VECTOR 2u  /* pos[b] */

/* size of the fixed device array behind gd_backend_sdpa_decode_positions_noalloc
 * (= GD_BACKEND_SDPA_DECODE_NOALLOC_SCRATCH_BYTES of the public header) */
#define GD_HIP_SDPA_NOALLOC_SCRATCH_BYTES (8u << 20)
#define GD_HIP_SDPA_MAX_DEVICES 16
/* The split-KV workspace starts with one arrival counter per (batch row, kv head) (zero between launches: the
 * piece that merges a row puts its counter back), the partial results follow.  A row is cut into at most
 * GD_HIP_SDPA_MAX_PIECES pieces when the last piece to arrive merges them inside the kernel. */
#define GD_HIP_SDPA_COUNTER_SLOTS 16384u
#define GD_HIP_SDPA_MAX_PIECES 16u
/* rows the PIECES form handles: every lane keeps the positions of its rows in registers */
#define GD_HIP_SDPA_PIECES_MAX_BATCH 256

typedef struct gd_hip_sdpa_decode_params {
    uint32_t batch, tq, tmax, hq, hkv, dh;
    uint32_t window, prefix_len;
    uint32_t pos_mode;
    int32_t cache_pos;
    float scale;
    uint32_t chunk;  /* keys per workgroup (split-KV kernel) */
    uint32_t nsplit; /* workgroups per (batch, kv head) */
    uint32_t dtype;  /* GD_BACKEND_DTYPE_F16 or _F32 (generic kernel) */
    uint32_t waves;  /* wavefronts per workgroup of the split-KV kernel: 4 or 8 */
    uint32_t unroll; /* key-row loads in flight per lane: 4 or 8 */
    uint32_t nontemporal; /* 1: K/V loads carry the streaming hint */
    uint32_t even_pieces; /* PIECES form: parts a row is cut into when all rows are about one length; 0: always at chunk */
} gd_hip_sdpa_decode_params;

#endif
