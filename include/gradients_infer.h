/*
 * gradients_infer.h - host-side public API of the inference decode path: the subset of the
 * reference's public headers that its decoder (examples/gpt_lm/gpt_lm_shared.c:825-1246)
 * calls, with the same names, argument order, struct layouts and status behaviour, so that
 * model code written against the reference compiles against this library.
 *
 *   status codes ........ reference include/gradients/status.h
 *   context, arenas ..... reference include/gradients/memory.h
 *   tensor descriptors .. reference include/gradients/tensor.h
 *   transfers ........... reference include/gradients/transfer.h
 *   operators ........... reference include/gradients/ops.h, ops_generated.h (forward only)
 *
 * Arena model (unchanged): weights in `params`, K/V caches in `state`, activations in the
 * `scratch` ring slot of the current step, token ids / positions in the `data` ring slot.
 * Operators allocate their outputs in scratch, so they need an open step
 * (gd_begin_step .. gd_end_step).  Buffers are HBM: span.host_ptr is NULL and host access goes
 * through gd_tensor_write / gd_tensor_read.
 *
 * New entry points (no counterpart in the reference) are marked NEW.
 */
#ifndef GRADIENTS_INFER_H
#define GRADIENTS_INFER_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#include "gd_backend_hip.h" /* gd_status */

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default) /* the library is built with hidden visibility: only these are exported */

const char *gd_status_string(gd_status status); /* status.h:21 */

/* ---- memory.h ------------------------------------------------------------------- */

typedef struct gd_context gd_context;
typedef struct gd_batch gd_batch;

typedef enum gd_arena_kind { /* memory.h:18-23 */
    GD_ARENA_PARAMS = 0,
    GD_ARENA_STATE = 1,
    GD_ARENA_SCRATCH = 2,
    GD_ARENA_DATA = 3
} gd_arena_kind;

typedef enum gd_scope_mode { /* memory.h:25-30 */
    GD_SCOPE_NONE = 0,
    GD_SCOPE_TRAIN = 1,
    GD_SCOPE_EVAL = 2,
    GD_SCOPE_INFER = 3
} gd_scope_mode;

typedef struct gd_memory_config { /* memory.h:32-40 */
    size_t params_bytes;
    size_t state_bytes;
    size_t scratch_slot_bytes;
    size_t data_slot_bytes;
    uint32_t scratch_slots;
    uint32_t data_slots;
    size_t default_alignment;
} gd_memory_config;

typedef struct gd_span { /* memory.h:42-51 */
    gd_arena_kind arena;
    int32_t slot;
    size_t offset;
    size_t nbytes;
    size_t alignment;
    uint64_t generation;
    void *buffer;   /* gd_backend_buffer* */
    void *host_ptr; /* NULL: arenas live in HBM */
} gd_span;

typedef struct gd_arena_stats { /* memory.h:53-59 */
    size_t capacity;
    size_t offset;
    size_t watermark;
    uint64_t generation;
    bool sealed;
} gd_arena_stats;

typedef struct gd_ring_stats { /* memory.h:61-68 */
    uint32_t slots;
    int32_t current_slot;
    size_t total_capacity;
    size_t total_watermark;
    size_t max_slot_watermark;
    uint64_t waits;
} gd_ring_stats;

typedef struct gd_memory_stats { /* memory.h:70-77 */
    gd_arena_stats params;
    gd_arena_stats state;
    gd_ring_stats scratch;
    gd_ring_stats data;
    uint64_t backend_waits;
    uint64_t last_scope_fence;
} gd_memory_stats;

gd_memory_config gd_memory_config_default(void);                                   /* memory.h:85 */
gd_status gd_context_create(const gd_memory_config *config, gd_context **out_ctx); /* :87 */
void gd_context_destroy(gd_context *ctx);
gd_status gd_context_status(const gd_context *ctx); /* :90-92 */
const char *gd_context_error(const gd_context *ctx);
void gd_context_clear_error(gd_context *ctx);
gd_status gd_context_seal_params(gd_context *ctx); /* :94 */

/* :96-97.  The decode path passes gd_batch_empty() (reference src/dataset/batch.c:23-31). */
gd_status gd_begin_step(gd_context *ctx, gd_scope_mode mode, gd_batch *batch);
gd_status gd_end_step(gd_context *ctx);
gd_batch *gd_batch_empty(void);

gd_status gd_alloc_params(gd_context *ctx, size_t nbytes, size_t alignment, gd_span *out); /* :99-102 */
gd_status gd_alloc_state(gd_context *ctx, size_t nbytes, size_t alignment, gd_span *out);
gd_status gd_alloc_scratch(gd_context *ctx, size_t nbytes, size_t alignment, gd_span *out);
gd_status gd_alloc_data(gd_context *ctx, size_t nbytes, size_t alignment, gd_span *out);

gd_status gd_memory_stats_query(const gd_context *ctx, gd_memory_stats *out); /* :126 */
void gd_debug_complete_all(gd_context *ctx);                                  /* :128-136 */
uint64_t gd_debug_heap_alloc_count(void);
void gd_debug_set_heap_guard(bool forbid_heap_allocations);
int32_t gd_debug_current_ring_slot(const gd_context *ctx, gd_arena_kind arena);
uint64_t gd_debug_ring_slot_generation(const gd_context *ctx, gd_arena_kind arena, uint32_t slot);

/* NEW: the backend behind a context, for the gd_backend_* extensions (timers, graphs). */
gd_backend *gd_context_backend(gd_context *ctx);

/* ---- tensor.h -------------------------------------------------------------------- */

#define GD_MAX_DIMS 8U

typedef struct gd_shape { /* tensor.h:21-24 */
    uint32_t rank;
    int64_t dims[GD_MAX_DIMS];
} gd_shape;

static inline gd_shape gd_shape_make(uint32_t rank, const int64_t *dims) /* tensor.h:33-46 */
{
    gd_shape s;
    uint32_t i;
    s.rank = rank;
    for (i = 0U; i < GD_MAX_DIMS; ++i) s.dims[i] = (dims != NULL && i < rank) ? dims[i] : 0;
    return s;
}
#define GD_SCALAR_SHAPE (gd_shape_make(0U, NULL))

typedef enum gd_dtype { /* tensor.h:49-57 */
    GD_DTYPE_INVALID = 0,
    GD_DTYPE_F16 = 1,
    GD_DTYPE_BF16 = 2,
    GD_DTYPE_F32 = 3,
    GD_DTYPE_I32 = 4,
    GD_DTYPE_U8 = 5,
    GD_DTYPE_U16 = 6
} gd_dtype;

typedef enum gd_device { GD_DEVICE_INVALID = 0, GD_DEVICE_GPU = 1 } gd_device; /* :59-62 */
typedef enum gd_layout { GD_LAYOUT_STRIDED = 0 } gd_layout;                     /* :64-66 */

typedef struct gd_tensor { /* tensor.h:69-83 */
    uint64_t id;
    uint32_t version;
    gd_dtype dtype;
    gd_device device;
    gd_layout layout;
    uint32_t rank;
    int64_t shape[GD_MAX_DIMS];
    int64_t strides[GD_MAX_DIMS]; /* elements */
    gd_span storage;
    size_t view_offset; /* bytes */
    bool is_view;
    bool requires_grad;
    bool is_leaf;
} gd_tensor;

size_t gd_dtype_size(gd_dtype dtype); /* tensor.h:85-86 */
const char *gd_dtype_name(gd_dtype dtype);

gd_status gd_tensor_empty(gd_context *ctx, gd_arena_kind arena, gd_dtype dtype, gd_shape shape,
                          size_t alignment, gd_tensor *out); /* :88-93 */
gd_status gd_tensor_zeros(gd_context *ctx, gd_arena_kind arena, gd_dtype dtype, gd_shape shape,
                          size_t alignment, gd_tensor *out); /* :94-99 */
gd_status gd_tensor_ones(gd_context *ctx, gd_arena_kind arena, gd_dtype dtype, gd_shape shape,
                         size_t alignment, gd_tensor *out); /* :100-105 */
gd_status gd_tensor_slice(gd_context *ctx, const gd_tensor *base, uint32_t dim, int64_t start,
                          int64_t length, gd_tensor *out); /* :124-129 */
gd_status gd_tensor_zero_(gd_context *ctx, gd_tensor *tensor); /* :138 */
bool gd_tensor_is_contiguous(const gd_tensor *tensor);         /* :147-148 */
size_t gd_tensor_storage_offset(const gd_tensor *tensor);
gd_status gd_tensor_numel(const gd_tensor *tensor, int64_t *out_numel); /* :150-153 */
gd_status gd_tensor_logical_nbytes(const gd_tensor *tensor, size_t *out_nbytes);
gd_status gd_tensor_validate(gd_context *ctx, const gd_tensor *tensor);

/* ---- transfer.h -------------------------------------------------------------------- */

gd_status gd_synchronize(gd_context *ctx);                                                    /* :16 */
gd_status gd_tensor_write(gd_context *ctx, gd_tensor *dst, const void *src, size_t nbytes);   /* :33-36 */
gd_status gd_tensor_read(gd_context *ctx, const gd_tensor *src, void *dst, size_t nbytes);
gd_status gd_tensor_write_f32(gd_context *ctx, gd_tensor *dst, const float *src, size_t count);
gd_status gd_tensor_read_f32(gd_context *ctx, const gd_tensor *src, float *dst, size_t count);

/* ---- ops.h (forward, inference) ------------------------------------------------------- */

/* ops.h:29-43 */
gd_status gd_linear(gd_context *ctx, const gd_tensor *x, const gd_tensor *w, const gd_tensor *bias, gd_tensor *out);
gd_status gd_linear_transposed_weight(gd_context *ctx, const gd_tensor *x, const gd_tensor *w,
                                      const gd_tensor *bias, gd_tensor *out);
/* ops.h:208-223 */
gd_status gd_swiglu_split(gd_context *ctx, const gd_tensor *x12, gd_tensor *out);
gd_status gd_swiglu_split_linear(gd_context *ctx, const gd_tensor *x12, const gd_tensor *w,
                                 const gd_tensor *bias, gd_tensor *out);
/* ops.h:238-241, 253-257 */
gd_status gd_embedding(gd_context *ctx, const gd_tensor *table, const gd_tensor *ids, gd_tensor *out);
gd_status gd_rms_norm(gd_context *ctx, const gd_tensor *x, const gd_tensor *weight, float eps, gd_tensor *out);
/* ops.h:306-309; metadata only */
gd_status gd_reshape(gd_context *ctx, const gd_tensor *x, gd_shape shape, gd_tensor *out);
/* ops_generated.h:27-30 */
gd_status gd_add(gd_context *ctx, const gd_tensor *x, const gd_tensor *y, gd_tensor *out);

typedef struct gd_rope_config { /* ops.h:338-342 */
    float theta;
    int32_t n_dims;
    bool interleaved;
} gd_rope_config;
/* ops.h:362-370 */
gd_status gd_qkv_split_rope(gd_context *ctx, const gd_tensor *qkv, const gd_tensor *pos_ids, int32_t n_heads,
                            int32_t head_dim, const gd_rope_config *config, gd_tensor *q, gd_tensor *k,
                            gd_tensor *v);

typedef struct gd_sdpa_varlen_config { /* ops.h:431-437 */
    float scale;
    bool causal;
    int32_t sliding_window;
    int32_t prefix_len;
    int32_t max_seqlen;
} gd_sdpa_varlen_config;
/* ops.h:439-445 */
gd_status gd_sdpa_varlen(gd_context *ctx, const gd_tensor *q, const gd_tensor *k, const gd_tensor *v,
                         const gd_tensor *cu_seqlens, const gd_sdpa_varlen_config *config, gd_tensor *out);

/* MiniMax-M3 block picker + block-sparse attention over packed sequences (ops.h:383-413): index_q / index_k
 * [N,H,Dh] give topk_idx I32 [H,N,topk] (scratch); sparse_attention attends over the keys j <= i of the listed
 * blocks.  F16, Dh <= 64, block_size <= 128 (<= 0: 128), topk <= 16 (<= 0: 4), max_seqlen <= 0: N; a NULL
 * configuration means one forced first and one forced last block. */
typedef struct gd_minimax_m3_sparse_config { /* ops.h:390-397 */
    float scale;
    int32_t block_size;
    int32_t topk;
    int32_t init_blocks;
    int32_t local_blocks;
    int32_t max_seqlen;
} gd_minimax_m3_sparse_config;
gd_status gd_minimax_m3_index_topk(gd_context *ctx, const gd_tensor *index_q, const gd_tensor *index_k,
                                   const gd_tensor *cu_seqlens, const gd_minimax_m3_sparse_config *config,
                                   gd_tensor *topk_idx);
gd_status gd_minimax_m3_sparse_attention(gd_context *ctx, const gd_tensor *q, const gd_tensor *k, const gd_tensor *v,
                                         const gd_tensor *cu_seqlens, const gd_tensor *topk_idx,
                                         const gd_minimax_m3_sparse_config *config, gd_tensor *out);

typedef struct gd_sdpa_decode_config { /* ops.h:461-465 */
    float scale;
    int32_t sliding_window;
    int32_t prefix_len;
} gd_sdpa_decode_config;
/* ops.h:468-494 */
gd_status gd_sdpa_decode(gd_context *ctx, const gd_tensor *q, const gd_tensor *k_cache, const gd_tensor *v_cache,
                         const gd_tensor *cache_pos, const gd_sdpa_decode_config *config, gd_tensor *out);
gd_status gd_sdpa_decode_at(gd_context *ctx, const gd_tensor *q, const gd_tensor *k_cache,
                            const gd_tensor *v_cache, int32_t cache_pos, const gd_sdpa_decode_config *config,
                            gd_tensor *out);
gd_status gd_sdpa_decode_positions(gd_context *ctx, const gd_tensor *q, const gd_tensor *k_cache,
                                   const gd_tensor *v_cache, const gd_tensor *cache_pos,
                                   const gd_sdpa_decode_config *config, gd_tensor *out);
/* ops.h:499-522 */
gd_status gd_kv_cache_append_at(gd_context *ctx, gd_tensor *k_cache, gd_tensor *v_cache, int32_t cache_pos,
                                const gd_tensor *k_new, const gd_tensor *v_new);
gd_status gd_kv_cache_append_positions(gd_context *ctx, gd_tensor *k_cache, gd_tensor *v_cache,
                                       const gd_tensor *cache_pos, const gd_tensor *k_new,
                                       const gd_tensor *v_new);
gd_status gd_kv_cache_append_packed(gd_context *ctx, gd_tensor *k_cache, gd_tensor *v_cache,
                                    const gd_tensor *cache_pos, const gd_tensor *cu_seqlens,
                                    const gd_tensor *k_new, const gd_tensor *v_new);

/* NEW: greedy next token per logits row on the device (the reference scans on the host,
 * examples/gpt_lm/gpt_lm_shared.c:1388-1400).  logits [rows, V] F16/F32 -> ids I32 [rows] and,
 * when gap != NULL, F32 [rows] best-minus-runner-up. */
gd_status gd_argmax_rows(gd_context *ctx, const gd_tensor *logits, gd_tensor *ids, gd_tensor *gap);

/* NEW: out[i,:] = x[rows[i],:] for a rank-2 x and I32 rows; replaces per-sequence slice + concat
 * (examples/gpt_lm/gpt_lm_shared.c:1117-1169). */
gd_status gd_gather_rows(gd_context *ctx, const gd_tensor *x, const gd_tensor *rows, gd_tensor *out);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif

#endif /* GRADIENTS_INFER_H */
