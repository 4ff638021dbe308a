/*
 * Internals of the host core: context, arenas, ring slots, error latch and the helpers the
 * operator front ends share (span checks, tensor -> backend view conversion).
 */
#ifndef GD_CORE_INTERNAL_H
#define GD_CORE_INTERNAL_H

#include <limits.h>
#include <string.h>

#include "gradients_infer.h"

#define GD_DEFAULT_ALIGNMENT 256U
#define GD_MAX_RING_SLOTS 16U
#define GD_MAX_SUBALLOC_ALIGNMENT 4096U

typedef struct gd_arena {
    gd_backend_buffer *buffer;
    gd_arena_kind kind;
    int32_t slot;
    size_t capacity, offset, watermark, alignment;
    uint64_t generation;
    bool sealed;
    /* ring slots only */
    gd_backend_fence fence;
    bool fence_pending;
    size_t last_alloc_offset, last_alloc_end; /* top allocation, for gd_context_release_scratch */
} gd_arena;

typedef struct gd_ring {
    gd_arena slots[GD_MAX_RING_SLOTS];
    uint32_t count;
    int32_t current;
    uint64_t waits;
} gd_ring;

struct gd_context {
    gd_backend *backend;
    gd_arena params, state;
    gd_ring scratch, data;
    gd_scope_mode mode;
    bool in_scope;
    uint64_t next_tensor_id;
    uint64_t scope_count;
    gd_status status;
    char error[160];
    /* F32 <-> F16 conversion staging of gd_tensor_write_f32 / read_f32, allocated with the context so that
     * transfers inside a step need no heap */
    uint16_t *pack;
    size_t pack_count;
};

/* reference src/core/memory.c:126-134: latch status + message, return the status */
gd_status gd_context_set_error(gd_context *ctx, gd_status status, const char *message);
gd_status gd_context_validate_span(gd_context *ctx, const gd_span *span, const char *message);
gd_status gd_context_alloc_span(gd_context *ctx, gd_arena_kind arena, size_t nbytes, size_t alignment, gd_span *out);
/* returns the span to its scratch slot when it is the most recent allocation (inference frees the
 * swiglu activation right after its consumer is enqueued, reference core_swiglu_split_linear.c:273-278) */
void gd_context_release_scratch(gd_context *ctx, const gd_span *span);
bool gd_context_in_scope(const gd_context *ctx);
gd_scope_mode gd_context_scope_mode(const gd_context *ctx);
uint64_t gd_context_next_tensor_id(gd_context *ctx);

/* tensor helpers (tensor.c) */
void gd_tensor_set_contiguous_strides(gd_tensor *t);
gd_status gd_tensor_alloc_like_shape(gd_context *ctx, gd_dtype dtype, uint32_t rank, const int64_t *shape,
                                     gd_tensor *out); /* scratch, default alignment, is_leaf=false */
bool gd_op_tensor_view(const gd_tensor *t, gd_backend_tensor_view *out);   /* contiguous tensors */
bool gd_op_matrix_view(const gd_tensor *t, gd_backend_matrix_view *out);   /* rank 2, last stride 1 */
bool gd_op_vector_view(const gd_tensor *t, gd_backend_vector_view *out);   /* rank 1 contiguous */
/* rank >= 1 tensor seen as [rows, last]: rank-2 tensors may be row-strided, others must be contiguous */
bool gd_op_rows_matrix_view(const gd_tensor *t, gd_backend_matrix_view *out);

uint16_t gd_f32_to_f16_bits(float value);
float gd_f16_bits_to_f32(uint16_t bits);

#endif
