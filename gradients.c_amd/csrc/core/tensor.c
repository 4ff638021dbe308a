/*
 * Tensor descriptors of the host core: allocation, validation, slices, and the conversion
 * of descriptors into the views the backend boundary takes.
 *
 * Contract restated from the reference's src/core/tensor.c (empty :452-500, validate :298-322,
 * slice :576-627) and src/ops/op_common.h:23-115 (view builders): descriptors are caller-owned
 * metadata, bytes live in arena spans; a tensor is valid while its span is live; slices share
 * storage and carry a byte view_offset; views handed to the backend are contiguous (tensors) or
 * row-strided with unit column stride (matrices).
 */
#include "core_internal.h"

size_t gd_dtype_size(gd_dtype dtype)
{
    switch (dtype) {
    case GD_DTYPE_F16: case GD_DTYPE_BF16: case GD_DTYPE_U16: return 2U;
    case GD_DTYPE_F32: case GD_DTYPE_I32: return 4U;
    case GD_DTYPE_U8: return 1U;
    default: return 0U;
    }
}

const char *gd_dtype_name(gd_dtype dtype)
{
    switch (dtype) {
    case GD_DTYPE_F16: return "f16";
    case GD_DTYPE_BF16: return "bf16";
    case GD_DTYPE_F32: return "f32";
    case GD_DTYPE_I32: return "i32";
    case GD_DTYPE_U8: return "u8";
    case GD_DTYPE_U16: return "u16";
    default: return "invalid";
    }
}

void gd_tensor_set_contiguous_strides(gd_tensor *t)
{
    int64_t stride = 1;
    uint32_t i;
    for (i = t->rank; i > 0U; --i) {
        t->strides[i - 1U] = stride;
        stride *= t->shape[i - 1U];
    }
}

gd_status gd_tensor_numel(const gd_tensor *t, int64_t *out)
{
    int64_t n = 1;
    uint32_t i;
    if (t == NULL || out == NULL || t->rank > GD_MAX_DIMS) return GD_ERR_INVALID_ARGUMENT;
    for (i = 0U; i < t->rank; ++i) {
        if (t->shape[i] <= 0) return GD_ERR_INVALID_ARGUMENT;
        if (n > INT64_MAX / t->shape[i]) return GD_ERR_OUT_OF_MEMORY;
        n *= t->shape[i];
    }
    *out = n;
    return GD_OK;
}

gd_status gd_tensor_logical_nbytes(const gd_tensor *t, size_t *out)
{
    int64_t n;
    size_t es;
    gd_status st = gd_tensor_numel(t, &n);
    if (st != GD_OK) return st;
    if (out == NULL) return GD_ERR_INVALID_ARGUMENT;
    es = gd_dtype_size(t->dtype);
    if (es == 0U) return GD_ERR_INVALID_ARGUMENT;
    if ((uint64_t)n > (uint64_t)(SIZE_MAX / es)) return GD_ERR_OUT_OF_MEMORY;
    *out = (size_t)n * es;
    return GD_OK;
}

bool gd_tensor_is_contiguous(const gd_tensor *t)
{
    int64_t stride = 1;
    uint32_t i;
    if (t == NULL || t->rank > GD_MAX_DIMS) return false;
    for (i = t->rank; i > 0U; --i) {
        if (t->shape[i - 1U] <= 0) return false;
        if (t->shape[i - 1U] != 1 && t->strides[i - 1U] != stride) return false;
        stride *= t->shape[i - 1U];
    }
    return true;
}

size_t gd_tensor_storage_offset(const gd_tensor *t) { return t != NULL ? t->storage.offset + t->view_offset : 0U; }

/* bytes from view_offset to one past the last addressed element */
static gd_status logical_span(const gd_tensor *t, size_t *out)
{
    uint64_t last = 0U;
    size_t es = gd_dtype_size(t->dtype);
    uint32_t i;
    for (i = 0U; i < t->rank; ++i) {
        if (t->shape[i] <= 0 || t->strides[i] < 0) return GD_ERR_INVALID_ARGUMENT;
        if (t->strides[i] != 0 && (uint64_t)(t->shape[i] - 1) > (UINT64_MAX / 4U) / (uint64_t)t->strides[i])
            return GD_ERR_OUT_OF_MEMORY;
        last += (uint64_t)(t->shape[i] - 1) * (uint64_t)t->strides[i];
        if (last > UINT64_MAX / 8U) return GD_ERR_OUT_OF_MEMORY;
    }
    *out = t->view_offset + (size_t)(last + 1U) * es;
    return GD_OK;
}

gd_status gd_tensor_validate(gd_context *ctx, const gd_tensor *t)
{
    size_t span;
    gd_status st;
    if (ctx == NULL || t == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (t->device != GD_DEVICE_GPU || t->layout != GD_LAYOUT_STRIDED || t->rank > GD_MAX_DIMS ||
        gd_dtype_size(t->dtype) == 0U)
        return gd_context_set_error(ctx, GD_ERR_INVALID_ARGUMENT, "invalid tensor descriptor");
    st = gd_context_validate_span(ctx, &t->storage, "tensor storage is stale");
    if (st != GD_OK) return st;
    st = logical_span(t, &span);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "invalid tensor shape or strides");
    if (span > t->storage.nbytes)
        return gd_context_set_error(ctx, GD_ERR_BAD_STATE, "tensor logical span exceeds allocation");
    return GD_OK;
}

gd_status gd_tensor_empty(gd_context *ctx, gd_arena_kind arena, gd_dtype dtype, gd_shape shape, size_t alignment,
                          gd_tensor *out)
{
    gd_tensor t;
    size_t nbytes;
    gd_status st;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    memset(&t, 0, sizeof(t));
    t.dtype = dtype;
    t.device = GD_DEVICE_GPU;
    t.layout = GD_LAYOUT_STRIDED;
    t.rank = shape.rank;
    if (shape.rank > GD_MAX_DIMS) return gd_context_set_error(ctx, GD_ERR_INVALID_ARGUMENT, "invalid tensor allocation shape");
    if (shape.rank > 0U) memcpy(t.shape, shape.dims, (size_t)shape.rank * sizeof(t.shape[0]));
    st = gd_tensor_logical_nbytes(&t, &nbytes);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "invalid tensor allocation shape");
    gd_tensor_set_contiguous_strides(&t);
    t.id = gd_context_next_tensor_id(ctx);
    st = gd_context_alloc_span(ctx, arena, nbytes, alignment, &t.storage);
    if (st != GD_OK) return st;
    t.is_leaf = true;
    *out = t;
    return GD_OK;
}

gd_status gd_tensor_alloc_like_shape(gd_context *ctx, gd_dtype dtype, uint32_t rank, const int64_t *shape, gd_tensor *out)
{
    gd_status st = gd_tensor_empty(ctx, GD_ARENA_SCRATCH, dtype, gd_shape_make(rank, shape), 256U, out);
    if (st == GD_OK) out->is_leaf = false;
    return st;
}

static gd_status fill_tensor(gd_context *ctx, gd_tensor *t, bool one)
{
    size_t es, count;
    uint32_t pattern = 0U;
    int64_t n;
    gd_status st = gd_tensor_validate(ctx, t);
    if (st != GD_OK) return st;
    if (!gd_tensor_is_contiguous(t)) return gd_context_set_error(ctx, GD_ERR_UNSUPPORTED, "fill requires contiguous tensor");
    st = gd_tensor_numel(t, &n);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "invalid tensor shape");
    es = gd_dtype_size(t->dtype);
    count = (size_t)n;
    if (one) {
        switch (t->dtype) {
        case GD_DTYPE_F16: pattern = 0x3c00U; break;
        case GD_DTYPE_BF16: pattern = 0x3f80U; break;
        case GD_DTYPE_F32: pattern = 0x3f800000U; break;
        default: pattern = 1U; break;
        }
    }
    st = gd_backend_fill(gd_context_backend(ctx), (gd_backend_buffer *)t->storage.buffer,
                         t->storage.offset + t->view_offset, count, es, pattern);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "backend fill failed");
    t->version += 1U;
    if (t->version == 0U) t->version = 1U;
    return GD_OK;
}

gd_status gd_tensor_zero_(gd_context *ctx, gd_tensor *t)
{
    if (ctx == NULL || t == NULL) return GD_ERR_INVALID_ARGUMENT;
    return fill_tensor(ctx, t, false);
}

static gd_status filled(gd_context *ctx, gd_arena_kind arena, gd_dtype dtype, gd_shape shape, size_t alignment,
                        gd_tensor *out, bool one)
{
    gd_tensor t;
    gd_status st;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    st = gd_tensor_empty(ctx, arena, dtype, shape, alignment, &t);
    if (st != GD_OK) return st;
    st = fill_tensor(ctx, &t, one);
    if (st != GD_OK) return st;
    *out = t;
    return GD_OK;
}

gd_status gd_tensor_zeros(gd_context *ctx, gd_arena_kind arena, gd_dtype dtype, gd_shape shape, size_t alignment, gd_tensor *out)
{
    return filled(ctx, arena, dtype, shape, alignment, out, false);
}

gd_status gd_tensor_ones(gd_context *ctx, gd_arena_kind arena, gd_dtype dtype, gd_shape shape, size_t alignment, gd_tensor *out)
{
    return filled(ctx, arena, dtype, shape, alignment, out, true);
}

gd_status gd_tensor_slice(gd_context *ctx, const gd_tensor *base, uint32_t dim, int64_t start, int64_t length,
                          gd_tensor *out)
{
    gd_tensor view;
    gd_status st;
    size_t es, delta;
    if (out != NULL) memset(out, 0, sizeof(*out));
    if (ctx == NULL || base == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    st = gd_tensor_validate(ctx, base);
    if (st != GD_OK) return st;
    if (dim >= base->rank || start < 0 || length <= 0 || start > base->shape[dim] || length > base->shape[dim] - start)
        return gd_context_set_error(ctx, GD_ERR_INVALID_ARGUMENT, "invalid tensor slice range");
    es = gd_dtype_size(base->dtype);
    if (base->strides[dim] != 0 && (uint64_t)start > (uint64_t)(SIZE_MAX / es) / (uint64_t)base->strides[dim])
        return gd_context_set_error(ctx, GD_ERR_OUT_OF_MEMORY, "tensor slice offset overflow");
    delta = (size_t)start * (size_t)base->strides[dim] * es;
    view = *base;
    view.id = gd_context_next_tensor_id(ctx);
    view.version = 0U;
    view.shape[dim] = length;
    view.view_offset = base->view_offset + delta;
    view.is_view = true;
    view.is_leaf = false;
    st = gd_tensor_validate(ctx, &view);
    if (st != GD_OK) return st;
    *out = view;
    return GD_OK;
}

/* ---- descriptors -> backend views ----------------------------------------------------- */

bool gd_op_tensor_view(const gd_tensor *t, gd_backend_tensor_view *out)
{
    int64_t n;
    uint32_t i;
    if (t == NULL || out == NULL || !gd_tensor_is_contiguous(t) || gd_tensor_numel(t, &n) != GD_OK) return false;
    memset(out, 0, sizeof(*out));
    out->buffer = (gd_backend_buffer *)t->storage.buffer;
    out->offset = t->storage.offset + t->view_offset;
    out->count = (size_t)n;
    out->dtype = (uint32_t)t->dtype;
    out->rank = t->rank;
    for (i = 0U; i < t->rank; ++i) out->shape[i] = t->shape[i];
    { /* canonical row-major strides (size-1 dims may carry anything in the descriptor) */
        int64_t stride = 1;
        for (i = t->rank; i > 0U; --i) {
            out->strides[i - 1U] = stride;
            stride *= t->shape[i - 1U];
        }
    }
    return out->buffer != NULL;
}

bool gd_op_matrix_view(const gd_tensor *t, gd_backend_matrix_view *out)
{
    size_t es;
    if (t == NULL || out == NULL || t->rank != 2U || t->strides[1] != 1 || t->strides[0] <= 0) return false;
    es = gd_dtype_size(t->dtype);
    if (es == 0U || t->shape[0] <= 0 || t->shape[1] <= 0 || t->shape[0] > (int64_t)UINT32_MAX ||
        t->shape[1] > (int64_t)UINT32_MAX || t->strides[0] < t->shape[1])
        return false;
    out->buffer = (gd_backend_buffer *)t->storage.buffer;
    out->offset = t->storage.offset + t->view_offset;
    out->rows = (uint32_t)t->shape[0];
    out->cols = (uint32_t)t->shape[1];
    out->row_bytes = (size_t)t->strides[0] * es;
    out->dtype = (uint32_t)t->dtype;
    return out->buffer != NULL;
}

bool gd_op_rows_matrix_view(const gd_tensor *t, gd_backend_matrix_view *out)
{
    int64_t n, cols;
    if (t == NULL || out == NULL || t->rank == 0U) return false;
    if (t->rank == 2U) return gd_op_matrix_view(t, out);
    if (!gd_tensor_is_contiguous(t) || gd_tensor_numel(t, &n) != GD_OK) return false;
    cols = t->shape[t->rank - 1U];
    if (n / cols > (int64_t)UINT32_MAX || cols > (int64_t)UINT32_MAX) return false;
    out->buffer = (gd_backend_buffer *)t->storage.buffer;
    out->offset = t->storage.offset + t->view_offset;
    out->rows = (uint32_t)(n / cols);
    out->cols = (uint32_t)cols;
    out->row_bytes = (size_t)cols * gd_dtype_size(t->dtype);
    out->dtype = (uint32_t)t->dtype;
    return out->buffer != NULL;
}

bool gd_op_vector_view(const gd_tensor *t, gd_backend_vector_view *out)
{
    if (t == NULL || out == NULL || t->rank != 1U || !gd_tensor_is_contiguous(t) || t->shape[0] > (int64_t)UINT32_MAX)
        return false;
    out->buffer = (gd_backend_buffer *)t->storage.buffer;
    out->offset = t->storage.offset + t->view_offset;
    out->length = (uint32_t)t->shape[0];
    out->dtype = (uint32_t)t->dtype;
    return out->buffer != NULL;
}
