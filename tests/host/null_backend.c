/*
 * TEST INFRASTRUCTURE ONLY: a backend without a device, so that the host core (arenas, ring slots and their
 * generations, tensor descriptors, transfers, operator front-end validation) can be tested on a machine with no
 * GPU.  Buffers are host memory, uploads and downloads are memcpy, fills are real; every operator entry point
 * computes NOTHING: it counts the call, remembers its name and returns GD_OK, so a front end's success path
 * (output allocation, shapes, version bumps) can be observed.  Lifecycle rules follow the HIP backend
 * (reference src/backends/metal/backend_metal.m:383-394, 541-544: a nested scope is GD_ERR_BAD_STATE).
 * Nothing under gradients.c_amd/ refers to this file; the product library never contains it.
 */
#include <stdbool.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/gd_backend_hip.h"

struct gd_backend {
    bool in_scope;
    uint64_t fences;
};

struct gd_backend_buffer {
    unsigned char *mem;
    size_t nbytes;
};

struct gd_backend_timer { int unused; };
struct gd_backend_graph { int unused; };

static uint64_t g_op_calls;
static const char *g_last_op = "";
static int g_ops_fail; /* when non-zero every operator returns this status instead of GD_OK */

int gd_null_backend_note(const char *name)
{
    g_op_calls += 1u;
    g_last_op = name;
    return g_ops_fail;
}

#pragma GCC visibility push(default)
uint64_t gd_null_backend_op_calls(void) { return g_op_calls; }
const char *gd_null_backend_last_op(void) { return g_last_op; }
void gd_null_backend_fail_ops(int status) { g_ops_fail = status; }

gd_status gd_backend_create_default(gd_backend **out)
{
    if (out == NULL) return GD_ERR_INVALID_ARGUMENT;
    *out = (gd_backend *)calloc(1, sizeof(gd_backend));
    return *out != NULL ? GD_OK : GD_ERR_OUT_OF_MEMORY;
}

void gd_backend_destroy(gd_backend *b) { free(b); }
gd_backend_kind gd_backend_kind_query(const gd_backend *b) { (void)b; return GD_BACKEND_HIP; }
const char *gd_backend_name(const gd_backend *b) { (void)b; return "null:host-memory"; }

gd_status gd_backend_buffer_create(gd_backend *b, size_t nbytes, gd_backend_buffer **out)
{
    gd_backend_buffer *buf;
    if (out != NULL) *out = NULL;
    if (b == NULL || out == NULL || nbytes == 0u) return GD_ERR_INVALID_ARGUMENT;
    buf = (gd_backend_buffer *)calloc(1, sizeof(*buf));
    if (buf == NULL) return GD_ERR_OUT_OF_MEMORY;
    buf->mem = (unsigned char *)malloc(nbytes);
    if (buf->mem == NULL) {
        free(buf);
        return GD_ERR_OUT_OF_MEMORY;
    }
    memset(buf->mem, 0xA5, nbytes); /* never-written memory is recognisable */
    buf->nbytes = nbytes;
    *out = buf;
    return GD_OK;
}

void gd_backend_buffer_destroy(gd_backend_buffer *buf)
{
    if (buf == NULL) return;
    free(buf->mem);
    free(buf);
}

size_t gd_backend_buffer_nbytes(const gd_backend_buffer *buf) { return buf != NULL ? buf->nbytes : 0u; }
void *gd_backend_buffer_host_ptr(gd_backend_buffer *buf) { (void)buf; return NULL; } /* like device memory */
bool gd_backend_buffer_is_host_visible(const gd_backend_buffer *buf) { (void)buf; return false; }
void *gd_backend_buffer_device_ptr(gd_backend_buffer *buf) { return buf != NULL ? buf->mem : NULL; }

gd_status gd_backend_scope_begin(gd_backend *b)
{
    if (b == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (b->in_scope) return GD_ERR_BAD_STATE;
    b->in_scope = true;
    return GD_OK;
}

gd_status gd_backend_flush(gd_backend *b) { return b != NULL ? GD_OK : GD_ERR_INVALID_ARGUMENT; }

gd_status gd_backend_record_fence(gd_backend *b, gd_backend_fence *out)
{
    if (b == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    b->in_scope = false;
    b->fences += 1u;
    out->handle = (void *)(uintptr_t)b->fences; /* already complete */
    return GD_OK;
}

bool gd_backend_fence_is_complete(gd_backend_fence *f) { (void)f; return true; }
gd_status gd_backend_fence_wait(gd_backend_fence *f) { (void)f; return GD_OK; }
void gd_backend_fence_destroy(gd_backend_fence *f) { if (f != NULL) f->handle = NULL; }

static bool range_ok(const gd_backend_buffer *buf, size_t offset, size_t nbytes)
{
    return buf != NULL && offset <= buf->nbytes && nbytes <= buf->nbytes - offset;
}

gd_status gd_backend_upload(gd_backend *b, gd_backend_buffer *buf, size_t offset, const void *src, size_t nbytes)
{
    if (b == NULL || (src == NULL && nbytes != 0u) || !range_ok(buf, offset, nbytes)) return GD_ERR_INVALID_ARGUMENT;
    if (nbytes != 0u) memcpy(buf->mem + offset, src, nbytes);
    return GD_OK;
}

gd_status gd_backend_download(gd_backend *b, gd_backend_buffer *buf, size_t offset, void *dst, size_t nbytes)
{
    if (b == NULL || (dst == NULL && nbytes != 0u) || !range_ok(buf, offset, nbytes)) return GD_ERR_INVALID_ARGUMENT;
    if (nbytes != 0u) memcpy(dst, buf->mem + offset, nbytes);
    return GD_OK;
}

gd_status gd_backend_fill(gd_backend *b, gd_backend_buffer *buf, size_t offset, size_t count, size_t elem_size,
                          uint32_t pattern)
{
    size_t i;
    if (b == NULL || buf == NULL || (elem_size != 1u && elem_size != 2u && elem_size != 4u) ||
        (offset % elem_size) != 0u || count > SIZE_MAX / elem_size || !range_ok(buf, offset, count * elem_size))
        return GD_ERR_INVALID_ARGUMENT;
    for (i = 0; i < count; ++i) memcpy(buf->mem + offset + i * elem_size, &pattern, elem_size); /* little endian */
    return GD_OK;
}

gd_status gd_backend_copy(gd_backend *b, gd_backend_buffer *dst, size_t dst_offset, gd_backend_buffer *src,
                          size_t src_offset, size_t nbytes)
{
    if (b == NULL || !range_ok(dst, dst_offset, nbytes) || !range_ok(src, src_offset, nbytes)) return GD_ERR_INVALID_ARGUMENT;
    memmove(dst->mem + dst_offset, src->mem + src_offset, nbytes);
    return GD_OK;
}

size_t gd_backend_sample_state_count(uint32_t rows) { return 8u + 10u * (size_t)rows; }
size_t gd_backend_sample_work_count(uint32_t rows, uint32_t cols)
{
    return (((size_t)rows * cols + 1u) & ~(size_t)1u) + 2u * (size_t)rows * (((size_t)cols + 2047u) / 2048u) * 258u;
}

gd_status gd_backend_device_info(const gd_backend *b, char *name, size_t name_bytes, int32_t *compute_units,
                                 uint64_t *global_mem)
{
    if (b == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (name != NULL && name_bytes > 0u) {
        strncpy(name, "null", name_bytes - 1u);
        name[name_bytes - 1u] = 0;
    }
    if (compute_units != NULL) *compute_units = 0;
    if (global_mem != NULL) *global_mem = 0u;
    return GD_OK;
}

gd_status gd_backend_set_tunable(gd_backend *b, const char *name, int64_t value)
{
    (void)b; (void)name; (void)value;
    return GD_ERR_UNSUPPORTED;
}

gd_status gd_backend_timer_create(gd_backend *b, gd_backend_timer **out)
{
    if (b == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    *out = (gd_backend_timer *)calloc(1, sizeof(gd_backend_timer));
    return *out != NULL ? GD_OK : GD_ERR_OUT_OF_MEMORY;
}
void gd_backend_timer_destroy(gd_backend_timer *t) { free(t); }
gd_status gd_backend_timer_start(gd_backend_timer *t) { (void)t; return GD_OK; }
gd_status gd_backend_timer_stop(gd_backend_timer *t) { (void)t; return GD_OK; }
gd_status gd_backend_timer_elapsed_ms(gd_backend_timer *t, float *ms)
{
    (void)t;
    if (ms != NULL) *ms = 0.0f;
    return GD_OK;
}

/* Graphs that record nothing: capture and replay succeed and are counted, so that the host logic of the resident
 * sessions (step accounting, the order of calls, what a session refuses) runs without a device. */
static int g_capturing;
static uint64_t g_graph_launches;
uint64_t gd_null_backend_graph_launches(void) { return g_graph_launches; }
gd_status gd_backend_graph_begin_capture(gd_backend *b)
{
    if (b == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (g_capturing) return GD_ERR_BAD_STATE;
    g_capturing = 1;
    return GD_OK;
}
gd_status gd_backend_graph_end_capture(gd_backend *b, gd_backend_graph **out)
{
    if (b == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (!g_capturing) return GD_ERR_BAD_STATE;
    g_capturing = 0;
    *out = (gd_backend_graph *)calloc(1, sizeof(gd_backend_graph));
    return *out != NULL ? GD_OK : GD_ERR_OUT_OF_MEMORY;
}
gd_status gd_backend_graph_launch(gd_backend *b, gd_backend_graph *g)
{
    if (b == NULL || g == NULL) return GD_ERR_INVALID_ARGUMENT;
    ++g_graph_launches;
    return GD_OK;
}
void gd_backend_graph_destroy(gd_backend_graph *g) { free(g); }
#pragma GCC visibility pop
