/*
 * Context, arenas and the step scope of the host core.
 *
 * Restates the contract of the reference's src/core/memory.c for the inference path:
 *   - four arenas backed by one backend buffer each (memory.c:965-1039): params (bump, can be
 *     sealed -> GD_ERR_FROZEN), state (bump), scratch and data rings of N slots;
 *   - gd_begin_step picks the next ring slots, waits on a slot's fence if the GPU still uses it,
 *     bumps the slot generation so tensors of the old step become stale (memory.c:701-735,
 *     1350-1421); gd_end_step records the fence that guards both slots (memory.c:1423-1474);
 *   - scratch/data allocation outside a step is GD_ERR_BAD_STATE (memory.c:936-946); a failed
 *     allocation clears the span (nbytes 0, buffer NULL, slot -1) and does not move the offset;
 *   - the context latches the last error and a 160-character message (memory.c:126-134);
 *   - heap allocations made by the core are counted and can be forbidden
 *     (gd_debug_set_heap_guard, memory.c:187-198): nothing allocates inside a step.
 * Buffers are HBM, so spans carry host_ptr == NULL and liveness is judged from arena, slot,
 * generation, buffer and range only.
 */
#include <stdio.h>
#include <stdlib.h>

#include "core_internal.h"

static uint64_t g_heap_allocs;
static bool g_heap_forbidden;
static gd_batch *const g_empty_batch = (gd_batch *)(uintptr_t)1;

static void *heap_alloc(size_t nbytes)
{
    void *p;
    if (g_heap_forbidden || nbytes == 0U) return NULL;
    p = calloc(1U, nbytes);
    if (p != NULL) g_heap_allocs += 1U;
    return p;
}

uint64_t gd_debug_heap_alloc_count(void) { return g_heap_allocs; }
void gd_debug_set_heap_guard(bool forbid) { g_heap_forbidden = forbid; }
gd_batch *gd_batch_empty(void) { return g_empty_batch; }

const char *gd_status_string(gd_status status)
{
    switch (status) {
    case GD_OK: return "ok";
    case GD_ERR_INVALID_ARGUMENT: return "invalid argument";
    case GD_ERR_OUT_OF_MEMORY: return "out of memory";
    case GD_ERR_FROZEN: return "frozen";
    case GD_ERR_BUSY: return "busy";
    case GD_ERR_BAD_STATE: return "bad state";
    case GD_ERR_UNSUPPORTED: return "unsupported";
    case GD_ERR_INTERNAL: return "internal error";
    case GD_ERR_NOT_IMPLEMENTED: return "not implemented";
    case GD_ERR_IO: return "io error";
    default: return "unknown status";
    }
}

gd_status gd_context_set_error(gd_context *ctx, gd_status status, const char *message)
{
    if (ctx != NULL) {
        ctx->status = status;
        snprintf(ctx->error, sizeof(ctx->error), "%s", message != NULL ? message : gd_status_string(status));
    }
    return status;
}

gd_status gd_context_status(const gd_context *ctx) { return ctx != NULL ? ctx->status : GD_ERR_INVALID_ARGUMENT; }
const char *gd_context_error(const gd_context *ctx) { return ctx != NULL ? ctx->error : "null context"; }
void gd_context_clear_error(gd_context *ctx)
{
    if (ctx != NULL) {
        ctx->status = GD_OK;
        ctx->error[0] = '\0';
    }
}
gd_backend *gd_context_backend(gd_context *ctx) { return ctx != NULL ? ctx->backend : NULL; }
bool gd_context_in_scope(const gd_context *ctx) { return ctx != NULL && ctx->in_scope; }
gd_scope_mode gd_context_scope_mode(const gd_context *ctx) { return ctx != NULL ? ctx->mode : GD_SCOPE_NONE; }
uint64_t gd_context_next_tensor_id(gd_context *ctx) { return ctx->next_tensor_id++; }

static bool is_pow2(size_t v) { return v != 0U && (v & (v - 1U)) == 0U; }

gd_memory_config gd_memory_config_default(void)
{
    gd_memory_config c;
    c.params_bytes = 128U * 1024U * 1024U;
    c.state_bytes = 64U * 1024U * 1024U;
    c.scratch_slot_bytes = 64U * 1024U * 1024U;
    c.data_slot_bytes = 8U * 1024U * 1024U;
    c.scratch_slots = 3U;
    c.data_slots = 3U;
    c.default_alignment = GD_DEFAULT_ALIGNMENT;
    return c;
}

static gd_status arena_init(gd_backend *backend, gd_arena *a, gd_arena_kind kind, int32_t slot, size_t capacity,
                            size_t alignment)
{
    memset(a, 0, sizeof(*a));
    a->kind = kind;
    a->slot = slot;
    a->capacity = capacity;
    a->alignment = alignment;
    a->generation = 1U;
    return gd_backend_buffer_create(backend, capacity, &a->buffer);
}

static void arena_destroy(gd_arena *a)
{
    if (a->fence_pending) {
        (void)gd_backend_fence_wait(&a->fence);
        gd_backend_fence_destroy(&a->fence);
        a->fence_pending = false;
    }
    if (a->buffer != NULL) gd_backend_buffer_destroy(a->buffer);
    a->buffer = NULL;
}

gd_status gd_context_create(const gd_memory_config *config, gd_context **out_ctx)
{
    gd_memory_config cfg;
    gd_context *ctx;
    gd_backend *backend = NULL;
    gd_status st;
    size_t align;
    uint32_t i;
    if (out_ctx == NULL) return GD_ERR_INVALID_ARGUMENT;
    *out_ctx = NULL;
    cfg = config != NULL ? *config : gd_memory_config_default();
    align = cfg.default_alignment == 0U ? GD_DEFAULT_ALIGNMENT : cfg.default_alignment;
    if (cfg.params_bytes == 0U || cfg.state_bytes == 0U || cfg.scratch_slot_bytes == 0U ||
        cfg.data_slot_bytes == 0U || cfg.scratch_slots == 0U || cfg.data_slots == 0U ||
        cfg.scratch_slots > GD_MAX_RING_SLOTS || cfg.data_slots > GD_MAX_RING_SLOTS || !is_pow2(align) ||
        align > GD_MAX_SUBALLOC_ALIGNMENT)
        return GD_ERR_INVALID_ARGUMENT;
    st = gd_backend_create_default(&backend);
    if (st != GD_OK) return st; /* GD_ERR_UNSUPPORTED without a device: callers skip */
    ctx = (gd_context *)heap_alloc(sizeof(*ctx));
    if (ctx == NULL) {
        gd_backend_destroy(backend);
        return GD_ERR_OUT_OF_MEMORY;
    }
    ctx->backend = backend;
    ctx->scratch.current = -1;
    ctx->data.current = -1;
    ctx->next_tensor_id = 1U;
    st = arena_init(backend, &ctx->params, GD_ARENA_PARAMS, -1, cfg.params_bytes, align);
    if (st == GD_OK) st = arena_init(backend, &ctx->state, GD_ARENA_STATE, -1, cfg.state_bytes, align);
    for (i = 0U; st == GD_OK && i < cfg.scratch_slots; ++i) {
        st = arena_init(backend, &ctx->scratch.slots[i], GD_ARENA_SCRATCH, (int32_t)i, cfg.scratch_slot_bytes, align);
        if (st == GD_OK) ctx->scratch.count = i + 1U;
    }
    for (i = 0U; st == GD_OK && i < cfg.data_slots; ++i) {
        st = arena_init(backend, &ctx->data.slots[i], GD_ARENA_DATA, (int32_t)i, cfg.data_slot_bytes, align);
        if (st == GD_OK) ctx->data.count = i + 1U;
    }
    if (st == GD_OK) {
        ctx->pack_count = (size_t)1U << 21; /* 4 MiB per transfer call */
        ctx->pack = (uint16_t *)heap_alloc(ctx->pack_count * sizeof(uint16_t));
        if (ctx->pack == NULL) st = GD_ERR_OUT_OF_MEMORY;
    }
    if (st != GD_OK) {
        gd_context_destroy(ctx);
        return st;
    }
    *out_ctx = ctx;
    return GD_OK;
}

void gd_context_destroy(gd_context *ctx)
{
    uint32_t i;
    if (ctx == NULL) return;
    if (ctx->backend != NULL) (void)gd_backend_flush(ctx->backend);
    arena_destroy(&ctx->params);
    arena_destroy(&ctx->state);
    for (i = 0U; i < GD_MAX_RING_SLOTS; ++i) {
        arena_destroy(&ctx->scratch.slots[i]);
        arena_destroy(&ctx->data.slots[i]);
    }
    if (ctx->backend != NULL) gd_backend_destroy(ctx->backend);
    free(ctx->pack);
    free(ctx);
}

gd_status gd_context_seal_params(gd_context *ctx)
{
    if (ctx == NULL) return GD_ERR_INVALID_ARGUMENT;
    ctx->params.sealed = true;
    return GD_OK;
}

/* ---- allocation ------------------------------------------------------------------- */

static void span_clear(gd_span *s)
{
    memset(s, 0, sizeof(*s));
    s->slot = -1;
}

static gd_status arena_alloc(gd_context *ctx, gd_arena *a, size_t nbytes, size_t alignment, gd_span *out)
{
    size_t start;
    if (alignment == 0U) alignment = a->alignment;
    if (nbytes == 0U || !is_pow2(alignment) || alignment > GD_MAX_SUBALLOC_ALIGNMENT)
        return gd_context_set_error(ctx, GD_ERR_INVALID_ARGUMENT, "invalid allocation size or alignment");
    if (a->sealed) return gd_context_set_error(ctx, GD_ERR_FROZEN, "arena is sealed");
    if (a->offset > SIZE_MAX - (alignment - 1U)) return gd_context_set_error(ctx, GD_ERR_OUT_OF_MEMORY, "arena offset overflow");
    start = (a->offset + alignment - 1U) & ~(alignment - 1U);
    if (start > a->capacity || nbytes > a->capacity - start)
        return gd_context_set_error(ctx, GD_ERR_OUT_OF_MEMORY, "arena out of memory");
    out->arena = a->kind;
    out->slot = a->slot;
    out->offset = start;
    out->nbytes = nbytes;
    out->alignment = alignment;
    out->generation = a->generation;
    out->buffer = a->buffer;
    out->host_ptr = NULL;
    a->last_alloc_offset = a->offset;
    a->offset = start + nbytes;
    a->last_alloc_end = a->offset;
    if (a->offset > a->watermark) a->watermark = a->offset;
    return GD_OK;
}

static gd_arena *ring_current(gd_ring *r)
{
    return (r->current >= 0 && (uint32_t)r->current < r->count) ? &r->slots[r->current] : NULL;
}

gd_status gd_context_alloc_span(gd_context *ctx, gd_arena_kind arena, size_t nbytes, size_t alignment, gd_span *out)
{
    gd_arena *a;
    if (out != NULL) span_clear(out);
    if (ctx == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    switch (arena) {
    case GD_ARENA_PARAMS: a = &ctx->params; break;
    case GD_ARENA_STATE: a = &ctx->state; break;
    case GD_ARENA_SCRATCH:
    case GD_ARENA_DATA:
        if (!ctx->in_scope)
            return gd_context_set_error(ctx, GD_ERR_BAD_STATE,
                                        arena == GD_ARENA_SCRATCH ? "scratch allocation outside a step scope"
                                                                  : "data allocation outside a step scope");
        a = ring_current(arena == GD_ARENA_SCRATCH ? &ctx->scratch : &ctx->data);
        if (a == NULL) return gd_context_set_error(ctx, GD_ERR_BAD_STATE, "ring has no current slot");
        break;
    default: return gd_context_set_error(ctx, GD_ERR_INVALID_ARGUMENT, "unknown arena");
    }
    {
        gd_status st = arena_alloc(ctx, a, nbytes, alignment, out);
        if (st != GD_OK) span_clear(out);
        return st;
    }
}

gd_status gd_alloc_params(gd_context *ctx, size_t n, size_t al, gd_span *out) { return gd_context_alloc_span(ctx, GD_ARENA_PARAMS, n, al, out); }
gd_status gd_alloc_state(gd_context *ctx, size_t n, size_t al, gd_span *out) { return gd_context_alloc_span(ctx, GD_ARENA_STATE, n, al, out); }
gd_status gd_alloc_scratch(gd_context *ctx, size_t n, size_t al, gd_span *out) { return gd_context_alloc_span(ctx, GD_ARENA_SCRATCH, n, al, out); }
gd_status gd_alloc_data(gd_context *ctx, size_t n, size_t al, gd_span *out) { return gd_context_alloc_span(ctx, GD_ARENA_DATA, n, al, out); }

void gd_context_release_scratch(gd_context *ctx, const gd_span *span)
{
    gd_arena *a;
    if (ctx == NULL || span == NULL || span->arena != GD_ARENA_SCRATCH || !ctx->in_scope) return;
    a = ring_current(&ctx->scratch);
    if (a == NULL || span->slot != a->slot || span->generation != a->generation) return;
    if (span->offset + span->nbytes == a->offset && a->last_alloc_end == a->offset) {
        a->offset = a->last_alloc_offset;
        a->last_alloc_end = 0U;
    }
}

static const gd_arena *span_arena(const gd_context *ctx, const gd_span *s)
{
    switch (s->arena) {
    case GD_ARENA_PARAMS: return s->slot == -1 ? &ctx->params : NULL;
    case GD_ARENA_STATE: return s->slot == -1 ? &ctx->state : NULL;
    case GD_ARENA_SCRATCH: return (s->slot >= 0 && (uint32_t)s->slot < ctx->scratch.count) ? &ctx->scratch.slots[s->slot] : NULL;
    case GD_ARENA_DATA: return (s->slot >= 0 && (uint32_t)s->slot < ctx->data.count) ? &ctx->data.slots[s->slot] : NULL;
    default: return NULL;
    }
}

/* reference memory.c:770-786: arena, slot, generation, buffer and range must still match */
gd_status gd_context_validate_span(gd_context *ctx, const gd_span *span, const char *message)
{
    const gd_arena *a;
    if (ctx == NULL || span == NULL) return GD_ERR_INVALID_ARGUMENT;
    a = span_arena(ctx, span);
    if (a == NULL || span->buffer == NULL || span->buffer != (void *)a->buffer || span->generation != a->generation ||
        span->nbytes == 0U || span->offset > a->capacity || span->nbytes > a->capacity - span->offset)
        return gd_context_set_error(ctx, GD_ERR_BAD_STATE, message);
    return GD_OK;
}

/* ---- step scope ---------------------------------------------------------------------- */

static gd_status ring_advance(gd_context *ctx, gd_ring *r)
{
    gd_arena *a;
    r->current = (int32_t)(((uint32_t)(r->current + 1)) % r->count);
    a = &r->slots[r->current];
    if (a->fence_pending) {
        if (!gd_backend_fence_is_complete(&a->fence)) {
            gd_status st;
            r->waits += 1U;
            st = gd_backend_fence_wait(&a->fence);
            if (st != GD_OK) return gd_context_set_error(ctx, st, "backend fence wait failed");
        }
        gd_backend_fence_destroy(&a->fence);
        a->fence_pending = false;
    }
    a->generation += 1U; /* tensors of the step that used this slot are stale from here on */
    a->offset = 0U;
    a->last_alloc_end = 0U;
    return GD_OK;
}

gd_status gd_begin_step(gd_context *ctx, gd_scope_mode mode, gd_batch *batch)
{
    gd_status st;
    if (ctx == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (mode != GD_SCOPE_TRAIN && mode != GD_SCOPE_EVAL && mode != GD_SCOPE_INFER)
        return gd_context_set_error(ctx, GD_ERR_INVALID_ARGUMENT, "invalid scope mode");
    if (batch != g_empty_batch)
        return gd_context_set_error(ctx, GD_ERR_UNSUPPORTED, "only gd_batch_empty() is supported (no dataloader)");
    if (ctx->in_scope) return gd_context_set_error(ctx, GD_ERR_BAD_STATE, "step scope already active");
    st = ring_advance(ctx, &ctx->data);
    if (st == GD_OK) st = ring_advance(ctx, &ctx->scratch);
    if (st != GD_OK) return st;
    st = gd_backend_scope_begin(ctx->backend);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "backend scope begin failed");
    ctx->in_scope = true;
    ctx->mode = mode;
    ctx->scope_count += 1U;
    return GD_OK;
}

gd_status gd_end_step(gd_context *ctx)
{
    gd_arena *s, *d;
    gd_status st;
    if (ctx == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (!ctx->in_scope) return gd_context_set_error(ctx, GD_ERR_BAD_STATE, "no active step scope");
    s = ring_current(&ctx->scratch);
    d = ring_current(&ctx->data);
    ctx->in_scope = false;
    ctx->mode = GD_SCOPE_NONE;
    st = gd_backend_record_fence(ctx->backend, &s->fence);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "backend fence record failed");
    s->fence_pending = true;
    st = gd_backend_record_fence(ctx->backend, &d->fence);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "backend fence record failed");
    d->fence_pending = true;
    return GD_OK;
}

void gd_debug_complete_all(gd_context *ctx)
{
    if (ctx != NULL) (void)gd_backend_flush(ctx->backend);
}

int32_t gd_debug_current_ring_slot(const gd_context *ctx, gd_arena_kind arena)
{
    if (ctx == NULL) return -1;
    if (arena == GD_ARENA_SCRATCH) return ctx->scratch.current;
    if (arena == GD_ARENA_DATA) return ctx->data.current;
    return -1;
}

uint64_t gd_debug_ring_slot_generation(const gd_context *ctx, gd_arena_kind arena, uint32_t slot)
{
    const gd_ring *r;
    if (ctx == NULL) return 0U;
    r = arena == GD_ARENA_SCRATCH ? &ctx->scratch : (arena == GD_ARENA_DATA ? &ctx->data : NULL);
    return (r != NULL && slot < r->count) ? r->slots[slot].generation : 0U;
}

static void arena_stats(const gd_arena *a, gd_arena_stats *o)
{
    o->capacity = a->capacity;
    o->offset = a->offset;
    o->watermark = a->watermark;
    o->generation = a->generation;
    o->sealed = a->sealed;
}

static void ring_stats(const gd_ring *r, gd_ring_stats *o)
{
    uint32_t i;
    memset(o, 0, sizeof(*o));
    o->slots = r->count;
    o->current_slot = r->current;
    o->waits = r->waits;
    for (i = 0U; i < r->count; ++i) {
        o->total_capacity += r->slots[i].capacity;
        o->total_watermark += r->slots[i].watermark;
        if (r->slots[i].watermark > o->max_slot_watermark) o->max_slot_watermark = r->slots[i].watermark;
    }
}

gd_status gd_memory_stats_query(const gd_context *ctx, gd_memory_stats *out)
{
    if (ctx == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    memset(out, 0, sizeof(*out));
    arena_stats(&ctx->params, &out->params);
    arena_stats(&ctx->state, &out->state);
    ring_stats(&ctx->scratch, &out->scratch);
    ring_stats(&ctx->data, &out->data);
    out->backend_waits = ctx->scratch.waits + ctx->data.waits;
    out->last_scope_fence = ctx->scope_count;
    return GD_OK;
}
