/*
 * HIP backend lifecycle: device, one stream, HBM buffers, step scope, fences,
 * transfers, timers and graph capture.  Plain C over the HIP runtime API.
 *
 * Mapping of the reference's Metal backend (src/backends/metal/backend_metal.m)
 * onto HIP: command queue + scoped command buffer -> one hipStream_t on which
 * every operator of a scope is enqueued in order; fence -> hipEvent_t recorded
 * at the end of the scope; flush -> hipStreamSynchronize; shared-storage
 * MTLBuffer -> hipMalloc (HBM, not host visible).
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "backend_hip_internal.h"

int gd_hip_launch_fill(hipStream_t stream, void *dst, size_t count, size_t elem_size, uint32_t pattern);
int gd_hip_launch_rand_uniform(hipStream_t stream, void *dst, uint64_t count, uint32_t dtype, uint64_t seed,
                               float low, float high);

int gd_hip_sdpa_decode_scratch_init(int device);

static gd_status status_of(hipError_t e)
{
    if (e == hipSuccess) return GD_OK;
    if (e == hipErrorOutOfMemory) return GD_ERR_OUT_OF_MEMORY;
    return GD_ERR_INTERNAL;
}

gd_status gd_hip_finish_op(gd_backend *backend, int hip_error)
{
    hipError_t e = (hipError_t)hip_error;
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return status_of(e);
    }
    if (!backend->scope_active && !backend->capturing) {
        return status_of(hipStreamSynchronize(backend->stream));
    }
    return GD_OK;
}

gd_status gd_hip_reserve_attn_ws(gd_backend *backend, size_t nbytes)
{
    void *p = NULL;
    if (nbytes <= backend->attn_ws_bytes) return GD_OK;
    if (backend->capturing) return GD_ERR_UNSUPPORTED; /* no allocation inside a capture */
    /* work already enqueued may still read the old block */
    if (hipStreamSynchronize(backend->stream) != hipSuccess) return GD_ERR_INTERNAL;
    nbytes = (nbytes + ((size_t)1 << 20) - 1u) & ~(((size_t)1 << 20) - 1u);
    /* a live graph replays kernels that write their partial results into the block it was captured with */
    if (backend->attn_ws != NULL && backend->live_graphs > 0 && backend->retired_ws_count == GD_HIP_MAX_RETIRED_WS)
        return GD_ERR_BUSY;
    if (hipMalloc(&p, nbytes) != hipSuccess) {
        (void)hipGetLastError();
        return GD_ERR_OUT_OF_MEMORY;
    }
    /* the block starts with arrival counters that the kernels find at zero and leave at zero */
    if (hipMemset(p, 0, nbytes) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(p);
        return GD_ERR_INTERNAL;
    }
    if (backend->attn_ws != NULL) {
        if (backend->live_graphs > 0) backend->retired_ws[backend->retired_ws_count++] = backend->attn_ws;
        else (void)hipFree(backend->attn_ws);
    }
    backend->attn_ws = p;
    backend->attn_ws_bytes = nbytes;
    return GD_OK;
}

static void free_retired_ws(gd_backend *backend)
{
    int i;
    for (i = 0; i < backend->retired_ws_count; ++i) (void)hipFree(backend->retired_ws[i]);
    backend->retired_ws_count = 0;
}

static int env_int(const char *name, int fallback, int lo, int hi)
{
    const char *s = getenv(name);
    long v;
    if (s == NULL || *s == '\0') return fallback;
    v = strtol(s, NULL, 10);
    if (v < lo || v > hi) return fallback;
    return (int)v;
}

gd_status gd_backend_create_default(gd_backend **out_backend)
{
    gd_backend *b;
    int count = 0;
    hipDeviceProp_t prop;
    const char *hv;
    if (out_backend == NULL) return GD_ERR_INVALID_ARGUMENT;
    *out_backend = NULL;
    /* How the HIP runtime replays a captured graph is its own choice, read from the environment when it starts: from
     * dispatch packets it recorded when the graph was instantiated (its default), or node by node through its usual
     * launch path.  The decode step is a chain of 17 short kernels (122 at 24 layers), and on MI355X the node-by-node
     * path ends each of them with lighter cache maintenance: 0.1082 against 0.1117 ms per step of the gpt_lm default
     * decoder at batch 64, while a batch-1 step becomes host-bound (79.5 against 70.6 us).  A process that wants it
     * says so with GD_HIP_GRAPH_NODE_REPLAY=1: the runtime's variable is then set here, in front of the process's
     * first HIP call, unless the user has set it; if something else has started the runtime already, this has no
     * effect and nothing breaks.  Without the request the runtime's default stays. */
    {
        const char *want = getenv("GD_HIP_GRAPH_NODE_REPLAY");
        if (want != NULL && want[0] == '1' && want[1] == '\0' && getenv("DEBUG_CLR_GRAPH_PACKET_CAPTURE") == NULL)
            (void)setenv("DEBUG_CLR_GRAPH_PACKET_CAPTURE", "0", 0);
    }
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return GD_ERR_UNSUPPORTED; /* "no GPU": the reference tests skip on this status */
    }
    b = (gd_backend *)calloc(1, sizeof(*b));
    if (b == NULL) return GD_ERR_OUT_OF_MEMORY;
    b->device = 0;
    if (hipSetDevice(b->device) != hipSuccess || hipGetDeviceProperties(&prop, b->device) != hipSuccess ||
        /* address of the fixed scratch array of the entry point that allocates nothing: looked up once per
         * device, with this device current */
        gd_hip_sdpa_decode_scratch_init(b->device) != (int)hipSuccess ||
        hipStreamCreateWithFlags(&b->stream, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        free(b);
        return GD_ERR_INTERNAL;
    }
    b->compute_units = prop.multiProcessorCount;
    b->global_mem = prop.totalGlobalMem;
    snprintf(b->name, sizeof(b->name), "hip:%.60s:%.40s", prop.name, prop.gcnArchName);
    hv = getenv("GD_HIP_HOST_VISIBLE");
    b->host_visible_buffers = hv != NULL && hv[0] == '1' && hv[1] == '\0';
    b->sdpa_chunk = env_int("GD_HIP_SDPA_CHUNK", 0, 32, 1 << 20);
    b->sdpa_waves = env_int("GD_HIP_SDPA_WAVES", 0, 4, 8);
    b->sdpa_unroll = env_int("GD_HIP_SDPA_UNROLL", 0, 2, 8);
    b->linear_wide = env_int("GD_HIP_LINEAR_WIDE", -1, -1, 1);
    b->sdpa_merge = env_int("GD_HIP_SDPA_MERGE", 1, 0, 2);
    b->sdpa_nontemporal = env_int("GD_HIP_SDPA_NONTEMPORAL", -1, -1, 1);
    b->linear_tiles = env_int("GD_HIP_LINEAR_TILES", 0, 1, 4);
    b->linear_waves = env_int("GD_HIP_LINEAR_WAVES", 0, 4, 8);
    *out_backend = b;
    return GD_OK;
}

void gd_backend_destroy(gd_backend *backend)
{
    if (backend == NULL) return;
    (void)hipStreamSynchronize(backend->stream);
    if (backend->attn_ws != NULL) (void)hipFree(backend->attn_ws);
    free_retired_ws(backend);
    {
        unsigned i;
        for (i = 0u; i < GD_HIP_GRAPH_RING; ++i) {
            if (backend->graph_events[i] != NULL) (void)hipEventDestroy(backend->graph_events[i]);
        }
    }
    (void)hipStreamDestroy(backend->stream);
    free(backend);
}

gd_backend_kind gd_backend_kind_query(const gd_backend *backend)
{
    (void)backend;
    return GD_BACKEND_HIP;
}

const char *gd_backend_name(const gd_backend *backend)
{
    return backend != NULL ? backend->name : "hip";
}

gd_status gd_backend_device_info(const gd_backend *backend, char *name, size_t name_len,
                                 int32_t *compute_units, uint64_t *global_mem_bytes)
{
    if (backend == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (name != NULL && name_len > 0u) snprintf(name, name_len, "%s", backend->name);
    if (compute_units != NULL) *compute_units = backend->compute_units;
    if (global_mem_bytes != NULL) *global_mem_bytes = (uint64_t)backend->global_mem;
    return GD_OK;
}

gd_status gd_backend_set_tunable(gd_backend *backend, const char *name, int64_t value)
{
    if (backend == NULL || name == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (strcmp(name, "sdpa_chunk") == 0) {
        if (value < 0 || value > (1 << 20)) return GD_ERR_INVALID_ARGUMENT;
        backend->sdpa_chunk = (int)value;
        return GD_OK;
    }
    if (strcmp(name, "m3_simple") == 0) {
        if (value != 0 && value != 1) return GD_ERR_INVALID_ARGUMENT;
        backend->m3_simple = (int)value;
        return GD_OK;
    }
    if (strcmp(name, "linear_wide") == 0) {
        if (value < -1 || value > 1) return GD_ERR_INVALID_ARGUMENT;
        backend->linear_wide = (int)value;
        return GD_OK;
    }
    if (strcmp(name, "sdpa_merge") == 0) {
        if (value < 0 || value > 2) return GD_ERR_INVALID_ARGUMENT;
        backend->sdpa_merge = (int)value;
        return GD_OK;
    }
    if (strcmp(name, "sdpa_nontemporal") == 0) {
        if (value != -1 && value != 0 && value != 1) return GD_ERR_INVALID_ARGUMENT;
        backend->sdpa_nontemporal = (int)value;
        return GD_OK;
    }
    if (strcmp(name, "linear_tiles") == 0) {
        if (value != 0 && value != 1 && value != 2 && value != 4) return GD_ERR_INVALID_ARGUMENT;
        backend->linear_tiles = (int)value;
        return GD_OK;
    }
    if (strcmp(name, "linear_waves") == 0) {
        if (value != 0 && value != 4 && value != 8) return GD_ERR_INVALID_ARGUMENT;
        backend->linear_waves = (int)value;
        return GD_OK;
    }
    if (strcmp(name, "linear_no_lds_stream") == 0) {
        if (value != 0 && value != 1) return GD_ERR_INVALID_ARGUMENT;
        backend->linear_no_lds_stream = (int)value;
        return GD_OK;
    }
    if (strcmp(name, "prefill_rope_epilogue") == 0) {
        if (value != 0 && value != 1) return GD_ERR_INVALID_ARGUMENT;
        backend->no_prefill_rope_epilogue = value == 0;
        return GD_OK;
    }
    if (strcmp(name, "sdpa_waves") == 0 || strcmp(name, "sdpa_unroll") == 0) {
        if (value != 0 && value != 4 && value != 8 && !(value == 2 && name[5] == 'u')) return GD_ERR_INVALID_ARGUMENT;
        if (name[5] == 'w') backend->sdpa_waves = (int)value;
        else backend->sdpa_unroll = (int)value;
        return GD_OK;
    }
    return GD_ERR_INVALID_ARGUMENT;
}

/* ---- buffers ---------------------------------------------------------------- */

gd_status gd_backend_buffer_create(gd_backend *backend, size_t nbytes, gd_backend_buffer **out_buffer)
{
    gd_backend_buffer *buf;
    hipError_t e;
    if (out_buffer != NULL) *out_buffer = NULL;
    if (backend == NULL || out_buffer == NULL || nbytes == 0u) return GD_ERR_INVALID_ARGUMENT;
    buf = (gd_backend_buffer *)calloc(1, sizeof(*buf));
    if (buf == NULL) return GD_ERR_OUT_OF_MEMORY;
    buf->backend = backend;
    buf->nbytes = nbytes;
    if (backend->host_visible_buffers) {
        e = hipHostMalloc(&buf->host_ptr, nbytes, hipHostMallocMapped);
        if (e == hipSuccess) e = hipHostGetDevicePointer(&buf->dptr, buf->host_ptr, 0);
    } else {
        e = hipMalloc(&buf->dptr, nbytes);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        if (buf->host_ptr != NULL) (void)hipHostFree(buf->host_ptr);
        free(buf);
        return e == hipErrorOutOfMemory ? GD_ERR_OUT_OF_MEMORY : GD_ERR_INTERNAL;
    }
    *out_buffer = buf;
    return GD_OK;
}

void gd_backend_buffer_destroy(gd_backend_buffer *buffer)
{
    if (buffer == NULL) return;
    (void)hipStreamSynchronize(buffer->backend->stream);
    if (buffer->host_ptr != NULL) (void)hipHostFree(buffer->host_ptr);
    else (void)hipFree(buffer->dptr);
    free(buffer);
}

size_t gd_backend_buffer_nbytes(const gd_backend_buffer *buffer) { return buffer != NULL ? buffer->nbytes : 0u; }
void *gd_backend_buffer_host_ptr(gd_backend_buffer *buffer) { return buffer != NULL ? buffer->host_ptr : NULL; }
bool gd_backend_buffer_is_host_visible(const gd_backend_buffer *buffer) { return buffer != NULL && buffer->host_ptr != NULL; }
void *gd_backend_buffer_device_ptr(gd_backend_buffer *buffer) { return buffer != NULL ? buffer->dptr : NULL; }

static bool range_ok(const gd_backend_buffer *buffer, size_t offset, size_t nbytes)
{
    return buffer != NULL && offset <= buffer->nbytes && nbytes <= buffer->nbytes - offset;
}

/* ---- scope, flush, fences ---------------------------------------------------- */

gd_status gd_backend_scope_begin(gd_backend *backend)
{
    if (backend == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (backend->scope_active) return GD_ERR_BAD_STATE;
    backend->scope_active = true;
    return GD_OK;
}

gd_status gd_backend_flush(gd_backend *backend)
{
    if (backend == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (backend->capturing) return GD_ERR_BAD_STATE;
    return status_of(hipStreamSynchronize(backend->stream));
}

gd_status gd_backend_record_fence(gd_backend *backend, gd_backend_fence *out_fence)
{
    hipEvent_t ev;
    if (backend == NULL || out_fence == NULL) return GD_ERR_INVALID_ARGUMENT;
    out_fence->handle = NULL;
    if (backend->capturing) return GD_ERR_BAD_STATE;
    backend->scope_active = false;
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess ||
        hipEventRecord(ev, backend->stream) != hipSuccess) {
        (void)hipGetLastError();
        return GD_ERR_INTERNAL;
    }
    out_fence->handle = (void *)ev;
    return GD_OK;
}

void gd_backend_fence_destroy(gd_backend_fence *fence)
{
    if (fence == NULL || fence->handle == NULL) return;
    (void)hipEventDestroy((hipEvent_t)fence->handle);
    fence->handle = NULL;
}

bool gd_backend_fence_is_complete(gd_backend_fence *fence)
{
    if (fence == NULL || fence->handle == NULL) return true;
    return hipEventQuery((hipEvent_t)fence->handle) == hipSuccess;
}

gd_status gd_backend_fence_wait(gd_backend_fence *fence)
{
    if (fence == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (fence->handle == NULL) return GD_OK;
    return status_of(hipEventSynchronize((hipEvent_t)fence->handle));
}

/* ---- transfers, fill, copy ----------------------------------------------------- */

gd_status gd_backend_upload(gd_backend *backend, gd_backend_buffer *buffer, size_t offset,
                            const void *src, size_t nbytes)
{
    if (backend == NULL || buffer == NULL || src == NULL || nbytes == 0u || !range_ok(buffer, offset, nbytes))
        return GD_ERR_INVALID_ARGUMENT;
    if (backend->capturing) return GD_ERR_BAD_STATE;
    if (hipMemcpyAsync((char *)buffer->dptr + offset, src, nbytes, hipMemcpyHostToDevice, backend->stream) != hipSuccess) {
        (void)hipGetLastError();
        return GD_ERR_INTERNAL;
    }
    return status_of(hipStreamSynchronize(backend->stream));
}

gd_status gd_backend_download(gd_backend *backend, gd_backend_buffer *buffer, size_t offset,
                              void *dst, size_t nbytes)
{
    if (backend == NULL || buffer == NULL || dst == NULL || nbytes == 0u || !range_ok(buffer, offset, nbytes))
        return GD_ERR_INVALID_ARGUMENT;
    if (backend->capturing) return GD_ERR_BAD_STATE;
    if (hipMemcpyAsync(dst, (char *)buffer->dptr + offset, nbytes, hipMemcpyDeviceToHost, backend->stream) != hipSuccess) {
        (void)hipGetLastError();
        return GD_ERR_INTERNAL;
    }
    return status_of(hipStreamSynchronize(backend->stream));
}

gd_status gd_backend_fill(gd_backend *backend, gd_backend_buffer *buffer, size_t offset,
                          size_t count, size_t elem_size, uint32_t pattern)
{
    if (backend == NULL || buffer == NULL || (elem_size != 1u && elem_size != 2u && elem_size != 4u) ||
        (offset % elem_size) != 0u || count > SIZE_MAX / elem_size || !range_ok(buffer, offset, count * elem_size))
        return GD_ERR_INVALID_ARGUMENT;
    if (count == 0u) return GD_OK;
    return gd_hip_finish_op(backend, gd_hip_launch_fill(backend->stream, (char *)buffer->dptr + offset,
                                                        count, elem_size, pattern));
}

gd_status gd_backend_rand_uniform(gd_backend *backend, gd_backend_buffer *buffer, size_t offset, size_t count,
                                  uint32_t dtype, uint64_t seed, float low, float high)
{
    size_t elem_size;
    if (dtype == GD_BACKEND_DTYPE_F16 || dtype == GD_BACKEND_DTYPE_BF16) elem_size = 2u;
    else if (dtype == GD_BACKEND_DTYPE_F32) elem_size = 4u;
    else return GD_ERR_UNSUPPORTED;
    if (backend == NULL || buffer == NULL || count > UINT32_MAX || !(low <= high) || (offset % elem_size) != 0u ||
        !range_ok(buffer, offset, count * elem_size))
        return GD_ERR_INVALID_ARGUMENT;
    if (count == 0u) return GD_OK;
    return gd_hip_finish_op(backend, gd_hip_launch_rand_uniform(backend->stream, (char *)buffer->dptr + offset, count,
                                                                dtype, seed, low, high));
}

gd_status gd_backend_copy(gd_backend *backend, gd_backend_buffer *dst, size_t dst_offset,
                          gd_backend_buffer *src, size_t src_offset, size_t nbytes)
{
    if (backend == NULL || !range_ok(dst, dst_offset, nbytes) || !range_ok(src, src_offset, nbytes))
        return GD_ERR_INVALID_ARGUMENT;
    if (nbytes == 0u) return GD_OK;
    return gd_hip_finish_op(backend, (int)hipMemcpyAsync((char *)dst->dptr + dst_offset,
                                                         (const char *)src->dptr + src_offset, nbytes,
                                                         hipMemcpyDeviceToDevice, backend->stream));
}

/* ---- timers --------------------------------------------------------------------- */

gd_status gd_backend_timer_create(gd_backend *backend, gd_backend_timer **out_timer)
{
    gd_backend_timer *t;
    if (backend == NULL || out_timer == NULL) return GD_ERR_INVALID_ARGUMENT;
    *out_timer = NULL;
    t = (gd_backend_timer *)calloc(1, sizeof(*t));
    if (t == NULL) return GD_ERR_OUT_OF_MEMORY;
    t->backend = backend;
    if (hipEventCreate(&t->start) != hipSuccess || hipEventCreate(&t->stop) != hipSuccess) {
        (void)hipGetLastError();
        free(t);
        return GD_ERR_INTERNAL;
    }
    *out_timer = t;
    return GD_OK;
}

void gd_backend_timer_destroy(gd_backend_timer *timer)
{
    if (timer == NULL) return;
    (void)hipEventDestroy(timer->start);
    (void)hipEventDestroy(timer->stop);
    free(timer);
}

gd_status gd_backend_timer_start(gd_backend_timer *timer)
{
    if (timer == NULL) return GD_ERR_INVALID_ARGUMENT;
    return status_of(hipEventRecord(timer->start, timer->backend->stream));
}

gd_status gd_backend_timer_stop(gd_backend_timer *timer)
{
    if (timer == NULL) return GD_ERR_INVALID_ARGUMENT;
    return status_of(hipEventRecord(timer->stop, timer->backend->stream));
}

gd_status gd_backend_timer_elapsed_ms(gd_backend_timer *timer, float *out_ms)
{
    if (timer == NULL || out_ms == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (hipEventSynchronize(timer->stop) != hipSuccess) return GD_ERR_INTERNAL;
    return status_of(hipEventElapsedTime(out_ms, timer->start, timer->stop));
}

/* ---- graph capture ------------------------------------------------------------------ */

gd_status gd_backend_graph_begin_capture(gd_backend *backend)
{
    if (backend == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (!backend->scope_active || backend->capturing) return GD_ERR_BAD_STATE;
    if (hipStreamBeginCapture(backend->stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
        (void)hipGetLastError();
        return GD_ERR_INTERNAL;
    }
    backend->capturing = true;
    return GD_OK;
}

gd_status gd_backend_graph_end_capture(gd_backend *backend, gd_backend_graph **out_graph)
{
    gd_backend_graph *g;
    hipGraph_t graph = NULL;
    if (out_graph != NULL) *out_graph = NULL;
    if (backend == NULL || out_graph == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (!backend->capturing) return GD_ERR_BAD_STATE;
    backend->capturing = false;
    if (hipStreamEndCapture(backend->stream, &graph) != hipSuccess || graph == NULL) {
        (void)hipGetLastError();
        return GD_ERR_INTERNAL;
    }
    g = (gd_backend_graph *)calloc(1, sizeof(*g));
    if (g == NULL) {
        (void)hipGraphDestroy(graph);
        return GD_ERR_OUT_OF_MEMORY;
    }
    g->backend = backend;
    g->graph = graph;
    if (hipGraphInstantiate(&g->exec, graph, NULL, NULL, 0) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipGraphDestroy(graph);
        free(g);
        return GD_ERR_INTERNAL;
    }
    backend->live_graphs += 1;
    *out_graph = g;
    return GD_OK;
}

gd_status gd_backend_graph_launch(gd_backend *backend, gd_backend_graph *graph)
{
    if (backend == NULL || graph == NULL || graph->backend != backend) return GD_ERR_INVALID_ARGUMENT;
    if (backend->capturing) return GD_ERR_BAD_STATE;
    {
        /* Keep the launches queued on the stream bounded (GD_HIP_GRAPH_RING * GD_HIP_GRAPH_STRIDE): each one holds
         * kernel-argument memory and queue packets of every node until it has run, and a caller may enqueue
         * thousands without a wait in between.  One event per GD_HIP_GRAPH_STRIDE launches keeps the cost of the
         * bound off the single step. */
        const unsigned n = backend->graph_launches;
        hipEvent_t *slot = &backend->graph_events[(n / GD_HIP_GRAPH_STRIDE) % GD_HIP_GRAPH_RING];
        hipError_t e;
        if ((n % GD_HIP_GRAPH_STRIDE) == 0u && n / GD_HIP_GRAPH_STRIDE >= GD_HIP_GRAPH_RING && *slot != NULL) {
            if (hipEventSynchronize(*slot) != hipSuccess) return GD_ERR_INTERNAL;
        }
        e = hipGraphLaunch(graph->exec, backend->stream);
        if (e == hipSuccess && (n % GD_HIP_GRAPH_STRIDE) == GD_HIP_GRAPH_STRIDE - 1u) {
            if (*slot == NULL && hipEventCreateWithFlags(slot, hipEventDisableTiming) != hipSuccess) {
                (void)hipGetLastError();
                *slot = NULL;
                return GD_ERR_INTERNAL;
            }
            e = hipEventRecord(*slot, backend->stream);
        }
        backend->graph_launches = n + 1u;
        return gd_hip_finish_op(backend, (int)e);
    }
}

void gd_backend_graph_destroy(gd_backend_graph *graph)
{
    if (graph == NULL) return;
    (void)hipStreamSynchronize(graph->backend->stream);
    (void)hipGraphExecDestroy(graph->exec);
    (void)hipGraphDestroy(graph->graph);
    graph->backend->live_graphs -= 1;
    if (graph->backend->live_graphs == 0) free_retired_ws(graph->backend);
    free(graph);
}
