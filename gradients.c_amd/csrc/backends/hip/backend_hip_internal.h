/*
 * Internal state of the HIP backend and the helpers every operator's host
 * dispatch uses: view checks, device pointers, the "finish" rule (operators
 * outside a scope complete before returning, reference
 * src/backends/metal/backend_metal.m:354-394).
 */
#ifndef GD_BACKEND_HIP_INTERNAL_H
#define GD_BACKEND_HIP_INTERNAL_H

#ifndef __HIP_PLATFORM_AMD__
#define __HIP_PLATFORM_AMD__ 1
#endif
#include <hip/hip_runtime_api.h>

#include "gd_backend_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define GD_HIP_MAX_RETIRED_WS 16
#define GD_HIP_GRAPH_STRIDE 8u
#define GD_HIP_GRAPH_RING 4u

struct gd_backend {
    int device;
    hipStream_t stream;
    bool scope_active;
    bool capturing;
    bool host_visible_buffers; /* GD_HIP_HOST_VISIBLE=1 */
    int compute_units;
    size_t global_mem;
    char name[128];
    /* scratch for split-KV attention partials, grown on demand outside capture */
    void *attn_ws;
    size_t attn_ws_bytes;
    /* instantiated graphs hold the workspace address of their capture: blocks replaced while any graph is alive
     * are kept here and freed when the last graph is destroyed (or with the backend) */
    int live_graphs;
    void *retired_ws[GD_HIP_MAX_RETIRED_WS];
    int retired_ws_count;
    /* graph launches in flight are bounded: an event after every GD_HIP_GRAPH_STRIDE launches, the host waits
     * for the one GD_HIP_GRAPH_RING events back */
    hipEvent_t graph_events[GD_HIP_GRAPH_RING];
    unsigned graph_launches;
    /* what the last sdpa_decode dispatch launched: 0 none, 1 split, 2 generic; D, G, W, U, streaming, prefix, grid */
    uint32_t last_sdpa[12];
    int last_linear_family; /* GD_HIP_LINEAR_FAMILY_* of the last projection call, 0 before the first */
    /* tunables read from the environment once at creation */
    int sdpa_chunk;      /* keys per workgroup in the split-KV decode kernel (0 = automatic) */
    int sdpa_waves;      /* 4 or 8 wavefronts per workgroup (0 = default 8) */
    int sdpa_unroll;     /* 4 or 8 key-row loads in flight per lane (0 = default 8) */
    int linear_wide;      /* few-row projections over large [N,K] weights: 1 always the wide kernel, 0 never, -1 from 4 MiB */
    int sdpa_merge;       /* ragged batches in pieces merged inside the kernel: 1 (default) where it pays, 0 never, 2 wherever it applies */
    int sdpa_nontemporal; /* streaming hint on the K/V loads: 1 always, 0 never, -1 by the size of the caches */
    int m3_simple;        /* 1: MiniMax-M3 operators always take the per-row kernels (tests compare the two paths) */
    int linear_tiles;    /* few-row projections: 16-column tiles per workgroup, 1 / 2 / 4 (0 = automatic) */
    int linear_waves;    /* few-row projections: wavefronts per workgroup = K split, 4 / 8 (0 = automatic) */
    int linear_no_lds_stream; /* few-row projections: 1 = never stage the weight stream through LDS (tests compare the two paths) */
    int no_prefill_rope_epilogue; /* 1: gd_backend_linear_qkv_rope_packed answers GD_ERR_UNSUPPORTED, so a caller stays with
                                     the separate operators (tests compare the two paths) */
};

struct gd_backend_buffer {
    gd_backend *backend;
    void *dptr;     /* device address */
    void *host_ptr; /* non-NULL only for host-visible buffers */
    size_t nbytes;
};

struct gd_backend_timer {
    gd_backend *backend;
    hipEvent_t start, stop;
};

struct gd_backend_graph {
    gd_backend *backend;
    hipGraph_t graph;
    hipGraphExec_t exec;
};

/* Maps a HIP error after a launch to a status; synchronises when no scope is open. */
gd_status gd_hip_finish_op(gd_backend *backend, int hip_error);

/* Ensures backend->attn_ws holds at least nbytes (UNSUPPORTED while capturing if it must grow). */
gd_status gd_hip_reserve_attn_ws(gd_backend *backend, size_t nbytes);

static inline size_t gd_hip_dtype_size(uint32_t dtype)
{
    switch (dtype) {
    case GD_BACKEND_DTYPE_F16: case GD_BACKEND_DTYPE_BF16: case GD_BACKEND_DTYPE_U16: return 2u;
    case GD_BACKEND_DTYPE_F32: case GD_BACKEND_DTYPE_I32: return 4u;
    case GD_BACKEND_DTYPE_U8: return 1u;
    default: return 0u;
    }
}

/* view lies inside its buffer (count * elem from offset) */
static inline bool gd_hip_view_in_range(const gd_backend_tensor_view *v)
{
    size_t es;
    if (v == NULL || v->buffer == NULL || v->rank > GD_BACKEND_MAX_DIMS) return false;
    es = gd_hip_dtype_size(v->dtype);
    if (es == 0u || v->offset > v->buffer->nbytes) return false;
    if (v->count > (v->buffer->nbytes - v->offset) / es) return false;
    return true;
}

/* positive dims, row-major strides, count == product of dims */
static inline bool gd_hip_view_contiguous(const gd_backend_tensor_view *v)
{
    int64_t stride = 1;
    uint32_t i;
    if (v == NULL || v->rank > GD_BACKEND_MAX_DIMS) return false;
    for (i = v->rank; i > 0u; --i) {
        const uint32_t d = i - 1u;
        if (v->shape[d] <= 0 || v->strides[d] != stride) return false;
        if (stride > INT64_MAX / v->shape[d]) return false;
        stride *= v->shape[d];
    }
    return (size_t)stride == v->count;
}

static inline bool gd_hip_view_ok(const gd_backend_tensor_view *v)
{
    return gd_hip_view_in_range(v) && gd_hip_view_contiguous(v);
}

static inline void *gd_hip_view_ptr(const gd_backend_tensor_view *v)
{
    return (void *)((char *)v->buffer->dptr + v->offset);
}

static inline bool gd_hip_matrix_ok(const gd_backend_matrix_view *m)
{
    size_t es, need;
    if (m == NULL || m->buffer == NULL || m->rows == 0u || m->cols == 0u) return false;
    es = gd_hip_dtype_size(m->dtype);
    if (es == 0u || m->row_bytes < (size_t)m->cols * es || (m->row_bytes % es) != 0u) return false;
    if (m->offset > m->buffer->nbytes) return false;
    need = (size_t)(m->rows - 1u) * m->row_bytes + (size_t)m->cols * es;
    return need <= m->buffer->nbytes - m->offset;
}

static inline void *gd_hip_matrix_ptr(const gd_backend_matrix_view *m)
{
    return (void *)((char *)m->buffer->dptr + m->offset);
}

static inline bool gd_hip_vector_ok(const gd_backend_vector_view *v)
{
    size_t es;
    if (v == NULL || v->buffer == NULL || v->length == 0u) return false;
    es = gd_hip_dtype_size(v->dtype);
    if (es == 0u || v->offset > v->buffer->nbytes) return false;
    return (size_t)v->length <= (v->buffer->nbytes - v->offset) / es;
}

static inline void *gd_hip_vector_ptr(const gd_backend_vector_view *v)
{
    return (void *)((char *)v->buffer->dptr + v->offset);
}

#ifdef __cplusplus
}
#endif

#endif /* GD_BACKEND_HIP_INTERNAL_H */
