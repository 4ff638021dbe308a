/*
 * Host dispatch of gd_backend_sdpa_decode{,_at,_positions}.  Validation restates the
 * reference dispatch src/ops/sdpa_decode/metal_sdpa_decode.m:60-150 with the head-size
 * limit raised from 64 to 128 for the split-KV kernel (256 for the generic one).
 */
#include <math.h>
#include <stdio.h>
#include <string.h>

#include "../../../backends/hip/backend_hip_internal.h"
#include "hip_sdpa_decode_types.h"

int gd_hip_launch_sdpa_decode_split(hipStream_t stream, const void *q, const void *k, const void *v,
                                    const int32_t *pos, void *out, float *ws,
                                    const gd_hip_sdpa_decode_params *params);
int gd_hip_launch_sdpa_decode_pieces(hipStream_t stream, const void *q, const void *k, const void *v,
                                     const int32_t *pos, void *out, float *ws,
                                     const gd_hip_sdpa_decode_params *params);
int gd_hip_launch_sdpa_decode_generic(hipStream_t stream, const void *q, const void *k, const void *v,
                                      const int32_t *pos, void *out, const gd_hip_sdpa_decode_params *params);

float *gd_hip_sdpa_decode_scratch(int device);

#define GD_HIP_SDPA_MAX_DH 256
/* keys per piece of a ragged batch (PIECES form) */
#define GD_HIP_SDPA_PIECE_KEYS 256u
_Static_assert(GD_HIP_SDPA_NOALLOC_SCRATCH_BYTES == GD_BACKEND_SDPA_DECODE_NOALLOC_SCRATCH_BYTES,
               "public constant and device array differ");

static bool common_ok(const gd_backend_tensor_view *q, const gd_backend_tensor_view *k,
                      const gd_backend_tensor_view *v, const gd_backend_tensor_view *out)
{
    uint32_t i;
    if (!gd_hip_view_ok(q) || !gd_hip_view_ok(k) || !gd_hip_view_ok(v) || !gd_hip_view_ok(out)) return false;
    if ((q->dtype != GD_BACKEND_DTYPE_F16 && q->dtype != GD_BACKEND_DTYPE_F32) || k->dtype != q->dtype ||
        v->dtype != q->dtype || out->dtype != q->dtype || q->rank != 4u || k->rank != 4u || v->rank != 4u ||
        out->rank != 4u)
        return false;
    for (i = 0u; i < 4u; ++i) {
        if (k->shape[i] != v->shape[i] || out->shape[i] != q->shape[i]) return false;
    }
    return q->shape[0] == k->shape[0] && q->shape[3] == k->shape[3] && (q->shape[2] % k->shape[2]) == 0 &&
           q->shape[0] <= (int64_t)INT32_MAX && q->shape[1] <= (int64_t)INT32_MAX &&
           k->shape[1] <= (int64_t)INT32_MAX && q->shape[2] <= 65535 && k->shape[2] <= 65535 &&
           q->shape[3] <= GD_HIP_SDPA_MAX_DH;
}

static bool args_ok(const gd_backend_sdpa_decode_args *a, const gd_backend_tensor_view *k)
{
    return a != NULL && a->scale == a->scale && a->scale > 0.0f && isfinite(a->scale) &&
           (int64_t)a->prefix_len <= k->shape[1] && a->sliding_window <= (uint32_t)INT32_MAX;
}

static gd_status dispatch(gd_backend *backend, const gd_backend_tensor_view *q, const gd_backend_tensor_view *k,
                          const gd_backend_tensor_view *v, const gd_backend_tensor_view *pos,
                          const gd_backend_tensor_view *out, const gd_backend_sdpa_decode_args *args,
                          uint32_t pos_mode, bool noalloc)
{
    gd_hip_sdpa_decode_params p;
    const int32_t *pos_ptr = pos != NULL ? (const int32_t *)gd_hip_view_ptr(pos) : NULL;
    uint32_t group;
    p.batch = (uint32_t)q->shape[0];
    p.tq = (uint32_t)q->shape[1];
    p.tmax = (uint32_t)k->shape[1];
    p.hq = (uint32_t)q->shape[2];
    p.hkv = (uint32_t)k->shape[2];
    p.dh = (uint32_t)q->shape[3];
    p.window = args->sliding_window;
    p.prefix_len = args->prefix_len;
    p.pos_mode = pos_mode;
    p.cache_pos = args->cache_pos;
    p.scale = args->scale;
    p.dtype = q->dtype;
    p.chunk = 0u;
    p.nsplit = 1u;
    /* measured on MI355X (512 keys, 64 rows x 8 heads): 4 wavefronts with trips of 2 row loads beat 8 wavefronts
     * with trips of 4 by 7 %: what is left to do when the last rows arrive is one short trip and a merge of 4 */
    p.waves = backend->sdpa_waves == 8 ? 8u : 4u;
    p.unroll = backend->sdpa_unroll != 0 ? (uint32_t)backend->sdpa_unroll : 2u;
    /* Cache rows are read once per launch.  Marked streaming they do not displace anything from the L2s and the
     * memory-side cache on their way, which is worth 10-13 % when the rows come from HBM (measured with launches
     * rotating over 0.5 GB of caches: 15.4 -> 13.6 us at 64 rows x 8 heads x 512 keys, 66.7 -> 58.7 us at 16 x 16
     * heads of 128 with 1024..4095 keys).  Caches small enough to stay in the 256 MB memory-side cache from one
     * decode step to the next (all layers together) are better left cacheable: the step then finds them there. */
    if (backend->sdpa_nontemporal >= 0) p.nontemporal = backend->sdpa_nontemporal != 0 ? 1u : 0u;
    else p.nontemporal = (uint64_t)p.batch * p.tmax * p.hkv * p.dh * 4u > (128ull << 20) ? 1u : 0u;
    group = p.hq / p.hkv;
    if (q->dtype == GD_BACKEND_DTYPE_F16 && p.tq == 1u && (p.dh == 64u || p.dh == 128u) &&
        (group == 1u || group == 2u || group == 3u || group == 4u || group == 6u || group == 8u) &&
        ((q->offset | k->offset | v->offset | out->offset) & 15u) == 0u && p.batch <= 65535u &&
        /* the kernel addresses the rows of one (batch row, kv head) with 24-bit factors and 32-bit byte offsets */
        p.tmax < (1u << 24) && (uint64_t)p.hkv * p.dh * 2u < (1u << 24) &&
        (uint64_t)p.tmax * p.hkv * p.dh * 2u < 0xffffffffull) {
        /* longest run of visible keys a row can have: the window, plus the prefix in front of it */
        uint32_t span = p.window > 0u && p.window < p.tmax ? p.window : p.tmax;
        if (p.window > 0u && p.prefix_len > 0u) span = span + p.prefix_len < p.tmax ? span + p.prefix_len : p.tmax;
        uint32_t chunk = (uint32_t)backend->sdpa_chunk;
        gd_status st;
        /* Ragged batches: rows cut into pieces, one workgroup each, the last piece of a row to arrive merges it
         * (sdpa_decode_pieces.hip).  Taken by itself when there is a (row, kv head) pair for every compute unit
         * (below that the key range is split to fill the device, as before) and rows can be long enough for
         * raggedness to matter; tunable "sdpa_merge": 0 never, 2 whenever the form applies.  The kernel keeps rows of
         * about one length whole, so an even batch costs about what one workgroup per row costs. */
        {
            const uint64_t pairs = (uint64_t)p.batch * p.hkv;
            uint32_t piece = chunk != 0u ? ((chunk + 31u) & ~31u) : GD_HIP_SDPA_PIECE_KEYS;
            uint32_t pieces;
            size_t need;
            if ((uint64_t)piece * GD_HIP_SDPA_MAX_PIECES < span)
                piece = ((span + GD_HIP_SDPA_MAX_PIECES - 1u) / GD_HIP_SDPA_MAX_PIECES + 31u) & ~31u;
            pieces = (span + piece - 1u) / piece;
            need = ((size_t)GD_HIP_SDPA_COUNTER_SLOTS + (size_t)p.batch * p.hq * pieces * (p.dh + 2u)) * sizeof(float);
            const bool applies = pos_mode == GD_HIP_SDPA_POS_VECTOR && p.batch <= GD_HIP_SDPA_PIECES_MAX_BATCH &&
                                 pairs <= GD_HIP_SDPA_COUNTER_SLOTS && pieces > 1u &&
                                 (!noalloc || need <= GD_HIP_SDPA_NOALLOC_SCRATCH_BYTES);
            const bool wanted = backend->sdpa_merge == 2 ||
                                (backend->sdpa_merge == 1 && chunk == 0u && pairs >= (uint64_t)backend->compute_units &&
                                 span >= 4u * GD_HIP_SDPA_PIECE_KEYS);
            if (applies && wanted) {
                float *ws;
                /* 4 wavefronts per workgroup; a requested chunk is taken literally, otherwise even rows stay whole
                 * when that leaves two workgroups per compute unit and are halved below that */
                p.waves = 4u;
                p.even_pieces = chunk != 0u ? 0u : (pairs >= 2u * (uint64_t)backend->compute_units ? 1u : 2u);
                p.chunk = piece;
                p.nsplit = pieces;
                if (noalloc) {
                    ws = gd_hip_sdpa_decode_scratch(backend->device);
                    if (ws == NULL) return GD_ERR_BAD_STATE;
                } else {
                    st = gd_hip_reserve_attn_ws(backend, need);
                    if (st != GD_OK) return st;
                    ws = (float *)backend->attn_ws;
                }
                {
                    const bool pfx = p.prefix_len > 0u;
                    const uint32_t rec[12] = {4u, p.dh, group, p.waves, group == 1u ? 2u : 4u, pfx ? 0u : p.nontemporal,
                                              pfx ? 1u : 0u, p.nsplit, p.hkv, p.batch, p.chunk, p.even_pieces};
                    memcpy(backend->last_sdpa, rec, sizeof(rec));
                }
                return gd_hip_finish_op(backend, gd_hip_launch_sdpa_decode_pieces(
                    backend->stream, gd_hip_view_ptr(q), gd_hip_view_ptr(k), gd_hip_view_ptr(v), pos_ptr,
                    gd_hip_view_ptr(out), ws, &p));
            }
            p.even_pieces = 0u;
        }
        if (chunk == 0u) {
            /* one workgroup per (batch row, kv head) as soon as that gives every compute unit one (a single pass, no
             * combine kernel: measured 6 % faster than two splits at 256 pairs x 4096 keys); below that, split the
             * key range to reach one workgroup per compute unit, never with less than 512 keys each */
            const uint64_t pairs = (uint64_t)p.batch * p.hkv;
            const uint64_t want = ((uint64_t)backend->compute_units + pairs - 1u) / pairs;
            chunk = (uint32_t)((span + want - 1u) / want);
            if (chunk < 512u) chunk = 512u;
        }
        chunk = (chunk + 31u) & ~31u;
        if (chunk > span) chunk = (span + 31u) & ~31u;
        p.chunk = chunk;
        p.nsplit = (span + chunk - 1u) / chunk;
        /* about 8 wavefronts per compute unit stream best: 4 per workgroup once there are two workgroups per unit */
        if (backend->sdpa_waves == 0)
            p.waves = (uint64_t)p.batch * p.hkv * p.nsplit >= 2u * (uint64_t)backend->compute_units ? 4u : 8u;
        float *ws = NULL;
        if (p.nsplit > 1u) {
            const size_t need = ((size_t)GD_HIP_SDPA_COUNTER_SLOTS +
                                 (size_t)p.batch * p.hq * p.nsplit * (p.dh + 2u)) * sizeof(float);
            if (noalloc) {
                /* partial results go to the fixed device array of this library; nothing is allocated */
                ws = gd_hip_sdpa_decode_scratch(backend->device);
                if (ws == NULL) return GD_ERR_BAD_STATE;
                if (need > GD_HIP_SDPA_NOALLOC_SCRATCH_BYTES) {
                    fprintf(stderr, "gd_backend_sdpa_decode_positions_noalloc: the split-KV partial results of this "
                                    "call need %zu bytes, the fixed scratch holds %u\n",
                            need, (unsigned)GD_HIP_SDPA_NOALLOC_SCRATCH_BYTES);
                    return GD_ERR_OUT_OF_MEMORY;
                }
            } else {
                st = gd_hip_reserve_attn_ws(backend, need);
                if (st != GD_OK) return st;
                ws = (float *)backend->attn_ws;
            }
        }
        {
            /* mirrors the instantiation choice of the launcher (sdpa_decode.hip: launch_split) */
            const bool pfx = p.prefix_len > 0u;
            const uint32_t w = pfx ? ((group == 1u && p.waves == 8u) ? 8u : 4u) : (group == 1u ? p.waves : 4u);
            const uint32_t u = pfx ? (group == 1u ? 2u : 4u)
                                   : (group == 1u ? ((p.unroll == 8u || p.unroll == 2u) ? p.unroll : 4u) : 4u);
            const uint32_t rec[12] = {1u, p.dh, group, w, u, pfx ? 0u : p.nontemporal, pfx ? 1u : 0u,
                                      p.nsplit, p.hkv, p.batch, p.chunk, !pfx && p.window == 0u ? 1u : 0u};
            memcpy(backend->last_sdpa, rec, sizeof(rec));
        }
        return gd_hip_finish_op(backend, gd_hip_launch_sdpa_decode_split(
            backend->stream, gd_hip_view_ptr(q), gd_hip_view_ptr(k), gd_hip_view_ptr(v), pos_ptr,
            gd_hip_view_ptr(out), ws, &p));
    }
    if ((uint64_t)p.batch * p.hq * p.tq > 0x7fffffffu) return GD_ERR_UNSUPPORTED;
    {
        const uint32_t rec[12] = {2u, p.dh, group, 1u, 0u, 0u, 0u, p.batch * p.hq * p.tq, 1u, 1u, 0u, 0u};
        memcpy(backend->last_sdpa, rec, sizeof(rec));
        backend->last_sdpa[5] = p.dtype;
    }
    return gd_hip_finish_op(backend, gd_hip_launch_sdpa_decode_generic(
        backend->stream, gd_hip_view_ptr(q), gd_hip_view_ptr(k), gd_hip_view_ptr(v), pos_ptr,
        gd_hip_view_ptr(out), &p));
}

gd_status gd_backend_sdpa_decode(gd_backend *backend, const gd_backend_tensor_view *q,
                                 const gd_backend_tensor_view *k_cache, const gd_backend_tensor_view *v_cache,
                                 const gd_backend_tensor_view *cache_pos, const gd_backend_tensor_view *out,
                                 const gd_backend_sdpa_decode_args *args)
{
    if (backend == NULL || !common_ok(q, k_cache, v_cache, out) || !gd_hip_view_ok(cache_pos) ||
        cache_pos->dtype != GD_BACKEND_DTYPE_I32 || cache_pos->rank != 0u || cache_pos->count != 1u ||
        (cache_pos->offset & 3u) != 0u || !args_ok(args, k_cache))
        return GD_ERR_INVALID_ARGUMENT;
    return dispatch(backend, q, k_cache, v_cache, cache_pos, out, args, GD_HIP_SDPA_POS_TENSOR0, false);
}

gd_status gd_backend_sdpa_decode_at(gd_backend *backend, const gd_backend_tensor_view *q,
                                    const gd_backend_tensor_view *k_cache, const gd_backend_tensor_view *v_cache,
                                    const gd_backend_tensor_view *out, const gd_backend_sdpa_decode_args *args)
{
    if (backend == NULL || !common_ok(q, k_cache, v_cache, out) || !args_ok(args, k_cache) ||
        args->cache_pos < 0 || (int64_t)args->cache_pos > k_cache->shape[1] ||
        q->shape[1] > k_cache->shape[1] - (int64_t)args->cache_pos)
        return GD_ERR_INVALID_ARGUMENT;
    return dispatch(backend, q, k_cache, v_cache, NULL, out, args, GD_HIP_SDPA_POS_SCALAR, false);
}

gd_status gd_backend_sdpa_decode_positions(gd_backend *backend, const gd_backend_tensor_view *q,
                                           const gd_backend_tensor_view *k_cache,
                                           const gd_backend_tensor_view *v_cache,
                                           const gd_backend_tensor_view *cache_pos,
                                           const gd_backend_tensor_view *out,
                                           const gd_backend_sdpa_decode_args *args)
{
    if (backend == NULL || !common_ok(q, k_cache, v_cache, out) || !gd_hip_view_ok(cache_pos) ||
        cache_pos->dtype != GD_BACKEND_DTYPE_I32 || cache_pos->rank != 1u || cache_pos->shape[0] != q->shape[0] ||
        (cache_pos->offset & 3u) != 0u || !args_ok(args, k_cache))
        return GD_ERR_INVALID_ARGUMENT;
    return dispatch(backend, q, k_cache, v_cache, cache_pos, out, args, GD_HIP_SDPA_POS_VECTOR, false);
}

/* The per-row-positions form for callers that cannot allocate device memory: same validation, same kernels and
 * therefore the same bits as gd_backend_sdpa_decode_positions; the split-KV partial results use the library's
 * fixed device array instead of the backend's grown workspace.  No hipMalloc / hipFree on any path. */
gd_status gd_backend_sdpa_decode_positions_noalloc(gd_backend *backend, const gd_backend_tensor_view *q,
                                                   const gd_backend_tensor_view *k_cache,
                                                   const gd_backend_tensor_view *v_cache,
                                                   const gd_backend_tensor_view *cache_pos,
                                                   const gd_backend_tensor_view *out,
                                                   const gd_backend_sdpa_decode_args *args)
{
    if (backend == NULL || !common_ok(q, k_cache, v_cache, out) || !gd_hip_view_ok(cache_pos) ||
        cache_pos->dtype != GD_BACKEND_DTYPE_I32 || cache_pos->rank != 1u || cache_pos->shape[0] != q->shape[0] ||
        (cache_pos->offset & 3u) != 0u || !args_ok(args, k_cache))
        return GD_ERR_INVALID_ARGUMENT;
    return dispatch(backend, q, k_cache, v_cache, cache_pos, out, args, GD_HIP_SDPA_POS_VECTOR, true);
}

gd_status gd_backend_sdpa_decode_last_kernel(gd_backend *backend, char *out, size_t capacity)
{
    const uint32_t *r;
    if (backend == NULL || out == NULL || capacity == 0u) return GD_ERR_INVALID_ARGUMENT;
    r = backend->last_sdpa;
    if (r[0] == 1u)
        /* template arguments as a kernel trace prints them: D, G, wavefronts, trip length, streaming loads[, prefix
         * [, pieces, first rows requested ahead of the position]] */
        snprintf(out, capacity, "gd_sdpa_decode_split_kernel<%u,%u,%u,%u,%s%s> [grid %u x %u x %u, %u keys per workgroup%s]",
                 r[1], r[2], r[3], r[4], r[5] ? "true" : "false",
                 r[6] ? ",true" : (r[11] ? ",false,false,true" : ""), r[7], r[8], r[9], r[10],
                 r[7] > 1u ? ", combine kernel" : "");
    else if (r[0] == 4u)
        snprintf(out, capacity, "gd_sdpa_decode_split_kernel<%u,%u,%u,%u,%s,%s,true> [grid %u x %u x %u, pieces of %u keys, "
                                "rows merged by the last piece%s]",
                 r[1], r[2], r[3], r[4], r[5] ? "true" : "false", r[6] ? "true" : "false", r[8], r[9], r[7], r[10],
                 r[11] == 1u ? ", even rows whole" : r[11] == 2u ? ", even rows halved" : "");
    else if (r[0] == 2u)
        snprintf(out, capacity, "gd_sdpa_decode_generic_kernel<%s> [grid %u]", r[5] == 1u ? "gd_half" : "float", r[7]);
    else
        return GD_ERR_BAD_STATE;
    return GD_OK;
}
