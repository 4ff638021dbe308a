/*
 * Host dispatch of gd_backend_minimax_m3_index_topk and gd_backend_minimax_m3_sparse_attention.  Validation
 * restates the reference's src/ops/minimax_m3_index_topk/metal_minimax_m3_index_topk.m:74-104 and the matching
 * checks of metal_minimax_m3_sparse_attention.m: contiguous F16 [N,H,Dh] tensors, I32 cu [B+1] and topk
 * [Hkv,N,topk], head size <= 64, topk <= 16, block size <= 128.  Head sizes 4, 8, 16, 32, 64 on 16-byte aligned
 * operands take kernels of their own (size 64 with block sizes 64 / 128: the matrix cores); every other head size
 * and alignment takes a half-by-half variant of the per-row kernels.
 */
#include "../../../backends/hip/backend_hip_internal.h"

typedef struct gd_hip_m3_params {
    uint32_t total, batch, hq, hkv, dh;
    uint32_t max_seqlen, block, topk, init_blocks, local_blocks;
    float scale;
    uint32_t unaligned; /* an operand starts off a 16-byte boundary */
} gd_hip_m3_params;

int gd_hip_launch_m3_index_topk(hipStream_t stream, const void *q, const void *k, const int32_t *cu, int32_t *topk,
                                const gd_hip_m3_params *p);
int gd_hip_launch_m3_sparse_attention(hipStream_t stream, const void *q, const void *k, const void *v,
                                      const int32_t *cu, const int32_t *topk, void *out, const gd_hip_m3_params *p);

/* matrix-core kernels for head size 64 and block sizes that are multiples of 64 (minimax_m3_mfma.hip) */
typedef struct gd_hip_m3f_params {
    uint32_t n_rows, batch, hq, hkv;
    uint32_t max_seqlen, block, topk, init_blocks, local_blocks;
    float scale;
} gd_hip_m3f_params;

int gd_hip_launch_m3_mfma(hipStream_t stream, int picker, const void *q, const void *k, const void *v, const int32_t *cu,
                          int32_t *topk, void *out, const gd_hip_m3f_params *p);

static bool mfma_shape(const gd_backend *backend, const gd_hip_m3_params *p)
{
    const uint64_t rows = p->max_seqlen < p->total ? p->max_seqlen : p->total;
    return backend->m3_simple == 0 && p->unaligned == 0u && p->dh == 64u && (p->block % 64u) == 0u && (rows + p->block - 1u) / p->block <= 2048u &&
           (uint64_t)p->total * p->hkv * 128u < 0xffffffffull && (uint64_t)p->total * p->hq * 128u < 0xffffffffull;
}

static void fast_params(const gd_hip_m3_params *p, gd_hip_m3f_params *f)
{
    f->n_rows = p->total;
    f->batch = p->batch;
    f->hq = p->hq;
    f->hkv = p->hkv;
    f->max_seqlen = p->max_seqlen;
    f->block = p->block;
    f->topk = p->topk;
    f->init_blocks = p->init_blocks;
    f->local_blocks = p->local_blocks;
    f->scale = p->scale;
}

#define M3_MAX_DH 64
#define M3_MAX_TOPK 16u
#define M3_MAX_BLOCK 128u

static bool contiguous(const gd_backend_tensor_view *v)
{
    int64_t stride = 1;
    uint32_t i;
    if (!gd_hip_view_ok(v)) return false;
    for (i = v->rank; i > 0u; --i) {
        if (v->shape[i - 1u] <= 0 || v->strides[i - 1u] != stride) return false;
        stride *= v->shape[i - 1u];
    }
    return true;
}

static bool args_ok(const gd_backend_minimax_m3_sparse_args *a)
{
    return a != NULL && a->topk > 0u && a->topk <= M3_MAX_TOPK && a->block_size > 0u && a->block_size <= M3_MAX_BLOCK &&
           a->max_seqlen > 0u;
}

static void fill(gd_hip_m3_params *p, const gd_backend_tensor_view *q, const gd_backend_tensor_view *k,
                 const gd_backend_tensor_view *cu, const gd_backend_minimax_m3_sparse_args *a)
{
    p->total = (uint32_t)q->shape[0];
    p->batch = (uint32_t)(cu->shape[0] - 1);
    p->hq = (uint32_t)q->shape[1];
    p->hkv = (uint32_t)k->shape[1];
    p->dh = (uint32_t)q->shape[2];
    p->max_seqlen = a->max_seqlen < p->total ? a->max_seqlen : p->total;
    p->block = a->block_size;
    p->topk = a->topk;
    p->init_blocks = a->init_blocks;
    p->local_blocks = a->local_blocks;
    p->scale = a->scale;
    p->unaligned = 0u;
}

gd_status gd_backend_minimax_m3_index_topk(gd_backend *backend, const gd_backend_tensor_view *q,
                                           const gd_backend_tensor_view *k, const gd_backend_tensor_view *cu,
                                           const gd_backend_tensor_view *topk,
                                           const gd_backend_minimax_m3_sparse_args *args)
{
    gd_hip_m3_params p;
    if (backend == NULL || !contiguous(q) || !contiguous(k) || !contiguous(cu) || !contiguous(topk) || !args_ok(args) ||
        q->dtype != GD_BACKEND_DTYPE_F16 || k->dtype != q->dtype || cu->dtype != GD_BACKEND_DTYPE_I32 ||
        topk->dtype != GD_BACKEND_DTYPE_I32 || q->rank != 3u || k->rank != 3u || cu->rank != 1u || topk->rank != 3u ||
        cu->shape[0] < 2 || k->shape[0] != q->shape[0] || k->shape[1] != q->shape[1] || k->shape[2] != q->shape[2] ||
        q->shape[2] > M3_MAX_DH || topk->shape[0] != k->shape[1] || topk->shape[1] != q->shape[0] ||
        topk->shape[2] != (int64_t)args->topk || q->shape[0] > 0x7fffffff || q->shape[1] > 65535 ||
        cu->shape[0] - 1 > 65535)
        return GD_ERR_INVALID_ARGUMENT;
    fill(&p, q, k, cu, args);
    p.unaligned = ((q->offset | k->offset) & 15u) != 0u;
    if (mfma_shape(backend, &p)) {
        gd_hip_m3f_params f;
        fast_params(&p, &f);
        return gd_hip_finish_op(backend, gd_hip_launch_m3_mfma(backend->stream, 1, gd_hip_view_ptr(q), gd_hip_view_ptr(k), NULL,
                                                               (const int32_t *)gd_hip_view_ptr(cu),
                                                               (int32_t *)gd_hip_view_ptr(topk), NULL, &f));
    }
    return gd_hip_finish_op(backend, gd_hip_launch_m3_index_topk(backend->stream, gd_hip_view_ptr(q), gd_hip_view_ptr(k),
                                                                 (const int32_t *)gd_hip_view_ptr(cu),
                                                                 (int32_t *)gd_hip_view_ptr(topk), &p));
}

gd_status gd_backend_minimax_m3_sparse_attention(gd_backend *backend, const gd_backend_tensor_view *q,
                                                 const gd_backend_tensor_view *k, const gd_backend_tensor_view *v,
                                                 const gd_backend_tensor_view *cu, const gd_backend_tensor_view *topk,
                                                 const gd_backend_tensor_view *out,
                                                 const gd_backend_minimax_m3_sparse_args *args)
{
    gd_hip_m3_params p;
    if (backend == NULL || !contiguous(q) || !contiguous(k) || !contiguous(v) || !contiguous(cu) || !contiguous(topk) ||
        !contiguous(out) || !args_ok(args) || q->dtype != GD_BACKEND_DTYPE_F16 || k->dtype != q->dtype ||
        v->dtype != q->dtype || out->dtype != q->dtype || cu->dtype != GD_BACKEND_DTYPE_I32 ||
        topk->dtype != GD_BACKEND_DTYPE_I32 || q->rank != 3u || k->rank != 3u || v->rank != 3u || out->rank != 3u ||
        cu->rank != 1u || topk->rank != 3u || cu->shape[0] < 2 || k->shape[0] != q->shape[0] ||
        k->shape[2] != q->shape[2] || v->shape[0] != k->shape[0] || v->shape[1] != k->shape[1] ||
        v->shape[2] != k->shape[2] || out->shape[0] != q->shape[0] || out->shape[1] != q->shape[1] ||
        out->shape[2] != q->shape[2] || k->shape[1] <= 0 || (q->shape[1] % k->shape[1]) != 0 ||
        q->shape[2] > M3_MAX_DH || topk->shape[0] != k->shape[1] || topk->shape[1] != q->shape[0] ||
        topk->shape[2] != (int64_t)args->topk || q->shape[0] > 0x7fffffff || q->shape[1] > 65535 ||
        cu->shape[0] - 1 > 65535 || !(args->scale > 0.0f))
        return GD_ERR_INVALID_ARGUMENT;
    fill(&p, q, k, cu, args);
    p.unaligned = ((q->offset | k->offset | v->offset | out->offset) & 15u) != 0u;
    if (mfma_shape(backend, &p)) {
        gd_hip_m3f_params f;
        fast_params(&p, &f);
        return gd_hip_finish_op(backend, gd_hip_launch_m3_mfma(backend->stream, 0, gd_hip_view_ptr(q), gd_hip_view_ptr(k),
                                                               gd_hip_view_ptr(v), (const int32_t *)gd_hip_view_ptr(cu),
                                                               (int32_t *)gd_hip_view_ptr(topk), gd_hip_view_ptr(out), &f));
    }
    return gd_hip_finish_op(backend, gd_hip_launch_m3_sparse_attention(
        backend->stream, gd_hip_view_ptr(q), gd_hip_view_ptr(k), gd_hip_view_ptr(v), (const int32_t *)gd_hip_view_ptr(cu),
        (const int32_t *)gd_hip_view_ptr(topk), gd_hip_view_ptr(out), &p));
}
