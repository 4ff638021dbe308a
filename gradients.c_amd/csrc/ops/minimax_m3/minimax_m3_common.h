/*
 * Limits and configuration defaults shared by the two MiniMax-M3 front ends (ops/minimax_m3_index_topk,
 * ops/minimax_m3_sparse_attention): the rules of the reference's
 * src/ops/minimax_m3_index_topk/core_minimax_m3_index_topk.c:9-60 and
 * src/ops/minimax_m3_sparse_attention/core_minimax_m3_sparse_attention.c:14-60: head size <= 64, block size <= 128
 * (default 128), topk <= 16 (default 4), init / local blocks default 1 without a configuration, scale <= 0
 * selects 1 / sqrt(Dh).
 */
#ifndef GD_MINIMAX_M3_COMMON_H
#define GD_MINIMAX_M3_COMMON_H
#include "../op_common.h"

#define M3_BLOCK_DEFAULT 128
#define M3_BLOCK_MAX 128
#define M3_TOPK_MAX 16
#define M3_DH_MAX 64

static inline gd_status gd_minimax_m3_resolve(gd_context *ctx, const gd_tensor *q, const gd_minimax_m3_sparse_config *c,
                         gd_backend_minimax_m3_sparse_args *a)
{
    const int32_t block = c != NULL && c->block_size > 0 ? c->block_size : M3_BLOCK_DEFAULT;
    const int32_t topk = c != NULL && c->topk > 0 ? c->topk : 4;
    const int32_t init_blocks = c != NULL ? c->init_blocks : 1, local_blocks = c != NULL ? c->local_blocks : 1;
    const int64_t max_seqlen = c != NULL && c->max_seqlen > 0 ? c->max_seqlen : q->shape[0];
    const double scale = c != NULL && c->scale > 0.0f ? (double)c->scale : 1.0 / sqrt((double)q->shape[2]);
    if (block > M3_BLOCK_MAX || topk > M3_TOPK_MAX || init_blocks < 0 || local_blocks < 0 || max_seqlen <= 0)
        GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "minimax_m3 sparse config out of range");
    if (!isfinite(scale) || scale <= 0.0) GD_FAIL(ctx, GD_ERR_INVALID_ARGUMENT, "minimax_m3 sparse scale must be finite");
    memset(a, 0, sizeof(*a));
    a->scale = (float)scale;
    a->block_size = (uint32_t)block;
    a->topk = (uint32_t)topk;
    a->init_blocks = (uint32_t)init_blocks;
    a->local_blocks = (uint32_t)local_blocks;
    a->max_seqlen = (uint32_t)(max_seqlen > (int64_t)UINT32_MAX ? UINT32_MAX : max_seqlen);
    return GD_OK;
}

#endif
