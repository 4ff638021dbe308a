/*
 * MiniMax-M3 block-sparse attention over packed sequences for gfx950, forward only: the block picker
 * ("lightning indexer") and the attention over the picked blocks.  Semantics restate the reference's
 * Metal kernels src/ops/minimax_m3_index_topk/metal_minimax_m3_index_topk.metal:20-137 and
 * src/ops/minimax_m3_sparse_attention/metal_minimax_m3_sparse_attention.metal:36-113.
 *
 * Both kernels give every query row its own thread, as every row has its own list of blocks: q lives in
 * registers as F16 pairs (products of two halfs are exact in F32, so v_dot2_f32_f16 loses nothing), scores and
 * the softmax state are F32.
 *   picker     one workgroup = 128 consecutive rows of one (sequence, kv head); the keys of the blocks these
 *              rows can see pass through LDS in tiles of 64 (every thread reads the same key: broadcast reads);
 *              the topk list is a register array kept sorted by a branch-free carry pass
 *   attention  64 rows per workgroup; every row walks its blocks in list order with an online softmax and reads
 *              its K / V rows straight from global memory (neighbouring rows mostly share their blocks, so the
 *              lines come from L2)
 * Head sizes 4, 8, 16, 32 and 64 have kernels of their own; any other size up to 64 (odd ones too), and any size
 * whose operands do not start on 16-byte boundaries, runs the size-64 code with ANY set: q, the LDS key tiles and the accumulators are padded with zeros to 64, global rows
 * keep their real stride and are read half by half.  The padding adds exact zeros, so results do not depend on
 * which of the two paths a size takes.
 * Bounds: picker = flops of a causal Q K^T (vector unit, not the matrix cores: a first version); attention =
 * rows x topk x block keys.
 */
#include "../../_shared/hip_device.h"

#define GD_M3_MAX_DH 64
#define GD_M3_MAX_TOPK 16
#define GD_M3_PICK_ROWS 128
#define GD_M3_PICK_TILE 64
#define GD_M3_ATTN_ROWS 64
#define GD_NEG_INF (-__builtin_inff())

struct gd_m3_params {
    uint32_t total, batch, hq, hkv, dh;
    uint32_t max_seqlen, block, topk, init_blocks, local_blocks;
    float scale;
    uint32_t unaligned; /* some operand does not start on a 16-byte boundary: take the half-by-half path */
};

/* q . k over DH halfs, q as pairs in registers, k as 16-byte chunks */
template <int DH>
__device__ __forceinline__ float gd_m3_dot(const gd_half2 (&q)[DH / 2], const gd_half *k)
{
    float d = 0.f;
    if (DH % 8 == 0) {
#pragma unroll
        for (int c = 0; c < DH / 8; ++c) {
            const gd_half8 kv = *reinterpret_cast<const gd_half8 *>(k + 8 * c);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                d = __builtin_amdgcn_fdot2(q[4 * c + e], (gd_half2){kv[2 * e], kv[2 * e + 1]}, d, false);
        }
    } else {
#pragma unroll
        for (int c = 0; c < DH / 2; ++c) d = __builtin_amdgcn_fdot2(q[c], (gd_half2){k[2 * c], k[2 * c + 1]}, d, false);
    }
    return d;
}

/* the same over a global row of dh <= DH halfs at any alignment; the missing tail counts as zeros */
template <int DH>
__device__ __forceinline__ float gd_m3_dot_any(const gd_half2 (&q)[DH / 2], const gd_half *k, int dh)
{
    float d = 0.f;
#pragma unroll
    for (int c = 0; c < DH / 2; ++c) {
        const gd_half k0 = 2 * c < dh ? k[2 * c] : (gd_half)0.f, k1 = 2 * c + 1 < dh ? k[2 * c + 1] : (gd_half)0.f;
        d = __builtin_amdgcn_fdot2(q[c], (gd_half2){k0, k1}, d, false);
    }
    return d;
}

template <int DH, bool ANY>
__global__ void __launch_bounds__(GD_M3_PICK_ROWS)
gd_m3_index_topk_kernel(const gd_half *__restrict__ q, const gd_half *__restrict__ k, const int32_t *__restrict__ cu,
                        int32_t *__restrict__ topk, gd_m3_params p)
{
    __shared__ __attribute__((aligned(16))) gd_half ks[GD_M3_PICK_TILE * DH];
    const int tid = threadIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int start = cu[b], T = cu[b + 1] - start;
    const int q0 = blockIdx.x * GD_M3_PICK_ROWS;
    if (q0 >= T) return;
    const int i = q0 + tid;
    const bool active = i < T && i < (int)p.max_seqlen; /* rows at or beyond max_seqlen are not processed */
    const int block = (int)p.block;
    const int valid = active ? (i + block) / block : 0;
    const int last_row = min(q0 + GD_M3_PICK_ROWS - 1, T - 1);
    const int max_valid = (last_row + block) / block;
    const int local_start = max(0, valid - (int)p.local_blocks);

    const int dh = ANY ? (int)p.dh : DH; /* halfs per row in global memory */
    gd_half2 qh[DH / 2];
    {
        const gd_half *qr = q + ((size_t)(start + (active ? i : 0)) * p.hkv + h) * dh;
#pragma unroll
        for (int c = 0; c < DH / 2; ++c) {
            const gd_half q0v = active && 2 * c < dh ? qr[2 * c] : (gd_half)0.f;
            const gd_half q1v = active && 2 * c + 1 < dh ? qr[2 * c + 1] : (gd_half)0.f;
            qh[c] = (gd_half2){q0v, q1v};
        }
    }
    float score[GD_M3_MAX_TOPK];
    int32_t index[GD_M3_MAX_TOPK];
#pragma unroll
    for (int t = 0; t < GD_M3_MAX_TOPK; ++t) {
        score[t] = GD_NEG_INF;
        index[t] = -1;
    }
    for (int blk = 0; blk < max_valid; ++blk) {
        const int k_begin = blk * block, k_end = min(k_begin + block, T);
        float best = GD_NEG_INF;
        for (int kb = k_begin; kb < k_end; kb += GD_M3_PICK_TILE) {
            const int tile = min(GD_M3_PICK_TILE, k_end - kb);
            __syncthreads(); /* the previous tile has been read */
            if (ANY) {
                for (int idx = tid; idx < tile * DH; idx += GD_M3_PICK_ROWS) {
                    const int jj = idx / DH, c = idx % DH;
                    ks[idx] = c < dh ? k[((size_t)(start + kb + jj) * p.hkv + h) * dh + c] : (gd_half)0.f;
                }
            } else {
                for (int idx = tid; idx < tile * DH / 2; idx += GD_M3_PICK_ROWS) {
                    const int jj = idx / (DH / 2), c = idx % (DH / 2);
                    reinterpret_cast<gd_half2 *>(ks)[idx] =
                        reinterpret_cast<const gd_half2 *>(k + ((size_t)(start + kb + jj) * p.hkv + h) * DH)[c];
                }
            }
            __syncthreads();
            if (blk < valid) {
                const int visible = min(tile, i - kb + 1); /* keys j <= i */
                for (int jj = 0; jj < visible; ++jj) best = fmaxf(best, gd_m3_dot<DH>(qh, ks + jj * DH));
            }
        }
        if (blk < valid) {
            /* fmaxf drops a NaN operand: a block whose every score is NaN stays at -inf, as in the reference.
             * First blocks rank highest, the last visible ones next (also when they are first blocks). */
            if (blk < (int)p.init_blocks) best = 1.0e30f;
            if (p.local_blocks > 0u && blk >= local_start) best = 1.0e29f;
            /* sorted insertion without branches: the candidate takes the first slot it beats; what it pushes
             * out is carried down and takes every following slot (it came from further up, so it wins ties) */
            float cs = best;
            int32_t ci = blk;
            bool carrying = false;
#pragma unroll
            for (int t = 0; t < GD_M3_MAX_TOPK; ++t) {
                if (t < (int)p.topk) {
                    const bool take = carrying || cs > score[t];
                    const float os = score[t];
                    const int32_t oi = index[t];
                    score[t] = take ? cs : os;
                    index[t] = take ? ci : oi;
                    cs = take ? os : cs;
                    ci = take ? oi : ci;
                    carrying = carrying || take;
                }
            }
        }
    }
    if (active) {
        int32_t *out = topk + ((size_t)h * p.total + (size_t)(start + i)) * p.topk;
#pragma unroll
        for (int t = 0; t < GD_M3_MAX_TOPK; ++t) {
            if (t < (int)p.topk) out[t] = t < valid ? index[t] : -1;
        }
    }
}

template <int DH, bool ANY>
__global__ void __launch_bounds__(GD_M3_ATTN_ROWS)
gd_m3_sparse_attention_kernel(const gd_half *__restrict__ q, const gd_half *__restrict__ k,
                              const gd_half *__restrict__ v, const int32_t *__restrict__ cu,
                              const int32_t *__restrict__ topk, gd_half *__restrict__ out, gd_m3_params p)
{
    const int hq = blockIdx.y, b = blockIdx.z;
    const int start = cu[b], T = cu[b + 1] - start;
    const int i = blockIdx.x * GD_M3_ATTN_ROWS + threadIdx.x;
    if (i >= T || i >= (int)p.max_seqlen) return; /* rows at or beyond max_seqlen are not processed */
    const int hkv = hq / (int)(p.hq / p.hkv);
    const size_t qg = (size_t)(start + i);
    const int dh = ANY ? (int)p.dh : DH; /* halfs per row in global memory */
    const gd_half *qr = q + (qg * p.hq + hq) * dh;
    gd_half2 qh[DH / 2];
#pragma unroll
    for (int c = 0; c < DH / 2; ++c)
        qh[c] = (gd_half2){2 * c < dh ? qr[2 * c] : (gd_half)0.f, 2 * c + 1 < dh ? qr[2 * c + 1] : (gd_half)0.f};
    float acc[DH];
#pragma unroll
    for (int c = 0; c < DH; ++c) acc[c] = 0.f;
    float m = GD_NEG_INF, l = 0.f;
    const float scale2 = p.scale * 1.4426950408889634f; /* softmax in the exp2 domain */
    const int32_t *list = topk + ((size_t)hkv * p.total + qg) * p.topk;
    for (uint32_t t = 0; t < p.topk; ++t) {
        const int blk = list[t];
        if (blk < 0) continue;
        const int k_begin = blk * (int)p.block;
        const int k_end = min(min(k_begin + (int)p.block, T), i + 1);
        for (int j = k_begin; j < k_end; ++j) {
            const size_t row = ((size_t)(start + j) * p.hkv + hkv) * dh;
            const float s = (ANY ? gd_m3_dot_any<DH>(qh, k + row, dh) : gd_m3_dot<DH>(qh, k + row)) * scale2;
            const float mn = fmaxf(m, s);
            const float corr = exp2f(m - mn), e = exp2f(s - mn); /* exp2(-inf) = 0 on the first key */
            l = l * corr + e;
            if (ANY) {
#pragma unroll
                for (int c = 0; c < DH; ++c) acc[c] = fmaf(e, c < dh ? (float)v[row + c] : 0.f, acc[c] * corr);
            } else if (DH % 8 == 0) {
#pragma unroll
                for (int c = 0; c < DH / 8; ++c) {
                    const gd_half8 vv = *reinterpret_cast<const gd_half8 *>(v + row + 8 * c);
#pragma unroll
                    for (int x = 0; x < 8; ++x) acc[8 * c + x] = fmaf(e, (float)vv[x], acc[8 * c + x] * corr);
                }
            } else {
#pragma unroll
                for (int c = 0; c < DH; ++c) acc[c] = fmaf(e, (float)v[row + c], acc[c] * corr);
            }
            m = mn;
        }
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
    gd_half *o = out + (qg * p.hq + hq) * dh;
#pragma unroll
    for (int c = 0; c < DH; ++c) {
        if (c < dh) o[c] = (gd_half)(acc[c] * inv);
    }
}

#define GD_M3_DISPATCH(PARAMS, STATEMENT)                                      \
    if ((PARAMS)->dh == 0u || (PARAMS)->dh > GD_M3_MAX_DH) return (int)hipErrorInvalidValue; \
    switch ((PARAMS)->unaligned != 0u ? 0u : (PARAMS)->dh) {                                                      \
    case 4: { constexpr int DH = 4; constexpr bool ANY = false; STATEMENT; break; }   \
    case 8: { constexpr int DH = 8; constexpr bool ANY = false; STATEMENT; break; }   \
    case 16: { constexpr int DH = 16; constexpr bool ANY = false; STATEMENT; break; } \
    case 32: { constexpr int DH = 32; constexpr bool ANY = false; STATEMENT; break; } \
    case 64: { constexpr int DH = 64; constexpr bool ANY = false; STATEMENT; break; } \
    default: { constexpr int DH = GD_M3_MAX_DH; constexpr bool ANY = true; STATEMENT; break; } \
    }

extern "C" int gd_hip_launch_m3_index_topk(hipStream_t stream, const void *q, const void *k, const int32_t *cu,
                                           int32_t *topk, const gd_m3_params *p)
{
    const dim3 grid((p->max_seqlen + GD_M3_PICK_ROWS - 1u) / GD_M3_PICK_ROWS, p->hkv, p->batch);
    GD_M3_DISPATCH(p, (gd_m3_index_topk_kernel<DH, ANY><<<grid, GD_M3_PICK_ROWS, 0, stream>>>(
                              (const gd_half *)q, (const gd_half *)k, cu, topk, *p)));
    return (int)hipGetLastError();
}

extern "C" int gd_hip_launch_m3_sparse_attention(hipStream_t stream, const void *q, const void *k, const void *v,
                                                 const int32_t *cu, const int32_t *topk, void *out,
                                                 const gd_m3_params *p)
{
    const dim3 grid((p->max_seqlen + GD_M3_ATTN_ROWS - 1u) / GD_M3_ATTN_ROWS, p->hq, p->batch);
    GD_M3_DISPATCH(p, (gd_m3_sparse_attention_kernel<DH, ANY><<<grid, GD_M3_ATTN_ROWS, 0, stream>>>(
                              (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, cu, topk, (gd_half *)out, *p)));
    return (int)hipGetLastError();
}
