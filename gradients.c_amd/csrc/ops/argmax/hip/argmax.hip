/*
 * Greedy next-token selection on the device for gfx950.  One workgroup per logits row;
 * HBM-bound (reads rows*cols values once).  Semantics restate the reference's host scan
 * examples/gpt_lm/gpt_lm_shared.c:1388-1400: largest finite value, lowest index on ties,
 * index 0 when the row holds no finite value.  Also returns best - runner-up (+inf when the row
 * has fewer than two finite values) so near-ties can be reported.
 */
#include "../../_shared/hip_device.h"

#define GD_ARGMAX_THREADS 256
#define GD_NEG_INF (-__builtin_inff())

struct gd_top2 {
    float best, second;
    int32_t idx; /* -1: nothing finite yet */
};

__device__ __forceinline__ void gd_top2_push(gd_top2 &t, float v, int32_t i)
{
    if (!isfinite(v)) return;
    if (t.idx < 0 || v > t.best || (v == t.best && i < t.idx)) {
        if (t.idx >= 0) t.second = fmaxf(t.second, t.best);
        t.best = v;
        t.idx = i;
    } else {
        t.second = fmaxf(t.second, v);
    }
}

__device__ __forceinline__ gd_top2 gd_top2_merge(const gd_top2 &a, const gd_top2 &b)
{
    if (a.idx < 0) return b;
    if (b.idx < 0) return a;
    gd_top2 r;
    const bool a_wins = a.best > b.best || (a.best == b.best && a.idx < b.idx);
    r.best = a_wins ? a.best : b.best;
    r.idx = a_wins ? a.idx : b.idx;
    r.second = fmaxf(fmaxf(a.second, b.second), a_wins ? b.best : a.best);
    return r;
}

template <typename T>
__global__ void __launch_bounds__(GD_ARGMAX_THREADS)
gd_argmax_rows_kernel(const T *__restrict__ logits, int32_t *__restrict__ ids, float *__restrict__ gap,
                      uint64_t cols)
{
    __shared__ gd_top2 sm[GD_ARGMAX_THREADS / 64];
    const T *row = logits + (uint64_t)blockIdx.x * cols;
    gd_top2 t;
    t.best = GD_NEG_INF;
    t.second = GD_NEG_INF;
    t.idx = -1;
    for (uint64_t c = threadIdx.x; c < cols; c += GD_ARGMAX_THREADS) gd_top2_push(t, (float)row[c], (int32_t)c);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        gd_top2 o;
        o.best = __shfl_xor(t.best, off, 64);
        o.second = __shfl_xor(t.second, off, 64);
        o.idx = __shfl_xor(t.idx, off, 64);
        t = gd_top2_merge(t, o);
    }
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = t;
    __syncthreads();
    if (threadIdx.x == 0) {
        gd_top2 r = sm[0];
        for (int w = 1; w < GD_ARGMAX_THREADS / 64; ++w) r = gd_top2_merge(r, sm[w]);
        ids[blockIdx.x] = r.idx < 0 ? 0 : r.idx;
        if (gap != nullptr)
            gap[blockIdx.x] = (r.idx >= 0 && r.second > GD_NEG_INF) ? r.best - r.second : __builtin_inff();
    }
}

extern "C" int gd_hip_launch_argmax_rows(hipStream_t stream, const void *logits, int32_t *ids, float *gap,
                                         uint64_t rows, uint64_t cols, int is_f16)
{
    if (rows == 0) return (int)hipSuccess;
    if (is_f16)
        gd_argmax_rows_kernel<gd_half><<<(unsigned)rows, GD_ARGMAX_THREADS, 0, stream>>>((const gd_half *)logits, ids, gap, cols);
    else
        gd_argmax_rows_kernel<float><<<(unsigned)rows, GD_ARGMAX_THREADS, 0, stream>>>((const float *)logits, ids, gap, cols);
    return (int)hipGetLastError();
}
