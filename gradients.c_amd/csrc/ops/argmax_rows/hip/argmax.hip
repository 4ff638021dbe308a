/*
 * Greedy next-token selection on the device for gfx950.  One workgroup per logits row;
 * HBM-bound (reads rows*cols values once).  Semantics restate the reference's host scan
 * examples/gpt_lm/gpt_lm_shared.c:1388-1400: largest finite value, lowest index on ties,
 * index 0 when the row holds no finite value.  Also returns best - runner-up (+inf when the row
 * has fewer than two finite values) so near-ties can be reported.
 */
#include "../../_shared/hip_device.h"

#define GD_ARGMAX_MAX_THREADS 1024 /* long rows; short rows run with 256 */
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

/* what a device-resident decode loop does with the chosen token, per row (one workgroup per row, so every
 * row keeps its own step counter) */
struct gd_hip_advance {
    int32_t *positions;     /* [rows] += pos_delta */
    int32_t *step_counters; /* [rows]: s = counter, record into slot s when s < max_steps, counter = s + 1 */
    int32_t *out_ids;       /* [max_steps * rows] */
    float *out_gaps;        /* [max_steps * rows] or NULL */
    uint32_t max_steps;
    int32_t pos_delta;
    /* optional: the chosen token's embedding row is copied to row b of next_x (the next step's input) */
    const unsigned char *table; /* [vocab, row_bytes] */
    unsigned char *next_x;      /* [rows, row_bytes] */
    uint32_t row_bytes;         /* multiple of 16 */
};

template <typename T, bool ADVANCE>
__global__ void __launch_bounds__(GD_ARGMAX_MAX_THREADS)
gd_argmax_rows_kernel(const T *__restrict__ logits, int32_t *__restrict__ ids, float *__restrict__ gap,
                      uint64_t cols, gd_hip_advance adv)
{
    __shared__ gd_top2 sm[GD_ARGMAX_MAX_THREADS / 64];
    __shared__ int32_t s_token;
    const T *row = logits + (uint64_t)blockIdx.x * cols;
    gd_top2 t;
    t.best = GD_NEG_INF;
    t.second = GD_NEG_INF;
    t.idx = -1;
    const uint32_t threads = blockDim.x;
    /* the row's step counter and position are requested here, in front of the scan, so that the pick at the end is not
     * followed by two more dependent round trips */
    int32_t counter = 0, position = 0;
    if (ADVANCE && threadIdx.x == 0) {
        counter = adv.step_counters[blockIdx.x];
        position = adv.positions[blockIdx.x];
    }
    uint64_t done = 0; /* columns covered by the vector part */
    if (sizeof(T) == 2 && (reinterpret_cast<uintptr_t>(row) & 15u) == 0u) {
        /* 8 halfs per lane and trip; lane-major order keeps the lowest-index rule: pushes of one lane ascend */
        const uint64_t whole = cols & ~(uint64_t)7;
        for (uint64_t c = (uint64_t)threadIdx.x * 8u; c < whole; c += (uint64_t)threads * 8u) {
            const gd_half8 v = *reinterpret_cast<const gd_half8 *>(row + c);
#pragma unroll
            for (int e = 0; e < 8; ++e) gd_top2_push(t, (float)v[e], (int32_t)(c + e));
        }
        done = whole;
    }
    for (uint64_t c = done + threadIdx.x; c < cols; c += threads) gd_top2_push(t, (float)row[c], (int32_t)c);
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
        for (uint32_t w = 1; w < threads / 64u; ++w) r = gd_top2_merge(r, sm[w]);
        const int32_t token = r.idx < 0 ? 0 : r.idx;
        const float g = (r.idx >= 0 && r.second > GD_NEG_INF) ? r.best - r.second : __builtin_inff();
        ids[blockIdx.x] = token;
        if (gap != nullptr) gap[blockIdx.x] = g;
        if (ADVANCE) {
            const int32_t s = counter;
            adv.positions[blockIdx.x] = position + adv.pos_delta;
            if (s >= 0 && (uint32_t)s < adv.max_steps) {
                adv.out_ids[(size_t)s * gridDim.x + blockIdx.x] = token;
                if (adv.out_gaps != nullptr) adv.out_gaps[(size_t)s * gridDim.x + blockIdx.x] = g;
            }
            adv.step_counters[blockIdx.x] = s + 1;
            s_token = token;
        }
    }
    if (ADVANCE && adv.table != nullptr) {
        __syncthreads();
        const gd_u128 *src = reinterpret_cast<const gd_u128 *>(adv.table + (size_t)s_token * adv.row_bytes);
        gd_u128 *dst = reinterpret_cast<gd_u128 *>(adv.next_x + (size_t)blockIdx.x * adv.row_bytes);
        for (uint32_t c = threadIdx.x; c < adv.row_bytes / 16u; c += threads) dst[c] = src[c];
    }
}

extern "C" int gd_hip_launch_argmax_rows(hipStream_t stream, const void *logits, int32_t *ids, float *gap,
                                         uint64_t rows, uint64_t cols, int is_f16)
{
    const gd_hip_advance none = {nullptr, nullptr, nullptr, nullptr, 0u, 0, nullptr, nullptr, 0u};
    if (rows == 0) return (int)hipSuccess;
    if (is_f16)
        gd_argmax_rows_kernel<gd_half, false><<<(unsigned)rows, cols >= 8192u ? GD_ARGMAX_MAX_THREADS : 256, 0, stream>>>((const gd_half *)logits, ids, gap, cols, none);
    else
        gd_argmax_rows_kernel<float, false><<<(unsigned)rows, cols >= 8192u ? GD_ARGMAX_MAX_THREADS : 256, 0, stream>>>((const float *)logits, ids, gap, cols, none);
    return (int)hipGetLastError();
}

extern "C" int gd_hip_launch_argmax_advance(hipStream_t stream, const void *logits, int32_t *ids, uint64_t rows,
                                            uint64_t cols, int is_f16, int32_t *positions, int32_t *step_counters,
                                            int32_t *out_ids, float *out_gaps, uint32_t max_steps, int32_t pos_delta,
                                            const void *table, void *next_x, uint32_t row_bytes)
{
    const gd_hip_advance adv = {positions, step_counters, out_ids, out_gaps, max_steps, pos_delta,
                                (const unsigned char *)table, (unsigned char *)next_x, row_bytes};
    if (rows == 0) return (int)hipSuccess;
    if (is_f16)
        gd_argmax_rows_kernel<gd_half, true><<<(unsigned)rows, cols >= 8192u ? GD_ARGMAX_MAX_THREADS : 256, 0, stream>>>((const gd_half *)logits, ids, nullptr, cols, adv);
    else
        gd_argmax_rows_kernel<float, true><<<(unsigned)rows, cols >= 8192u ? GD_ARGMAX_MAX_THREADS : 256, 0, stream>>>((const float *)logits, ids, nullptr, cols, adv);
    return (int)hipGetLastError();
}
