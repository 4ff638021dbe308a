/*
 * sdpa_varlen forward for gfx950: packed causal / windowed / prefix attention over cu_seqlens
 * (prefill).  Replaces the reference kernel src/ops/sdpa_varlen/metal_sdpa_varlen.metal:137-228;
 * mask :30-55.  q [N,Hq,D], k/v [N,Hkv,D]; segment b covers rows [cu[b], cu[b+1]) and positions
 * are relative to the segment start.  Queries at or past max_seqlen inside a longer segment get
 * zeros (the reference sizes its launch grid from max_seqlen and never reaches them).
 *
 * One wavefront per (query row, head): lane-per-key scores, online softmax over 64-key chunks,
 * lane-per-channel accumulation.
 */
#include "../../_shared/hip_device.h"

#define GD_NEG_INF (-__builtin_inff())

struct gd_hip_sdpa_varlen_params {
    uint32_t n_rows, batch, hq, hkv, dh;
    uint32_t causal, window, prefix_len, max_seqlen;
    float scale;
};

__device__ __forceinline__ bool gd_varlen_allowed(int i, int j, int causal, int window, int prefix_len)
{
    if (causal) {
        if (prefix_len > 0) {
            if (i < prefix_len) {
                if (j >= prefix_len) return false;
            } else if (j > i) {
                return false;
            }
        } else if (j > i) {
            return false;
        }
    }
    if (window > 0) {
        if (prefix_len > 0) {
            if (i >= prefix_len && j >= prefix_len && (i - j) >= window) return false;
        } else if ((i - j) >= window) {
            return false;
        }
    }
    return true;
}

template <typename T>
__global__ void __launch_bounds__(64)
gd_sdpa_varlen_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
                      const int32_t *__restrict__ cu, T *__restrict__ out, gd_hip_sdpa_varlen_params p)
{
    __shared__ float qs[256];
    __shared__ float ps[64];
    const int lane = threadIdx.x;
    const uint32_t hq = blockIdx.x % p.hq;
    const uint32_t n = blockIdx.x / p.hq;
    const int D = (int)p.dh;
    if (cu[0] < 0 || (int32_t)n < cu[0] || (int32_t)n >= cu[p.batch]) return;
    uint32_t lo = 0u, hi = p.batch;
    while (lo + 1u < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (cu[mid] <= (int32_t)n) lo = mid; else hi = mid;
    }
    const int start = cu[lo], end = cu[lo + 1u];
    if (end <= start || (int)n >= end || end > (int)p.n_rows) return;
    const int T_len = end - start;
    const int i = (int)n - start;
    const size_t obase = ((size_t)n * p.hq + hq) * D;
    if (p.max_seqlen > 0u && i >= (int)p.max_seqlen) {
        for (int c = lane; c < D; c += 64) out[obase + c] = (T)0.f;
        return;
    }
    const uint32_t hkv = hq / (p.hq / p.hkv);
    for (int c = lane; c < D; c += 64) qs[c] = (float)q[obase + c];
    __syncthreads();

    int jend = T_len, jbeg = 0;
    if (p.causal) jend = (p.prefix_len > 0u && i < (int)p.prefix_len) ? min(T_len, (int)p.prefix_len) : i + 1;
    if (p.window > 0u && p.prefix_len == 0u) jbeg = max(0, i - (int)p.window + 1) & ~63;
    float m = GD_NEG_INF, l = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int j0 = jbeg; j0 < jend; j0 += 64) {
        const int j = j0 + lane;
        const bool ok = j < jend && gd_varlen_allowed(i, j, (int)p.causal, (int)p.window, (int)p.prefix_len);
        float s = GD_NEG_INF;
        if (ok) {
            const T *kr = k + ((size_t)(start + j) * p.hkv + hkv) * D;
            float dot = 0.f;
            for (int c = 0; c < D; ++c) dot = fmaf(qs[c], (float)kr[c], dot);
            s = dot * p.scale;
        }
        const float cm = gd_wave_max(s);
        if (cm == GD_NEG_INF) continue;
        const float mn = fmaxf(m, cm);
        const float corr = (m == GD_NEG_INF) ? 0.f : expf(m - mn);
        const float pr = ok ? expf(s - mn) : 0.f;
        l = l * corr + gd_wave_sum(pr);
        __syncthreads();
        ps[lane] = pr;
        __syncthreads();
        const int cnt = min(64, jend - j0);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int c = lane + 64 * rr;
            if (c < D) {
                float a = acc[rr] * corr;
                const T *vr = v + ((size_t)(start + j0) * p.hkv + hkv) * D + c;
                for (int jj = 0; jj < cnt; ++jj) a = fmaf(ps[jj], (float)vr[(size_t)jj * p.hkv * D], a);
                acc[rr] = a;
            }
        }
        m = mn;
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        const int c = lane + 64 * rr;
        if (c < D) out[obase + c] = (T)(acc[rr] * inv);
    }
}

extern "C" int gd_hip_launch_sdpa_varlen(hipStream_t stream, const void *q, const void *k, const void *v,
                                         const int32_t *cu, void *out, uint32_t n_rows, uint32_t batch,
                                         uint32_t hq, uint32_t hkv, uint32_t dh, uint32_t causal, uint32_t window,
                                         uint32_t prefix_len, uint32_t max_seqlen, float scale, int is_f16)
{
    gd_hip_sdpa_varlen_params p = {n_rows, batch, hq, hkv, dh, causal, window, prefix_len, max_seqlen, scale};
    const uint64_t blocks = (uint64_t)n_rows * hq;
    if (blocks == 0) return (int)hipSuccess;
    if (is_f16)
        gd_sdpa_varlen_kernel<gd_half><<<(unsigned)blocks, 64, 0, stream>>>(
            (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, cu, (gd_half *)out, p);
    else
        gd_sdpa_varlen_kernel<float><<<(unsigned)blocks, 64, 0, stream>>>(
            (const float *)q, (const float *)k, (const float *)v, cu, (float *)out, p);
    return (int)hipGetLastError();
}
