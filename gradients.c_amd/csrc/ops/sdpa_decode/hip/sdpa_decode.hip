/*
 * sdpa_decode for gfx950: attention of the newest query token(s) over the K/V cache.
 *
 * Replaces the reference kernels src/ops/sdpa_decode/metal_sdpa_decode.metal:86-175
 * (Tq=1 window fast path) and :177-281 (general path, one active thread per query).
 *
 * The path is HBM-bound: every live K and V row is read once (algorithmic bytes =
 * sum_b T_b * Hkv * D * 2 * 2 + q/out).  Split-KV kernel, F16, Tq == 1:
 *   - grid (nsplit, Hkv, B); a workgroup of 4 wavefronts owns `chunk` consecutive keys of one
 *     (batch, kv head) and all G = Hq/Hkv query heads that share it, so K/V bytes are read once;
 *   - a wavefront load covers 64 lanes x 16 B = 1 KiB: D/8 lanes hold one key row (8 halfs each),
 *     so one instruction fetches 8 (D=64) or 4 (D=128) whole rows, each a full 128/256-byte line;
 *   - the dot product is reduced over the D/8 lanes of a row with shuffles; every row slot keeps
 *     its own running max/sum (online softmax in the exp2 domain) and an F32 accumulator for its
 *     8 channels, so the inner loop has no cross-slot traffic;
 *   - slots are merged with shuffles, wavefronts through LDS; with nsplit == 1 the result is
 *     normalised and stored as F16 directly, otherwise (max, sum, acc) partials go to a
 *     workspace and a small combine kernel finishes.
 * Ragged batches with at least one (row, kv head) pair per compute unit take the same kernel in its PIECES form
 * (sdpa_decode_pieces.hip): persistent workgroups walk pieces of the rows and the last piece of a row to arrive
 * merges it, one launch.
 * Everything else (F32 caches, Tq > 1, other head sizes) takes the generic
 * kernel: one wavefront per query row, lane-per-key scores, lane-per-channel accumulation.
 *
 * Semantics (both kernels): live = min(pos + Tq, Tmax), query position pos + i, mask
 * reference metal_sdpa_decode.metal:30-53, out = 0 when no key is visible, rows with a
 * negative position are left untouched.
 */
#include "sdpa_decode_split_kernel.h"

template <int D>
__global__ void __launch_bounds__(D)
gd_sdpa_decode_combine_kernel(const float *__restrict__ ws, const int32_t *__restrict__ pos_ptr,
                              gd_half *__restrict__ out, gd_hip_sdpa_decode_params p)
{
    const int hq = blockIdx.x, b = blockIdx.y, c = threadIdx.x;
    if (gd_decode_pos(pos_ptr, p, b) < 0) return;
    const float *w = ws + GD_HIP_SDPA_COUNTER_SLOTS + ((size_t)b * p.hq + hq) * p.nsplit * (D + 2);
    float mm = GD_NEG_INF;
    for (uint32_t s = 0; s < p.nsplit; ++s) mm = fmaxf(mm, w[(size_t)s * (D + 2)]);
    float ll = 0.f, aa = 0.f;
    for (uint32_t s = 0; s < p.nsplit; ++s) {
        const float ms = w[(size_t)s * (D + 2)];
        if (ms == GD_NEG_INF) continue;
        const float cw = exp2f(ms - mm);
        ll += w[(size_t)s * (D + 2) + 1] * cw;
        aa += w[(size_t)s * (D + 2) + 2 + c] * cw;
    }
    out[((size_t)b * p.hq + hq) * D + c] = (gd_half)(ll > 0.f ? aa / ll : 0.f);
}

/* ---- generic kernel -------------------------------------------------------------- */

template <typename T>
__global__ void __launch_bounds__(64)
gd_sdpa_decode_generic_kernel(const T *__restrict__ q, const T *__restrict__ kc, const T *__restrict__ vc,
                              const int32_t *__restrict__ pos_ptr, T *__restrict__ out,
                              gd_hip_sdpa_decode_params p)
{
    __shared__ float qs[256];
    __shared__ float ps[64];
    const int lane = threadIdx.x;
    int r = blockIdx.x;
    const int i = r % (int)p.tq;
    r /= (int)p.tq;
    const int hq = r % (int)p.hq;
    const int b = r / (int)p.hq;
    const int pos = gd_decode_pos(pos_ptr, p, b);
    if (pos < 0) return;
    const int D = (int)p.dh;
    const int hkv = hq / (int)(p.hq / p.hkv);
    const int live = (int)min((long long)pos + (long long)p.tq, (long long)p.tmax);
    const int qpos = pos + i;
    const size_t qbase = (((size_t)b * p.tq + i) * p.hq + hq) * D;
    for (int c = lane; c < D; c += 64) qs[c] = (float)q[qbase + c];
    __syncthreads();

    float m = GD_NEG_INF, l = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
    int jstart = 0;
    if (p.window > 0u && p.prefix_len == 0u) jstart = max(0, qpos - (int)p.window + 1) & ~63;
    for (int j0 = jstart; j0 < live; j0 += 64) {
        const int j = j0 + lane;
        const bool ok = j < live && gd_attn_allowed(qpos, j, (int)p.window, (int)p.prefix_len);
        float s = GD_NEG_INF;
        if (ok) {
            const T *kr = kc + (((size_t)b * p.tmax + j) * p.hkv + hkv) * D;
            float dot = 0.f;
            for (int c = 0; c < D; ++c) dot = fmaf(qs[c], (float)kr[c], dot);
            s = dot * p.scale;
        }
        const float cm = gd_wave_max(s);
        if (cm == GD_NEG_INF) continue; /* uniform across the wavefront */
        const float mn = fmaxf(m, cm);
        const float corr = (m == GD_NEG_INF) ? 0.f : expf(m - mn);
        const float pr = ok ? expf(s - mn) : 0.f;
        l = l * corr + gd_wave_sum(pr);
        __syncthreads();
        ps[lane] = pr;
        __syncthreads();
        const int n = min(64, live - j0);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int c = lane + 64 * rr;
            if (c < D) {
                float a = acc[rr] * corr;
                const T *vr = vc + (((size_t)b * p.tmax + j0) * p.hkv + hkv) * D + c;
                for (int jj = 0; jj < n; ++jj) a = fmaf(ps[jj], (float)vr[(size_t)jj * p.hkv * D], a);
                acc[rr] = a;
            }
        }
        m = mn;
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        const int c = lane + 64 * rr;
        if (c < D) out[qbase + c] = (T)(acc[rr] * inv);
    }
}

/* ---- fixed scratch of the entry point that allocates nothing ------------------------------ */

/* Split-KV partial results of gd_backend_sdpa_decode_positions_noalloc live here instead of a hipMalloc'd
 * workspace.  Every device that loads this code object holds its own copy at its own address until the
 * process ends; the address is looked up once per device (with that device current) and kept, and host code
 * uses the kept pointer only: the array's name is a host-side stand-in, not a device address.  The split
 * kernel writes (max, sum) of every (row, head, split) slot, also of splits without keys, and the combine
 * kernel skips the accumulator of such a slot, so nothing has to be cleared between calls. */
static __device__ __align__(256) float scratch[GD_HIP_SDPA_NOALLOC_SCRATCH_BYTES / sizeof(float)];
static float *gd_scratch_ptr[GD_HIP_SDPA_MAX_DEVICES];

extern "C" int gd_hip_sdpa_decode_scratch_init(int device)
{
    float *ptr = nullptr;
    if (device < 0 || device >= GD_HIP_SDPA_MAX_DEVICES) return (int)hipErrorInvalidDevice;
    if (gd_scratch_ptr[device] != nullptr) return (int)hipSuccess;
    const hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    gd_scratch_ptr[device] = ptr;
    return (int)hipSuccess;
}

/* NULL until gd_hip_sdpa_decode_scratch_init(device) has succeeded. */
extern "C" float *gd_hip_sdpa_decode_scratch(int device)
{
    return device >= 0 && device < GD_HIP_SDPA_MAX_DEVICES ? gd_scratch_ptr[device] : nullptr;
}

/* ---- launchers ----------------------------------------------------------------------- */

template <int D, int G>
static int launch_split(hipStream_t stream, const void *q, const void *k, const void *v, const int32_t *pos,
                        void *out, float *ws, const gd_hip_sdpa_decode_params &p)
{
    dim3 grid(p.nsplit, p.hkv, p.batch);
#define GD_GO(W, U)                                                                                          \
    do {                                                                                                     \
        if (p.nontemporal && p.window == 0u)                                                                 \
            gd_sdpa_decode_split_kernel<D, G, W, U, true, false, false, true><<<grid, W * 64, 0, stream>>>(   \
                (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, ws, p);        \
        else if (p.nontemporal)                                                                              \
            gd_sdpa_decode_split_kernel<D, G, W, U, true><<<grid, W * 64, 0, stream>>>(                       \
                (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, ws, p);        \
        else if (p.window == 0u)                                                                             \
            gd_sdpa_decode_split_kernel<D, G, W, U, false, false, false, true><<<grid, W * 64, 0, stream>>>(  \
                (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, ws, p);        \
        else                                                                                                 \
            gd_sdpa_decode_split_kernel<D, G, W, U, false><<<grid, W * 64, 0, stream>>>(                      \
                (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, ws, p);        \
    } while (0)
    if (p.prefix_len > 0u) {
        /* one instantiation per wavefront count: the tunables for trip length and streaming loads do not apply */
        constexpr int U = G == 1 ? 2 : 4;
        if (G == 1 && p.waves == 8u)
            gd_sdpa_decode_split_kernel<D, G, 8, U, false, true><<<grid, 8 * 64, 0, stream>>>(
                (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, ws, p);
        else
            gd_sdpa_decode_split_kernel<D, G, 4, U, false, true><<<grid, 4 * 64, 0, stream>>>(
                (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, ws, p);
    } else if constexpr (G == 1) {
        if (p.waves == 8u && p.unroll == 8u) GD_GO(8, 8);
        else if (p.waves == 8u && p.unroll == 2u) GD_GO(8, 2);
        else if (p.waves == 8u) GD_GO(8, 4);
        else if (p.unroll == 8u) GD_GO(4, 8);
        else if (p.unroll == 2u) GD_GO(4, 2);
        else GD_GO(4, 4);
    } else {
        GD_GO(4, 4);
    }
#undef GD_GO
    if (p.nsplit > 1u) {
        dim3 cgrid(p.hq, p.batch);
        gd_sdpa_decode_combine_kernel<D><<<cgrid, D, 0, stream>>>(ws, pos, (gd_half *)out, p);
    }
    return (int)hipGetLastError();
}

/* Returns hipErrorInvalidValue when (D, G) has no split-KV instantiation. */
extern "C" int gd_hip_launch_sdpa_decode_split(hipStream_t stream, const void *q, const void *k, const void *v,
                                               const int32_t *pos, void *out, float *ws,
                                               const gd_hip_sdpa_decode_params *params)
{
    const gd_hip_sdpa_decode_params &p = *params;
    const uint32_t g = p.hq / p.hkv;
#define GD_CASE(DD, GG) if (p.dh == DD && g == GG) return launch_split<DD, GG>(stream, q, k, v, pos, out, ws, p)
    GD_CASE(64, 1); GD_CASE(64, 2); GD_CASE(64, 3); GD_CASE(64, 4); GD_CASE(64, 6); GD_CASE(64, 8);
    GD_CASE(128, 1); GD_CASE(128, 2); GD_CASE(128, 3); GD_CASE(128, 4); GD_CASE(128, 6); GD_CASE(128, 8);
#undef GD_CASE
    return (int)hipErrorInvalidValue;
}

extern "C" int gd_hip_launch_sdpa_decode_generic(hipStream_t stream, const void *q, const void *k, const void *v,
                                                 const int32_t *pos, void *out,
                                                 const gd_hip_sdpa_decode_params *params)
{
    const gd_hip_sdpa_decode_params &p = *params;
    const unsigned blocks = p.batch * p.hq * p.tq;
    if (p.dtype == 1u)
        gd_sdpa_decode_generic_kernel<gd_half><<<blocks, 64, 0, stream>>>(
            (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, p);
    else
        gd_sdpa_decode_generic_kernel<float><<<blocks, 64, 0, stream>>>(
            (const float *)q, (const float *)k, (const float *)v, pos, (float *)out, p);
    return (int)hipGetLastError();
}
