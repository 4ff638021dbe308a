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
 * Everything else (F32 caches, Tq > 1, other head sizes) takes the generic
 * kernel: one wavefront per query row, lane-per-key scores, lane-per-channel accumulation.
 *
 * Semantics (both kernels): live = min(pos + Tq, Tmax), query position pos + i, mask
 * reference metal_sdpa_decode.metal:30-53, out = 0 when no key is visible, rows with a
 * negative position are left untouched.
 */
#include "sdpa_decode_device.h"

/* PFX: a prefix of always-visible keys in front of the window (prefix_len > 0).  The visible keys are then two
 * runs, [0, a_len) and [b0, live); the kernel walks a virtual index over both (v < a_len: key v, else key
 * v - a_len + b0) and the split of the range counts virtual indices.  Without PFX there is one run and the index is
 * the key row itself. */
template <int D, int G, int WAVES, int UNROLL, bool NT, bool PFX = false>
__global__ void __launch_bounds__(WAVES * 64)
gd_sdpa_decode_split_kernel(const gd_half *__restrict__ q, const gd_half *__restrict__ kc,
                            const gd_half *__restrict__ vc, const int32_t *__restrict__ pos_ptr,
                            gd_half *__restrict__ out, float *__restrict__ ws, gd_hip_sdpa_decode_params p)
{
    constexpr int LPK = D / 8;      /* lanes per key row */
    constexpr int KPW = 64 / LPK;   /* key rows per wavefront load */
    constexpr int KPB = KPW * WAVES;
    /* Every kernel argument this path reads is requested from the argument segment here, in one batch with
     * one wait.  Left to the compiler, each load sits in front of its first use behind the early exits, and
     * a wavefront goes through five dependent round trips before its first K/V load. */
    asm volatile("" ::"s"(q), "s"(kc), "s"(vc), "s"(pos_ptr), "s"(out), "s"(ws), "s"(p.tmax), "s"(p.hq), "s"(p.hkv),
                 "s"(p.window), "s"(p.pos_mode), "s"(p.cache_pos), "s"(p.scale), "s"(p.chunk), "s"(p.nsplit));
    const int split = blockIdx.x, hkv = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int slot = lane / LPK, sub = lane % LPK;

    const int pos = gd_decode_pos(pos_ptr, p, b);
    if (pos < 0) return;
    const int live = min(pos + 1, (int)p.tmax);
    const int first = p.window > 0u ? max(0, pos - (int)p.window + 1) : 0;
    /* reference mask (metal_sdpa_decode.metal:25-52): a query inside the prefix sees the prefix keys that exist; one
     * behind it sees the whole prefix plus its window (everything up to itself without a window) */
    const int a_len = PFX ? min((int)p.prefix_len, live) : 0;
    const int b0 = PFX ? (pos < (int)p.prefix_len ? live : min(max(a_len, first), live)) : first;
    const int r0 = PFX ? split * (int)p.chunk : first + split * (int)p.chunk;
    const int r1 = PFX ? min(r0 + (int)p.chunk, a_len + live - b0) : min(r0 + (int)p.chunk, live);
    float *ws_row = ws + (((size_t)b * p.hq + (size_t)hkv * G) * p.nsplit + split) * (D + 2);
    if (r0 >= r1) {
        if (p.nsplit > 1u) {
            if (threadIdx.x < G) {
                float *w = ws_row + (size_t)threadIdx.x * p.nsplit * (D + 2);
                w[0] = GD_NEG_INF;
                w[1] = 0.f;
            }
        } else {
            for (int idx = threadIdx.x; idx < G * D; idx += WAVES * 64)
                out[((size_t)b * p.hq + (size_t)hkv * G) * D + idx] = (gd_half)0.f;
        }
        return;
    }

    /* Addresses: one scalar base per cache for this (batch row, kv head), plus a 32-bit byte offset per lane
     * made by one 24-bit multiply-add (the host checks that tmax, the row pitch and their product fit).  The
     * four wavefronts of a SIMD start together and share its issue slots, so every vector instruction in
     * front of the first row loads delays all of them. */
    const uint32_t pitch = p.hkv * (uint32_t)(D * 2); /* bytes between consecutive keys */
    const size_t slab = ((size_t)b * p.tmax * p.hkv + (size_t)hkv) * (size_t)(D * 2);
    const unsigned char *kslab = reinterpret_cast<const unsigned char *>(kc) + slab;
    const unsigned char *vslab = reinterpret_cast<const unsigned char *>(vc) + slab;
    const uint32_t lane_off = (uint32_t)sub * 16u;

    /* Row loads of trip t+1 are issued before the arithmetic of trip t (two register buffers), so
     * the memory pipe stays busy while the wavefront computes.  All K rows of a trip are requested before
     * its V rows: the scores need every K row, the accumulation takes the V rows one by one.  s0: the
     * wavefront's first row of the trip (scalar); rows past the range re-read the last row and are masked
     * in the arithmetic. */
    auto load_trip = [&](gd_half8 (&kv)[UNROLL], gd_half8 (&vv)[UNROLL], int s0) __attribute__((always_inline)) {
        uint32_t off[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            int row = min(s0 + u * KPB + slot, r1 - 1);
            if (PFX) row = row < a_len ? row : row - a_len + b0;
            off[u] = __umul24((uint32_t)row, pitch) + lane_off;
        }
        /* every cache row is read exactly once per launch: optionally mark the loads streaming */
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const gd_half8 *kp = reinterpret_cast<const gd_half8 *>(kslab + off[u]);
            kv[u] = NT ? __builtin_nontemporal_load(kp) : *kp;
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const gd_half8 *vp = reinterpret_cast<const gd_half8 *>(vslab + off[u]);
            vv[u] = NT ? __builtin_nontemporal_load(vp) : *vp;
        }
    };

    constexpr int STEP = KPB * UNROLL;
    /* trips are decided per wavefront (scalar branches), rows past the range are masked per lane */
    const int jw = r0 + wave * KPW;
    const bool any_rows = jw < r1;
    gd_half8 kA[UNROLL], vA[UNROLL], kB[UNROLL], vB[UNROLL];
    if (any_rows) load_trip(kA, vA, jw);
    __builtin_amdgcn_sched_barrier(0); /* nothing below moves in front of the first loads */

    /* query rows of the G heads that share this kv head stay in F16: products of two halfs are
     * exact in F32, so v_dot2_f32_f16 loses nothing; the softmax scale (exp2 domain) is applied
     * to the reduced dot product */
    const float qscale = p.scale * 1.4426950408889634f;
    gd_half2 qh[G][4];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const gd_half8 qv = *reinterpret_cast<const gd_half8 *>(q + ((size_t)b * p.hq + (size_t)hkv * G + g) * D + sub * 8);
#pragma unroll
        for (int e = 0; e < 4; ++e) qh[g][e] = (gd_half2){qv[2 * e], qv[2 * e + 1]};
    }

    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = GD_NEG_INF;
        l[g] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
    }

    auto compute_trip = [&](const gd_half8 (&kv)[UNROLL], const gd_half8 (&vv)[UNROLL], int s0)
        __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            /* scores of the UNROLL rows, then one rescale of the running state for all of them */
            float sc[UNROLL];
            float mt = GD_NEG_INF;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                float d = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    d = __builtin_amdgcn_fdot2(qh[g][e], (gd_half2){kv[u][2 * e], kv[u][2 * e + 1]}, d, false);
                d = gd_row_group_sum<LPK>(d);
                sc[u] = (s0 + u * KPB + slot < r1) ? d * qscale : GD_NEG_INF;
                mt = fmaxf(mt, sc[u]);
            }
            /* a lane whose rows of this and all earlier trips lie past the range has mt = m = -inf: the
             * reference point 0 then makes every factor below exp2(-inf) = 0 instead of exp2(nan) */
            const float mx = fmaxf(m[g], mt);
            const float mn = mx == GD_NEG_INF ? 0.f : mx;
            const float corr = exp2f(m[g] - mn); /* exp2(-inf) = 0 on the first trip */
            float lsum = l[g] * corr;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[g][e] *= corr;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const float pr = exp2f(sc[u] - mn); /* 0 for rows past the range */
                lsum += pr;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(pr, (float)vv[u][e], acc[g][e]);
            }
            l[g] = lsum;
            m[g] = mx;
        }
    };

    if (any_rows) {
        int sa = jw; /* first row of the wavefront's trip, the same in every lane */
        /* The arithmetic of a trip is written once per branch on purpose: where the two paths (a further trip
         * was requested / was not) meet in front of shared code, the compiler has to wait for ALL outstanding
         * loads there, and every wavefront would start computing only after its last row has arrived. */
        while (true) {
            const int sb = sa + STEP;
            if (sb < r1) {
                load_trip(kB, vB, sb);
                compute_trip(kA, vA, sa);
            } else {
                compute_trip(kA, vA, sa);
                break;
            }
            sa = sb + STEP;
            if (sa < r1) {
                load_trip(kA, vA, sa);
                compute_trip(kB, vB, sb);
            } else {
                compute_trip(kB, vB, sb);
                break;
            }
        }
    }

    /* merge the KPW row slots of the wavefront: common maximum first, one rescale, then plain sums; every
     * lane of the wavefront ends up with the totals.  Exchanges stay in the vector unit: a rotation inside
     * the 16-lane row (distance 8) and the row / half swaps of gfx950 (distances 16 and 32). */
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const float mw = gd_slot_max<LPK>(m[g]);
        const float c = (m[g] == GD_NEG_INF) ? 0.f : exp2f(m[g] - mw);
        l[g] = gd_slot_sum<LPK>(l[g] * c);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = gd_slot_sum<LPK>(acc[g][e] * c);
        m[g] = mw;
    }

    /* merge the wavefronts through LDS */
    __shared__ float sm_acc[WAVES][G][D];
    __shared__ float sm_m[WAVES][G], sm_l[WAVES][G];
    if (slot == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
            for (int e = 0; e < 8; ++e) sm_acc[wave][g][sub * 8 + e] = acc[g][e];
            if (sub == 0) {
                sm_m[wave][g] = m[g];
                sm_l[wave][g] = l[g];
            }
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * D; idx += WAVES * 64) {
        const int g = idx / D, c = idx % D;
        float mm = GD_NEG_INF;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) mm = fmaxf(mm, sm_m[w][g]);
        float ll = 0.f, aa = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float cw = (sm_m[w][g] == GD_NEG_INF) ? 0.f : exp2f(sm_m[w][g] - mm);
            ll += sm_l[w][g] * cw;
            aa += sm_acc[w][g][c] * cw;
        }
        if (p.nsplit > 1u) {
            float *w = ws_row + (size_t)g * p.nsplit * (D + 2);
            w[2 + c] = aa;
            if (c == 0) {
                w[0] = mm;
                w[1] = ll;
            }
        } else {
            out[((size_t)b * p.hq + (size_t)hkv * G + g) * D + c] = (gd_half)(ll > 0.f ? aa / ll : 0.f);
        }
    }
}

template <int D>
__global__ void __launch_bounds__(D)
gd_sdpa_decode_combine_kernel(const float *__restrict__ ws, const int32_t *__restrict__ pos_ptr,
                              gd_half *__restrict__ out, gd_hip_sdpa_decode_params p)
{
    const int hq = blockIdx.x, b = blockIdx.y, c = threadIdx.x;
    if (gd_decode_pos(pos_ptr, p, b) < 0) return;
    const float *w = ws + ((size_t)b * p.hq + hq) * p.nsplit * (D + 2);
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
#define GD_GO(W, U)                                                                                   \
    do {                                                                                              \
        if (p.nontemporal)                                                                            \
            gd_sdpa_decode_split_kernel<D, G, W, U, true><<<grid, W * 64, 0, stream>>>(                \
                (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, ws, p); \
        else                                                                                          \
            gd_sdpa_decode_split_kernel<D, G, W, U, false><<<grid, W * 64, 0, stream>>>(               \
                (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, ws, p); \
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
