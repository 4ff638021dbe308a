/*
 * sdpa_decode for rows of very different lengths (per-row positions, long caches): the same arithmetic as the
 * split-KV kernel of sdpa_decode.hip, with the keys dealt to the workgroups by COUNT instead of by row.
 *
 * Replaces the reference kernels src/ops/sdpa_decode/metal_sdpa_decode.metal:86-175 and :177-281 for that case.
 *
 * One workgroup per (batch row, kv head) lets the longest row decide the time of the launch: a compute unit
 * streams its row at the rate its own loads in flight allow (about 30 GB/s of the 8 TB/s), so a 4095-key row
 * next to 1024-key rows finishes long after them.  Here the visible keys of all rows are laid end to end
 * (batch row major, then kv head, then key: L = Hkv * sum_b len_b entries), the line is cut into equal SHARES of
 * R entries, one per wavefront of the grid, and wavefront w streams share w: one or more SEGMENTS, each a run of
 * keys of one (batch row, kv head).  A wavefront works alone (no barrier, no LDS) and its loads run on across
 * segment ends: the first rows of the next segment are requested before the last ones of the current segment
 * are multiplied.  Every segment leaves a partial result (accumulator, running maximum, sum) in the workspace at
 * slot (row index + w): going along the line, every boundary crossed raises either the row index or w by one,
 * so the slots of consecutive segments are consecutive and no two segments share one.  The combine kernel
 * recomputes where its row starts on the line, which shares it touches, and merges those slots.
 *
 * The positions live on the device, so every wavefront first derives the cut from them (a sum and a prefix
 * search over the batch rows: a dependent load and a few cross-lane steps in front of the first cache row,
 * which only pays where a launch streams for tens of microseconds: the host chooses this kernel by cache size).
 *
 * Semantics as in sdpa_decode.hip: live = min(pos + 1, Tmax), window mask of metal_sdpa_decode.metal:30-53
 * (no always-visible prefix here), rows with a negative position are left untouched.
 */
#include "sdpa_decode_device.h"

/* first visible key and number of visible keys of batch row b (0 keys for a negative position) */
__device__ __forceinline__ void gd_bal_row(const int32_t *__restrict__ pos_ptr, uint32_t tmax, uint32_t window, int b,
                                           int *first, int *len)
{
    const int pos = pos_ptr[b];
    const int live = min(pos + 1, (int)tmax);
    const int f = window > 0u ? max(0, pos - (int)window + 1) : 0;
    *first = f;
    *len = pos < 0 ? 0 : live - f;
}

__device__ __forceinline__ uint32_t gd_bal_share(uint32_t line, uint32_t shares)
{
    return (((line + shares - 1u) / shares) + 63u) & ~63u;
}

__device__ __forceinline__ uint32_t gd_wave_sum_u32(uint32_t v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += (uint32_t)__shfl_xor((int)v, off, 64);
    return v;
}

/* floats per partial result in the workspace: accumulator [D], maximum, sum, two unused (16-byte rows) */
#define GD_BAL_STRIDE(D) ((D) + 4)

template <int D, int G, bool NT>
__global__ void __launch_bounds__(256)
gd_sdpa_decode_balanced_kernel(const gd_half *__restrict__ q, const gd_half *__restrict__ kc,
                               const gd_half *__restrict__ vc, const int32_t *__restrict__ pos_ptr,
                               float *__restrict__ ws, gd_hip_sdpa_decode_params p)
{
    constexpr int WAVES = 4, UNROLL = 2;
    constexpr int LPK = D / 8;    /* lanes per key row */
    constexpr int KPW = 64 / LPK; /* key rows per wavefront load */
    constexpr int STEP = KPW * UNROLL;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int slot = lane / LPK, sub = lane % LPK;
    const int B = (int)p.batch, HKV = (int)p.hkv;
    /* a wavefront is a share of its own: no barrier, no LDS; neighbouring wavefronts stream neighbouring shares */
    const uint32_t w = blockIdx.x * WAVES + (uint32_t)wave, shares = gridDim.x * WAVES;

    /* ---- the cut: every wavefront computes the same numbers from the positions ---- */
    uint32_t keys = 0u;
    for (int c = 0; c < B; c += 64) {
        int f, n = 0;
        if (c + lane < B) gd_bal_row(pos_ptr, p.tmax, p.window, c + lane, &f, &n);
        keys += gd_wave_sum_u32((uint32_t)n);
    }
    const uint32_t line = __builtin_amdgcn_readfirstlane(keys) * (uint32_t)HKV;
    const uint32_t share = gd_bal_share(line, shares);
    const uint32_t x0 = w * share, x1 = min(x0 + share, line);
    if (x0 >= line) return;

    /* the batch row whose stretch of the line holds x0: the first one that ends behind x0 */
    int b = 0, first_b = 0, len_b = 0;
    uint32_t start_b = 0u;
    {
        uint32_t base = 0u;
        for (int c = 0; c < B; c += 64) {
            int f = 0, n = 0;
            if (c + lane < B) gd_bal_row(pos_ptr, p.tmax, p.window, c + lane, &f, &n);
            uint32_t incl = (uint32_t)n;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const uint32_t up = (uint32_t)__shfl_up((int)incl, off, 64);
                if (lane >= off) incl += up;
            }
            const uint64_t behind = __ballot((base + incl) * (uint32_t)HKV > x0);
            if (behind != 0ull) {
                const int j = __builtin_ctzll(behind);
                b = c + j;
                len_b = __builtin_amdgcn_readlane(n, j);
                first_b = __builtin_amdgcn_readlane(f, j);
                start_b = (base + (uint32_t)__builtin_amdgcn_readlane((int)incl, j) - (uint32_t)len_b) * (uint32_t)HKV;
                break;
            }
            base += (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        }
    }
    int h = (int)((x0 - start_b) / (uint32_t)len_b);
    int t = (int)((x0 - start_b) % (uint32_t)len_b);

    const uint32_t pitch = p.hkv * (uint32_t)(D * 2); /* bytes between consecutive keys */
    const uint32_t lane_off = (uint32_t)sub * 16u;
    const float qscale = p.scale * 1.4426950408889634f;
    const unsigned char *kbase = reinterpret_cast<const unsigned char *>(kc);
    const unsigned char *vbase = reinterpret_cast<const unsigned char *>(vc);

    /* one trip = STEP keys of one segment; `slab` = byte offset of (batch row, kv head) in both caches, rows
     * s0 .. of that slab, masked from r1 on (rows past the segment re-read its last row) */
    auto load_trip = [&](gd_half8 (&kv)[UNROLL], gd_half8 (&vv)[UNROLL], size_t slab, int s0, int r1)
        __attribute__((always_inline)) {
        uint32_t off[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) off[u] = __umul24((uint32_t)min(s0 + u * KPW + slot, r1 - 1), pitch) + lane_off;
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const gd_half8 *kp = reinterpret_cast<const gd_half8 *>(kbase + slab + off[u]);
            kv[u] = NT ? __builtin_nontemporal_load(kp) : *kp;
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const gd_half8 *vp = reinterpret_cast<const gd_half8 *>(vbase + slab + off[u]);
            vv[u] = NT ? __builtin_nontemporal_load(vp) : *vp;
        }
    };
    auto load_q = [&](gd_half8 (&qv)[G], int bb, int hh) __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < G; ++g)
            qv[g] = *reinterpret_cast<const gd_half8 *>(q + ((size_t)bb * p.hq + (size_t)hh * G + g) * D + sub * 8);
    };

    float m[G], l[G], acc[G][8];
    auto reset = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            m[g] = GD_NEG_INF;
            l[g] = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
        }
    };
    auto compute_trip = [&](const gd_half8 (&kv)[UNROLL], const gd_half8 (&vv)[UNROLL], const gd_half8 (&qv)[G], int s0,
                            int r1) __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float sc[UNROLL];
            float mt = GD_NEG_INF;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                float d = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    d = __builtin_amdgcn_fdot2((gd_half2){qv[g][2 * e], qv[g][2 * e + 1]},
                                               (gd_half2){kv[u][2 * e], kv[u][2 * e + 1]}, d, false);
                d = gd_row_group_sum<LPK>(d);
                sc[u] = (s0 + u * KPW + slot < r1) ? d * qscale : GD_NEG_INF;
                mt = fmaxf(mt, sc[u]);
            }
            const float mx = fmaxf(m[g], mt);
            const float mn = mx == GD_NEG_INF ? 0.f : mx;
            const float corr = exp2f(m[g] - mn);
            float lsum = l[g] * corr;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[g][e] *= corr;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const float pr = exp2f(sc[u] - mn);
                lsum += pr;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(pr, (float)vv[u][e], acc[g][e]);
            }
            l[g] = lsum;
            m[g] = mx;
        }
    };
    /* the segment's partial result: row slots merged inside the wavefront, written by the lanes of slot 0 */
    auto flush = [&](int bb, int hh) __attribute__((always_inline)) {
        float *dst = ws + ((size_t)bb * p.hkv + (size_t)hh + (size_t)w) * (size_t)(G * GD_BAL_STRIDE(D));
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float mw = gd_slot_max<LPK>(m[g]);
            const float c = (m[g] == GD_NEG_INF) ? 0.f : exp2f(m[g] - mw);
            const float lw = gd_slot_sum<LPK>(l[g] * c);
            gd_float4 a0, a1;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                a0[e] = gd_slot_sum<LPK>(acc[g][e] * c);
                a1[e] = gd_slot_sum<LPK>(acc[g][4 + e] * c);
            }
            if (slot == 0) {
                float *d = dst + (size_t)g * GD_BAL_STRIDE(D);
                *reinterpret_cast<gd_float4 *>(d + sub * 8) = a0;
                *reinterpret_cast<gd_float4 *>(d + sub * 8 + 4) = a1;
                if (sub == 0) {
                    d[D] = mw;
                    d[D + 1] = lw;
                }
            }
        }
    };

    /* ---- the stream: trips follow one another across segment ends, so the loads never stop ---- */
    /* scalar state of the trip in flight ("cur") and of the one after it ("nxt") */
    int seg = min((int)(x1 - x0), len_b - t);
    uint32_t x = x0;
    int cb = b, ch = h;                 /* (batch row, kv head) of the current trip's segment */
    int s0 = first_b + t, r1 = s0 + seg; /* its first row and the segment's end */
    size_t slab = ((size_t)b * p.tmax * p.hkv + (size_t)h) * (size_t)(D * 2);

    gd_half8 kA[UNROLL], vA[UNROLL], kB[UNROLL], vB[UNROLL], qc[G], qn[G];
    load_trip(kA, vA, slab, s0, r1);
    load_q(qc, cb, ch);
    reset();

    /* moves (b, h, t, x, seg, len_b, first_b) to the segment after the current one; false at the end of the share */
    auto next_segment = [&]() __attribute__((always_inline)) -> bool {
        x += (uint32_t)seg;
        t += seg;
        if (x >= x1) return false;
        if (t == len_b) {
            t = 0;
            if (++h == HKV) {
                h = 0;
                len_b = 0;
                while (len_b == 0 && ++b < B) {
                    int f, n;
                    gd_bal_row(pos_ptr, p.tmax, p.window, b, &f, &n);
                    first_b = __builtin_amdgcn_readfirstlane(f);
                    len_b = __builtin_amdgcn_readfirstlane(n);
                }
                if (b >= B) return false;
            }
        }
        seg = min((int)(x1 - x), len_b - t);
        return true;
    };

    while (true) {
        /* context of the trip after the current one */
        int n_s0 = s0 + STEP, n_r1 = r1, nb = cb, nh = ch;
        size_t n_slab = slab;
        bool newseg = false, more = true;
        if (n_s0 >= r1) {
            more = next_segment();
            newseg = true;
            nb = b;
            nh = h;
            n_s0 = first_b + t;
            n_r1 = n_s0 + seg;
            n_slab = ((size_t)b * p.tmax * p.hkv + (size_t)h) * (size_t)(D * 2);
        }
        if (!more) {
            compute_trip(kA, vA, qc, s0, r1);
            flush(cb, ch);
            break;
        }
        load_trip(kB, vB, n_slab, n_s0, n_r1);
        if (newseg) load_q(qn, nb, nh);
        compute_trip(kA, vA, qc, s0, r1);
        if (newseg) {
            flush(cb, ch);
            reset();
#pragma unroll
            for (int g = 0; g < G; ++g) qc[g] = qn[g];
        }
        s0 = n_s0; r1 = n_r1; cb = nb; ch = nh; slab = n_slab;

        /* the same with the register sets exchanged */
        n_s0 = s0 + STEP; n_r1 = r1; nb = cb; nh = ch; n_slab = slab;
        newseg = false;
        more = true;
        if (n_s0 >= r1) {
            more = next_segment();
            newseg = true;
            nb = b;
            nh = h;
            n_s0 = first_b + t;
            n_r1 = n_s0 + seg;
            n_slab = ((size_t)b * p.tmax * p.hkv + (size_t)h) * (size_t)(D * 2);
        }
        if (!more) {
            compute_trip(kB, vB, qc, s0, r1);
            flush(cb, ch);
            break;
        }
        load_trip(kA, vA, n_slab, n_s0, n_r1);
        if (newseg) load_q(qn, nb, nh);
        compute_trip(kB, vB, qc, s0, r1);
        if (newseg) {
            flush(cb, ch);
            reset();
#pragma unroll
            for (int g = 0; g < G; ++g) qc[g] = qn[g];
        }
        s0 = n_s0; r1 = n_r1; cb = nb; ch = nh; slab = n_slab;
    }
}

/* One workgroup of D threads per (query head, batch row): finds the row's stretch of the line, the shares that
 * overlap it, and merges their slots. */
template <int D, int G>
__global__ void __launch_bounds__(D)
gd_sdpa_decode_balanced_combine_kernel(const float *__restrict__ ws, const int32_t *__restrict__ pos_ptr,
                                       gd_half *__restrict__ out, gd_hip_sdpa_decode_params p, uint32_t shares)
{
    const int hq = blockIdx.x, b = blockIdx.y, c = threadIdx.x;
    const int B = (int)p.batch;
    if (pos_ptr[b] < 0) return;
    __shared__ uint32_t s_sum[2][D / 64];
    uint32_t before = 0u, keys = 0u;
    for (int bb = c; bb < B; bb += D) {
        int f, n;
        gd_bal_row(pos_ptr, p.tmax, p.window, bb, &f, &n);
        keys += (uint32_t)n;
        if (bb < b) before += (uint32_t)n;
    }
    before = gd_wave_sum_u32(before);
    keys = gd_wave_sum_u32(keys);
    if ((c & 63) == 0) {
        s_sum[0][c >> 6] = before;
        s_sum[1][c >> 6] = keys;
    }
    __syncthreads();
    before = keys = 0u;
#pragma unroll
    for (int i = 0; i < D / 64; ++i) {
        before += s_sum[0][i];
        keys += s_sum[1][i];
    }
    int first_b, len_b;
    gd_bal_row(pos_ptr, p.tmax, p.window, b, &first_b, &len_b);
    const uint32_t share = gd_bal_share(keys * p.hkv, shares);
    const uint32_t hkv = (uint32_t)hq / G, g = (uint32_t)hq % G;
    const uint32_t s0 = before * p.hkv + hkv * (uint32_t)len_b;
    const uint32_t w0 = s0 / share, w1 = (s0 + (uint32_t)len_b - 1u) / share;
    const float *row = ws + (((size_t)b * p.hkv + hkv) * G + g) * (size_t)GD_BAL_STRIDE(D);
    const size_t per_share = (size_t)G * GD_BAL_STRIDE(D);
    float mm = GD_NEG_INF;
    for (uint32_t w = w0; w <= w1; ++w) mm = fmaxf(mm, row[(size_t)w * per_share + D]);
    float ll = 0.f, aa = 0.f;
    for (uint32_t w = w0; w <= w1; ++w) {
        const float ms = row[(size_t)w * per_share + D];
        if (ms == GD_NEG_INF) continue;
        const float cw = exp2f(ms - mm);
        ll += row[(size_t)w * per_share + D + 1] * cw;
        aa += row[(size_t)w * per_share + c] * cw;
    }
    out[((size_t)b * p.hq + hq) * D + c] = (gd_half)(ll > 0.f ? aa / ll : 0.f);
}

template <int D, int G>
static int launch_balanced(hipStream_t stream, const void *q, const void *k, const void *v, const int32_t *pos,
                           void *out, float *ws, const gd_hip_sdpa_decode_params &p, uint32_t shares)
{
    /* shares are wavefronts: four to a workgroup */
    if (p.nontemporal)
        gd_sdpa_decode_balanced_kernel<D, G, true><<<shares / 4u, 256, 0, stream>>>(
            (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, ws, p);
    else
        gd_sdpa_decode_balanced_kernel<D, G, false><<<shares / 4u, 256, 0, stream>>>(
            (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, ws, p);
    dim3 cgrid(p.hq, p.batch);
    gd_sdpa_decode_balanced_combine_kernel<D, G><<<cgrid, D, 0, stream>>>(ws, pos, (gd_half *)out, p, shares);
    return (int)hipGetLastError();
}

/* shares: a multiple of 4.  ws: (batch * hkv + shares) * (hq / hkv) * (dh + 4) floats.  Returns hipErrorInvalidValue when (dh, group) has
 * no instantiation. */
extern "C" int gd_hip_launch_sdpa_decode_balanced(hipStream_t stream, const void *q, const void *k, const void *v,
                                                  const int32_t *pos, void *out, float *ws,
                                                  const gd_hip_sdpa_decode_params *params, uint32_t shares)
{
    const gd_hip_sdpa_decode_params &p = *params;
    const uint32_t g = p.hq / p.hkv;
#define GD_CASE(DD, GG) \
    if (p.dh == DD && g == GG) return launch_balanced<DD, GG>(stream, q, k, v, pos, out, ws, p, shares)
    GD_CASE(64, 1); GD_CASE(64, 2); GD_CASE(64, 4); GD_CASE(64, 8);
    GD_CASE(128, 1); GD_CASE(128, 2); GD_CASE(128, 4); GD_CASE(128, 8);
#undef GD_CASE
    return (int)hipErrorInvalidValue;
}
