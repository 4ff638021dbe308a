/*
 * The split-KV decode attention kernel of gfx950 (F16, one query token per row, head size 64 or 128), shared by
 * its two translation units: sdpa_decode.hip (one workgroup per (piece, kv head, row), a combine kernel behind it
 * when rows are cut) and sdpa_decode_pieces.hip (PIECES: the rows of a ragged batch in pieces, one workgroup each,
 * merged inside the kernel by the last piece of a row to arrive).  Replaces the reference kernels
 * src/ops/sdpa_decode/metal_sdpa_decode.metal:86-175 (Tq=1 window fast path) and :177-281 (general path).
 */
#ifndef GD_SDPA_DECODE_SPLIT_KERNEL_H
#define GD_SDPA_DECODE_SPLIT_KERNEL_H
#include "sdpa_decode_device.h"

/* PFX: a prefix of always-visible keys in front of the window (prefix_len > 0).  The visible keys are then two
 * runs, [0, a_len) and [b0, live); the kernel walks a virtual index over both (v < a_len: key v, else key
 * v - a_len + b0) and the split of the range counts virtual indices.  Without PFX there is one run and the index is
 * the key row itself. */
template <int D, int G, int WAVES, int UNROLL, bool NT, bool PFX = false, bool PIECES = false, bool AHEAD = false>
__global__ void __launch_bounds__(WAVES * 64)
gd_sdpa_decode_split_kernel(const gd_half *__restrict__ q, const gd_half *__restrict__ kc,
                            const gd_half *__restrict__ vc, const int32_t *__restrict__ pos_ptr,
                            gd_half *__restrict__ out, float *__restrict__ ws, gd_hip_sdpa_decode_params p)
{
    constexpr int LPK = D / 8;      /* lanes per key row */
    constexpr int KPW = 64 / LPK;   /* key rows per wavefront load */
    constexpr int KPB = KPW * WAVES;
    constexpr int STEP = KPB * UNROLL;
    /* AHEAD (chosen by the launcher: no window, no prefix, not the PIECES form): the wavefront's first rows are
     * requested before the row's position is known, see below */
    constexpr bool ahead = AHEAD && !PIECES && !PFX;
    /* Every kernel argument this path reads is requested from the argument segment here, in one batch with
     * one wait.  Left to the compiler, each load sits in front of its first use behind the early exits, and
     * a wavefront goes through five dependent round trips before its first K/V load. */
    asm volatile("" ::"s"(q), "s"(kc), "s"(vc), "s"(pos_ptr), "s"(out), "s"(ws), "s"(p.tmax), "s"(p.hq), "s"(p.hkv),
                 "s"(p.window), "s"(p.pos_mode), "s"(p.cache_pos), "s"(p.scale), "s"(p.chunk), "s"(p.nsplit), "s"(p.even_pieces));
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int slot = lane / LPK, sub = lane % LPK;
    const uint32_t pitch = p.hkv * (uint32_t)(D * 2); /* bytes between consecutive keys */
    const uint32_t lane_off = (uint32_t)sub * 16u;
    const float qscale = p.scale * 1.4426950408889634f;
    __shared__ float sm_acc[WAVES][G][D];
    __shared__ float sm_m[WAVES][G], sm_l[WAVES][G];
    __shared__ uint32_t sm_last;

    /* visible keys of a row at position `at`: [0, a_len) and [b0, live).  Reference mask
     * (metal_sdpa_decode.metal:25-52): a query inside the prefix sees the prefix keys that exist; one behind it sees
     * the whole prefix plus its window (everything up to itself without a window) */
    auto visible = [&](int at, int &live_, int &first_, int &a_len_, int &b0_) __attribute__((always_inline)) {
        live_ = min(at + 1, (int)p.tmax);
        first_ = p.window > 0u ? max(0, at - (int)p.window + 1) : 0;
        a_len_ = PFX ? min((int)p.prefix_len, live_) : 0;
        b0_ = PFX ? (at < (int)p.prefix_len ? live_ : min(max(a_len_, first_), live_)) : first_;
        return PFX ? a_len_ + live_ - b0_ : live_ - first_;
    };

    /* PIECES: grid (Hkv, B, pieces): the visible keys of a row are cut into pieces of `chunk` keys, one workgroup
     * each, so that the long rows of a ragged batch spread over the compute units its short rows leave idle; the
     * first pieces of all rows hold the lowest workgroup numbers, the pieces a short row does not have (they leave
     * at once) the highest.  Every wavefront looks at the positions of all rows (lane l holds rows l, l + 64, ...;
     * the same arithmetic everywhere, so all workgroups agree): rows of about one length (the longest within 1.25
     * of the mean) are cut into p.even_pieces equal parts instead (one part: the row stays whole and nothing is
     * merged), which is the one-workgroup-per-row kernel again. */
    const int split = PIECES ? blockIdx.z : blockIdx.x, hkv = PIECES ? blockIdx.x : blockIdx.y;
    const int b = PIECES ? blockIdx.y : blockIdx.z;
    int pos, pos_lane = 0, chunk = (int)p.chunk;
    /* PIECES without a window or a prefix: the first piece of a row requests its first rows ahead of the positions */
    const bool pieces_ahead = PIECES && !PFX && p.window == 0u;

    /* Addresses: one scalar base per cache for this (batch row, kv head), plus a 32-bit byte offset per lane
     * made by one 24-bit multiply-add (the host checks that tmax, the row pitch and their product fit).  The
     * four wavefronts of a SIMD start together and share its issue slots, so every vector instruction in
     * front of the first row loads delays all of them. */
    const size_t slab = ((size_t)b * p.tmax * p.hkv + (size_t)hkv) * (size_t)(D * 2);
    const unsigned char *kslab = reinterpret_cast<const unsigned char *>(kc) + slab;
    const unsigned char *vslab = reinterpret_cast<const unsigned char *>(vc) + slab;
    /* rows first .. first + UNROLL * KPB of the wavefront, no row past `last`: all K rows of a trip are requested
     * before its V rows (the scores need every K row, the accumulation takes the V rows one by one) */
    auto load_rows = [&](gd_half8 (&kv)[UNROLL], gd_half8 (&vv)[UNROLL], int s0, int last, int a_len_, int b0_)
        __attribute__((always_inline)) {
        uint32_t off[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            int row = min(s0 + u * KPB + slot, last);
            if (PFX) row = row < a_len_ ? row : row - a_len_ + b0_;
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
    gd_half8 kA[UNROLL], vA[UNROLL], kB[UNROLL], vB[UNROLL];
    auto load_rows_early = [&](int s0) __attribute__((always_inline)) { load_rows(kA, vA, s0, (int)p.tmax - 1, 0, 0); };

    if (PIECES) {
        constexpr int RS = GD_HIP_SDPA_PIECES_MAX_BATCH / 64;
        int longest = 0, total = 0, rows = 0;
        pos = -1;
        int at_row[RS];
#pragma unroll
        for (int i = 0; i < RS; ++i) {
            const int r = i * 64 + lane;
            at_row[i] = r < (int)p.batch ? pos_ptr[r] : -1;
        }
        /* The first piece of a row starts at key 0 whatever the positions say (no window, no prefix), and the first
         * pieces hold the lowest workgroup numbers: they are the workgroups the launch starts with.  Their first rows
         * are requested here, behind the requests for the positions and in front of their first use, so that the two
         * round trips overlap at the start of the launch (later pieces start next to running ones, and pieces a row
         * does not have must not load anything). */
        __builtin_amdgcn_sched_barrier(0);
        if (pieces_ahead && split == 0) load_rows_early(wave * KPW);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < RS; ++i) {
            const int at = at_row[i];
            int l_, f_, a_, b_;
            const int n = at >= 0 ? max(visible(at, l_, f_, a_, b_), 0) : 0;
            longest = max(longest, n);
            total += n;
            rows += at >= 0 ? 1 : 0;
            if ((b >> 6) == i) pos = __builtin_amdgcn_readlane(at, b & 63);
        }
        longest = gd_wave_reduce_i32(longest, [](int x, int y) { return max(x, y); });
        total = gd_wave_reduce_i32(total, [](int x, int y) { return x + y; });
        rows = gd_wave_reduce_i32(rows, [](int x, int y) { return x + y; });
        /* p.even_pieces is 0 (never), 1 or 2; p.chunk times the pieces of the grid covers the longest row there can be */
        if (p.even_pieces != 0u && 4.f * (float)longest * (float)rows <= 5.f * (float)total)
            chunk = max((((longest + (int)p.even_pieces - 1) >> (p.even_pieces >> 1)) + 31) & ~31, 32);
    } else {
        if (ahead) {
            /* the position is requested through a lane address the compiler cannot prove uniform, so that it stays
             * in a vector register (no wait) until the wavefront's first rows have been requested */
            pos_lane = p.cache_pos;
            if (p.pos_mode != GD_HIP_SDPA_POS_SCALAR) {
                int idx = p.pos_mode == GD_HIP_SDPA_POS_VECTOR ? b : 0;
                asm volatile("" : "+v"(idx));
                pos_lane = pos_ptr[idx];
            }
            pos = 0;
        } else {
            pos = gd_decode_pos(pos_ptr, p, b);
        }
    }

    /* Without a window the wavefront's first rows do not depend on the row's position: they are requested here,
     * behind the request for the position and in front of its first use, so that the two round trips overlap.  What
     * the position then says does not exist (rows from the live length on; they lie inside the cache, so the loads
     * are harmless) is masked in the first trip's arithmetic, values included: such rows may hold anything. */
    __builtin_amdgcn_sched_barrier(0);
    if (ahead) load_rows(kA, vA, split * chunk + wave * KPW, (int)p.tmax - 1, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    if (ahead) pos = __builtin_amdgcn_readfirstlane(pos_lane);
    const bool ahead_now = ahead || (pieces_ahead && split == 0); /* the first rows are on their way */
    /* (the early exits below read a loaded register, which keeps the loads above in front of the branches) */
    if (pos < 0) {
        if (ahead_now) asm volatile("" ::"v"(kA[0]), "v"(vA[0]));
        return;
    }
    int live, first, a_len, b0;
    const int n_vis = visible(pos, live, first, a_len, b0);
    const int r0 = PFX ? split * chunk : first + split * chunk;
    const int r1 = PFX ? min(r0 + chunk, n_vis) : min(r0 + chunk, live);
    /* the first GD_HIP_SDPA_COUNTER_SLOTS words of the workspace are the rows' arrival counters; a row's partial
     * results follow each other (room for p.nsplit of them) */
    const uint32_t stride = p.nsplit;
    float *ws_row = ws + GD_HIP_SDPA_COUNTER_SLOTS + (((size_t)b * p.hq + (size_t)hkv * G) * stride + split) * (D + 2);
    /* pieces this row has (PIECES); a row of one piece stores its result itself */
    const uint32_t npieces = ((uint32_t)max(n_vis, 0) + (uint32_t)chunk - 1u) / (uint32_t)chunk;
    const bool partial = PIECES ? npieces > 1u : p.nsplit > 1u;
    if (r0 >= r1) {
        if (ahead_now) asm volatile("" ::"v"(kA[0]), "v"(vA[0]));
        if (PIECES) {
            /* a piece the row does not have; the first piece of a row without a visible key stores zeros */
            if (split != 0) return;
            for (int idx = threadIdx.x; idx < G * D; idx += WAVES * 64)
                out[((size_t)b * p.hq + (size_t)hkv * G) * D + idx] = (gd_half)0.f;
        } else if (p.nsplit > 1u) {
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

    /* Row loads of trip t+1 are issued before the arithmetic of trip t (two register buffers), so
     * the memory pipe stays busy while the wavefront computes.  s0: the wavefront's first row of the trip (scalar);
     * rows past the range re-read the last row and are masked in the arithmetic. */
    auto load_trip = [&](gd_half8 (&kv)[UNROLL], gd_half8 (&vv)[UNROLL], int s0) __attribute__((always_inline)) {
        load_rows(kv, vv, s0, r1 - 1, a_len, b0);
    };

    /* trips are decided per wavefront (scalar branches), rows past the range are masked per lane */
    const int jw = r0 + wave * KPW;
    const bool any_rows = jw < r1;
    if (any_rows && !ahead_now) load_trip(kA, vA, jw);
    __builtin_amdgcn_sched_barrier(0); /* nothing below moves in front of the first loads */

    /* query rows of the G heads that share this kv head stay in F16: products of two halfs are
     * exact in F32, so v_dot2_f32_f16 loses nothing; the softmax scale (exp2 domain) is applied
     * to the reduced dot product */
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

    bool unchecked = ahead_now; /* the buffers hold rows that were requested before the live length was known */
    auto compute_trip = [&](const gd_half8 (&kv)[UNROLL], const gd_half8 (&vin)[UNROLL], int s0)
        __attribute__((always_inline)) {
        gd_half8 vv[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            vv[u] = vin[u];
            if (unchecked && !(s0 + u * KPB + slot < r1)) vv[u] = (gd_half8)(gd_half)0.f;
        }
        unchecked = false;
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
        if (partial) {
            float *w = ws_row + (size_t)g * stride * (D + 2);
            if (PIECES) {
                /* write-through stores: the merging workgroup may run on another XCD, whose L2 is not this one's */
                gd_agent_store(w + 2 + c, aa);
                if (c == 0) {
                    gd_agent_store(w, mm);
                    gd_agent_store(w + 1, ll);
                }
            } else {
                w[2 + c] = aa;
                if (c == 0) {
                    w[0] = mm;
                    w[1] = ll;
                }
            }
        } else {
            out[((size_t)b * p.hq + (size_t)hkv * G + g) * D + c] = (gd_half)(ll > 0.f ? aa / ll : 0.f);
        }
    }
    if (PIECES && partial) {

    /* The piece that arrives last merges the row.  The barrier waits for every thread's stores above (they have
     * left this XCD by then); one relaxed device-scope add per piece counts the arrivals; the last one puts the
     * counter back to zero for the next launch and reads all partials past its own L2.  Nobody waits for anybody. */
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t *cnt = reinterpret_cast<uint32_t *>(ws) + (size_t)b * p.hkv + hkv;
        const uint32_t seen = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (seen + 1u == npieces) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sm_last = seen + 1u == npieces ? 1u : 0u;
    }
    __syncthreads();
    if (sm_last != 0u)
    for (int idx = threadIdx.x; idx < G * D; idx += WAVES * 64) {
        const int g = idx / D, c = idx % D;
        const float *w = ws_row - (size_t)split * (D + 2) + (size_t)g * stride * (D + 2);
        float ms[GD_HIP_SDPA_MAX_PIECES], ls[GD_HIP_SDPA_MAX_PIECES], as[GD_HIP_SDPA_MAX_PIECES];
        /* all loads of the merge are requested before the first is used */
#pragma unroll
        for (uint32_t s = 0; s < GD_HIP_SDPA_MAX_PIECES; ++s) {
            const bool have = s < npieces;
            const float *ws_s = w + (size_t)(have ? s : 0u) * (D + 2);
            ms[s] = gd_agent_load(ws_s);
            ls[s] = gd_agent_load(ws_s + 1);
            as[s] = gd_agent_load(ws_s + 2 + c);
            if (!have) ms[s] = GD_NEG_INF;
        }
        float mm = GD_NEG_INF;
#pragma unroll
        for (uint32_t s = 0; s < GD_HIP_SDPA_MAX_PIECES; ++s) mm = fmaxf(mm, ms[s]);
        float ll = 0.f, aa = 0.f;
#pragma unroll
        for (uint32_t s = 0; s < GD_HIP_SDPA_MAX_PIECES; ++s) {
            const float cw = ms[s] == GD_NEG_INF ? 0.f : exp2f(ms[s] - mm);
            ll += ls[s] * cw;
            aa += as[s] * cw;
        }
        out[((size_t)b * p.hq + (size_t)hkv * G + g) * D + c] = (gd_half)(ll > 0.f ? aa / ll : 0.f);
    }
    }
}

#endif
