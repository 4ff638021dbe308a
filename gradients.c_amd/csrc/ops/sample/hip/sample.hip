/*
 * Next-token sampling on the device for gfx950: soft cap, repetition penalty, temperature / min-p
 * draw and the bookkeeping of a generation loop, so that a device-resident loop never moves the
 * logits to the host.  Restates the host code of the reference's example,
 * examples/gpt_lm/gpt_lm_shared.c: gpt_apply_logits_softcap (:1322-1331),
 * gpt_apply_repetition_penalty (:1347-1369), gpt_sample_next_token (:1371-1442) and the loop
 * around them (:1586-1600, 1606-1680): one generator shared by the rows, advanced once per row
 * that really draws, in row order; a row ends at the stop token or when its history is full.
 *
 * A row is cut into parts of 2048 tokens, one workgroup of 256 threads each, every thread owning a
 * segment of 8 consecutive tokens:
 *   prepare  capped and penalised logits -> work[row] (F32); leader of the part; then, relative to the
 *            row's leader, the mass of every segment and of the part, and "will draw".  A row of one
 *            part does this in one launch; with more parts the row's leader has to be agreed on
 *            first, so the launch is split in two.  One more workgroup meanwhile steps the generator
 *            once per row (the draws this step can need at most).
 *   pick     one workgroup per row: the row's draw (its rank among the drawing rows selects it),
 *            search over part masses, segment masses, then the tokens of one segment; history /
 *            finished / ids / positions / record update, optional gather of the next embedding row
 * HBM traffic per row: logits read once, work and the masses written once (work read once more when
 * the launch is split); the pick reads the part masses, one part's segment masses and one segment.
 *
 * Arithmetic as in the reference: F32 cap (tanhf) and penalty, F64 mass (exp) and target.  Sums are
 * formed in another order than the reference's left-to-right loop, so the total and the running
 * sums can differ in the last bits; the chosen token differs only when the drawn point lies within
 * that distance of a boundary between two tokens.
 */
#include "../../_shared/hip_device.h"

#define GD_SAMPLE_THREADS 256
#define GD_SAMPLE_SEG 8
#define GD_SAMPLE_PART (GD_SAMPLE_THREADS * GD_SAMPLE_SEG) /* tokens per workgroup */
#define GD_SAMPLE_MAX_PARTS 128u
#define GD_NEG_INF (-__builtin_inff())

struct __attribute__((aligned(8))) gd_sample_rec {
    double best_value, sum;
    int32_t best, draws;
    int32_t pad[2];
};

/* device-resident generator and per-row records; the caller provides it as an I32 tensor of
 * 8 + 10 * rows elements, 8-byte aligned: header, rec[rows], then draw_state[rows] */
struct __attribute__((aligned(8))) gd_sample_state {
    unsigned long long rng[2]; /* slot (epoch & 1) is current */
    uint32_t epoch;            /* +1 per sample_advance call */
    uint32_t pad[3];
    gd_sample_rec rec[1];
};

struct gd_sample_cfg {
    float temperature, min_p, penalty, softcap;
    int32_t stop_token;
    uint32_t cols, hist_cap;
    uint32_t parts; /* workgroups per row */
};

/* leader of one part: largest finite value and its token; index < 0: nothing finite */
struct __attribute__((aligned(8))) gd_sample_part {
    float value;
    int32_t index;
};

/* scratch behind the rows' values, per row and part: 256 segment masses, the part's mass, the part's leader */
struct gd_sample_scratch {
    float *work;
    double *seg_mass, *part_mass;
    gd_sample_part *part_max;
};

__device__ __forceinline__ unsigned long long gd_splitmix64(unsigned long long x)
{
    x += 0x9e3779b97f4a7c15ull;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
    return x ^ (x >> 31);
}

__device__ __forceinline__ unsigned long long *gd_sample_draw_states(gd_sample_state *st, uint32_t rows)
{
    return reinterpret_cast<unsigned long long *>(&st->rec[rows]);
}

/* mass of one token relative to the leader; valid = the reference's loop does not skip it */
__device__ __forceinline__ double gd_sample_mass(float logit, double best, double temp, double threshold, bool &valid)
{
    const double v = (double)logit;
    valid = false;
    if (!isfinite(v) || v < threshold) return 0.0;
    const double p = exp((v - best) / temp);
    if (!isfinite(p)) return 0.0;
    valid = true;
    return p;
}

__device__ __forceinline__ double gd_sample_threshold(const gd_sample_cfg &c, double best)
{
    return c.min_p > 0.0f ? best + (double)c.temperature * log((double)c.min_p) : -__builtin_inf();
}

/* (value, index) a replaces b?  larger value, lower index among equals; index < 0 never wins */
__device__ __forceinline__ bool gd_sample_leads(float av, int32_t ai, float bv, int32_t bi)
{
    return ai >= 0 && (bi < 0 || av > bv || (av == bv && ai < bi));
}

/* PHASE 0: everything for a row of one part.  PHASE 1: values and the part's leader.  PHASE 2: masses, once every
 * part's leader is known.  Workgroup rows * parts of PHASE 0 / 1 steps the generator. */
template <typename T, int PHASE>
__global__ void __launch_bounds__(GD_SAMPLE_THREADS)
gd_sample_prepare_kernel(const T *__restrict__ logits, gd_sample_scratch s, gd_sample_state *__restrict__ st,
                         const int32_t *__restrict__ history, const int32_t *__restrict__ hist_len,
                         const int32_t *__restrict__ finished, uint32_t rows, gd_sample_cfg c)
{
    __shared__ uint32_t seen[GD_SAMPLE_PART / 32]; /* one bit per token of the part: occurs in the row's history */
    __shared__ float s_val[GD_SAMPLE_THREADS / 64];
    __shared__ int32_t s_idx[GD_SAMPLE_THREADS / 64];
    __shared__ double s_sum[GD_SAMPLE_THREADS / 64];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    constexpr uint32_t nw = GD_SAMPLE_THREADS / 64;
    if (blockIdx.x == rows * c.parts) {
        /* draw number k of this step uses the state after k + 1 steps of the generator; which rows draw is only
         * known after this launch, so all `rows` states are laid out while the other workgroups do their rows.
         * Every lane of the first wavefront walks the same chain, so the 64-bit arithmetic runs on the scalar unit
         * (the values are made uniform below); lane 0 stores */
        if (PHASE != 2 && tid < 64u) {
            const uint32_t epoch = st->epoch + 1u;
            unsigned long long *draw_state = gd_sample_draw_states(st, rows);
            const unsigned long long start = st->rng[epoch & 1u];
            unsigned long long state =
                ((unsigned long long)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(start >> 32)) << 32) |
                (unsigned long long)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)start);
            if (tid == 0) st->epoch = epoch;
            for (uint32_t k = 0; k < rows; ++k) {
                state = gd_splitmix64(state);
                if (tid == 0) draw_state[k] = state;
            }
        }
        return;
    }
    const uint32_t b = blockIdx.x / c.parts, part = blockIdx.x % c.parts;
    gd_sample_rec *rec = &st->rec[b];
    if (finished[b] != 0) {
        if (PHASE != 1 && part == 0 && tid == 0) {
            rec->best_value = 0.0;
            rec->sum = 0.0;
            rec->best = 0;
            rec->draws = 0;
        }
        return;
    }
    const T *row = logits + (size_t)b * c.cols;
    float *w = s.work + (size_t)b * c.cols;
    const uint32_t p0 = part * GD_SAMPLE_PART;
    const uint32_t c0 = min(p0 + tid * GD_SAMPLE_SEG, c.cols), c1 = min(c0 + GD_SAMPLE_SEG, c.cols);
    const bool whole = c0 + GD_SAMPLE_SEG <= c.cols;
    float v[GD_SAMPLE_SEG];
    float bv = GD_NEG_INF;
    int32_t bi = -1;
    if (PHASE != 2) {
        /* the first 1024 history tokens are fetched before the row's length is known (the buffer has hist_cap places
         * per row, so the loads stay inside it), and the values before the history pass: neither waits for the other */
        const int32_t *h = history + (size_t)b * c.hist_cap;
        int32_t early[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t i = tid + (uint32_t)k * GD_SAMPLE_THREADS;
            early[k] = i < c.hist_cap ? h[i] : -1;
        }
        const int32_t len = min(max(hist_len[b], 0), (int32_t)c.hist_cap);
        const bool penalise = isfinite(c.penalty) && c.penalty > 1.0f && len > 0;
        const bool vec = sizeof(T) == 2 && whole && (reinterpret_cast<uintptr_t>(row + c0) & 15u) == 0u;
        gd_half8 raw;
        if (vec) raw = *reinterpret_cast<const gd_half8 *>(row + c0);
        if (penalise) {
            if (tid < GD_SAMPLE_PART / 32) seen[tid] = 0u;
            __syncthreads();
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int32_t i = (int32_t)tid + k * GD_SAMPLE_THREADS;
                const uint32_t t = (uint32_t)early[k] - p0; /* a negative or foreign token lands outside the part */
                if (i < len && t < (uint32_t)GD_SAMPLE_PART && t + p0 < c.cols) atomicOr(&seen[t >> 5], 1u << (t & 31u));
            }
            for (int32_t i = (int32_t)tid + 4 * GD_SAMPLE_THREADS; i < len; i += GD_SAMPLE_THREADS) {
                const uint32_t t = (uint32_t)h[i] - p0;
                if (t < (uint32_t)GD_SAMPLE_PART && t + p0 < c.cols) atomicOr(&seen[t >> 5], 1u << (t & 31u));
            }
            __syncthreads();
        }
        /* capped and penalised value of every token; leader = largest finite one, lowest index among equals (a
         * thread meets its tokens in ascending order and only a larger value replaces) */
#pragma unroll
        for (int e = 0; e < GD_SAMPLE_SEG; ++e) {
            const uint32_t i = c0 + (uint32_t)e;
            float x = GD_NEG_INF;
            if (i < c1) {
                x = vec ? (float)raw[e] : (float)row[i];
                if (c.softcap > 0.0f) x = c.softcap * tanhf(x / c.softcap);
                if (penalise && ((seen[(i - p0) >> 5] >> ((i - p0) & 31u)) & 1u) != 0u)
                    x = x > 0.0f ? x / c.penalty : x * c.penalty;
                w[i] = x;
                if (isfinite(x) && (bi < 0 || x > bv)) {
                    bv = x;
                    bi = (int32_t)i;
                }
            }
            v[e] = x;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int32_t oi = __shfl_xor(bi, off, 64);
            if (gd_sample_leads(ov, oi, bv, bi)) {
                bv = ov;
                bi = oi;
            }
        }
        if (lane == 0) {
            s_val[wave] = bv;
            s_idx[wave] = bi;
        }
        __syncthreads();
        bv = s_val[0];
        bi = s_idx[0];
#pragma unroll
        for (uint32_t k = 1; k < nw; ++k) {
            if (gd_sample_leads(s_val[k], s_idx[k], bv, bi)) {
                bv = s_val[k];
                bi = s_idx[k];
            }
        }
        if (PHASE == 1) {
            if (tid == 0) {
                gd_sample_part m;
                m.value = bv;
                m.index = bi;
                s.part_max[(size_t)b * c.parts + part] = m;
            }
            return;
        }
    } else {
        /* the row's leader from the parts' leaders (every wavefront works it out for itself), and this thread's
         * values back from work[] */
        for (uint32_t j = lane; j < c.parts; j += 64u) {
            const gd_sample_part m = s.part_max[(size_t)b * c.parts + j];
            if (gd_sample_leads(m.value, m.index, bv, bi)) {
                bv = m.value;
                bi = m.index;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int32_t oi = __shfl_xor(bi, off, 64);
            if (gd_sample_leads(ov, oi, bv, bi)) {
                bv = ov;
                bi = oi;
            }
        }
        if (whole && (reinterpret_cast<uintptr_t>(w + c0) & 15u) == 0u) {
            const gd_float4 lo = *reinterpret_cast<const gd_float4 *>(w + c0);
            const gd_float4 hi = *reinterpret_cast<const gd_float4 *>(w + c0 + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] = lo[e];
                v[4 + e] = hi[e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < GD_SAMPLE_SEG; ++e) v[e] = c0 + (uint32_t)e < c1 ? w[c0 + (uint32_t)e] : GD_NEG_INF;
        }
    }
    if (bi < 0 || !isfinite(c.temperature) || c.temperature <= 0.0f) {
        if (part == 0 && tid == 0) {
            rec->best_value = (double)bv;
            rec->sum = 0.0;
            rec->best = bi < 0 ? 0 : bi;
            rec->draws = 0;
        }
        return;
    }
    /* mass of this thread's segment and of the part (kept for the pick) */
    const double best = (double)bv, temp = (double)c.temperature, threshold = gd_sample_threshold(c, best);
    double sum = 0.0;
#pragma unroll
    for (int e = 0; e < GD_SAMPLE_SEG; ++e) {
        bool valid;
        if (c0 + (uint32_t)e < c1) sum += gd_sample_mass(v[e], best, temp, threshold, valid);
    }
    s.seg_mass[((size_t)b * c.parts + part) * GD_SAMPLE_THREADS + tid] = sum;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0) s_sum[wave] = sum;
    __syncthreads();
    if (tid == 0) {
        double total = 0.0;
        for (uint32_t k = 0; k < nw; ++k) total += s_sum[k];
        s.part_mass[(size_t)b * c.parts + part] = total;
        if (part == 0) {
            /* the leader's own mass is exp(0) = 1 unless min_p > 1 puts the threshold above it, and no mass exceeds
             * 1: the row's mass is positive and finite exactly when min_p is not above 1 */
            rec->best_value = best;
            rec->sum = 0.0;
            rec->best = bi;
            rec->draws = c.min_p > 1.0f ? 0 : 1;
        }
    }
}

/* what the loop does with the chosen token (one workgroup per row) */
struct gd_sample_advance {
    int32_t *history, *hist_len, *finished;
    int32_t *ids;           /* [rows]: the next step's input token */
    int32_t *positions;     /* [rows] += pos_delta */
    int32_t *step_counters; /* [rows] */
    int32_t *out_ids;       /* [max_steps * rows]: the token appended to the row's history, or -1 */
    uint32_t max_steps;
    int32_t pos_delta;
    const unsigned char *table;
    unsigned char *next_x;
    uint32_t row_bytes;
};

/* inclusive prefix sum over the wavefront */
__device__ __forceinline__ double gd_wave_scan(double x, uint32_t lane)
{
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const double y = __shfl_up(x, off, 64);
        if ((int)lane >= off) x += y;
    }
    return x;
}

/* First of 64 * N ascending entries (lane l holds entries l, 64 + l, ...; `count` of them exist) at which the running
 * sum reaches rem; rem is left at what remains at the start of that entry.  Returns count if none does. */
template <int N>
__device__ __forceinline__ uint32_t gd_sample_search(const double (&x)[N], uint32_t count, uint32_t lane, double &rem)
{
#pragma unroll
    for (int q = 0; q < N; ++q) {
        const uint32_t k = 64u * (uint32_t)q + lane;
        if (64u * (uint32_t)q >= count) break;
        const double run = gd_wave_scan(k < count ? x[q] : 0.0, lane);
        const unsigned long long hit = __ballot(k < count && rem - run <= 0.0);
        if (hit != 0ull) {
            const int f = __builtin_ctzll(hit);
            const double before = __shfl(run, f > 0 ? f - 1 : 0, 64);
            if (f > 0) rem -= before;
            return 64u * (uint32_t)q + (uint32_t)f;
        }
        rem -= __shfl(run, 63, 64);
    }
    return count;
}

__global__ void __launch_bounds__(GD_SAMPLE_THREADS)
gd_sample_pick_kernel(gd_sample_scratch s, gd_sample_state *__restrict__ st, gd_sample_cfg c, gd_sample_advance adv)
{
    __shared__ int32_t s_token;
    const uint32_t b = blockIdx.x, rows = gridDim.x, tid = threadIdx.x, nt = blockDim.x, lane = tid & 63u;
    const gd_sample_rec rec = st->rec[b];
    const bool was_finished = adv.finished[b] != 0;
    const bool draws = !was_finished && rec.draws != 0;
    const uint32_t epoch = st->epoch;
    if (tid < 64u) { /* the first wavefront picks; the others only help with the copy at the end */
        int32_t token = rec.best;
        /* fetched now, needed at the end: nothing in between writes them */
        const int32_t len0 = adv.hist_len[b], step0 = adv.step_counters[b], pos0 = adv.positions[b];
        double pm[2] = {0.0, 0.0}, sm[4] = {0.0, 0.0, 0.0, 0.0};
        unsigned long long my_state = 0ull;
        if (draws) {
            if (lane < c.parts) pm[0] = s.part_mass[(size_t)b * c.parts + lane];
            if (64u + lane < c.parts) pm[1] = s.part_mass[(size_t)b * c.parts + 64u + lane];
            if (lane < rows) my_state = gd_sample_draw_states(st, rows)[lane]; /* state number rank, if rows <= 64 */
            if (c.parts == 1u) {
                const double *segs = s.seg_mass + (size_t)b * GD_SAMPLE_THREADS;
#pragma unroll
                for (int q = 0; q < 4; ++q) sm[q] = segs[64u * (uint32_t)q + lane];
            }
        }
        /* draws of the rows before this one and of all rows */
        uint32_t rank = 0, total = 0;
        for (uint32_t j = lane; j < rows; j += 64u) {
            const uint32_t d = st->rec[j].draws != 0 ? 1u : 0u;
            total += d;
            rank += j < b ? d : 0u;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            rank += __shfl_xor(rank, off, 64);
            total += __shfl_xor(total, off, 64);
        }
        if (draws) {
            const double best = rec.best_value, temp = (double)c.temperature, threshold = gd_sample_threshold(c, best);
            const float *w = s.work + (size_t)b * c.cols;
            /* this row's place in the generator's sequence: after the draws of the rows before it */
            const unsigned long long state = rows <= 64u ? __shfl(my_state, (int)rank, 64)
                                                         : gd_sample_draw_states(st, rows)[rank];
            double row_mass = pm[0] + pm[1];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) row_mass += __shfl_xor(row_mass, off, 64);
            double rem = ((double)(state >> 11) * (1.0 / 9007199254740992.0)) * row_mass;
            /* part, then segment, in which the running mass reaches the drawn point */
            const uint32_t part = gd_sample_search<2>(pm, c.parts, lane, rem);
            uint32_t start = c.cols; /* token from which to walk */
            if (part < c.parts) {
                if (c.parts > 1u) {
                    const double *segs = s.seg_mass + ((size_t)b * c.parts + part) * GD_SAMPLE_THREADS;
#pragma unroll
                    for (int q = 0; q < 4; ++q) sm[q] = segs[64u * (uint32_t)q + lane];
                }
                const uint32_t seg = gd_sample_search<4>(sm, GD_SAMPLE_THREADS, lane, rem);
                start = min(part * GD_SAMPLE_PART + seg * GD_SAMPLE_SEG, c.cols);
            }
            /* the token: normally among the next 8; further on only if the rounding of the sums says so */
            int32_t found = -1;
            for (uint32_t base = start; base < c.cols && found < 0; base += 64u) {
                const uint32_t i = base + lane;
                bool valid = false;
                const double x = gd_wave_scan(i < c.cols ? gd_sample_mass(w[i], best, temp, threshold, valid) : 0.0, lane);
                const unsigned long long hit = __ballot(valid && rem - x <= 0.0);
                if (hit != 0ull) found = (int32_t)(base + (uint32_t)__builtin_ctzll(hit));
                rem -= __shfl(x, 63, 64);
            }
            if (found >= 0) token = found;
            /* the last draw of the step leaves the generator's next state */
            if (lane == 0 && rank + 1u == total) st->rng[(epoch + 1u) & 1u] = state;
        }
        if (b == 0 && lane == 0 && total == 0u) st->rng[(epoch + 1u) & 1u] = st->rng[epoch & 1u];
        if (lane == 0) {
            int32_t fin = was_finished ? 1 : 0, appended = 0;
            if (!fin) {
                const int32_t len = max(len0, 0);
                if (c.stop_token >= 0 && token == c.stop_token) {
                    fin = 1;
                } else if (len >= (int32_t)c.hist_cap) {
                    fin = 1;
                } else {
                    adv.history[(size_t)b * c.hist_cap + (size_t)len] = token;
                    adv.hist_len[b] = len + 1;
                    appended = 1;
                }
                adv.finished[b] = fin;
            }
            const int32_t next = fin ? (c.stop_token >= 0 ? c.stop_token : 0) : token;
            adv.ids[b] = next;
            adv.positions[b] = pos0 + adv.pos_delta;
            if (step0 >= 0 && (uint32_t)step0 < adv.max_steps) adv.out_ids[(size_t)step0 * rows + b] = appended ? token : -1;
            adv.step_counters[b] = step0 + 1;
            s_token = next;
        }
    }
    if (adv.table != nullptr) {
        __syncthreads();
        const gd_u128 *src = reinterpret_cast<const gd_u128 *>(adv.table + (size_t)s_token * adv.row_bytes);
        gd_u128 *dst = reinterpret_cast<gd_u128 *>(adv.next_x + (size_t)b * adv.row_bytes);
        for (uint32_t i = tid; i < adv.row_bytes / 16u; i += nt) dst[i] = src[i];
    }
}

template <typename T>
static void gd_sample_launch_prepare(hipStream_t stream, const void *logits, const gd_sample_scratch &s,
                                     gd_sample_state *st, uint32_t rows, const gd_sample_cfg &cfg,
                                     const gd_sample_advance *adv)
{
    const T *in = (const T *)logits;
    const uint32_t blocks = rows * cfg.parts;
    if (cfg.parts == 1u) {
        gd_sample_prepare_kernel<T, 0><<<blocks + 1u, GD_SAMPLE_THREADS, 0, stream>>>(in, s, st, adv->history, adv->hist_len, adv->finished, rows, cfg);
    } else {
        gd_sample_prepare_kernel<T, 1><<<blocks + 1u, GD_SAMPLE_THREADS, 0, stream>>>(in, s, st, adv->history, adv->hist_len, adv->finished, rows, cfg);
        gd_sample_prepare_kernel<T, 2><<<blocks, GD_SAMPLE_THREADS, 0, stream>>>(in, s, st, adv->history, adv->hist_len, adv->finished, rows, cfg);
    }
}

/* work: F32 [rows * cols] values (an even count), then per row and part 256 + 1 F64 masses and one leader */
extern "C" int gd_hip_launch_sample_advance(hipStream_t stream, const void *logits, int is_f16, float *work, void *state,
                                            uint32_t rows, const gd_sample_cfg *cfg_in, const gd_sample_advance *adv)
{
    gd_sample_state *st = (gd_sample_state *)state;
    gd_sample_cfg cfg = *cfg_in;
    gd_sample_scratch s;
    if (rows == 0u) return (int)hipSuccess;
    cfg.parts = (cfg.cols + GD_SAMPLE_PART - 1u) / GD_SAMPLE_PART;
    if (cfg.parts > GD_SAMPLE_MAX_PARTS) return (int)hipErrorInvalidValue;
    const size_t values = ((size_t)rows * cfg.cols + 1u) & ~(size_t)1u, cells = (size_t)rows * cfg.parts;
    s.work = work;
    s.seg_mass = reinterpret_cast<double *>(work + values);
    s.part_mass = s.seg_mass + cells * GD_SAMPLE_THREADS;
    s.part_max = reinterpret_cast<gd_sample_part *>(s.part_mass + cells);
    if (is_f16) gd_sample_launch_prepare<gd_half>(stream, logits, s, st, rows, cfg, adv);
    else gd_sample_launch_prepare<float>(stream, logits, s, st, rows, cfg, adv);
    gd_sample_pick_kernel<<<rows, GD_SAMPLE_THREADS, 0, stream>>>(s, st, cfg, *adv);
    return (int)hipGetLastError();
}
