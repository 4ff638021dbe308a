/*
 * Next-token sampling on the device for gfx950: soft cap, repetition penalty, temperature / min-p
 * draw and the bookkeeping of a generation loop, so that a device-resident loop never moves the
 * logits to the host.  Restates the host code of the reference's example,
 * examples/gpt_lm/gpt_lm_shared.c: gpt_apply_logits_softcap (:1322-1331),
 * gpt_apply_repetition_penalty (:1347-1369), gpt_sample_next_token (:1371-1442) and the loop
 * around them (:1586-1600, 1606-1680): one generator shared by the rows, advanced once per row
 * that really draws, in row order; a row ends at the stop token or when its history is full.
 *
 * Two launches, one workgroup per row each:
 *   prepare  capped and penalised logits -> work[row] (F32), leader, total mass, "will draw"
 *   pick     the row's draw (its rank among the drawing rows gives its place in the generator's
 *            sequence), inverse CDF over work[row], history / finished / ids / positions /
 *            record update, optional gather of the next embedding row
 * HBM traffic per row: logits once, work written once and read three times (L2-resident).
 *
 * Arithmetic as in the reference: F32 cap (tanhf) and penalty, F64 mass (exp) and target.  Sums are
 * formed in another order than the reference's left-to-right loop, so the total and the running
 * sums can differ in the last bits; the chosen token differs only when the drawn point lies within
 * that distance of a boundary between two tokens.
 */
#include "../../_shared/hip_device.h"

#define GD_SAMPLE_MAX_THREADS 1024
#define GD_NEG_INF (-__builtin_inff())

struct __attribute__((aligned(8))) gd_sample_rec {
    double best_value, sum;
    int32_t best, draws;
    int32_t pad[2];
};

/* device-resident generator and per-row records; the caller provides it as an I32 tensor of
 * 8 + 8 * rows elements, 8-byte aligned */
struct __attribute__((aligned(8))) gd_sample_state {
    unsigned long long rng[2]; /* slot (epoch & 1) is current */
    uint32_t epoch;            /* +1 per prepare launch */
    uint32_t pad[3];
    gd_sample_rec rec[1];
};

struct gd_sample_cfg {
    float temperature, min_p, penalty, softcap;
    int32_t stop_token;
    uint32_t cols, hist_cap;
};

__device__ __forceinline__ unsigned long long gd_splitmix64(unsigned long long x)
{
    x += 0x9e3779b97f4a7c15ull;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
    return x ^ (x >> 31);
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

template <typename T>
__global__ void __launch_bounds__(GD_SAMPLE_MAX_THREADS)
gd_sample_prepare_kernel(const T *__restrict__ logits, float *__restrict__ work, gd_sample_state *__restrict__ st,
                         const int32_t *__restrict__ history, const int32_t *__restrict__ hist_len,
                         const int32_t *__restrict__ finished, gd_sample_cfg c)
{
    extern __shared__ uint32_t seen[]; /* one bit per token: already penalised */
    __shared__ float s_val[GD_SAMPLE_MAX_THREADS / 64];
    __shared__ int32_t s_idx[GD_SAMPLE_MAX_THREADS / 64];
    __shared__ double s_sum[GD_SAMPLE_MAX_THREADS / 64];
    __shared__ float s_best;
    __shared__ int32_t s_best_idx;
    const uint32_t b = blockIdx.x, tid = threadIdx.x, nt = blockDim.x, lane = tid & 63u, wave = tid >> 6;
    gd_sample_rec *rec = &st->rec[b];
    if (b == 0 && tid == 0) st->epoch += 1u;
    if (finished[b] != 0) {
        if (tid == 0) {
            rec->best_value = 0.0;
            rec->sum = 0.0;
            rec->best = 0;
            rec->draws = 0;
        }
        return;
    }
    const T *row = logits + (size_t)b * c.cols;
    float *w = work + (size_t)b * c.cols;
    const int32_t len = min(max(hist_len[b], 0), (int32_t)c.hist_cap);
    const bool penalise = isfinite(c.penalty) && c.penalty > 1.0f && len > 0;
    if (penalise) {
        for (uint32_t i = tid; i < (c.cols + 31u) / 32u; i += nt) seen[i] = 0u;
    }
    for (uint32_t i = tid; i < c.cols; i += nt) {
        float v = (float)row[i];
        if (c.softcap > 0.0f) v = c.softcap * tanhf(v / c.softcap);
        w[i] = v;
    }
    __syncthreads();
    if (penalise) {
        const int32_t *h = history + (size_t)b * c.hist_cap;
        for (int32_t i = (int32_t)tid; i < len; i += (int32_t)nt) {
            const int32_t t = h[i];
            if (t < 0 || (uint32_t)t >= c.cols) continue;
            const uint32_t bit = 1u << (t & 31);
            if ((atomicOr(&seen[t >> 5], bit) & bit) != 0u) continue; /* another occurrence got there first */
            const float v = w[t];
            w[t] = v > 0.0f ? v / c.penalty : v * c.penalty;
        }
        __syncthreads();
    }
    /* leader: largest finite value, lowest index among equals */
    float bv = GD_NEG_INF;
    int32_t bi = -1;
    for (uint32_t i = tid; i < c.cols; i += nt) {
        const float v = w[i];
        if (isfinite(v) && (bi < 0 || v > bv)) {
            bv = v;
            bi = (int32_t)i;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int32_t oi = __shfl_xor(bi, off, 64);
        if (oi >= 0 && (bi < 0 || ov > bv || (ov == bv && oi < bi))) {
            bv = ov;
            bi = oi;
        }
    }
    if (lane == 0) {
        s_val[wave] = bv;
        s_idx[wave] = bi;
    }
    __syncthreads();
    if (tid == 0) {
        for (uint32_t k = 1; k < nt / 64u; ++k) {
            const float ov = s_val[k];
            const int32_t oi = s_idx[k];
            if (oi >= 0 && (bi < 0 || ov > bv || (ov == bv && oi < bi))) {
                bv = ov;
                bi = oi;
            }
        }
        s_best = bv;
        s_best_idx = bi;
    }
    __syncthreads();
    bv = s_best;
    bi = s_best_idx;
    if (bi < 0 || !isfinite(c.temperature) || c.temperature <= 0.0f) {
        if (tid == 0) {
            rec->best_value = (double)bv;
            rec->sum = 0.0;
            rec->best = bi < 0 ? 0 : bi;
            rec->draws = 0;
        }
        return;
    }
    const double best = (double)bv, temp = (double)c.temperature, threshold = gd_sample_threshold(c, best);
    double sum = 0.0;
    for (uint32_t i = tid; i < c.cols; i += nt) {
        bool valid;
        sum += gd_sample_mass(w[i], best, temp, threshold, valid);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0) s_sum[wave] = sum;
    __syncthreads();
    if (tid == 0) {
        double total = 0.0;
        for (uint32_t k = 0; k < nt / 64u; ++k) total += s_sum[k];
        rec->best_value = best;
        rec->sum = total;
        rec->best = bi;
        rec->draws = (total > 0.0 && isfinite(total)) ? 1 : 0;
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

#define GD_SAMPLE_MAX_COLS 262144u /* 64-token segments: 4096 partial sums in LDS; penalty bitmap 32 KiB */

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

__global__ void __launch_bounds__(GD_SAMPLE_MAX_THREADS)
gd_sample_pick_kernel(const float *__restrict__ work, gd_sample_state *__restrict__ st, gd_sample_cfg c,
                      gd_sample_advance adv)
{
    __shared__ double part[GD_SAMPLE_MAX_COLS / 64u]; /* mass of every 64-token segment */
    __shared__ int32_t s_token;
    const uint32_t b = blockIdx.x, rows = gridDim.x, tid = threadIdx.x, nt = blockDim.x, lane = tid & 63u;
    const uint32_t wave = tid >> 6, nw = nt >> 6;
    const gd_sample_rec rec = st->rec[b];
    const bool was_finished = adv.finished[b] != 0;
    const bool draws = !was_finished && rec.draws != 0;
    const float *w = work + (size_t)b * c.cols;
    const uint32_t epoch = st->epoch;
    if (tid == 0) s_token = rec.best;
    if (draws) {
        const double best = rec.best_value, temp = (double)c.temperature, threshold = gd_sample_threshold(c, best);
        const uint32_t nseg = (c.cols + 63u) / 64u;
        for (uint32_t seg = wave; seg < nseg; seg += nw) {
            const uint32_t i = seg * 64u + lane;
            bool valid;
            double x = i < c.cols ? gd_sample_mass(w[i], best, temp, threshold, valid) : 0.0;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
            if (lane == 0) part[seg] = x;
        }
        __syncthreads();
        if (wave == 0) {
            double rem = 0.0;
            if (lane == 0) {
                /* this row's place in the generator's sequence: after the draws of the rows before it */
                uint32_t rank = 0;
                for (uint32_t j = 0; j < b; ++j) rank += st->rec[j].draws != 0 ? 1u : 0u;
                unsigned long long state = st->rng[epoch & 1u];
                for (uint32_t k = 0; k <= rank; ++k) state = gd_splitmix64(state);
                rem = ((double)(state >> 11) * (1.0 / 9007199254740992.0)) * rec.sum;
            }
            rem = __shfl(rem, 0, 64);
            /* segment in which the running sum reaches the drawn point */
            uint32_t first = nseg;
            for (uint32_t base = 0; base < nseg && first == nseg; base += 64u) {
                const uint32_t k = base + lane;
                const double x = gd_wave_scan(k < nseg ? part[k] : 0.0, lane);
                const unsigned long long hit = __ballot(k < nseg && rem - x <= 0.0);
                if (hit != 0ull) {
                    const int f = __builtin_ctzll(hit);
                    const double before = __shfl(x, f > 0 ? f - 1 : 0, 64);
                    first = base + (uint32_t)f;
                    if (f > 0) rem -= before;
                } else {
                    rem -= __shfl(x, 63, 64);
                }
            }
            /* the token inside it (the next segments only if rounding of the segment sums says so) */
            int32_t found = -1;
            for (uint32_t seg = first; seg < nseg && found < 0; ++seg) {
                const uint32_t i = seg * 64u + lane;
                bool valid = false;
                const double x = gd_wave_scan(i < c.cols ? gd_sample_mass(w[i], best, temp, threshold, valid) : 0.0, lane);
                const unsigned long long hit = __ballot(valid && rem - x <= 0.0);
                if (hit != 0ull) found = (int32_t)(seg * 64u + (uint32_t)__builtin_ctzll(hit));
                rem -= __shfl(x, 63, 64);
            }
            if (lane == 0 && found >= 0) s_token = found;
        }
    }
    __syncthreads();
    if (tid == 0) {
        const int32_t token = s_token;
        int32_t fin = was_finished ? 1 : 0, appended = 0;
        if (!fin) {
            const int32_t len = max(adv.hist_len[b], 0);
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
        adv.positions[b] += adv.pos_delta;
        const int32_t s = adv.step_counters[b];
        if (s >= 0 && (uint32_t)s < adv.max_steps) adv.out_ids[(size_t)s * rows + b] = appended ? token : -1;
        adv.step_counters[b] = s + 1;
        s_token = next;
        if (b == 0) {
            /* the generator moves on by the number of draws of this step; the other slot is written because
             * the other rows' workgroups may still be reading the current one */
            uint32_t total = 0;
            for (uint32_t j = 0; j < rows; ++j) total += st->rec[j].draws != 0 ? 1u : 0u;
            unsigned long long state = st->rng[epoch & 1u];
            for (uint32_t k = 0; k < total; ++k) state = gd_splitmix64(state);
            st->rng[(epoch + 1u) & 1u] = state;
        }
    }
    if (adv.table != nullptr) {
        __syncthreads();
        const gd_u128 *src = reinterpret_cast<const gd_u128 *>(adv.table + (size_t)s_token * adv.row_bytes);
        gd_u128 *dst = reinterpret_cast<gd_u128 *>(adv.next_x + (size_t)b * adv.row_bytes);
        for (uint32_t i = tid; i < adv.row_bytes / 16u; i += nt) dst[i] = src[i];
    }
}

extern "C" int gd_hip_launch_sample_advance(hipStream_t stream, const void *logits, int is_f16, float *work, void *state,
                                            uint32_t rows, const gd_sample_cfg *cfg, const gd_sample_advance *adv)
{
    const unsigned threads = cfg->cols >= 8192u ? GD_SAMPLE_MAX_THREADS : 256u;
    const size_t lds = (size_t)((cfg->cols + 31u) / 32u) * sizeof(uint32_t);
    gd_sample_state *st = (gd_sample_state *)state;
    if (rows == 0u) return (int)hipSuccess;
    if (is_f16)
        gd_sample_prepare_kernel<gd_half><<<rows, threads, lds, stream>>>((const gd_half *)logits, work, st, adv->history,
                                                                          adv->hist_len, adv->finished, *cfg);
    else
        gd_sample_prepare_kernel<float><<<rows, threads, lds, stream>>>((const float *)logits, work, st, adv->history,
                                                                        adv->hist_len, adv->finished, *cfg);
    gd_sample_pick_kernel<<<rows, threads, 0, stream>>>(work, st, *cfg, *adv);
    return (int)hipGetLastError();
}
