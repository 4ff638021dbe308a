/*
 * gd_oracle.c - CPU restatement of the gradients.c inference decode path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP backend is compared
 * against; it is built into oracle/libgd_oracle.so and may be loaded only by the
 * test-suite, the smoke check and the CPU-baseline leg of the benchmark.  Nothing
 * in the product library links, loads or falls back to it.
 *
 * The reference has no CPU execution path.  Every function below restates either
 * (a) one of the double/float reference routines the reference keeps inside its
 * own C tests, or (b) the arithmetic of the reference's Metal kernel for that
 * operator, with the same rounding points (F16 loads, wide accumulation, one F16
 * rounding per stored value).  The citation above each function names the
 * reference lines it follows.  Accumulation is done in double where the
 * reference's in-test oracle does so (attention) and in double for dot products
 * (the reference kernels use F32 there; both approximate the exact value and the
 * reference's own tolerance covers the difference).
 *
 * Pinning status (what fixes each function besides this text is listed in
 * tests/test_oracle_pinning.py): every function has at least one check against a
 * golden vector of the reference's tests, a closed form, a brute-force model or
 * a library routine.  No function is "parity unpinned".
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define GDO_API __attribute__((visibility("default")))

/* ---- F16 <-> F32, round to nearest even ---------------------------------- */

/* reference src/core/dtype_internal.h:6-60 */
GDO_API uint16_t gdo_f32_to_f16(float value)
{
    union { float f; uint32_t u; } in;
    in.f = value;
    const uint32_t sign = (in.u >> 16) & 0x8000u;
    const uint32_t biased = (in.u >> 23) & 0xffu;
    uint32_t frac = in.u & 0x7fffffu;
    if (biased == 0xffu) {
        return (uint16_t)(sign | (frac ? 0x7e00u : 0x7c00u)); /* NaN collapses to 0x7e00 */
    }
    const int32_t e = (int32_t)biased - 127;
    if (e > 15) {
        return (uint16_t)(sign | 0x7c00u);
    }
    if (e < -14) { /* subnormal half or zero */
        const int32_t shift = -14 - e;
        /* |value| < 2^-25 rounds to zero.  The reference tests `shift > 24` here and
         * then shifts a 32-bit word by shift+13 (up to 37 bits), which is undefined
         * for 2^-39 <= |value| < 2^-33; this restatement keeps the IEEE result. */
        if (shift > 11) {
            return (uint16_t)sign;
        }
        frac |= 0x800000u;
        const uint32_t drop = (uint32_t)shift + 13u;
        uint32_t kept = frac >> drop;
        const uint32_t rest = frac & ((1u << drop) - 1u);
        const uint32_t half = 1u << (drop - 1u);
        if (rest > half || (rest == half && (kept & 1u))) {
            kept += 1u;
        }
        return (uint16_t)(sign | kept);
    }
    uint32_t he = (uint32_t)(e + 15);
    uint32_t hm = frac >> 13;
    const uint32_t rest = frac & 0x1fffu;
    if (rest > 0x1000u || (rest == 0x1000u && (hm & 1u))) {
        hm += 1u;
        if (hm == 0x400u) {
            hm = 0u;
            he += 1u;
            if (he >= 31u) {
                return (uint16_t)(sign | 0x7c00u);
            }
        }
    }
    return (uint16_t)(sign | (he << 10) | hm);
}

/* reference src/core/dtype_internal.h:62-88 */
GDO_API float gdo_f16_to_f32(uint16_t bits)
{
    union { uint32_t u; float f; } out;
    const uint32_t sign = ((uint32_t)bits & 0x8000u) << 16;
    int32_t e = (int32_t)((bits >> 10) & 0x1fu);
    uint32_t m = (uint32_t)bits & 0x3ffu;
    if (e == 0) {
        if (m == 0u) {
            out.u = sign;
            return out.f;
        }
        e = 1;
        while (!(m & 0x400u)) {
            m <<= 1;
            e -= 1;
        }
        m &= 0x3ffu;
    } else if (e == 31) {
        out.u = sign | 0x7f800000u | (m << 13);
        return out.f;
    }
    out.u = sign | ((uint32_t)(e + 112) << 23) | (m << 13);
    return out.f;
}

GDO_API void gdo_f32_to_f16_array(const float *src, uint16_t *dst, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = gdo_f32_to_f16(src[i]);
}

GDO_API void gdo_f16_to_f32_array(const uint16_t *src, float *dst, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = gdo_f16_to_f32(src[i]);
}

static inline double h2d(uint16_t h) { return (double)gdo_f16_to_f32(h); }

/* ---- deterministic input generators -------------------------------------- */

/* reference examples/gpt_lm/gpt_lm_shared.c:32-48 */
static uint64_t mix64(uint64_t x)
{
    x = (x ^ (x >> 30)) * UINT64_C(0xbf58476d1ce4e5b9);
    x = (x ^ (x >> 27)) * UINT64_C(0x94d049bb133111eb);
    return x ^ (x >> 31);
}

GDO_API uint64_t gdo_splitmix64(uint64_t x) { return mix64(x + UINT64_C(0x9e3779b97f4a7c15)); }

static uint64_t stream_next(uint64_t *state)
{
    *state += UINT64_C(0x9e3779b97f4a7c15);
    return mix64(*state);
}

/* reference examples/gpt_lm/gpt_lm_shared.c:196-218: uniform in (0,1], Box-Muller
 * pairs (cos first, then sin), scaled by stddev in double, stored as float. */
GDO_API void gdo_fill_normal(float *values, size_t count, uint64_t seed, float stddev)
{
    uint64_t state = seed;
    size_t i = 0;
    while (i < count) {
        const double u1 = ((double)(stream_next(&state) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
        const double u2 = ((double)(stream_next(&state) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
        const double radius = sqrt(-2.0 * log(u1));
        const double angle = 6.283185307179586476925286766559 * u2;
        values[i++] = (float)(radius * cos(angle) * (double)stddev);
        if (i < count) {
            values[i++] = (float)(radius * sin(angle) * (double)stddev);
        }
    }
}

GDO_API void gdo_fill_normal_f16(uint16_t *values, size_t count, uint64_t seed, float stddev)
{
    /* same stream as gdo_fill_normal, rounded to F16 the way gd_tensor_write_f32
     * does (reference src/core/transfer.c uses gd_f32_to_f16_bits). */
    uint64_t state = seed;
    size_t i = 0;
    while (i < count) {
        const double u1 = ((double)(stream_next(&state) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
        const double u2 = ((double)(stream_next(&state) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
        const double radius = sqrt(-2.0 * log(u1));
        const double angle = 6.283185307179586476925286766559 * u2;
        values[i++] = gdo_f32_to_f16((float)(radius * cos(angle) * (double)stddev));
        if (i < count) {
            values[i++] = gdo_f32_to_f16((float)(radius * sin(angle) * (double)stddev));
        }
    }
}

/* reference src/backends/metal/primitives/random/metal_random.metal:8-30 (gd_backend_rand_uniform):
 * element i is low + (high - low) * u with u = bits [40,64) of splitmix64(seed + i) times 2^-24,
 * evaluated in F32 as one fused multiply-add (the shader source writes low + span * u and its compiler
 * contracts by default; the HIP kernel pins the same single rounding), stored as F32. */
GDO_API void gdo_rand_uniform_f32(float *values, size_t count, uint64_t seed, float low, float high)
{
    const float span = high - low;
    for (size_t i = 0; i < count; ++i) {
        const uint32_t mant = (uint32_t)((gdo_splitmix64(seed + (uint64_t)i) >> 40) & 0xffffffu);
        const float u = (float)mant * (1.0f / 16777216.0f);
        values[i] = fmaf(span, u, low);
    }
}

/* Uniform integers in [lo, hi] from the same splitmix64 stream (modulo draw). */
GDO_API void gdo_fill_uniform_i32(int32_t *values, size_t count, uint64_t seed, int32_t lo, int32_t hi)
{
    uint64_t state = seed;
    const uint64_t span = (uint64_t)((int64_t)hi - (int64_t)lo + 1);
    for (size_t i = 0; i < count; ++i) {
        values[i] = (int32_t)((int64_t)lo + (int64_t)((stream_next(&state) >> 11) % span));
    }
}

/* reference tests/test_sdpa_varlen.c:149-156 */
GDO_API void gdo_fill_tokens(uint16_t *x, uint32_t count, float base)
{
    for (uint32_t i = 0; i < count; ++i) {
        x[i] = gdo_f32_to_f16(base + 0.03125f * (float)((i * 17u + 3u) % 19u) -
                              0.015625f * (float)(i % 5u));
    }
}

/* reference tests/test_linear.c:61-67 */
GDO_API void gdo_fill_values(float *dst, size_t count, float scale, float bias)
{
    for (size_t i = 0; i < count; ++i) {
        dst[i] = bias + scale * (float)((i * 17u + 5u) % 31u) - 0.5f * scale * (float)(i % 7u);
    }
}

/* ---- A1: K/V cache append ------------------------------------------------- */

/* reference src/ops/kv_cache_append/metal_kv_cache_append.metal:30-63.
 * cache [B,Tmax,row_bytes], fresh [B,Tnew,row_bytes] as raw bytes.  pos == NULL
 * selects the scalar position.  A batch row is skipped when its position is
 * negative or pos + Tnew > Tmax. */
GDO_API void gdo_kv_cache_append(uint8_t *k_cache, uint8_t *v_cache, const uint8_t *k_new,
                                 const uint8_t *v_new, const int32_t *pos, int32_t scalar_pos,
                                 int64_t batch, int64_t tnew, int64_t tmax, int64_t row_bytes)
{
    for (int64_t b = 0; b < batch; ++b) {
        const int64_t p = pos ? pos[b] : scalar_pos;
        if (p < 0 || p + tnew > tmax) {
            continue;
        }
        for (int64_t t = 0; t < tnew; ++t) {
            const size_t dst = (size_t)((b * tmax + p + t) * row_bytes);
            const size_t src = (size_t)((b * tnew + t) * row_bytes);
            memcpy(k_cache + dst, k_new + src, (size_t)row_bytes);
            memcpy(v_cache + dst, v_new + src, (size_t)row_bytes);
        }
    }
}

/* reference src/ops/kv_cache_append/metal_kv_cache_append.metal:65-122.
 * fresh rows packed [N,row_bytes]; row -> batch by the largest b with cu[b] <= row
 * (binary search over b in [0,B)); nothing is written when cu[0] != 0, rows at or
 * past cu[B] are ignored, and a sequence is skipped when its range is malformed
 * or pos + len > Tmax. */
GDO_API void gdo_kv_cache_append_packed(uint8_t *k_cache, uint8_t *v_cache, const uint8_t *k_new,
                                        const uint8_t *v_new, const int32_t *pos, const int32_t *cu,
                                        int64_t batch, int64_t n_rows, int64_t tmax, int64_t row_bytes)
{
    if (batch <= 0 || cu[0] != 0) {
        return;
    }
    for (int64_t row = 0; row < n_rows; ++row) {
        if ((int32_t)row >= cu[batch]) {
            continue;
        }
        uint32_t lo = 0, hi = (uint32_t)batch;
        while (lo + 1u < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if ((uint32_t)cu[mid] <= (uint32_t)row) lo = mid; else hi = mid;
        }
        const int32_t start = cu[lo], end = cu[lo + 1];
        const int32_t t = (int32_t)row - start;
        const int32_t p = pos[lo];
        if (start < 0 || end < start || t < 0 || p < 0 || (int64_t)p + (end - start) > tmax) {
            continue;
        }
        const size_t dst = (size_t)(((int64_t)lo * tmax + p + t) * row_bytes);
        const size_t src = (size_t)(row * row_bytes);
        memcpy(k_cache + dst, k_new + src, (size_t)row_bytes);
        memcpy(v_cache + dst, v_new + src, (size_t)row_bytes);
    }
}

/* ---- attention mask -------------------------------------------------------- */

/* reference tests/test_sdpa_varlen.c:122-147 and
 * src/ops/sdpa_decode/metal_sdpa_decode.metal:30-53 (causal fixed to 1 there). */
GDO_API int gdo_attn_allowed(int i, int j, int causal, int window, int prefix_len)
{
    if (causal) {
        if (prefix_len > 0) {
            if (i < prefix_len) {
                if (j >= prefix_len) return 0;
            } else if (j > i) {
                return 0;
            }
        } else if (j > i) {
            return 0;
        }
    }
    if (window > 0) {
        if (prefix_len > 0) {
            if (i >= prefix_len && j >= prefix_len && (i - j) >= window) return 0;
        } else if ((i - j) >= window) {
            return 0;
        }
    }
    return 1;
}

/* ---- A2: sdpa_decode ------------------------------------------------------- */

/* reference tests/test_sdpa_varlen.c:604-677 (ref_decode), generalised from one
 * scalar position to one position per batch row as
 * src/ops/sdpa_decode/metal_sdpa_decode.metal:199-212 does: live = min(pos+Tq,
 * Tmax), qpos = pos + i, two-pass softmax in double, out = sum(e v)/sum(e), zero
 * when no key is visible.  Rows with pos < 0 keep `out` as passed in (the kernel
 * returns before storing, metal:205-207).  q/out [B,Tq,Hq,D], caches
 * [B,Tmax,Hkv,D], all F16 bit patterns; out_f32 receives the unrounded result. */
GDO_API void gdo_sdpa_decode_f16(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                                 const int32_t *pos, int64_t B, int64_t Tq, int64_t Tmax,
                                 int64_t Hq, int64_t Hkv, int64_t D, float scale, int window,
                                 int prefix_len, float *out_f32)
{
    const int64_t group = Hq / Hkv;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t hq = 0; hq < Hq; ++hq) {
            const int32_t p = pos[b];
            if (p < 0) continue;
            const int64_t hkv = hq / group;
            int64_t live = (int64_t)p + Tq;
            if (live > Tmax) live = Tmax;
            double *scores = (double *)malloc((size_t)(live > 0 ? live : 1) * sizeof(double));
            double acc[256];
            for (int64_t i = 0; i < Tq; ++i) {
                const int qpos = p + (int)i;
                const uint16_t *qrow = q + ((b * Tq + i) * Hq + hq) * D;
                float *orow = out_f32 + ((b * Tq + i) * Hq + hq) * D;
                double m = -HUGE_VAL, sum = 0.0;
                for (int64_t j = 0; j < live; ++j) {
                    if (!gdo_attn_allowed(qpos, (int)j, 1, window, prefix_len)) continue;
                    const uint16_t *krow = k + ((b * Tmax + j) * Hkv + hkv) * D;
                    double s = 0.0;
                    for (int64_t c = 0; c < D; ++c) s += h2d(qrow[c]) * h2d(krow[c]);
                    s *= (double)scale;
                    scores[j] = s;
                    if (s > m) m = s;
                }
                for (int64_t c = 0; c < D; ++c) acc[c] = 0.0;
                for (int64_t j = 0; j < live; ++j) {
                    if (!gdo_attn_allowed(qpos, (int)j, 1, window, prefix_len)) continue;
                    const uint16_t *vrow = v + ((b * Tmax + j) * Hkv + hkv) * D;
                    const double e = exp(scores[j] - m);
                    sum += e;
                    for (int64_t c = 0; c < D; ++c) acc[c] += e * h2d(vrow[c]);
                }
                for (int64_t c = 0; c < D; ++c) orow[c] = sum > 0.0 ? (float)(acc[c] / sum) : 0.0f;
            }
            free(scores);
        }
    }
}

/* F32 caches: same arithmetic on float inputs (the reference's append/decode
 * consistency tests use F32 tensors, tests/test_kv_cache_decode.c:181-303). */
GDO_API void gdo_sdpa_decode_f32(const float *q, const float *k, const float *v, const int32_t *pos,
                                 int64_t B, int64_t Tq, int64_t Tmax, int64_t Hq, int64_t Hkv,
                                 int64_t D, float scale, int window, int prefix_len, float *out)
{
    const int64_t group = Hq / Hkv;
    for (int64_t b = 0; b < B; ++b) {
        const int32_t p = pos[b];
        if (p < 0) continue;
        int64_t live = (int64_t)p + Tq;
        if (live > Tmax) live = Tmax;
        for (int64_t hq = 0; hq < Hq; ++hq) {
            const int64_t hkv = hq / group;
            for (int64_t i = 0; i < Tq; ++i) {
                const int qpos = p + (int)i;
                const float *qrow = q + ((b * Tq + i) * Hq + hq) * D;
                float *orow = out + ((b * Tq + i) * Hq + hq) * D;
                double m = -HUGE_VAL, sum = 0.0, acc[256];
                for (int64_t j = 0; j < live; ++j) {
                    if (!gdo_attn_allowed(qpos, (int)j, 1, window, prefix_len)) continue;
                    const float *krow = k + ((b * Tmax + j) * Hkv + hkv) * D;
                    double s = 0.0;
                    for (int64_t c = 0; c < D; ++c) s += (double)qrow[c] * (double)krow[c];
                    s *= (double)scale;
                    if (s > m) m = s;
                }
                for (int64_t c = 0; c < D; ++c) acc[c] = 0.0;
                for (int64_t j = 0; j < live; ++j) {
                    if (!gdo_attn_allowed(qpos, (int)j, 1, window, prefix_len)) continue;
                    const float *krow = k + ((b * Tmax + j) * Hkv + hkv) * D;
                    const float *vrow = v + ((b * Tmax + j) * Hkv + hkv) * D;
                    double s = 0.0;
                    for (int64_t c = 0; c < D; ++c) s += (double)qrow[c] * (double)krow[c];
                    const double e = exp((double)scale * s - m);
                    sum += e;
                    for (int64_t c = 0; c < D; ++c) acc[c] += e * (double)vrow[c];
                }
                for (int64_t c = 0; c < D; ++c) orow[c] = sum > 0.0 ? (float)(acc[c] / sum) : 0.0f;
            }
        }
    }
}

/* ---- A11: packed variable-length attention -------------------------------- */

/* reference tests/test_sdpa_varlen.c:158-230 (ref_varlen_fwd).  q [N,Hq,D],
 * k/v [N,Hkv,D]; segment b covers rows [cu[b],cu[b+1]); positions are relative
 * to the segment start.  max_seqlen > 0 truncates a longer segment's queries to
 * the first max_seqlen rows, the launch-grid effect noted for
 * src/ops/sdpa_varlen/metal_sdpa_varlen.m:359; rows past it stay zero. */
GDO_API void gdo_sdpa_varlen_f16(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                                 const int32_t *cu, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                 float scale, int causal, int window, int prefix_len,
                                 int64_t max_seqlen, float *out_f32)
{
    const int64_t group = Hq / Hkv;
    memset(out_f32, 0, (size_t)cu[B] * (size_t)Hq * (size_t)D * sizeof(float));
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t hq = 0; hq < Hq; ++hq) {
            const int64_t start = cu[b], T = (int64_t)cu[b + 1] - cu[b];
            const int64_t hkv = hq / group;
            if (T <= 0) continue;
            double *scores = (double *)malloc((size_t)T * sizeof(double));
            double acc[256];
            const int64_t tq = (max_seqlen > 0 && T > max_seqlen) ? max_seqlen : T;
            for (int64_t i = 0; i < tq; ++i) {
                const uint16_t *qrow = q + ((start + i) * Hq + hq) * D;
                float *orow = out_f32 + ((start + i) * Hq + hq) * D;
                double m = -HUGE_VAL, sum = 0.0;
                for (int64_t j = 0; j < T; ++j) {
                    if (!gdo_attn_allowed((int)i, (int)j, causal, window, prefix_len)) continue;
                    const uint16_t *krow = k + ((start + j) * Hkv + hkv) * D;
                    double s = 0.0;
                    for (int64_t c = 0; c < D; ++c) s += h2d(qrow[c]) * h2d(krow[c]);
                    s *= (double)scale;
                    scores[j] = s;
                    if (s > m) m = s;
                }
                for (int64_t c = 0; c < D; ++c) acc[c] = 0.0;
                for (int64_t j = 0; j < T; ++j) {
                    if (!gdo_attn_allowed((int)i, (int)j, causal, window, prefix_len)) continue;
                    const uint16_t *vrow = v + ((start + j) * Hkv + hkv) * D;
                    const double e = exp(scores[j] - m);
                    sum += e;
                    for (int64_t c = 0; c < D; ++c) acc[c] += e * h2d(vrow[c]);
                }
                if (sum > 0.0) {
                    for (int64_t c = 0; c < D; ++c) orow[c] = (float)(acc[c] / sum);
                }
            }
            free(scores);
        }
    }
}

/* ---- A3: rms_norm ---------------------------------------------------------- */

/* reference tests/test_rms_norm.c:56-105 (rms_reference) and
 * src/ops/rms_norm/metal_rms_norm.metal:29-67: ss = sum x^2, inv = 1/sqrt(ss/cols
 * + eps), y = half(x * w * inv).  The sum is taken in double, inv and the product
 * in float as the kernel does. */
GDO_API void gdo_rms_norm_f16(const uint16_t *x, const uint16_t *w, int64_t rows, int64_t cols,
                              float eps, uint16_t *out)
{
#pragma omp parallel for
    for (int64_t r = 0; r < rows; ++r) {
        double ss = 0.0;
        for (int64_t c = 0; c < cols; ++c) {
            const double xv = h2d(x[r * cols + c]);
            ss += xv * xv;
        }
        const float inv = (float)(1.0 / sqrt(ss / (double)cols + (double)eps));
        for (int64_t c = 0; c < cols; ++c) {
            out[r * cols + c] =
                gdo_f32_to_f16(gdo_f16_to_f32(x[r * cols + c]) * gdo_f16_to_f32(w[c]) * inv);
        }
    }
}

GDO_API void gdo_rms_norm_f32(const float *x, const float *w, int64_t rows, int64_t cols, float eps,
                              float *out)
{
    for (int64_t r = 0; r < rows; ++r) {
        double ss = 0.0;
        for (int64_t c = 0; c < cols; ++c) ss += (double)x[r * cols + c] * (double)x[r * cols + c];
        const float inv = (float)(1.0 / sqrt(ss / (double)cols + (double)eps));
        for (int64_t c = 0; c < cols; ++c) out[r * cols + c] = x[r * cols + c] * w[c] * inv;
    }
}

/* ---- A4: qkv split + rotary embedding ------------------------------------- */

/* reference src/ops/qkv_split_rope/metal_qkv_split_rope.metal:6-36,57-104 and
 * metal_qkv_split_rope.m:228 (freq_scale = -2*log2f(theta)/n_dims, float):
 * angle = float(pos) * exp2f(pair * freq_scale) in float; cos/sin of that float
 * angle (taken in double here); pairs (p, p+D/2) or (2p, 2p+1) when interleaved;
 * q,k rotated in float then rounded; v copied bit for bit.  Matches rope_ref of
 * reference tests/test_rope.c:67-104 up to the float rounding of the frequency. */
GDO_API void gdo_qkv_split_rope_f16(const uint16_t *qkv, const int32_t *pos, int64_t N, int64_t H,
                                    int64_t D, float theta, int interleaved, uint16_t *q,
                                    uint16_t *k, uint16_t *v)
{
    const int64_t area = H * D, half_d = D / 2;
    const float freq_scale = -2.0f * log2f(theta) / (float)D;
#pragma omp parallel for
    for (int64_t n = 0; n < N; ++n) {
        const uint16_t *src = qkv + n * 3 * area;
        for (int64_t p = 0; p < half_d; ++p) {
            const float angle = (float)pos[n] * exp2f((float)p * freq_scale);
            const float c = (float)cos((double)angle), s = (float)sin((double)angle);
            const int64_t a = interleaved ? 2 * p : p;
            const int64_t bb = interleaved ? 2 * p + 1 : p + half_d;
            for (int64_t h = 0; h < H; ++h) {
                const int64_t base = h * D;
                const float q0 = gdo_f16_to_f32(src[base + a]), q1 = gdo_f16_to_f32(src[base + bb]);
                const float k0 = gdo_f16_to_f32(src[area + base + a]);
                const float k1 = gdo_f16_to_f32(src[area + base + bb]);
                q[n * area + base + a] = gdo_f32_to_f16(q0 * c - q1 * s);
                q[n * area + base + bb] = gdo_f32_to_f16(q0 * s + q1 * c);
                k[n * area + base + a] = gdo_f32_to_f16(k0 * c - k1 * s);
                k[n * area + base + bb] = gdo_f32_to_f16(k0 * s + k1 * c);
                v[n * area + base + a] = src[2 * area + base + a];
                v[n * area + base + bb] = src[2 * area + base + bb];
            }
        }
    }
}

/* ---- A5/A6: projections ---------------------------------------------------- */

/* reference tests/test_linear.c:126-146 (ref_linear_transposed_weight_forward)
 * with the rounding points of the reference's two kernels
 * (src/ops/linear_transposed_weight/core_linear_transposed_weight.c:51,76):
 * t = half(sum_k x[m,k] w[n,k]); y = half(t + bias[n]) when a bias is given. */
GDO_API void gdo_linear_nt_f16(const uint16_t *x, const uint16_t *w, const uint16_t *bias, int64_t M,
                               int64_t K, int64_t N, uint16_t *y)
{
#pragma omp parallel for
    for (int64_t n = 0; n < N; ++n) {
        for (int64_t m = 0; m < M; ++m) {
            double acc = 0.0;
            for (int64_t kk = 0; kk < K; ++kk) acc += h2d(x[m * K + kk]) * h2d(w[n * K + kk]);
            uint16_t t = gdo_f32_to_f16((float)acc);
            if (bias) t = gdo_f32_to_f16(gdo_f16_to_f32(t) + gdo_f16_to_f32(bias[n]));
            y[m * N + n] = t;
        }
    }
}

/* reference tests/test_linear.c:69-89 (ref_linear_forward) with the single
 * rounding of src/ops/_shared/gemm/metal_gemm_common.h:125-132:
 * y = half(sum_k x[m,k] w[k,n] + bias[n]). */
GDO_API void gdo_linear_f16(const uint16_t *x, const uint16_t *w, const uint16_t *bias, int64_t M,
                            int64_t K, int64_t N, uint16_t *y)
{
#pragma omp parallel for
    for (int64_t m = 0; m < M; ++m) {
        double *acc = (double *)calloc((size_t)N, sizeof(double));
        for (int64_t kk = 0; kk < K; ++kk) {
            const double xv = h2d(x[m * K + kk]);
            const uint16_t *wr = w + kk * N;
            for (int64_t n = 0; n < N; ++n) acc[n] += xv * h2d(wr[n]);
        }
        for (int64_t n = 0; n < N; ++n) {
            y[m * N + n] = gdo_f32_to_f16((float)(acc[n] + (bias ? h2d(bias[n]) : 0.0)));
        }
        free(acc);
    }
}

/* ---- A8: add --------------------------------------------------------------- */

/* reference src/ops/add/metal_add.metal:37-59: half + half, i.e. the exactly
 * computed sum rounded once to F16.  y_count divides x_count: y is broadcast over
 * the trailing dimension (bias rows) or equals x in shape (residual). */
GDO_API void gdo_add_f16(const uint16_t *x, const uint16_t *y, int64_t x_count, int64_t y_count,
                         uint16_t *out)
{
    for (int64_t i = 0; i < x_count; ++i) {
        out[i] = gdo_f32_to_f16(gdo_f16_to_f32(x[i]) + gdo_f16_to_f32(y[i % y_count]));
    }
}

/* ---- A7: swiglu ------------------------------------------------------------ */

/* reference tests/test_swiglu.c:52-67 (sigmoid_stable, swiglu_gate) and
 * src/ops/swiglu/metal_swiglu.metal:94-118: out[r,c] = half(x12[r,c] * z *
 * sigmoid(z)), z = x12[r,H+c] (the gate is the second half). */
GDO_API void gdo_swiglu_split_f16(const uint16_t *x12, int64_t rows, int64_t H, uint16_t *out)
{
#pragma omp parallel for
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t c = 0; c < H; ++c) {
            const float a = gdo_f16_to_f32(x12[r * 2 * H + c]);
            const float z = gdo_f16_to_f32(x12[r * 2 * H + H + c]);
            const double sg = z >= 0.0f ? 1.0 / (1.0 + exp(-(double)z))
                                        : exp((double)z) / (1.0 + exp((double)z));
            out[r * H + c] = gdo_f32_to_f16(a * (z * (float)sg));
        }
    }
}

/* ---- A9: embedding --------------------------------------------------------- */

/* reference src/ops/embedding/metal_embedding.metal:11-33: row copy, id outside
 * [0,vocab) -> F16 NaN (0x7e00) in every column. */
GDO_API void gdo_embedding_f16(const uint16_t *table, const int32_t *ids, int64_t n_ids,
                               int64_t vocab, int64_t dim, uint16_t *out)
{
    for (int64_t i = 0; i < n_ids; ++i) {
        if (ids[i] < 0 || ids[i] >= vocab) {
            for (int64_t c = 0; c < dim; ++c) out[i * dim + c] = 0x7e00u;
        } else {
            memcpy(out + i * dim, table + (int64_t)ids[i] * dim, (size_t)dim * 2u);
        }
    }
}

/* ---- A10: greedy next token ------------------------------------------------ */

/* reference examples/gpt_lm/gpt_lm_shared.c:1388-1400: scan left to right, skip
 * non-finite values, keep the first strictly largest; 0 when nothing is finite.
 * gap = best - runner-up among finite values (+inf with fewer than two). */
GDO_API void gdo_argmax_rows_f16(const uint16_t *logits, int64_t rows, int64_t cols, int32_t *ids,
                                 float *gap)
{
    for (int64_t r = 0; r < rows; ++r) {
        int best = 0, have = 0;
        double bv = -HUGE_VAL, second = -HUGE_VAL;
        for (int64_t i = 0; i < cols; ++i) {
            const double val = h2d(logits[r * cols + i]);
            if (!isfinite(val)) continue;
            if (!have || val > bv) {
                if (have) second = bv;
                bv = val;
                best = (int)i;
                have = 1;
            } else if (val > second) {
                second = val;
            }
        }
        ids[r] = best;
        if (gap) gap[r] = (have && second > -HUGE_VAL) ? (float)(bv - second) : INFINITY;
    }
}

/* ---- MiniMax-M3 block-sparse attention over packed sequences --------------- */

/* Block picker.  reference src/ops/minimax_m3_index_topk/metal_minimax_m3_index_topk.metal:20-137
 * (the in-test model tests/test_minimax_m3_sparse_attention.c:145-213 states the same): row i of a
 * sequence sees the blocks 0 .. i / block; a block's score is the largest q_i . k_j over its keys
 * j <= i (NaN counts as -inf); the first init_blocks blocks score 1e30, the last local_blocks
 * visible ones 1e29 (which also overrides 1e30); the topk best are kept in descending order, an equal
 * score never displaces an earlier block; slots beyond the number of visible blocks, and slots no
 * block with a score above -inf reached, hold -1.  q, k [N,H,Dh]; out [H,N,topk]. */
GDO_API void gdo_minimax_m3_index_topk_f16(const uint16_t *q, const uint16_t *k, const int32_t *cu, int64_t B,
                                           int64_t H, int64_t Dh, int64_t block, int64_t topk,
                                           int64_t init_blocks, int64_t local_blocks, int32_t *out)
{
    const int64_t N = cu[B];
    for (int64_t i = 0; i < H * N * topk; ++i) out[i] = -1;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t h = 0; h < H; ++h) {
            const int64_t start = cu[b], T = cu[b + 1] - cu[b];
            double *score = (double *)malloc((size_t)topk * sizeof(double));
            int32_t *idx = (int32_t *)malloc((size_t)topk * sizeof(int32_t));
            for (int64_t i = 0; i < T; ++i) {
                const int64_t valid = (i + block) / block;
                const int64_t local_start = valid > local_blocks ? valid - local_blocks : 0;
                for (int64_t t = 0; t < topk; ++t) {
                    score[t] = -HUGE_VAL;
                    idx[t] = -1;
                }
                for (int64_t blk = 0; blk < valid; ++blk) {
                    const int64_t k0 = blk * block, k1 = k0 + block < T ? k0 + block : T;
                    double best = -HUGE_VAL;
                    for (int64_t j = k0; j < k1 && j <= i; ++j) {
                        double dot = 0.0;
                        for (int64_t c = 0; c < Dh; ++c)
                            dot += h2d(q[((start + i) * H + h) * Dh + c]) * h2d(k[((start + j) * H + h) * Dh + c]);
                        if (dot > best) best = dot;
                    }
                    if (blk < init_blocks) best = 1.0e30;
                    if (local_blocks > 0 && blk >= local_start) best = 1.0e29;
                    for (int64_t slot = 0; slot < topk; ++slot) {
                        if (best > score[slot]) {
                            for (int64_t move = topk - 1; move > slot; --move) {
                                score[move] = score[move - 1];
                                idx[move] = idx[move - 1];
                            }
                            score[slot] = best;
                            idx[slot] = (int32_t)blk;
                            break;
                        }
                    }
                }
                for (int64_t t = 0; t < topk; ++t) out[(h * N + start + i) * topk + t] = t < valid ? idx[t] : -1;
            }
            free(score);
            free(idx);
        }
    }
}

/* Attention of every row over the keys j <= i of its listed blocks.  reference
 * src/ops/minimax_m3_sparse_attention/metal_minimax_m3_sparse_attention.metal:36-113 (in-test models
 * tests/test_minimax_m3_sparse_attention.c:231-288, 423-483): blocks are visited in list order, -1
 * entries skipped, a block listed twice counts twice; q [N,Hq,Dh], k / v [N,Hkv,Dh], topk
 * [Hkv,N,topk]; a row without visible keys gives zeros.  F64 softmax, one F16 rounding. */
GDO_API void gdo_minimax_m3_sparse_attention_f16(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                                                 const int32_t *cu, const int32_t *topk, int64_t B, int64_t Hq,
                                                 int64_t Hkv, int64_t Dh, int64_t block, int64_t tk, float scale,
                                                 uint16_t *out)
{
    const int64_t N = cu[B], group = Hq / Hkv;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t hq = 0; hq < Hq; ++hq) {
            const int64_t start = cu[b], T = cu[b + 1] - cu[b], hkv = hq / group;
            double *acc = (double *)malloc((size_t)Dh * sizeof(double));
            double *sc = (double *)malloc((size_t)(tk * block) * sizeof(double));
            for (int64_t i = 0; i < T; ++i) {
                const int32_t *list = topk + (hkv * N + start + i) * tk;
                const uint16_t *qr = q + ((start + i) * Hq + hq) * Dh;
                double m = -HUGE_VAL, l = 0.0;
                int64_t n = 0;
                for (int64_t t = 0; t < tk; ++t) {
                    if (list[t] < 0) continue;
                    const int64_t k0 = (int64_t)list[t] * block, k1 = k0 + block < T ? k0 + block : T;
                    for (int64_t j = k0; j < k1 && j <= i; ++j) {
                        double dot = 0.0;
                        for (int64_t c = 0; c < Dh; ++c) dot += h2d(qr[c]) * h2d(k[((start + j) * Hkv + hkv) * Dh + c]);
                        sc[n] = (double)scale * dot;
                        if (sc[n] > m) m = sc[n];
                        ++n;
                    }
                }
                for (int64_t c = 0; c < Dh; ++c) acc[c] = 0.0;
                n = 0;
                for (int64_t t = 0; t < tk; ++t) {
                    if (list[t] < 0) continue;
                    const int64_t k0 = (int64_t)list[t] * block, k1 = k0 + block < T ? k0 + block : T;
                    for (int64_t j = k0; j < k1 && j <= i; ++j) {
                        const double e = exp(sc[n++] - m);
                        l += e;
                        for (int64_t c = 0; c < Dh; ++c) acc[c] += e * h2d(v[((start + j) * Hkv + hkv) * Dh + c]);
                    }
                }
                for (int64_t c = 0; c < Dh; ++c)
                    out[((start + i) * Hq + hq) * Dh + c] = gdo_f32_to_f16((float)(l > 0.0 ? acc[c] / l : 0.0));
            }
            free(acc);
            free(sc);
        }
    }
}

/* ---- sampling front end (the step after the logits) ------------------------ */

/* reference examples/gpt_lm/gpt_lm_shared.c:1322-1331 */
GDO_API void gdo_logits_softcap(float *logits, int64_t n, float cap)
{
    if (!(cap > 0.0f)) return;
    for (int64_t i = 0; i < n; ++i) logits[i] = cap * tanhf(logits[i] / cap);
}

/* reference :1347-1369: every distinct token of the history is penalised once */
GDO_API void gdo_repetition_penalty(float *logits, int64_t vocab, const int32_t *history, int64_t len,
                                    float penalty)
{
    if (len <= 0 || !isfinite(penalty) || penalty <= 1.0f) return;
    for (int64_t i = 0; i < len; ++i) {
        const int64_t token = history[i];
        int seen = 0;
        if (token < 0 || token >= vocab) continue;
        for (int64_t j = 0; j < i && !seen; ++j) seen = history[j] == token;
        if (seen) continue;
        if (logits[token] > 0.0f) logits[token] /= penalty;
        else logits[token] *= penalty;
    }
}

/* reference :1371-1442.  logits are modified in place by the penalty, *rng advances by one
 * splitmix64 application only when a draw is made.  margin (may be NULL) receives how far the
 * drawn point lies from the nearest boundary between two tokens' intervals, as a fraction of
 * the total mass (+inf when no draw was made): an implementation that sums in another order
 * may pick the neighbouring token only when this is tiny. */
GDO_API int32_t gdo_sample_next_token(float *logits, int64_t vocab, const int32_t *history, int64_t len,
                                      float temperature, float min_p, float penalty, uint64_t *rng,
                                      double *margin)
{
    int best = 0, have = 0;
    double best_value = -HUGE_VAL;
    if (margin) *margin = HUGE_VAL;
    gdo_repetition_penalty(logits, vocab, history, len, penalty);
    for (int64_t i = 0; i < vocab; ++i) {
        const double value = (double)logits[i];
        if (!isfinite(value)) continue;
        if (!have || value > best_value) {
            best_value = value;
            best = (int)i;
            have = 1;
        }
    }
    if (!have || !isfinite(temperature) || temperature <= 0.0f) return best;
    const double temp = (double)temperature;
    const double threshold = min_p > 0.0f ? best_value + temp * log((double)min_p) : -HUGE_VAL;
    double sum = 0.0;
    for (int64_t i = 0; i < vocab; ++i) {
        const double value = (double)logits[i];
        if (!isfinite(value) || value < threshold) continue;
        const double p = exp((value - best_value) / temp);
        if (isfinite(p)) sum += p;
    }
    if (!(sum > 0.0) || !isfinite(sum)) return best;
    *rng = gdo_splitmix64(*rng);
    double target = ((double)(*rng >> 11) * (1.0 / 9007199254740992.0)) * sum;
    for (int64_t i = 0; i < vocab; ++i) {
        const double value = (double)logits[i];
        if (!isfinite(value) || value < threshold) continue;
        const double p = exp((value - best_value) / temp);
        if (!isfinite(p)) continue;
        target -= p;
        if (target <= 0.0) {
            if (margin) *margin = fmin(-target, target + p) / sum;
            return (int32_t)i;
        }
    }
    if (margin) *margin = 0.0;
    return best;
}

/* ---- A13: decoder (call sequence of the reference example) ----------------- */

typedef struct gdo_decoder {
    int64_t vocab, d_model, n_layers, n_heads, head_dim, mlp_hidden, max_seq, batch;
    float rms_eps, rope_theta;
    int window;
    uint16_t *embed;      /* [V,Dm] */
    uint16_t *lm_head;    /* [V,Dm]; == embed while the head is tied (reference :393-402) */
    uint16_t *lm_bias;    /* [V] */
    uint16_t *final_norm; /* [Dm] */
    uint16_t **attn_norm, **mlp_norm;    /* [Dm] */
    uint16_t **w_qkv, **b_qkv;           /* [3Dm,Dm], [3Dm] */
    uint16_t **w_attn, **b_attn;         /* [Dm,Dm], [Dm] */
    uint16_t **w_upgate, **b_upgate;     /* [2Hm,Dm], [2Hm] */
    uint16_t **w_down, **b_down;         /* [Hm,Dm], [Dm] */
    uint16_t **k_cache, **v_cache;       /* [B,Tmax,H,D] per layer */
    int32_t *pos;                        /* [B] live length of each sequence */
    /* MiniMax-M3 architecture (reference gpt_lm_shared.c:588-600, 918-933): block_size > 0 switches the packed
     * prefill to picked blocks when the context is long enough; the decode step stays dense */
    int64_t m3_block, m3_topk, m3_init, m3_local;
} gdo_decoder;

static uint16_t *alloc_h(size_t n) { return (uint16_t *)calloc(n ? n : 1, sizeof(uint16_t)); }

static uint16_t *normal_h(size_t n, uint64_t seed, float stddev)
{
    uint16_t *p = alloc_h(n);
    gdo_fill_normal_f16(p, n, seed, stddev);
    return p;
}

static uint16_t *ones_h(size_t n)
{
    uint16_t *p = alloc_h(n);
    for (size_t i = 0; i < n; ++i) p[i] = 0x3c00u;
    return p;
}

/* Weights as the reference example initialises them
 * (examples/gpt_lm/gpt_lm_shared.c:290-345, 353-402): per-block seed =
 * seed ^ (index << 8); qkv/up_gate N(0,0.02), attn/down N(0, 0.02/sqrt(2L)),
 * biases zero, norm weights one, embedding N(0,0.02) with the LM head tied. */
GDO_API gdo_decoder *gdo_decoder_create(int64_t vocab, int64_t d_model, int64_t n_layers,
                                        int64_t n_heads, int64_t head_dim, int64_t mlp_hidden,
                                        int64_t max_seq, int64_t batch, int window, uint64_t seed)
{
    gdo_decoder *d = (gdo_decoder *)calloc(1, sizeof(*d));
    const size_t L = (size_t)n_layers;
    const float std = 0.02f, resid = 0.02f / sqrtf(2.0f * (float)n_layers);
    d->vocab = vocab; d->d_model = d_model; d->n_layers = n_layers; d->n_heads = n_heads;
    d->head_dim = head_dim; d->mlp_hidden = mlp_hidden; d->max_seq = max_seq; d->batch = batch;
    d->rms_eps = 1.0e-5f; d->rope_theta = 10000.0f; d->window = window;
    d->embed = normal_h((size_t)(vocab * d_model), gdo_splitmix64(seed ^ UINT64_C(0xabc001)), std);
    d->lm_head = d->embed;
    d->lm_bias = alloc_h((size_t)vocab);
    d->final_norm = ones_h((size_t)d_model);
#define ARR(name) d->name = (uint16_t **)calloc(L, sizeof(uint16_t *))
    ARR(attn_norm); ARR(mlp_norm); ARR(w_qkv); ARR(b_qkv); ARR(w_attn); ARR(b_attn);
    ARR(w_upgate); ARR(b_upgate); ARR(w_down); ARR(b_down); ARR(k_cache); ARR(v_cache);
#undef ARR
    for (size_t l = 0; l < L; ++l) {
        const uint64_t bs = seed ^ ((uint64_t)l << 8);
        d->attn_norm[l] = ones_h((size_t)d_model);
        d->mlp_norm[l] = ones_h((size_t)d_model);
        d->w_qkv[l] = normal_h((size_t)(3 * d_model * d_model), gdo_splitmix64(bs ^ 1u), std);
        d->b_qkv[l] = alloc_h((size_t)(3 * d_model));
        d->w_attn[l] = normal_h((size_t)(d_model * d_model), gdo_splitmix64(bs ^ 2u), resid);
        d->b_attn[l] = alloc_h((size_t)d_model);
        d->w_upgate[l] = normal_h((size_t)(2 * mlp_hidden * d_model), gdo_splitmix64(bs ^ 3u), std);
        d->b_upgate[l] = alloc_h((size_t)(2 * mlp_hidden));
        d->w_down[l] = normal_h((size_t)(mlp_hidden * d_model), gdo_splitmix64(bs ^ 4u), resid);
        d->b_down[l] = alloc_h((size_t)d_model);
        d->k_cache[l] = alloc_h((size_t)(batch * max_seq * n_heads * head_dim));
        d->v_cache[l] = alloc_h((size_t)(batch * max_seq * n_heads * head_dim));
    }
    d->pos = (int32_t *)calloc((size_t)batch, sizeof(int32_t));
    return d;
}

GDO_API void gdo_decoder_destroy(gdo_decoder *d)
{
    if (!d) return;
    for (int64_t l = 0; l < d->n_layers; ++l) {
        free(d->attn_norm[l]); free(d->mlp_norm[l]); free(d->w_qkv[l]); free(d->b_qkv[l]);
        free(d->w_attn[l]); free(d->b_attn[l]); free(d->w_upgate[l]); free(d->b_upgate[l]);
        free(d->w_down[l]); free(d->b_down[l]); free(d->k_cache[l]); free(d->v_cache[l]);
    }
    free(d->attn_norm); free(d->mlp_norm); free(d->w_qkv); free(d->b_qkv); free(d->w_attn);
    free(d->b_attn); free(d->w_upgate); free(d->b_upgate); free(d->w_down); free(d->b_down);
    if (d->lm_head != d->embed) free(d->lm_head);
    free(d->k_cache); free(d->v_cache); free(d->embed); free(d->lm_bias); free(d->final_norm);
    free(d->pos); free(d);
}

/* Tensor access for tests: name in {embed, lm_bias, final_norm, attn_norm, mlp_norm,
 * w_qkv, b_qkv, w_attn, b_attn, w_upgate, b_upgate, w_down, b_down, k_cache, v_cache}. */
GDO_API uint16_t *gdo_decoder_tensor(gdo_decoder *d, const char *name, int64_t layer)
{
#define ONE(n) if (!strcmp(name, #n)) return d->n
#define PER(n) if (!strcmp(name, #n)) return d->n[layer]
    ONE(embed); ONE(lm_head); ONE(lm_bias); ONE(final_norm);
    PER(attn_norm); PER(mlp_norm); PER(w_qkv); PER(b_qkv); PER(w_attn); PER(b_attn);
    PER(w_upgate); PER(b_upgate); PER(w_down); PER(b_down); PER(k_cache); PER(v_cache);
#undef ONE
#undef PER
    return NULL;
}

GDO_API int32_t *gdo_decoder_positions(gdo_decoder *d) { return d->pos; }

/* Gives the LM head its own [V,Dm] weight, N(0,0.02) from splitmix64(seed ^ 0xabc002). */
GDO_API void gdo_decoder_untie_lm_head(gdo_decoder *d, uint64_t seed)
{
    if (d->lm_head == d->embed) d->lm_head = alloc_h((size_t)(d->vocab * d->d_model));
    gdo_fill_normal_f16(d->lm_head, (size_t)(d->vocab * d->d_model), gdo_splitmix64(seed ^ UINT64_C(0xabc002)), 0.02f);
}

/* One transformer block over `rows` token rows; `attend` runs the attention for
 * this block.  Order of operators: reference examples/gpt_lm/gpt_lm_shared.c:
 * 1017-1070 (decode) and 895-958 (prefill). */
typedef void (*gdo_attend_fn)(gdo_decoder *d, int64_t layer, int64_t rows, const uint16_t *q,
                              const uint16_t *k, const uint16_t *v, const void *ctx, uint16_t *attn);

static void block_forward(gdo_decoder *d, int64_t l, int64_t rows, const int32_t *positions,
                          uint16_t *x, gdo_attend_fn attend, const void *actx)
{
    const int64_t Dm = d->d_model, Hm = d->mlp_hidden, H = d->n_heads, D = d->head_dim;
    uint16_t *normed = alloc_h((size_t)(rows * Dm)), *qkv = alloc_h((size_t)(rows * 3 * Dm));
    uint16_t *q = alloc_h((size_t)(rows * Dm)), *k = alloc_h((size_t)(rows * Dm));
    uint16_t *v = alloc_h((size_t)(rows * Dm)), *attn = alloc_h((size_t)(rows * Dm));
    uint16_t *proj = alloc_h((size_t)(rows * Dm)), *ug = alloc_h((size_t)(rows * 2 * Hm));
    uint16_t *act = alloc_h((size_t)(rows * Hm));
    gdo_rms_norm_f16(x, d->attn_norm[l], rows, Dm, d->rms_eps, normed);
    gdo_linear_nt_f16(normed, d->w_qkv[l], d->b_qkv[l], rows, Dm, 3 * Dm, qkv);
    gdo_qkv_split_rope_f16(qkv, positions, rows, H, D, d->rope_theta, 0, q, k, v);
    attend(d, l, rows, q, k, v, actx, attn);
    gdo_linear_nt_f16(attn, d->w_attn[l], d->b_attn[l], rows, Dm, Dm, proj);
    gdo_add_f16(x, proj, rows * Dm, rows * Dm, x);
    gdo_rms_norm_f16(x, d->mlp_norm[l], rows, Dm, d->rms_eps, normed);
    gdo_linear_nt_f16(normed, d->w_upgate[l], d->b_upgate[l], rows, Dm, 2 * Hm, ug);
    gdo_swiglu_split_f16(ug, rows, Hm, act);
    gdo_linear_f16(act, d->w_down[l], d->b_down[l], rows, Hm, Dm, proj);
    gdo_add_f16(x, proj, rows * Dm, rows * Dm, x);
    free(normed); free(qkv); free(q); free(k); free(v); free(attn); free(proj); free(ug); free(act);
}

static void attend_decode(gdo_decoder *d, int64_t l, int64_t rows, const uint16_t *q,
                          const uint16_t *k, const uint16_t *v, const void *ctx, uint16_t *attn)
{
    (void)ctx;
    const int64_t H = d->n_heads, D = d->head_dim;
    float *o = (float *)calloc((size_t)(rows * H * D), sizeof(float));
    gdo_kv_cache_append((uint8_t *)d->k_cache[l], (uint8_t *)d->v_cache[l], (const uint8_t *)k,
                        (const uint8_t *)v, d->pos, 0, rows, 1, d->max_seq, H * D * 2);
    gdo_sdpa_decode_f16(q, d->k_cache[l], d->v_cache[l], d->pos, rows, 1, d->max_seq, H, H, D,
                        (float)(1.0 / sqrt((double)D)), d->window, 0, o);
    gdo_f32_to_f16_array(o, attn, (size_t)(rows * H * D));
    free(o);
}

typedef struct { const int32_t *cu; int64_t n_seq; const int32_t *cache_pos; } prefill_ctx;

static void attend_prefill(gdo_decoder *d, int64_t l, int64_t rows, const uint16_t *q,
                           const uint16_t *k, const uint16_t *v, const void *ctx, uint16_t *attn)
{
    const prefill_ctx *p = (const prefill_ctx *)ctx;
    const int64_t H = d->n_heads, D = d->head_dim;
    float *o = (float *)calloc((size_t)(rows * H * D), sizeof(float));
    gdo_kv_cache_append_packed((uint8_t *)d->k_cache[l], (uint8_t *)d->v_cache[l],
                               (const uint8_t *)k, (const uint8_t *)v, p->cache_pos, p->cu,
                               p->n_seq, rows, d->max_seq, H * D * 2);
    if (d->m3_block > 0 && d->m3_topk > 0 && d->max_seq > d->m3_block * 8 && d->m3_block * d->m3_topk * 2 < d->max_seq) {
        int32_t *idx = (int32_t *)malloc((size_t)(H * rows * d->m3_topk) * sizeof(int32_t));
        gdo_minimax_m3_index_topk_f16(q, k, p->cu, p->n_seq, H, D, d->m3_block, d->m3_topk, d->m3_init, d->m3_local, idx);
        gdo_minimax_m3_sparse_attention_f16(q, k, v, p->cu, idx, p->n_seq, H, H, D, d->m3_block, d->m3_topk,
                                            (float)(1.0 / sqrt((double)D)), attn);
        free(idx);
        free(o);
        return;
    }
    gdo_sdpa_varlen_f16(q, k, v, p->cu, p->n_seq, H, H, D, (float)(1.0 / sqrt((double)D)), 1,
                        d->window, 0, d->max_seq, o);
    gdo_f32_to_f16_array(o, attn, (size_t)(rows * H * D));
    free(o);
}

GDO_API void gdo_decoder_set_minimax_m3(gdo_decoder *d, int64_t block, int64_t topk, int64_t init_blocks,
                                        int64_t local_blocks)
{
    d->m3_block = block;
    d->m3_topk = topk;
    d->m3_init = init_blocks;
    d->m3_local = local_blocks;
}

static void head_forward(gdo_decoder *d, int64_t rows, const uint16_t *x, uint16_t *logits)
{
    uint16_t *normed = alloc_h((size_t)(rows * d->d_model));
    gdo_rms_norm_f16(x, d->final_norm, rows, d->d_model, d->rms_eps, normed);
    gdo_linear_nt_f16(normed, d->lm_head, d->lm_bias, rows, d->d_model, d->vocab, logits);
    free(normed);
}

/* One batched decode step: reference examples/gpt_lm/gpt_lm_shared.c:1204-1246.
 * ids [B]; rope position and cache position are both the live length of each
 * sequence; writes logits [B,V] (F16), the greedy ids and their top-2 gaps, then
 * advances every position by one. */
GDO_API void gdo_decoder_step(gdo_decoder *d, const int32_t *ids, uint16_t *logits,
                              int32_t *next_ids, float *gaps)
{
    const int64_t B = d->batch, Dm = d->d_model;
    uint16_t *x = alloc_h((size_t)(B * Dm));
    uint16_t *lg = logits ? logits : alloc_h((size_t)(B * d->vocab));
    gdo_embedding_f16(d->embed, ids, B, d->vocab, Dm, x);
    for (int64_t l = 0; l < d->n_layers; ++l) {
        block_forward(d, l, B, d->pos, x, attend_decode, NULL);
    }
    head_forward(d, B, x, lg);
    if (next_ids) gdo_argmax_rows_f16(lg, B, d->vocab, next_ids, gaps);
    for (int64_t b = 0; b < B; ++b) d->pos[b] += 1;
    if (!logits) free(lg);
    free(x);
}

/* Packed prefill: reference examples/gpt_lm/gpt_lm_shared.c:1073-1202.  ids [N]
 * packed by cu [B+1]; rope positions restart at 0 in every segment; caches are
 * written from position 0; logits are produced for the last row of each segment
 * only; positions become the segment lengths.  hidden_out (optional, [N,Dm])
 * receives the block-stack output of every row. */
GDO_API void gdo_decoder_prefill(gdo_decoder *d, const int32_t *ids, const int32_t *cu,
                                 uint16_t *logits, int32_t *next_ids, float *gaps,
                                 uint16_t *hidden_out)
{
    const int64_t B = d->batch, Dm = d->d_model, N = cu[B];
    uint16_t *x = alloc_h((size_t)(N * Dm)), *last = alloc_h((size_t)(B * Dm));
    uint16_t *lg = logits ? logits : alloc_h((size_t)(B * d->vocab));
    int32_t *positions = (int32_t *)calloc((size_t)N, sizeof(int32_t));
    int32_t *zero = (int32_t *)calloc((size_t)B, sizeof(int32_t));
    for (int64_t b = 0; b < B; ++b) {
        for (int32_t r = cu[b]; r < cu[b + 1]; ++r) positions[r] = r - cu[b];
    }
    prefill_ctx pc = {cu, B, zero};
    gdo_embedding_f16(d->embed, ids, N, d->vocab, Dm, x);
    for (int64_t l = 0; l < d->n_layers; ++l) {
        block_forward(d, l, N, positions, x, attend_prefill, &pc);
    }
    if (hidden_out) memcpy(hidden_out, x, (size_t)(N * Dm) * 2u);
    for (int64_t b = 0; b < B; ++b) {
        memcpy(last + b * Dm, x + ((int64_t)cu[b + 1] - 1) * Dm, (size_t)Dm * 2u);
        d->pos[b] = cu[b + 1] - cu[b];
    }
    head_forward(d, B, last, lg);
    if (next_ids) gdo_argmax_rows_f16(lg, B, d->vocab, next_ids, gaps);
    if (!logits) free(lg);
    free(x); free(last); free(positions); free(zero);
}
