/*
 * Instantiations and launcher of gd_linear_wide_kernel (linear_wide_kernel.h): the few-row projections of the wide
 * decoders.  A translation unit of its own, like linear_lds.hip, so that the code object of linear.hip stays as it
 * is laid out without it.
 */
#include "linear_wide_kernel.h"

template <int NT, int MT, int PMAX, int PRO, int EPI>
static void launch_wide(hipStream_t stream, const void *x, const void *w, const void *bias, const void *residual,
                        const void *norm_w, void *y, const gd_hip_linear_params &p, const gd_hip_rope_epilogue &rope)
{
    constexpr bool PAIRED = EPI != GD_WIDE_EPI_PLAIN;
    const uint32_t cols = PAIRED ? 8u * NT : 16u * NT; /* output (first-of-pair) columns per workgroup */
    const uint32_t outs = EPI == GD_WIDE_EPI_ROPE ? p.N / 2u : (EPI == GD_WIDE_EPI_SWIGLU ? p.swiglu_cols : p.N);
    const uint32_t n_tiles = outs / cols;
    dim3 grid(n_tiles, (p.M + 16u * MT - 1u) / (16u * MT));
    gd_linear_wide_kernel<NT, MT, PMAX, 8, PRO, EPI><<<grid, 512, 0, stream>>>(
        (const gd_half *)x, (const gd_half *)w, (const gd_half *)bias, (const gd_half *)residual,
        (const gd_half *)norm_w, (gd_half *)y, p, n_tiles, rope);
}

/* 8 columns per workgroup (narrow outputs, one row tile): see gd_linear_wide_half_kernel */
template <int QMAX>
static void launch_wide_half(hipStream_t stream, const void *x, const void *w, const void *bias, const void *residual,
                             void *y, const gd_hip_linear_params &p)
{
    const uint32_t n_tiles = p.N / 8u;
    dim3 grid(n_tiles, (p.M + 15u) / 16u);
    gd_linear_wide_half_kernel<QMAX, 8><<<grid, 512, 0, stream>>>(
        (const gd_half *)x, (const gd_half *)w, (const gd_half *)bias, (const gd_half *)residual, (gd_half *)y, p, n_tiles);
}

/* persistent form: K = 2048 behind an rms_norm, at most 8 tiles per workgroup, one workgroup per compute unit */
template <int NT, int MT, int EPI>
static void launch_persistent(hipStream_t stream, const void *x, const void *w, const void *bias, const void *residual,
                              const void *norm_w, void *y, const gd_hip_linear_params &p, const gd_hip_rope_epilogue &rope,
                              uint32_t units, bool narrow)
{
    constexpr bool PAIRED = EPI != GD_WIDE_EPI_PLAIN;
    /* as deep as LDS allows next to the sums of the wavefronts (NT x MT x 8 KB): 8 x RING x 2 KB; an eighth group for
     * the two-tile forms changed nothing (12.5 against 12.2 us at 16 x 2048 -> 6144) */
    constexpr int RING = NT * MT <= 4 ? 7 : 5;
    const uint32_t cols = PAIRED ? 8u * NT : 16u * NT;
    const uint32_t outs = EPI == GD_WIDE_EPI_ROPE ? p.N / 2u : (EPI == GD_WIDE_EPI_SWIGLU ? p.swiglu_cols : p.N);
    uint32_t n_tiles = outs / cols, tile_w = cols;
    /* fewer full tiles than compute units (5632 gated outputs: 176 tiles of 32): narrower tiles, one per unit, so
     * that every unit streams its share of the weights (22 columns each; the 3072 rotation pairs of a 6144-row qkv
     * weight: 12 pairs each).  Narrow rope tiles straddle heads: only when half the head size is a power of two. */
    const uint32_t hd2 = p.rope_head_dim / 2u;
    const bool may_straddle = EPI != GD_WIDE_EPI_ROPE || (hd2 != 0u && (hd2 & (hd2 - 1u)) == 0u);
    if (may_straddle && n_tiles < units && narrow && 2u * ((outs + units - 1u) / units) > cols) {
        tile_w = (outs + units - 1u) / units; /* more than half of a tile's columns stay in use */
        n_tiles = (outs + tile_w - 1u) / tile_w;
    }
    uint32_t groups = n_tiles < units ? n_tiles : units;
    if ((n_tiles + groups - 1u) / groups > 8u) groups = (n_tiles + 7u) / 8u;
    dim3 grid(groups, (p.M + 16u * MT - 1u) / (16u * MT));
    gd_linear_wide_persistent_kernel<NT, MT, 4, RING, EPI, 8><<<grid, 512, 0, stream>>>(
        (const gd_half *)x, (const gd_half *)w, (const gd_half *)bias, (const gd_half *)residual,
        (const gd_half *)norm_w, (gd_half *)y, p, n_tiles, tile_w, rope);
}

/* Returns 1 when the launch was taken (hipGetLastError() then tells how it went), 0 when this kernel family does
 * not cover the call and the caller goes on to the stream kernel.  Covered: [N,K] weights of at least min_bytes
 * whose K is a multiple of 64 and splits over the eight wavefronts into at most 4 (behind an rms_norm) or 12 (no
 * prologue) pairs of steps each, fewer than 128 rows, and
 *   plain epilogue:   no prologue, 16 columns per workgroup (8 where that leaves compute units without one);
 *                     rms_norm prologue, 64 columns per workgroup;
 *   swiglu epilogue:  rms_norm prologue, 32 (tiles == 2) or 64 weight rows per workgroup;
 *   rope epilogue:    rms_norm prologue, 32 weight rows per workgroup (head size a multiple of 32). */
extern "C" int gd_hip_try_launch_linear_wide(hipStream_t stream, const void *x, const void *w, const void *bias,
                                             const void *residual, const void *norm_w, void *y,
                                             const gd_hip_linear_params *params, const gd_hip_rope_epilogue *rope_epilogue,
                                             uint64_t min_bytes, uint32_t tiles, uint32_t units)
{
    const gd_hip_rope_epilogue no_rope = {nullptr, nullptr, nullptr, nullptr, nullptr};
    const gd_hip_rope_epilogue &rope = rope_epilogue != nullptr ? *rope_epilogue : no_rope;
    const gd_hip_linear_params &p = *params;
    if (!p.w_is_nk || p.M == 0u || p.M >= 128u || p.K == 0u || (p.K % 64u) != 0u ||
        (uint64_t)p.N * p.K * 2u < min_bytes || (uint64_t)p.N * p.ldw * 4u >= 0x7fffffffull ||
        (uint64_t)p.M * p.ldx * 2u >= 0x7fffffffull)
        return 0;
    const uint32_t ppw = (p.K / 64u + 7u) / 8u; /* pairs of steps per wavefront */
    const int epi = p.rope_head_dim != 0u ? GD_WIDE_EPI_ROPE : (p.swiglu_cols != 0u ? GD_WIDE_EPI_SWIGLU : GD_WIDE_EPI_PLAIN);
    const uint32_t mt = p.M <= 16u ? 1u : (p.M <= 32u ? 2u : 4u);
    const bool persistent = tiles != 1u; /* "linear_tiles" = 1 asks for the one-tile-per-workgroup form (for comparison) */
#define GD_W(NT, MT, PMAX, PRO, EPI) \
    do { launch_wide<NT, MT, PMAX, PRO, EPI>(stream, x, w, bias, residual, norm_w, y, p, rope); return 1; } while (0)
#define GD_W_MT(NT, PMAX, PRO, EPI) \
    do { if (mt == 1u) GD_W(NT, 1, PMAX, PRO, EPI); if (mt == 2u) GD_W(NT, 2, PMAX, PRO, EPI); GD_W(NT, 4, PMAX, PRO, EPI); } while (0)
    if (p.prologue == GD_HIP_PRO_NONE && epi == GD_WIDE_EPI_PLAIN && (p.N % 16u) == 0u) {
        /* 16 columns per workgroup: these are the narrow outputs (N = d_model), where further row tiles are worth
         * more as workgroups of their own (16 x 2048 x 2048 and 32 x ...: 6.0 us with one row tile per workgroup,
         * 8.2 us with both in one; the second reader of a weight line finds it in L2) */
        /* up to 16 rows and fewer 16-column tiles than compute units: 8 columns per workgroup, so that every unit
         * streams (16 x 5632 -> 2048: 256 workgroups instead of 128) */
        if (p.M <= 16u && p.N / 16u < units && tiles != 1u && (p.K % 128u) == 0u && (p.N % 8u) == 0u) {
            const uint32_t qpw = (p.K / 128u + 7u) / 8u; /* pieces of 128 per wavefront */
            if (qpw <= 2u) { launch_wide_half<2>(stream, x, w, bias, residual, y, p); return 1; }
            if (qpw <= 6u) { launch_wide_half<6>(stream, x, w, bias, residual, y, p); return 1; }
        }
        if (ppw <= 4u) GD_W(1, 1, 4, GD_HIP_PRO_NONE, GD_WIDE_EPI_PLAIN);
        if (ppw <= 12u) GD_W(1, 1, 12, GD_HIP_PRO_NONE, GD_WIDE_EPI_PLAIN);
        return 0;
    }
    if (p.prologue != GD_HIP_PRO_RMS_NORM || ppw > 4u) return 0;
    /* K = 2048: the persistent form, where its LDS holds the sums of MT x NT tiles next to the ring */
#define GD_P(NT, MT, EPI) \
    do { launch_persistent<NT, MT, EPI>(stream, x, w, bias, residual, norm_w, y, p, rope, units, tiles != 4u); return 1; } while (0)
    if (p.K == 2048u && persistent) {
        if (epi == GD_WIDE_EPI_PLAIN && (p.N % 64u) == 0u && mt <= 2u) {
            if (mt == 1u) GD_P(4, 1, GD_WIDE_EPI_PLAIN);
            GD_P(4, 2, GD_WIDE_EPI_PLAIN);
        }
        /* four row tiles: the sums of 4 x 4 tiles would not fit next to the ring, so 32 columns per tile */
        if (epi == GD_WIDE_EPI_PLAIN && (p.N % 32u) == 0u) GD_P(2, 4, GD_WIDE_EPI_PLAIN);
        if (epi == GD_WIDE_EPI_SWIGLU && tiles != 2u && (p.swiglu_cols % 32u) == 0u && mt <= 2u) {
            if (mt == 1u) GD_P(4, 1, GD_WIDE_EPI_SWIGLU);
            GD_P(4, 2, GD_WIDE_EPI_SWIGLU);
        }
        if (epi == GD_WIDE_EPI_SWIGLU && (p.swiglu_cols % 16u) == 0u) {
            if (mt == 1u) GD_P(2, 1, GD_WIDE_EPI_SWIGLU);
            if (mt == 2u) GD_P(2, 2, GD_WIDE_EPI_SWIGLU);
            GD_P(2, 4, GD_WIDE_EPI_SWIGLU);
        }
        if (epi == GD_WIDE_EPI_ROPE && (p.rope_head_dim % 32u) == 0u && p.N == 3u * p.rope_heads * p.rope_head_dim) {
            if (mt == 1u) GD_P(2, 1, GD_WIDE_EPI_ROPE);
            if (mt == 2u) GD_P(2, 2, GD_WIDE_EPI_ROPE);
            /* 33 rows or more: the stream kernel's four workgroups per column tile are faster here (20.7 against
             * 22.3 us at 64 x 2048 -> 6144), the rotation of 64 rows weighs more than the second pass over L2 */
            return 0;
        }
    }
#undef GD_P
    if (epi == GD_WIDE_EPI_PLAIN && (p.N % 64u) == 0u) GD_W_MT(4, 4, GD_HIP_PRO_RMS_NORM, GD_WIDE_EPI_PLAIN);
    if (epi == GD_WIDE_EPI_SWIGLU && p.swiglu_cols == p.N) {
        if (tiles != 2u && (p.swiglu_cols % 32u) == 0u) GD_W_MT(4, 4, GD_HIP_PRO_RMS_NORM, GD_WIDE_EPI_SWIGLU);
        if ((p.swiglu_cols % 16u) == 0u) GD_W_MT(2, 4, GD_HIP_PRO_RMS_NORM, GD_WIDE_EPI_SWIGLU);
    }
    if (epi == GD_WIDE_EPI_ROPE && (p.rope_head_dim % 32u) == 0u && p.N == 3u * p.rope_heads * p.rope_head_dim && mt <= 2u)
        GD_W_MT(2, 4, GD_HIP_PRO_RMS_NORM, GD_WIDE_EPI_ROPE);
#undef GD_W_MT
#undef GD_W
    return 0;
}
