/*
 * F16 projections with F32 accumulation for gfx950 (MFMA 16x16x32 F16).
 *
 * Replaces the reference GEMM kernels src/ops/_shared/gemm/metal_gemm_common.h:54-135 (NN,
 * bias fused in F32) and :161-237 (NT) plus the separate bias add of
 * src/ops/linear_transposed_weight/core_linear_transposed_weight.c:51,76.
 *
 * Weight-streaming kernel (decode, up to 64 rows per pass): the weight matrix is read once from
 * HBM, the activation tile is small and stays in cache, so the kernel is HBM-bound on
 * N*K*2 bytes and, for the small matrices of a decode step, latency-bound.  A workgroup of
 * WAVES wavefronts owns 16 output columns; the wavefronts split K and are summed through LDS,
 * which gives N/16 workgroups x WAVES independent weight streams even for narrow outputs.  Every
 * wavefront issues the fragment loads of several K steps before the first MFMA, so a short K
 * range costs one memory round trip instead of one per step.  With w stored [N,K] both MFMA
 * operands are K-contiguous: every lane fetches its 8-half fragment with one 16-byte load
 * straight from global memory (16 rows x 64 B per wavefront load), no LDS staging.  With w stored
 * [K,N] the B fragment is gathered with 2-byte loads (16 lanes read 32 contiguous bytes of a
 * weight row).
 *
 * MFMA operand layout used here (v_mfma_f32_16x16x32_f16): lane l supplies row/col l%16 and the
 * 8 consecutive K values starting at 8*(l/16); the result lane holds column l%16, rows
 * 4*(l/16)..+3.
 *
 * Rounding points: F32 accumulate; GD_HIP_EPI_BIAS_F32 adds the bias before the single F16
 * rounding; GD_HIP_EPI_BIAS_F16 rounds, then adds the bias in F16 (the reference's two-kernel
 * NT path).  The optional prologues (swiglu gate, rms_norm) round the activation to F16 before the
 * MFMA exactly like the reference's separate kernels, and the optional residual is added last in
 * F16 like the reference's separate add.
 */
#include "linear_stream_kernel.h"

/* Any shape or alignment: one thread per output, F32 dot product.  Correctness path only. */
__global__ void __launch_bounds__(256)
gd_linear_scalar_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w,
                        const gd_half *__restrict__ bias, const gd_half *__restrict__ residual,
                        const gd_half *__restrict__ norm_w, gd_half *__restrict__ y, gd_hip_linear_params p)
{
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)p.M * p.N) return;
    const uint32_t m = (uint32_t)(gid / p.N), n = (uint32_t)(gid % p.N);
    const gd_half *xr = x + (size_t)m * p.ldx;
    float inv = 1.f;
    if (p.prologue == GD_HIP_PRO_RMS_NORM) {
        float ss = 0.f;
        for (uint32_t k = 0; k < p.K; ++k) ss = fmaf((float)xr[k], (float)xr[k], ss);
        inv = rsqrtf(ss / (float)p.K + p.eps);
    }
    float acc = 0.f;
    for (uint32_t k = 0; k < p.K; ++k) {
        gd_half a = xr[k];
        if (p.prologue == GD_HIP_PRO_SWIGLU) a = (gd_half)((float)a * gd_lin_silu((float)xr[p.K + k]));
        if (p.prologue == GD_HIP_PRO_RMS_NORM) a = (gd_half)((float)a * (float)norm_w[k] * inv);
        const gd_half b = p.w_is_nk ? w[(size_t)n * p.ldw + k] : w[(size_t)k * p.ldw + n];
        acc = fmaf((float)a, (float)b, acc);
    }
    gd_half h;
    if (p.epilogue == GD_HIP_EPI_BIAS_F32) h = (gd_half)(acc + (float)bias[n]);
    else if (p.epilogue == GD_HIP_EPI_BIAS_F16) h = (gd_half)acc + bias[n];
    else h = (gd_half)acc;
    if (p.has_residual) h = residual[(size_t)m * p.ldr + n] + h;
    y[(size_t)m * p.ldy + n] = h;
}

/* linear_lds.hip: gd_linear_stream_kernel<4, 8, [N,K], rms_norm, resident, LDS stream> */
extern "C" void gd_hip_launch_linear_lds(hipStream_t stream, const void *x, const void *w, const void *bias,
                                         const void *residual, const void *norm_w, void *y,
                                         const gd_hip_linear_params *p, uint32_t n_tiles,
                                         const gd_hip_rope_epilogue *rope, uint32_t grid_x, uint32_t grid_y);

template <int NT, int WAVES>
static void launch_stream(hipStream_t stream, const gd_half *x, const gd_half *w, const gd_half *bias,
                          const gd_half *residual, const gd_half *norm_w, gd_half *y, const gd_hip_linear_params &p,
                          const gd_hip_rope_epilogue &rope)
{
    const bool paired = p.swiglu_cols != 0u || p.rope_head_dim != 0u;
    const uint32_t cols = paired ? 8u * NT : 16u * NT; /* first-of-pair / plain output columns per workgroup */
    const uint32_t n_tiles = p.rope_head_dim != 0u ? (p.N / 2u) / cols : (p.N + cols - 1u) / cols;
    dim3 grid(n_tiles, (p.M + 15u) / 16u);
    const int threads = WAVES * 64;
    /* the whole K slice of a wavefront fits the resident registers (8 steps of 32) */
    const bool res = ((p.K + 31u) / 32u + WAVES - 1u) / WAVES <= 8u;
#define GD_GO(NK, PRO, RES) gd_linear_stream_kernel<NT, WAVES, NK, PRO, RES, false><<<grid, threads, 0, stream>>>(x, w, bias, residual, norm_w, y, p, n_tiles, rope)
    if (p.w_is_nk) {
        if (p.prologue == GD_HIP_PRO_SWIGLU) GD_GO(true, GD_HIP_PRO_SWIGLU, false);
        else if (p.prologue == GD_HIP_PRO_RMS_NORM) {
            /* 64 columns, 8 wavefronts, resident activation slice: the form whose weight stream goes through LDS
             * (linear_lds.hip); same sums to the bit */
            if (res && NT == 4 && WAVES == 8 && p.no_lds_stream == 0u)
                gd_hip_launch_linear_lds(stream, x, w, bias, residual, norm_w, y, &p, n_tiles, &rope, grid.x, grid.y);
            else if (res) GD_GO(true, GD_HIP_PRO_RMS_NORM, true);
            else GD_GO(true, GD_HIP_PRO_RMS_NORM, false);
        }
        else GD_GO(true, GD_HIP_PRO_NONE, false);
    } else {
        if (p.prologue == GD_HIP_PRO_SWIGLU) GD_GO(false, GD_HIP_PRO_SWIGLU, false);
        else if (p.prologue == GD_HIP_PRO_RMS_NORM) { if (res) GD_GO(false, GD_HIP_PRO_RMS_NORM, true); else GD_GO(false, GD_HIP_PRO_RMS_NORM, false); }
        else GD_GO(false, GD_HIP_PRO_NONE, false);
    }
#undef GD_GO
}

/* linear_wide.hip: the projections of the wide decoders (megabytes of [N,K] weights, fewer than 128 rows) */
extern "C" int gd_hip_try_launch_linear_wide(hipStream_t stream, const void *x, const void *w, const void *bias,
                                             const void *residual, const void *norm_w, void *y,
                                             const gd_hip_linear_params *params, const gd_hip_rope_epilogue *rope_epilogue,
                                             uint64_t min_bytes, uint32_t tiles, uint32_t units);

extern "C" int gd_hip_launch_linear_tile(hipStream_t stream, const void *x, const void *w, const void *bias,
                                         const void *residual, const void *norm_w, void *y,
                                         const gd_hip_linear_params *params, int big_tiles, int vector_store,
                                         int compute_units);

/* vector_ok: K % 8 == 0 and every pointer / pitch allows 16-byte fragment loads (for w only when it is [N,K]);
 * kn_vector_ok: w stored [K,N] with N % 8 == 0 and 16-byte aligned rows; store_vector_ok: y (and the residual)
 * rows allow 16-byte accesses.  min_workgroups: about two per compute unit.  wide_mode: see below. */
extern "C" int gd_hip_launch_linear(hipStream_t stream, const void *x, const void *w, const void *bias,
                                    const void *residual, const void *norm_w, void *y,
                                    const gd_hip_linear_params *params, int vector_ok, int kn_vector_ok,
                                    int store_vector_ok, int min_workgroups, const gd_hip_rope_epilogue *rope_epilogue,
                                    int wide_mode, int *family)
{
    /* *family: which kernel family took the call (GD_HIP_LINEAR_FAMILY_*), for logs and tests */
    *family = GD_HIP_LINEAR_FAMILY_STREAM;
    const gd_hip_rope_epilogue no_rope = {nullptr, nullptr, nullptr, nullptr, nullptr};
    const gd_hip_rope_epilogue &rope = rope_epilogue != nullptr ? *rope_epilogue : no_rope;
    const gd_hip_linear_params &p = *params;
    const gd_half *xp = (const gd_half *)x, *wp = (const gd_half *)w, *bp = (const gd_half *)bias;
    const gd_half *rp = (const gd_half *)residual, *np = (const gd_half *)norm_w;
    gd_half *yp = (gd_half *)y;
    if (p.M == 0 || p.N == 0) return (int)hipSuccess;
    if (!vector_ok || p.K == 0 || (!p.w_is_nk && !kn_vector_ok)) {
        const uint64_t total = (uint64_t)p.M * p.N;
        gd_linear_scalar_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(xp, wp, bp, rp, np, yp, p);
        *family = GD_HIP_LINEAR_FAMILY_SCALAR;
    } else if (p.M >= 128u && (p.w_is_nk || kn_vector_ok) && p.rope_head_dim == 0u) {
        /* matrix-core bound: LDS-tiled kernel; the 256 x 256 tile once it still gives every compute unit
         * a workgroup, the 128 x 128 tile below that */
        const uint32_t out_cols = p.swiglu_cols != 0u ? 128u : 256u; /* output columns of a 256-wide weight tile */
        const uint64_t big = (uint64_t)((p.M + 255u) / 256u) * ((p.N + out_cols - 1u) / out_cols);
        const uint32_t units = min_workgroups > 0 ? (uint32_t)min_workgroups / 2u : 256u;
        *family = GD_HIP_LINEAR_FAMILY_TILE;
        return gd_hip_launch_linear_tile(stream, x, w, bias, residual, norm_w, y, params, big >= units, store_vector_ok, (int)units);
    } else if (wide_mode != 0 && p.w_is_nk &&
               gd_hip_try_launch_linear_wide(stream, x, w, bias, residual, norm_w, y, params, rope_epilogue,
                                             wide_mode > 0 ? 0u : (4ull << 20), p.force_tiles,
                                             min_workgroups > 0 ? (uint32_t)min_workgroups / 2u : 256u)) {
        /* weight matrices of megabytes: the kernel built around the weight stream (wide_mode: 0 never, 1 whenever it
         * covers the call, -1 from 4 MiB of weights on; below that the launch latency decides and the stream kernel
         * is shorter) */
        *family = GD_HIP_LINEAR_FAMILY_WIDE;
    } else {
        /* columns per workgroup: 64, 32 or 16 (rows: always 16, further rows in grid.y; their weight re-reads
         * come from L2).  More columns reuse each activation fragment for more MFMAs and repeat the prologue
         * in fewer workgroups, but leave fewer workgroups; the grid keeps at least one per compute unit.
         * Paired modes (swiglu / rope epilogue) need 2 or 4 tiles; rope with 4 tiles needs head_dim % 64 == 0. */
        const uint64_t mt = (p.M + 15u) / 16u;
        const uint32_t target = min_workgroups > 0 ? (uint32_t)min_workgroups / 2u : 256u;
        const bool paired = p.rope_head_dim != 0u || p.swiglu_cols != 0u;
        const uint32_t outs = p.rope_head_dim != 0u ? p.N / 2u : p.N; /* columns that count towards the grid */
        const uint32_t per4 = paired ? 32u : 64u, per2 = paired ? 16u : 32u;
        uint32_t nt;
        const uint64_t wgs4 = ((outs + per4 - 1u) / per4) * mt;
        if (wgs4 >= target || (p.K >= 1024u && wgs4 * 2u >= target && p.rope_head_dim == 0u)) nt = 4u; /* deep K: the repeated prologue weighs more */
        else if (paired || ((outs + per2 - 1u) / per2) * mt >= target) nt = 2u;
        else nt = 1u;
        if (p.force_tiles != 0u && !(paired && p.force_tiles == 1u)) nt = p.force_tiles;
        if (p.rope_head_dim != 0u && nt == 4u && (p.rope_head_dim % 64u) != 0u) nt = 2u;
        /* short K: splitting it eight ways leaves a wavefront one or two steps; four wavefronts then */
        uint32_t waves = (p.K + 31u) / 32u <= 16u ? 4u : 8u;
        /* very long K without a prologue (the down projection of the wide decoders): the stream is long enough to
         * hide the round trips with four wavefronts, and four leave less to add up (13.6 against 14.7 us at
         * 16 x 5632 x 2048) */
        if (p.K >= 4096u && p.prologue == GD_HIP_PRO_NONE) waves = 4u;
        if (p.force_waves != 0u) waves = p.force_waves;
#define GD_LS(NTV, WV) launch_stream<NTV, WV>(stream, xp, wp, bp, rp, np, yp, p, rope)
        if (waves == 4u) {
            if (nt == 4u) GD_LS(4, 4); else if (nt == 2u) GD_LS(2, 4); else GD_LS(1, 4);
        } else {
            if (nt == 4u) GD_LS(4, 8); else if (nt == 2u) GD_LS(2, 8); else GD_LS(1, 8);
        }
#undef GD_LS
    }
    return (int)hipGetLastError();
}
