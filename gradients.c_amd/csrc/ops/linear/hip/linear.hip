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
#include "../../_shared/hip_device.h"
#include "hip_linear_types.h"

__device__ __forceinline__ float gd_lin_silu(float z)
{
    const float e = __expf(-fabsf(z));
    const float inv = 1.0f / (1.0f + e);
    return z * (z >= 0.0f ? inv : e * inv);
}

template <int MT, int WAVES, bool W_NK, int PRO>
__global__ void __launch_bounds__(WAVES * 64)
gd_linear_stream_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w,
                        const gd_half *__restrict__ bias, const gd_half *__restrict__ residual,
                        const gd_half *__restrict__ norm_w, gd_half *__restrict__ y, gd_hip_linear_params p,
                        uint32_t n_tiles)
{
    constexpr int U = 4; /* K steps whose loads are in flight together */
    __shared__ float sm[WAVES][MT][64][4];
    __shared__ float s_inv[MT * 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 15, lg = lane >> 4;
    /* XCD-aware tile order: workgroup ids are dealt round-robin to the 8 XCDs, so give each XCD a
     * contiguous run of column tiles (neighbouring tiles share weight cache lines when w is [K,N]) */
    uint32_t tile = blockIdx.x;
    if ((n_tiles & 7u) == 0u) tile = (blockIdx.x & 7u) * (n_tiles >> 3) + (blockIdx.x >> 3);
    const uint32_t n0 = tile * 16u;
    const uint32_t m0 = blockIdx.y * (MT * 16u);
    const uint32_t n = min(n0 + li, p.N - 1u); /* clamped: out-of-range columns are never stored */

    if (PRO == GD_HIP_PRO_RMS_NORM) {
        /* row norms of this tile: one wavefront per row, 8 halfs per lane and trip */
        for (uint32_t r = wave; r < MT * 16u; r += WAVES) {
            const uint32_t row = min(m0 + r, p.M - 1u);
            const gd_half *xr = x + (size_t)row * p.ldx;
            float ss = 0.f;
            for (uint32_t k = lane * 8u; k < p.K; k += 512u) {
                const gd_half8 v = *reinterpret_cast<const gd_half8 *>(xr + k);
#pragma unroll
                for (int e = 0; e < 8; ++e) ss = fmaf((float)v[e], (float)v[e], ss);
            }
            ss = gd_wave_sum(ss);
            if (lane == 0) s_inv[r] = rsqrtf(ss / (float)p.K + p.eps);
        }
        __syncthreads();
    }

    /* K range of this wavefront, in steps of 32 */
    const uint32_t ksteps = (p.K + 31u) / 32u;
    const uint32_t per_wave = (ksteps + WAVES - 1u) / WAVES;
    const uint32_t s_begin = wave * per_wave, s_end = min(s_begin + per_wave, ksteps);

    gd_float4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = (gd_float4){0.f, 0.f, 0.f, 0.f};

    uint32_t mrow[MT];
    float minv[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        mrow[t] = min(m0 + t * 16u + li, p.M - 1u);
        minv[t] = PRO == GD_HIP_PRO_RMS_NORM ? s_inv[t * 16 + li] : 1.f;
    }

    for (uint32_t s0 = s_begin; s0 < s_end; s0 += U) {
        gd_half8 bf[U], af[U][MT], zf[U][MT], nf[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t k = (s0 + u) * 32u + lg * 8u; /* K % 8 == 0: a fragment is all-valid or all-out */
            const bool kok = (s0 + u) < s_end && k < p.K;
            bf[u] = (gd_half8)(gd_half)0.f;
            if (kok) {
                if (W_NK) {
                    bf[u] = *reinterpret_cast<const gd_half8 *>(w + (size_t)n * p.ldw + k);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) bf[u][e] = w[(size_t)(k + e) * p.ldw + n];
                }
                if (PRO == GD_HIP_PRO_RMS_NORM) nf[u] = *reinterpret_cast<const gd_half8 *>(norm_w + k);
            }
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                af[u][t] = (gd_half8)(gd_half)0.f;
                if (kok) {
                    const gd_half *xr = x + (size_t)mrow[t] * p.ldx + k;
                    af[u][t] = *reinterpret_cast<const gd_half8 *>(xr);
                    if (PRO == GD_HIP_PRO_SWIGLU) zf[u][t] = *reinterpret_cast<const gd_half8 *>(xr + p.K);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t k = (s0 + u) * 32u + lg * 8u;
            const bool kok = (s0 + u) < s_end && k < p.K;
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                gd_half8 a = af[u][t];
                if (PRO == GD_HIP_PRO_SWIGLU && kok) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) a[e] = (gd_half)((float)a[e] * gd_lin_silu((float)zf[u][t][e]));
                }
                if (PRO == GD_HIP_PRO_RMS_NORM && kok) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) a[e] = (gd_half)((float)a[e] * (float)nf[u][e] * minv[t]);
                }
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bf[u], acc[t], 0, 0, 0);
            }
        }
    }

#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int r = 0; r < 4; ++r) sm[wave][t][lane][r] = acc[t][r];
    }
    __syncthreads();
    /* (result lane, register) pairs of the MT tiles are spread over the workgroup's threads */
    for (int idx = threadIdx.x; idx < MT * 256; idx += WAVES * 64) {
        const int t = idx >> 8, rl = idx & 63, rr = (idx >> 6) & 3;
        const uint32_t col = n0 + (rl & 15);
        const uint32_t row = m0 + t * 16u + 4u * (rl >> 4) + rr;
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) v += sm[wv][t][rl][rr];
        if (row < p.M && col < p.N) {
            gd_half h;
            if (p.epilogue == GD_HIP_EPI_BIAS_F32) h = (gd_half)(v + (float)bias[col]);
            else if (p.epilogue == GD_HIP_EPI_BIAS_F16) h = (gd_half)v + bias[col];
            else h = (gd_half)v;
            if (p.has_residual) h = residual[(size_t)row * p.ldr + col] + h;
            y[(size_t)row * p.ldy + col] = h;
        }
    }
}

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

template <int MT, int WAVES>
static void launch_stream(hipStream_t stream, const gd_half *x, const gd_half *w, const gd_half *bias,
                          const gd_half *residual, const gd_half *norm_w, gd_half *y, const gd_hip_linear_params &p)
{
    const uint32_t n_tiles = (p.N + 15u) / 16u;
    dim3 grid(n_tiles, (p.M + MT * 16u - 1u) / (MT * 16u));
    const int threads = WAVES * 64;
#define GD_GO(NK, PRO) gd_linear_stream_kernel<MT, WAVES, NK, PRO><<<grid, threads, 0, stream>>>(x, w, bias, residual, norm_w, y, p, n_tiles)
    if (p.w_is_nk) {
        if (p.prologue == GD_HIP_PRO_SWIGLU) GD_GO(true, GD_HIP_PRO_SWIGLU);
        else if (p.prologue == GD_HIP_PRO_RMS_NORM) GD_GO(true, GD_HIP_PRO_RMS_NORM);
        else GD_GO(true, GD_HIP_PRO_NONE);
    } else {
        if (p.prologue == GD_HIP_PRO_SWIGLU) GD_GO(false, GD_HIP_PRO_SWIGLU);
        else if (p.prologue == GD_HIP_PRO_RMS_NORM) GD_GO(false, GD_HIP_PRO_RMS_NORM);
        else GD_GO(false, GD_HIP_PRO_NONE);
    }
#undef GD_GO
}

extern "C" int gd_hip_launch_linear_tile(hipStream_t stream, const void *x, const void *w, const void *bias,
                                         const void *residual, const void *norm_w, void *y,
                                         const gd_hip_linear_params *params, int big_tiles, int vector_store);

/* vector_ok: K % 8 == 0 and every pointer / pitch allows 16-byte fragment loads (for w only when it is [N,K]);
 * kn_vector_ok: w stored [K,N] with N % 8 == 0 and 16-byte aligned rows; store_vector_ok: y (and the residual)
 * rows allow 16-byte accesses.  min_workgroups: about two per compute unit. */
extern "C" int gd_hip_launch_linear(hipStream_t stream, const void *x, const void *w, const void *bias,
                                    const void *residual, const void *norm_w, void *y,
                                    const gd_hip_linear_params *params, int vector_ok, int kn_vector_ok,
                                    int store_vector_ok, int min_workgroups)
{
    const gd_hip_linear_params &p = *params;
    const gd_half *xp = (const gd_half *)x, *wp = (const gd_half *)w, *bp = (const gd_half *)bias;
    const gd_half *rp = (const gd_half *)residual, *np = (const gd_half *)norm_w;
    gd_half *yp = (gd_half *)y;
    if (p.M == 0 || p.N == 0) return (int)hipSuccess;
    if (!vector_ok || p.K == 0) {
        const uint64_t total = (uint64_t)p.M * p.N;
        gd_linear_scalar_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(xp, wp, bp, rp, np, yp, p);
    } else if (p.M >= 128u && (p.w_is_nk || kn_vector_ok)) {
        /* matrix-core bound: LDS-tiled kernel; the 256 x 256 tile once it still gives every compute unit
         * a workgroup, the 128 x 128 tile below that */
        const uint64_t big = (uint64_t)((p.M + 255u) / 256u) * ((p.N + 255u) / 256u);
        const uint32_t units = min_workgroups > 0 ? (uint32_t)min_workgroups / 2u : 256u;
        return gd_hip_launch_linear_tile(stream, x, w, bias, residual, norm_w, y, params, big >= units, store_vector_ok);
    } else {
        /* rows per workgroup: 16, 32 or 64.  More rows reuse each weight fragment for more MFMAs but
         * leave fewer workgroups; narrow outputs take 16 rows so that the grid still covers the chip
         * (the re-read weights come from L2). */
        const uint64_t n_tiles = (p.N + 15u) / 16u;
        const uint32_t target = min_workgroups > 0 ? (uint32_t)min_workgroups : 512u;
        if (p.M > 32u && n_tiles * ((p.M + 63u) / 64u) >= target) launch_stream<4, 8>(stream, xp, wp, bp, rp, np, yp, p);
        else if (p.M > 16u && n_tiles * ((p.M + 31u) / 32u) >= target) launch_stream<2, 8>(stream, xp, wp, bp, rp, np, yp, p);
        else launch_stream<1, 8>(stream, xp, wp, bp, rp, np, yp, p);
    }
    return (int)hipGetLastError();
}
