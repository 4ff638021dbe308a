/*
 * F16 projections with F32 accumulation for gfx950 (MFMA 16x16x32 F16).
 *
 * Replaces the reference GEMM kernels src/ops/_shared/gemm/metal_gemm_common.h:54-135 (NN,
 * bias fused in F32) and :161-237 (NT) plus the separate bias add of
 * src/ops/linear_transposed_weight/core_linear_transposed_weight.c:51,76.
 *
 * Weight-streaming kernel (decode, M <= 64 rows per pass): the weight matrix is read once from
 * HBM, the activation tile is small and stays in cache, so the kernel is HBM-bound on
 * N*K*2 bytes.  A workgroup of 4 wavefronts owns 16 output columns; the wavefronts split K
 * four ways and are summed through LDS, which gives N/16 workgroups x 4 wavefronts of
 * independent weight streams even for narrow outputs.  With w stored [N,K] both MFMA operands
 * are K-contiguous: every lane fetches its 8-half fragment with one 16-byte load straight from
 * global memory (16 rows x 64 B per wavefront load) and no LDS staging is needed.  With w stored
 * [K,N] the B fragment is gathered with 2-byte loads (16 lanes read 32 contiguous bytes of a
 * weight row).
 *
 * MFMA operand layout used here (v_mfma_f32_16x16x32_f16): lane l supplies row/col l%16 and the
 * 8 consecutive K values starting at 8*(l/16); the result lane holds column l%16, rows
 * 4*(l/16)..+3.
 *
 * Rounding points: F32 accumulate; GD_HIP_EPI_BIAS_F32 adds the bias before the single F16
 * rounding; GD_HIP_EPI_BIAS_F16 rounds, then adds the bias in F16 (the reference's two-kernel
 * NT path).  The optional swiglu prologue rounds the activation to F16 before the MFMA exactly
 * like the reference's separate swiglu kernel, and the optional residual is added last in F16.
 */
#include "../../_shared/hip_device.h"
#include "hip_linear_types.h"

#define GD_LIN_WAVES 4

__device__ __forceinline__ float gd_lin_silu(float z)
{
    const float e = __expf(-fabsf(z));
    const float inv = 1.0f / (1.0f + e);
    return z * (z >= 0.0f ? inv : e * inv);
}

template <int MT, bool W_NK, bool SWIGLU>
__global__ void __launch_bounds__(GD_LIN_WAVES * 64)
gd_linear_stream_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w,
                        const gd_half *__restrict__ bias, const gd_half *__restrict__ residual,
                        gd_half *__restrict__ y, gd_hip_linear_params p, uint32_t n_tiles)
{
    __shared__ float sm[GD_LIN_WAVES][MT][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 15, lg = lane >> 4;
    /* XCD-aware tile order: workgroup ids are dealt round-robin to the 8 XCDs, so give each XCD a
     * contiguous run of column tiles (neighbouring tiles share weight cache lines when w is [K,N]) */
    uint32_t tile = blockIdx.x;
    if ((n_tiles & 7u) == 0u) tile = (blockIdx.x & 7u) * (n_tiles >> 3) + (blockIdx.x >> 3);
    const uint32_t n0 = tile * 16u;
    const uint32_t m0 = blockIdx.y * (MT * 16u);
    const uint32_t n = min(n0 + li, p.N - 1u); /* clamped: out-of-range columns are never stored */

    /* K range of this wavefront, in steps of 32 */
    const uint32_t ksteps = (p.K + 31u) / 32u;
    const uint32_t per_wave = (ksteps + GD_LIN_WAVES - 1u) / GD_LIN_WAVES;
    const uint32_t s_begin = wave * per_wave, s_end = min(s_begin + per_wave, ksteps);

    gd_float4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = (gd_float4){0.f, 0.f, 0.f, 0.f};

    uint32_t mrow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) mrow[t] = min(m0 + t * 16u + li, p.M - 1u);

    for (uint32_t s = s_begin; s < s_end; ++s) {
        const uint32_t k = s * 32u + lg * 8u; /* K % 8 == 0, so a fragment is all-valid or all-out */
        const bool kok = k < p.K;
        gd_half8 bf = (gd_half8)(gd_half)0.f;
        if (kok) {
            if (W_NK) {
                bf = *reinterpret_cast<const gd_half8 *>(w + (size_t)n * p.ldw + k);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) bf[e] = w[(size_t)(k + e) * p.ldw + n];
            }
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            gd_half8 af = (gd_half8)(gd_half)0.f;
            if (kok) {
                const gd_half *xr = x + (size_t)mrow[t] * p.ldx + k;
                af = *reinterpret_cast<const gd_half8 *>(xr);
                if (SWIGLU) {
                    const gd_half8 z = *reinterpret_cast<const gd_half8 *>(xr + p.K);
#pragma unroll
                    for (int e = 0; e < 8; ++e) af[e] = (gd_half)((float)af[e] * gd_lin_silu((float)z[e]));
                }
            }
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, bf, acc[t], 0, 0, 0);
        }
    }

#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int r = 0; r < 4; ++r) sm[wave][t][lane][r] = acc[t][r];
    }
    __syncthreads();
    /* thread -> (result lane, register): 256 threads cover the 64 x 4 values of one 16x16 tile */
    const int rl = threadIdx.x & 63, rr = threadIdx.x >> 6;
    const uint32_t col = n0 + (rl & 15);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const uint32_t row = m0 + t * 16u + 4u * (rl >> 4) + rr;
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < GD_LIN_WAVES; ++wv) v += sm[wv][t][rl][rr];
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
                        gd_half *__restrict__ y, gd_hip_linear_params p)
{
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)p.M * p.N) return;
    const uint32_t m = (uint32_t)(gid / p.N), n = (uint32_t)(gid % p.N);
    float acc = 0.f;
    for (uint32_t k = 0; k < p.K; ++k) {
        gd_half a = x[(size_t)m * p.ldx + k];
        if (p.swiglu) a = (gd_half)((float)a * gd_lin_silu((float)x[(size_t)m * p.ldx + p.K + k]));
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

template <int MT>
static void launch_stream(hipStream_t stream, const gd_half *x, const gd_half *w, const gd_half *bias,
                          const gd_half *residual, gd_half *y, const gd_hip_linear_params &p)
{
    const uint32_t n_tiles = (p.N + 15u) / 16u;
    dim3 grid(n_tiles, (p.M + MT * 16u - 1u) / (MT * 16u));
    const int threads = GD_LIN_WAVES * 64;
    if (p.w_is_nk) {
        if (p.swiglu) gd_linear_stream_kernel<MT, true, true><<<grid, threads, 0, stream>>>(x, w, bias, residual, y, p, n_tiles);
        else gd_linear_stream_kernel<MT, true, false><<<grid, threads, 0, stream>>>(x, w, bias, residual, y, p, n_tiles);
    } else {
        if (p.swiglu) gd_linear_stream_kernel<MT, false, true><<<grid, threads, 0, stream>>>(x, w, bias, residual, y, p, n_tiles);
        else gd_linear_stream_kernel<MT, false, false><<<grid, threads, 0, stream>>>(x, w, bias, residual, y, p, n_tiles);
    }
}

/* vector_ok: K % 8 == 0 and every pointer / pitch allows 16-byte fragment loads */
extern "C" int gd_hip_launch_linear(hipStream_t stream, const void *x, const void *w, const void *bias,
                                    const void *residual, void *y, const gd_hip_linear_params *params,
                                    int vector_ok)
{
    const gd_hip_linear_params &p = *params;
    const gd_half *xp = (const gd_half *)x, *wp = (const gd_half *)w, *bp = (const gd_half *)bias;
    const gd_half *rp = (const gd_half *)residual;
    gd_half *yp = (gd_half *)y;
    if (p.M == 0 || p.N == 0) return (int)hipSuccess;
    if (!vector_ok || p.K == 0) {
        const uint64_t total = (uint64_t)p.M * p.N;
        gd_linear_scalar_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(xp, wp, bp, rp, yp, p);
    } else if (p.M <= 16u) {
        launch_stream<1>(stream, xp, wp, bp, rp, yp, p);
    } else if (p.M <= 32u) {
        launch_stream<2>(stream, xp, wp, bp, rp, yp, p);
    } else {
        launch_stream<4>(stream, xp, wp, bp, rp, yp, p);
    }
    return (int)hipGetLastError();
}
