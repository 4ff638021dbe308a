/*
 * The few-row projection kernel (gd_linear_stream_kernel) as a template, shared by linear.hip, which instantiates
 * every form with the weight fragments loaded straight into registers, and linear_lds.hip, which instantiates the one
 * form that stages its weight stream through LDS.  Two translation units on purpose: the kernels of a decode step
 * at the small configuration are latency chains of a few microseconds, and their timing moved by 4 % with nothing
 * but their placement in the code object when the LDS form was compiled next to them.
 */
#ifndef GD_LINEAR_STREAM_KERNEL_H
#define GD_LINEAR_STREAM_KERNEL_H
#include "../../_shared/hip_device.h"
#include "hip_linear_types.h"
#include "../../qkv_split_rope/hip/rope_device.h"
#include <type_traits>

__device__ __forceinline__ float gd_lin_silu(float z)
{
    const float e = __expf(-fabsf(z));
    const float inv = 1.0f / (1.0f + e);
    return z * (z >= 0.0f ? inv : e * inv);
}

/* 16 bytes per lane from global memory straight into LDS: lane l's data lands at lds_byte_address + 16*l.
 * Assembly, because the kernel counts these loads itself (s_waitcnt vmcnt) instead of waiting for all of them. */
__device__ __forceinline__ void gd_lin_load_lds16(const unsigned char *uniform_base, uint32_t lane_byte_offset,
                                                  uint32_t lds_byte_address)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_byte_address), "v"(lane_byte_offset), "s"(uniform_base)
                 : "memory");
}

template <int NT, int WAVES, bool W_NK, int PRO, bool RES, bool LDS_STREAM>
__global__ void __launch_bounds__(WAVES * 64)
gd_linear_stream_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w,
                        const gd_half *__restrict__ bias, const gd_half *__restrict__ residual,
                        const gd_half *__restrict__ norm_w, gd_half *__restrict__ y, gd_hip_linear_params p,
                        uint32_t n_tiles, gd_hip_rope_epilogue rope)
{
    constexpr int U = NT >= 4 ? 2 : 4;  /* K steps per register set; two sets alternate */
    constexpr int RES_STEPS = 8;        /* RES: the wavefront's whole K slice of the activation stays in registers */
    constexpr uint32_t COLS = 16u * NT; /* output columns of a workgroup */
    typedef short gd_short4 __attribute__((ext_vector_type(4)));
    __shared__ float sm[WAVES][NT][64][4];
    __shared__ float s_inv[16];
    __shared__ float s_part[WAVES][16];
    /* w stored [K,N]: a 32(k) x COLS(n) tile per wavefront, turned by the transposing LDS read */
    __shared__ __align__(16) gd_half s_tr[W_NK ? 1 : WAVES][W_NK ? 8 : 32 * COLS];
    /* Weight stream through LDS (long-K [N,K] projections behind an rms_norm whose activation slice is resident:
     * the qkv, up/gate and LM-head projections of the wide decoders).  A load that goes straight to registers must
     * follow the MFMA operand layout, 4 lanes = 64 bytes per weight row and instruction, and such half-line requests
     * stream about a fifth slower than whole lines.  Lane order in LDS is free, so here one instruction fetches
     * 8 weight rows x 128 bytes (two K steps) into a wavefront-private ring and the fragments are read from there
     * (16-byte chunks XOR-swizzled by the row so that the reads spread over the banks).  A group = the 16 rows of
     * one column tile x 128 bytes = two instructions; RING groups are in flight per wavefront.  The MFMAs run in
     * the order of the register path, so the sums are the same to the bit. */
    constexpr bool LDSW = LDS_STREAM && W_NK && RES && WAVES == 8 && NT >= 4 && PRO == GD_HIP_PRO_RMS_NORM;
    constexpr int RING = 6;
    __shared__ __align__(16) unsigned char s_ring[LDSW ? WAVES * RING * 2048 : 16];
    /* every kernel argument the kernel reads, requested in one batch with one wait (left alone, the compiler puts
     * each load in front of its first use, one dependent round trip after the other) */
    asm volatile("" ::"s"(x), "s"(w), "s"(bias), "s"(residual), "s"(norm_w), "s"(y), "s"(p.M), "s"(p.N), "s"(p.K),
                 "s"(p.ldx), "s"(p.ldw), "s"(p.ldy), "s"(p.epilogue), "s"(p.has_residual), "s"(p.ldr), "s"(p.eps),
                 "s"(p.swiglu_cols), "s"(p.rope_head_dim), "s"(n_tiles));
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15, lg = lane >> 4;
    /* XCD-aware tile order: workgroup ids are dealt round-robin to the 8 XCDs, so give each XCD a
     * contiguous run of column tiles (neighbouring tiles share weight cache lines when w is [K,N]) */
    uint32_t tile = blockIdx.x;
    if ((n_tiles & 7u) == 0u) tile = (blockIdx.x & 7u) * (n_tiles >> 3) + (blockIdx.x >> 3);
    /* gated (swiglu epilogue): the first NT/2 column tiles are value columns, the others the matching gate columns
     * swiglu_cols further down the weight; the workgroup then owns COLS/2 output columns */
    /* roped (rope + append epilogue): the same pairing inside one head: columns c and c + head_dim/2 */
    const bool roped = NT >= 2 && p.rope_head_dim != 0u;
    const bool gated = NT >= 2 && (p.swiglu_cols != 0u || roped);
    const uint32_t pair_offset = roped ? p.rope_head_dim / 2u : p.swiglu_cols;
    uint32_t n0 = tile * (gated ? COLS / 2u : COLS);
    if (roped) {
        const uint32_t per_head = (p.rope_head_dim / 2u) / (COLS / 2u); /* workgroups per head and section */
        n0 = (tile / per_head) * p.rope_head_dim + (tile % per_head) * (COLS / 2u);
    }
    const uint32_t m0 = blockIdx.y * 16u;
    const uint32_t mrow = min(m0 + (uint32_t)li, p.M - 1u);

    /* What the epilogue will need of other tensors (bias values, the residual, the positions of the rope + append
     * form) is requested here, in front of everything else: read behind the sum of the wavefronts, each would be one
     * more dependent round trip at the end of a kernel that is a chain of round trips. */
    constexpr int NTO_MAX = NT >= 2 ? NT : 1; /* output column tiles of the plain form (the paired forms have NT / 2) */
    constexpr int EPT = (NTO_MAX * 256 + WAVES * 64 - 1) / (WAVES * 64);
    gd_half pf_b1[EPT], pf_b2[EPT], pf_res[EPT];
    int32_t pf_pos[EPT], pf_cpos[EPT];
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
        const int idx = (int)threadIdx.x + i * WAVES * 64;
        const int j = idx >> 8, rl = idx & 63, rr = (idx >> 6) & 3;
        const uint32_t col = min(n0 + 16u * j + (rl & 15), p.N - 1u);
        const uint32_t row = min(m0 + 4u * (rl >> 4) + rr, p.M - 1u);
        pf_b1[i] = pf_b2[i] = pf_res[i] = (gd_half)0.f;
        pf_pos[i] = pf_cpos[i] = 0;
        if (idx < (gated ? NT / 2 : NT) * 256) {
            if (p.epilogue != GD_HIP_EPI_NONE) {
                pf_b1[i] = bias[col];
                if (gated) pf_b2[i] = bias[pair_offset + col];
            }
            if (!gated && p.has_residual) pf_res[i] = residual[(size_t)row * p.ldr + col];
            if (roped) {
                pf_pos[i] = rope.rope_pos[row];
                pf_cpos[i] = rope.cache_pos[row];
            }
        }
    }

    /* K range of this wavefront, in steps of 32 */
    const uint32_t ksteps = (p.K + 31u) / 32u;
    const uint32_t per_wave = (ksteps + WAVES - 1u) / WAVES;
    const uint32_t s_begin = wave * per_wave, s_end = min(s_begin + per_wave, ksteps);

    gd_half8 bf[2][U][NT];
    gd_half8 af[2][RES ? 1 : U], zf[2][PRO == GD_HIP_PRO_SWIGLU ? U : 1], nf[2][(PRO == GD_HIP_PRO_RMS_NORM && !RES) ? U : 1];
    gd_half8 ar[RES ? RES_STEPS : 1], nr[(RES && PRO == GD_HIP_PRO_RMS_NORM) ? RES_STEPS : 1];
    const gd_half8 zero8 = (gd_half8)(gd_half)0.f;
    const gd_half *xrow = x + (size_t)mrow * p.ldx;

    /* Fast path (whole steps of 32, byte offsets that fit 32 bits, all columns of a [K,N] tile in range): the
     * loads carry no guards and take a scalar base that advances with the step plus one per-lane offset computed
     * once, so a register set is requested by a run of load instructions with nothing in between.  The four to
     * eight wavefronts of a workgroup share the issue slots of their SIMDs: what sits in front of the first loads
     * is paid by every one of them before the memory round trip even starts. */
    const bool off32 = (W_NK ? (uint64_t)(p.N + pair_offset) * p.ldw : (uint64_t)p.K * p.ldw) < 0x7fffffffull &&
                       (uint64_t)p.M * p.ldx + 2u * (uint64_t)p.K < 0x7fffffffull;
    const bool fast = (p.K & 31u) == 0u && off32 && (W_NK || n0 + COLS <= p.N);
    const unsigned char *wb = reinterpret_cast<const unsigned char *>(w);
    const unsigned char *xb = reinterpret_cast<const unsigned char *>(x);
    const unsigned char *nb = reinterpret_cast<const unsigned char *>(norm_w);
    uint32_t woff[NT]; /* bytes from w to the lane's fragment of step 0 */
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        if (W_NK) {
            const uint32_t n = (gated && j >= NT / 2)
                                   ? pair_offset + min(n0 + 16u * (uint32_t)(j - NT / 2) + (uint32_t)li, p.N - 1u)
                                   : min(n0 + 16u * (uint32_t)j + (uint32_t)li, p.N - 1u);
            woff[j] = (n * p.ldw + (uint32_t)lg * 8u) * 2u;
        } else {
            woff[j] = (((uint32_t)j * (32u / NT) + (uint32_t)lane / (2u * NT)) * p.ldw + n0 + ((uint32_t)lane % (2u * NT)) * 8u) * 2u;
        }
    }
    const uint32_t xoff = (mrow * p.ldx + (uint32_t)lg * 8u) * 2u;
    const uint32_t wstep = W_NK ? 64u : 64u * p.ldw; /* bytes per step of 32 k */

    /* requests the operands of steps s0 .. s0+U-1 into register set `set` */
    auto load_set_impl = [&](auto set_tag, auto full_tag, uint32_t s0) __attribute__((always_inline)) {
        constexpr int set = decltype(set_tag)::value;
        constexpr bool FULL = decltype(full_tag)::value;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (FULL) {
                const unsigned char *ws = wb + (size_t)(s0 + u) * wstep;
#pragma unroll
                for (int j = 0; j < NT; ++j) bf[set][u][j] = *reinterpret_cast<const gd_half8 *>(ws + woff[j]);
                if (!RES) {
                    const unsigned char *xs = xb + (size_t)(s0 + u) * 64u;
                    af[set][u] = *reinterpret_cast<const gd_half8 *>(xs + xoff);
                    if (PRO == GD_HIP_PRO_SWIGLU) zf[set][u] = *reinterpret_cast<const gd_half8 *>(xs + (size_t)p.K * 2u + xoff);
                    if (PRO == GD_HIP_PRO_RMS_NORM)
                        nf[set][u] = *reinterpret_cast<const gd_half8 *>(nb + (size_t)(s0 + u) * 64u + (uint32_t)lg * 16u);
                }
                continue;
            }
            const bool sok = (s0 + u) < s_end;
            const uint32_t k = (s0 + u) * 32u + lg * 8u; /* K % 8 == 0: a fragment is all-valid or all-out */
            const bool kok = sok && k < p.K;
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                bf[set][u][j] = zero8;
                if (W_NK) {
                    /* clamped: out-of-range columns are never stored */
                    const uint32_t n = (gated && j >= NT / 2)
                                           ? pair_offset + min(n0 + 16u * (uint32_t)(j - NT / 2) + (uint32_t)li, p.N - 1u)
                                           : min(n0 + 16u * (uint32_t)j + (uint32_t)li, p.N - 1u);
                    if (kok) bf[set][u][j] = *reinterpret_cast<const gd_half8 *>(w + (size_t)n * p.ldw + k);
                } else {
                    /* load j fetches k-rows j*32/NT .. of the 32 x COLS tile: 2*NT chunks of 8 columns per row */
                    const uint32_t kr = (s0 + u) * 32u + (uint32_t)j * (32u / NT) + (uint32_t)lane / (2u * NT);
                    const uint32_t nc = n0 + ((uint32_t)lane % (2u * NT)) * 8u;
                    if (sok && kr < p.K && nc < p.N)
                        bf[set][u][j] = *reinterpret_cast<const gd_half8 *>(w + (size_t)kr * p.ldw + nc);
                }
            }
            if (!RES) {
                af[set][u] = kok ? *reinterpret_cast<const gd_half8 *>(xrow + k) : zero8;
                if (PRO == GD_HIP_PRO_SWIGLU) zf[set][u] = kok ? *reinterpret_cast<const gd_half8 *>(xrow + p.K + k) : zero8;
                if (PRO == GD_HIP_PRO_RMS_NORM) nf[set][u] = kok ? *reinterpret_cast<const gd_half8 *>(norm_w + k) : zero8;
            }
        }
    };
    auto load_set = [&](auto set_tag, uint32_t s0) __attribute__((always_inline)) {
        if (fast && s0 + (uint32_t)U <= s_end) load_set_impl(set_tag, std::true_type{}, s0);
        else load_set_impl(set_tag, std::false_type{}, s0);
    };

    gd_float4 acc[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[j] = (gd_float4){0.f, 0.f, 0.f, 0.f};
    float minv = 1.f;

    /* multiplies the steps of register set `set`; `base` = index of its first step within the wavefront's slice */
    auto compute_set = [&](auto set_tag, auto base_tag) __attribute__((always_inline)) {
        constexpr int set = decltype(set_tag)::value;
        constexpr int base = decltype(base_tag)::value;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            gd_half8 a = RES ? ar[(base + u) < RES_STEPS ? (base + u) : 0] : af[set][u];
            if (PRO == GD_HIP_PRO_SWIGLU) {
#pragma unroll
                for (int e = 0; e < 8; ++e) a[e] = (gd_half)((float)a[e] * gd_lin_silu((float)zf[set][u][e]));
            }
            if (PRO == GD_HIP_PRO_RMS_NORM) {
                const gd_half8 nw = RES ? nr[(base + u) < RES_STEPS ? (base + u) : 0] : nf[set][u];
#pragma unroll
                for (int e = 0; e < 8; ++e) a[e] = (gd_half)((float)a[e] * (float)nw[e] * minv);
            }
            if (!W_NK) {
                gd_half *tr = &s_tr[wave][0];
#pragma unroll
                for (int j = 0; j < NT; ++j)
                    *reinterpret_cast<gd_half8 *>(tr + ((uint32_t)j * (32u / NT) + (uint32_t)lane / (2u * NT)) * COLS +
                                                  ((uint32_t)lane % (2u * NT)) * 8u) = bf[set][u][j];
            }
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                gd_half8 b = bf[set][u][j];
                if (!W_NK) {
                    /* lane q + 4e of a 16-lane group addresses k-row 8*lg + e (+4), columns 4q .. 4q+3 of column tile j;
                     * lane i then receives column i of four consecutive k-rows */
                    const gd_half *src = &s_tr[wave][0] + (8 * lg + ((lane >> 2) & 3)) * COLS + 16 * j + (lane & 3) * 4;
                    union { gd_short4 s[2]; gd_half8 h; } t2;
                    t2.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) gd_short4 *)src);
                    t2.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) gd_short4 *)(src + 4 * COLS));
                    b = t2.h;
                }
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[j], 0, 0, 0);
            }
        }
    };
    using gd_s0 = std::integral_constant<int, 0>;
    using gd_s1 = std::integral_constant<int, 1>;

    /* LDS path: every step of the wavefront exists (8 steps = 4 line pairs per column tile) */
    const bool ldsw = LDSW && fast && s_begin + (uint32_t)RES_STEPS <= s_end;
    uint32_t goff[NT][2]; /* bytes from the group's base to the lane's 16 bytes: row 8*half + lane/8, swizzled chunk */
    const uint32_t ring_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)s_ring + (uint32_t)wave * (RING * 2048u);
    auto issue_group = [&](uint32_t g) __attribute__((always_inline)) {
        /* g = pair * NT + j: K steps 2*pair, 2*pair+1 of column tile j */
        const uint32_t pair = g / NT, j = g % NT, slot = ring_base + (g % RING) * 2048u;
        const unsigned char *src = wb + (size_t)(s_begin + 2u * pair) * 64u;
        gd_lin_load_lds16(src, goff[j][0], slot);
        gd_lin_load_lds16(src, goff[j][1], slot + 1024u);
    };
    if (LDSW && ldsw) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t rowi = 8u * h + (uint32_t)lane / 8u;
                const uint32_t n = (gated && j >= NT / 2)
                                       ? pair_offset + min(n0 + 16u * (uint32_t)(j - NT / 2) + rowi, p.N - 1u)
                                       : min(n0 + 16u * (uint32_t)j + rowi, p.N - 1u);
                goff[j][h] = (n * p.ldw + ((((uint32_t)lane % 8u) ^ ((uint32_t)lane / 8u)) * 8u)) * 2u;
            }
        }
#pragma unroll
        for (int g = 0; g < RING; ++g) issue_group((uint32_t)g);
    } else {
        /* the first weights are requested before anything else so that the row norms below overlap their flight */
        load_set(gd_s0{}, s_begin);
    }

    if (RES) {
        /* the wavefront's whole activation slice (at most RES_STEPS steps): one batch of loads, and the row's sum of
         * squares comes from these registers instead of a second pass over x */
        float ss = 0.f;
        if (fast && s_begin + (uint32_t)RES_STEPS <= s_end) {
#pragma unroll
            for (int r = 0; r < RES_STEPS; ++r) {
                ar[r] = *reinterpret_cast<const gd_half8 *>(xb + (size_t)(s_begin + r) * 64u + xoff);
                if (PRO == GD_HIP_PRO_RMS_NORM)
                    nr[r] = *reinterpret_cast<const gd_half8 *>(nb + (size_t)(s_begin + r) * 64u + (uint32_t)lg * 16u);
            }
        } else {
#pragma unroll
            for (int r = 0; r < RES_STEPS; ++r) {
                const uint32_t k = (s_begin + r) * 32u + lg * 8u;
                const bool kok = (s_begin + r) < s_end && k < p.K;
                ar[r] = kok ? *reinterpret_cast<const gd_half8 *>(xrow + k) : zero8;
                if (PRO == GD_HIP_PRO_RMS_NORM) nr[r] = kok ? *reinterpret_cast<const gd_half8 *>(norm_w + k) : zero8;
            }
        }
        /* the second register set is requested here too: behind the barrier of the row norms its round trip would
         * start only when the first one has ended */
        if (!(LDSW && ldsw)) load_set(gd_s1{}, s_begin + U);
        if (PRO == GD_HIP_PRO_RMS_NORM) {
#pragma unroll
            for (int r = 0; r < RES_STEPS; ++r)
#pragma unroll
                for (int e = 0; e < 8; ++e) ss = fmaf((float)ar[r][e], (float)ar[r][e], ss);
            ss += __shfl_xor(ss, 16, 64);
            ss += __shfl_xor(ss, 32, 64);
            if (lg == 0) s_part[wave][li] = ss;
            __syncthreads();
            float tot = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) tot += s_part[wv][li];
            minv = rsqrtf(tot / (float)p.K + p.eps);
        }
    } else if (PRO == GD_HIP_PRO_RMS_NORM) {
        /* row norms by a separate pass over x: one wavefront per row, 8 halfs per lane and trip */
        for (uint32_t r = wave; r < 16u; r += WAVES) {
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
        minv = s_inv[li];
    }

    /* two register sets alternate: the next U steps are in flight while the current ones are multiplied */
    if (LDSW && ldsw) {
        const uint32_t li8 = (uint32_t)li % 8u, half_rows = ((uint32_t)li / 8u) * 1024u;
        const uint32_t rd0 = half_rows + (li8 * 8u + ((uint32_t)lg ^ li8)) * 16u;
        const uint32_t rd1 = half_rows + (li8 * 8u + ((4u + (uint32_t)lg) ^ li8)) * 16u;
        const unsigned char *ring = &s_ring[0] + (size_t)wave * (RING * 2048);
        constexpr int NG = (RES_STEPS / 2) * NT;
        /* the normalised activation fragments, rounded to F16 like the separate rms_norm */
#pragma unroll
        for (int r = 0; r < RES_STEPS; ++r) {
#pragma unroll
            for (int e = 0; e < 8; ++e) ar[r][e] = (gd_half)((float)ar[r][e] * (float)nr[r][e] * minv);
        }
        /* group g is read from its slot while the MFMAs of group g-1 run; the slot of g-1 is refilled only behind
         * those MFMAs, which could not issue before its reads had returned */
        gd_half8 f0, f1, pf0 = zero8, pf1 = zero8;
#pragma unroll
        for (int g = 0; g <= NG; ++g) {
            if (g < NG) {
                /* loads return in order: group g has landed once only the groups requested after it are outstanding */
                const int issued = g < 2 ? RING - 1 : (g - 2 + RING < NG - 1 ? g - 2 + RING : NG - 1);
                const int later = issued - g;
                if (later >= 7) asm volatile("s_waitcnt vmcnt(14)" ::: "memory");
                else if (later == 6) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
                else if (later == 5) asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
                else if (later == 4) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
                else if (later == 3) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
                else if (later == 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                else if (later == 1) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                const unsigned char *slot = ring + (g % RING) * 2048;
                f0 = *reinterpret_cast<const gd_half8 *>(slot + rd0);
                f1 = *reinterpret_cast<const gd_half8 *>(slot + rd1);
            }
            if (g >= 1) {
                const int q = g - 1, pair = q / NT, j = q % NT;
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar[2 * pair], pf0, acc[j], 0, 0, 0);
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar[2 * pair + 1], pf1, acc[j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (q + RING < NG) issue_group((uint32_t)(q + RING));
            }
            pf0 = f0;
            pf1 = f1;
        }
    } else if (RES) {
        /* at most RES_STEPS steps: fully unrolled so that the resident fragments are indexed statically */
        compute_set(gd_s0{}, std::integral_constant<int, 0>{});
        if (2 * U < RES_STEPS) {
            load_set(gd_s0{}, s_begin + 2u * U);
            compute_set(gd_s1{}, std::integral_constant<int, U>{});
            load_set(gd_s1{}, s_begin + 3u * U);
            compute_set(gd_s0{}, std::integral_constant<int, 2 * U>{});
            compute_set(gd_s1{}, std::integral_constant<int, 3 * U>{});
        } else {
            compute_set(gd_s1{}, std::integral_constant<int, U>{});
        }
    } else {
        for (uint32_t s0 = s_begin; s0 < s_end; s0 += 2u * U) {
            load_set(gd_s1{}, s0 + U);
            compute_set(gd_s0{}, std::integral_constant<int, 0>{});
            load_set(gd_s0{}, s0 + 2u * U);
            compute_set(gd_s1{}, std::integral_constant<int, 0>{});
        }
    }

#pragma unroll
    for (int j = 0; j < NT; ++j) {
#pragma unroll
        for (int r = 0; r < 4; ++r) sm[wave][j][lane][r] = acc[j][r];
    }
    __syncthreads();
    if (gated) {
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
            const int idx = (int)threadIdx.x + i * WAVES * 64;
            if (idx >= (NT / 2) * 256) break;
            const int j = idx >> 8, rl = idx & 63, rr = (idx >> 6) & 3;
            const uint32_t col = n0 + 16u * j + (rl & 15);
            const uint32_t row = m0 + 4u * (rl >> 4) + rr;
            float v1 = 0.f, v2 = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) {
                v1 += sm[wv][j][rl][rr];
                v2 += sm[wv][j + NT / 2][rl][rr];
            }
            if (row < p.M && col < p.N) {
                gd_half h1, h2;
                if (p.epilogue == GD_HIP_EPI_BIAS_F32) {
                    h1 = (gd_half)(v1 + (float)pf_b1[i]);
                    h2 = (gd_half)(v2 + (float)pf_b2[i]);
                } else if (p.epilogue == GD_HIP_EPI_BIAS_F16) {
                    h1 = (gd_half)v1 + pf_b1[i];
                    h2 = (gd_half)v2 + pf_b2[i];
                } else {
                    h1 = (gd_half)v1;
                    h2 = (gd_half)v2;
                }
                if (!roped) {
                    y[(size_t)row * p.ldy + col] = (gd_half)((float)h1 * gd_lin_silu((float)h2));
                } else {
                    /* col = (section * heads + head) * head_dim + pair: q is rotated into its own tensor, k rotated and
                     * v copied into row cache_pos of the sequence's caches (skipped when that row does not exist) */
                    const uint32_t D = p.rope_head_dim, area = p.rope_heads * D;
                    const uint32_t section = col / area, within = col % area, pair = within % D;
                    gd_half o1 = h1, o2 = h2;
                    if (section < 2u) {
                        float c, sn;
                        gd_rope_cos_sin((float)pf_pos[i], pair, p.rope_freq_scale, &c, &sn);
                        gd_rope_rotate((float)h1, (float)h2, c, sn, &o1, &o2);
                    }
                    if (section == 0u) {
                        gd_half *dst = (gd_half *)rope.q + (size_t)row * area + within;
                        dst[0] = o1;
                        dst[D / 2u] = o2;
                    } else {
                        const int32_t cp = pf_cpos[i];
                        if (cp >= 0 && (uint32_t)cp < p.rope_tmax) {
                            gd_half *dst = (gd_half *)(section == 1u ? rope.k_cache : rope.v_cache) +
                                           ((size_t)row * p.rope_tmax + (size_t)cp) * area + within;
                            dst[0] = o1;
                            dst[D / 2u] = o2;
                        }
                    }
                }
            }
        }
        return;
    }
    /* (result lane, register) pairs of the NT tiles are spread over the workgroup's threads */
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
        const int idx = (int)threadIdx.x + i * WAVES * 64;
        if (idx >= NT * 256) break;
        const int j = idx >> 8, rl = idx & 63, rr = (idx >> 6) & 3;
        const uint32_t col = n0 + 16u * j + (rl & 15);
        const uint32_t row = m0 + 4u * (rl >> 4) + rr;
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) v += sm[wv][j][rl][rr];
        if (row < p.M && col < p.N) {
            gd_half h;
            if (p.epilogue == GD_HIP_EPI_BIAS_F32) h = (gd_half)(v + (float)pf_b1[i]);
            else if (p.epilogue == GD_HIP_EPI_BIAS_F16) h = (gd_half)v + pf_b1[i];
            else h = (gd_half)v;
            if (p.has_residual) h = pf_res[i] + h;
            y[(size_t)row * p.ldy + col] = h;
        }
    }
}

#endif
