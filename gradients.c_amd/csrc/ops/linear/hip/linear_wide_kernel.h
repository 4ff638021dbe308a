/*
 * Few-row projections over LARGE [N,K] weight matrices (megabytes: the projections of the wide decoders at decode
 * time, 1 to 64 activation rows): gd_linear_wide_kernel.  Same arithmetic and rounding points as
 * gd_linear_stream_kernel (MFMA 16x16x32 F16, F32 accumulation, prologue rounded to F16, bias / residual / swiglu /
 * rope epilogues), built around the weight stream instead of around the launch latency:
 *
 *   - every weight byte is read once, also for 32 or 64 activation rows: a workgroup keeps MT row tiles of 16 and
 *     multiplies each weight fragment MT times (the stream kernel runs one workgroup per row tile and re-reads
 *     the weights through L2);
 *   - the weights go from global memory straight into LDS in whole 128-byte lines (one instruction = 8 weight
 *     rows x 128 bytes; a load into registers must follow the MFMA operand layout, 16 rows x 64 bytes, and such
 *     half-line requests stream about a fifth slower), into a ring of RING groups of 2 KB per wavefront, so a
 *     compute unit has 8 x (RING - 1) x 2 KB of weights in flight without spending registers on them;
 *   - the activation slice of a wavefront (its K range of all MT row tiles) is loaded once, up front, into
 *     registers, and the operands the epilogue needs (bias, residual, positions) are requested before
 *     anything else, so no dependent round trip is left behind the stream; the slice is requested in front of
 *     the ring with loads the kernel counts itself (gd_wide_request16), because a wait placed by the compiler
 *     would also wait for the ring: the row sums of the rms_norm and the first matrix instructions then run
 *     while the first weight groups are still on their way (measured per phase with time stamps: the slice
 *     usable 3.4 instead of 5.7 us after entry at 16 x 2048 -> 6144);
 *   - the eight wavefronts of a workgroup split K and are summed through LDS (the ring's memory, reused).
 *
 * Reference semantics: src/ops/_shared/gemm/metal_gemm_common.h:161-237 (NT GEMM) with the separate bias add of
 * src/ops/linear_transposed_weight/core_linear_transposed_weight.c:51,76; rms_norm, swiglu and rope + append as the
 * separate operators round them.
 */
#ifndef GD_LINEAR_WIDE_KERNEL_H
#define GD_LINEAR_WIDE_KERNEL_H
#include "linear_stream_kernel.h"

#define GD_WIDE_EPI_PLAIN 0  /* bias (both rounding modes), optional residual */
#define GD_WIDE_EPI_SWIGLU 1 /* value / gate column pairs: y = half(value) * silu(half(gate)) */
#define GD_WIDE_EPI_ROPE 2   /* qkv of a decode step: rotation pairs, q stored, k / v appended to the caches */

/* Register loads the kernel counts itself.  The compiler does not see the global -> LDS loads of the ring, so a wait
 * it places for a load of its own is a wait for everything outstanding, the ring included: a wavefront would start
 * on its activation slice only when all of its first weight groups had crossed the chip.  Loads requested this way,
 * in front of the ring, are waited for with gd_wide_wait_groups (loads return in order: once only the ring's
 * instructions are outstanding, everything older has arrived); gd_wide_arrived then hands the registers to the
 * compiler, which must not touch them before. */
__device__ __forceinline__ gd_half8 gd_wide_request16(const unsigned char *uniform_base, uint32_t lane_byte_offset)
{
    gd_half8 v;
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(lane_byte_offset), "s"(uniform_base) : "memory");
    return v;
}
__device__ __forceinline__ uint32_t gd_wide_request2(const void *uniform_base, uint32_t lane_byte_offset)
{
    uint32_t v;
    asm volatile("global_load_ushort %0, %1, %2" : "=v"(v) : "v"(lane_byte_offset), "s"(uniform_base) : "memory");
    return v;
}
__device__ __forceinline__ uint32_t gd_wide_request4(const void *uniform_base, uint32_t lane_byte_offset)
{
    uint32_t v;
    asm volatile("global_load_dword %0, %1, %2" : "=v"(v) : "v"(lane_byte_offset), "s"(uniform_base) : "memory");
    return v;
}
template <typename T>
__device__ __forceinline__ void gd_wide_arrived(T &v)
{
    asm volatile("" : "+v"(v) : : "memory");
}
__device__ __forceinline__ gd_half gd_wide_half_of(uint32_t bits)
{
    union { unsigned short u; gd_half h; } c;
    c.u = (unsigned short)bits;
    return c.h;
}

/* waits until at most 2 * later of the wavefront's vector-memory loads are outstanding (later uniform, 0..8) */
__device__ __forceinline__ void gd_wide_wait_groups(int later)
{
    switch (later) {
    case 8: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
    case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
    case 3: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    case 5: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(14)" ::: "memory"); break;
    }
}

/* NT column tiles of 16 and MT row tiles of 16 per workgroup; a wavefront's K range is at most PMAX pairs of
 * 32-wide steps (64 columns of K each); PRO: GD_HIP_PRO_NONE or GD_HIP_PRO_RMS_NORM; EPI: GD_WIDE_EPI_*.
 * Host guarantees: K % 64 == 0, ceil(K / 64 / 8) <= PMAX, byte offsets below 2^31, N a multiple of 16 * NT (of the
 * pairing for the paired epilogues), 16-byte aligned rows. */
template <int NT, int MT, int PMAX, int RING, int PRO, int EPI>
__global__ void __launch_bounds__(512)
gd_linear_wide_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w, const gd_half *__restrict__ bias,
                      const gd_half *__restrict__ residual, const gd_half *__restrict__ norm_w,
                      gd_half *__restrict__ y, gd_hip_linear_params p, uint32_t n_tiles, gd_hip_rope_epilogue rope)
{
    constexpr int WAVES = 8;
    constexpr int SMAX = 2 * PMAX;  /* K steps of 32 per wavefront */
    constexpr int NGMAX = PMAX * NT; /* weight groups per wavefront: (pair, column tile) */
    constexpr bool PAIRED = EPI != GD_WIDE_EPI_PLAIN;
    constexpr int NTO = PAIRED ? NT / 2 : NT;               /* column tiles that produce outputs */
    constexpr int EPT = (NTO * MT * 256 + 511) / 512;       /* outputs per thread */
    static_assert(!PAIRED || NT >= 2, "paired epilogues need two column tiles");
    static_assert(RING >= 2 && RING <= 8, "ring depth");
    /* the ring during the stream, the partial sums of the wavefronts after it */
    constexpr int RING_BYTES = WAVES * RING * 2048, SUM_BYTES = WAVES * MT * NT * 1024;
    __shared__ __align__(16) unsigned char s_mem[RING_BYTES > SUM_BYTES ? RING_BYTES : SUM_BYTES];
    __shared__ float s_part[WAVES][MT][16];

    asm volatile("" ::"s"(x), "s"(w), "s"(bias), "s"(residual), "s"(norm_w), "s"(y), "s"(p.M), "s"(p.N), "s"(p.K),
                 "s"(p.ldx), "s"(p.ldw), "s"(p.ldy), "s"(p.epilogue), "s"(p.has_residual), "s"(p.ldr), "s"(p.eps),
                 "s"(p.swiglu_cols), "s"(p.rope_head_dim), "s"(n_tiles));
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15, lg = lane >> 4;
    /* XCD-aware tile order: workgroup ids are dealt round-robin to the 8 XCDs; each XCD gets a run of tiles */
    uint32_t tile = blockIdx.x;
    if ((n_tiles & 7u) == 0u) tile = (blockIdx.x & 7u) * (n_tiles >> 3) + (blockIdx.x >> 3);
    constexpr uint32_t COLS = 16u * NT;
    const uint32_t pair_offset = EPI == GD_WIDE_EPI_ROPE ? p.rope_head_dim / 2u : (EPI == GD_WIDE_EPI_SWIGLU ? p.swiglu_cols : 0u);
    uint32_t n0 = tile * (PAIRED ? COLS / 2u : COLS);
    if (EPI == GD_WIDE_EPI_ROPE) {
        const uint32_t per_head = (p.rope_head_dim / 2u) / (COLS / 2u); /* workgroups per head and section */
        n0 = (tile / per_head) * p.rope_head_dim + (tile % per_head) * (COLS / 2u);
    }
    const uint32_t m0 = blockIdx.y * (16u * MT);

    /* ---- 1. what the epilogue will need, requested first ---- */
    gd_half pf_b1[EPT], pf_b2[EPT], pf_res[EPT];
    int32_t pf_pos[EPT], pf_cpos[EPT];
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
        const int idx = (int)threadIdx.x + 512 * i;
        const int jj = idx >> 8, mt = jj / NTO, j = jj % NTO, rl = idx & 63, rr = (idx >> 6) & 3;
        const uint32_t col = min(n0 + 16u * j + (rl & 15), p.N - 1u);
        const uint32_t row = min(m0 + 16u * mt + 4u * (rl >> 4) + rr, p.M - 1u);
        pf_b1[i] = pf_b2[i] = pf_res[i] = (gd_half)0.f;
        pf_pos[i] = pf_cpos[i] = 0;
        if (jj < NTO * MT) {
            if (p.epilogue != GD_HIP_EPI_NONE) {
                pf_b1[i] = bias[col];
                if (PAIRED) pf_b2[i] = bias[pair_offset + col];
            }
            if (EPI == GD_WIDE_EPI_PLAIN && p.has_residual) pf_res[i] = residual[(size_t)row * p.ldr + col];
            if (EPI == GD_WIDE_EPI_ROPE) {
                pf_pos[i] = rope.rope_pos[row];
                pf_cpos[i] = rope.cache_pos[row];
            }
        }
    }

    /* ---- 2. the wavefront's K range (pairs of steps) ---- */
    const uint32_t kpairs = p.K / 64u;
    const uint32_t per_wave = (kpairs + WAVES - 1u) / WAVES;
    const uint32_t p_begin = min((uint32_t)wave * per_wave, kpairs);
    const int np = (int)(min(p_begin + per_wave, kpairs) - p_begin); /* 0..PMAX */
    const int ng = np * NT;
    const unsigned char *wb = reinterpret_cast<const unsigned char *>(w) + (size_t)p_begin * 128u;
    /* (a wavefront without a K range requests the first step of the row instead of one past its end) */
    const unsigned char *xb = reinterpret_cast<const unsigned char *>(x) + (size_t)(np > 0 ? p_begin : 0u) * 128u;
    const unsigned char *nb = reinterpret_cast<const unsigned char *>(norm_w) + (size_t)(np > 0 ? p_begin : 0u) * 128u;
    const gd_half8 zero8 = (gd_half8)(gd_half)0.f;
    /* ---- 3. the weight stream: group g = pair * NT + j, two instructions of 8 rows x 128 bytes ---- */
    uint32_t goff[NT][2]; /* bytes from the pair's base to the lane's 16 bytes: row 8*half + lane/8, swizzled chunk */
#pragma unroll
    for (int j = 0; j < NT; ++j) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t rowi = 8u * h + (uint32_t)lane / 8u;
            const uint32_t n = (PAIRED && j >= NT / 2) ? pair_offset + min(n0 + 16u * (uint32_t)(j - NT / 2) + rowi, p.N - 1u)
                                                       : min(n0 + 16u * (uint32_t)j + rowi, p.N - 1u);
            goff[j][h] = (n * p.ldw + ((((uint32_t)lane % 8u) ^ ((uint32_t)lane / 8u)) * 8u)) * 2u;
        }
    }
    const uint32_t ring_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)s_mem +
                               (uint32_t)wave * (RING * 2048u);
    auto issue_group = [&](int g) __attribute__((always_inline)) {
        const int pair = g / NT, j = g % NT;
        const uint32_t slot = ring_base + (uint32_t)(g % RING) * 2048u;
        const unsigned char *src = wb + (size_t)pair * 128u;
        gd_lin_load_lds16(src, goff[j][0], slot);
        gd_lin_load_lds16(src, goff[j][1], slot + 1024u);
    };
    /* ---- 3a. the activation slice of the wavefront (and the norm weights of its K range), resident: requested in
     *          front of the ring and counted by hand, so that it is usable while the ring is still on its way.  Steps
     *          past the wavefront's range re-read its first one (never multiplied with a landed weight group, but the
     *          row sums of the rms_norm must not see them: zeroed after arrival) ---- */
    gd_half8 ar[MT][SMAX], nr[PRO == GD_HIP_PRO_RMS_NORM ? SMAX : 1];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const uint32_t mrow = min(m0 + 16u * mt + (uint32_t)li, p.M - 1u);
        const uint32_t xoff = (mrow * p.ldx + (uint32_t)lg * 8u) * 2u;
#pragma unroll
        for (int s = 0; s < SMAX; ++s) ar[mt][s] = gd_wide_request16(xb, (s < 2 * np ? (uint32_t)s * 64u : 0u) + xoff);
    }
    if (PRO == GD_HIP_PRO_RMS_NORM) {
#pragma unroll
        for (int s = 0; s < SMAX; ++s) nr[s] = gd_wide_request16(nb, (s < 2 * np ? (uint32_t)s * 64u : 0u) + (uint32_t)lg * 16u);
    }
    int first_groups = 0;
#pragma unroll
    for (int g = 0; g < RING && g < NGMAX; ++g) {
        if (g < ng) {
            issue_group(g);
            first_groups = g + 1;
        }
    }
    gd_wide_wait_groups(first_groups);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
            gd_wide_arrived(ar[mt][s]);
            if (s >= 2 * np) ar[mt][s] = zero8;
        }
    if (PRO == GD_HIP_PRO_RMS_NORM) {
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
            gd_wide_arrived(nr[s]);
            if (s >= 2 * np) nr[s] = zero8;
        }
    }

    /* ---- 4. prologue on the resident activation slice ---- */
    if (PRO == GD_HIP_PRO_RMS_NORM) {
        float ss[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            ss[mt] = 0.f;
#pragma unroll
            for (int s = 0; s < SMAX; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e) ss[mt] = fmaf((float)ar[mt][s][e], (float)ar[mt][s][e], ss[mt]);
            ss[mt] += __shfl_xor(ss[mt], 16, 64);
            ss[mt] += __shfl_xor(ss[mt], 32, 64);
            if (lg == 0) s_part[wave][mt][li] = ss[mt];
        }
        /* LDS writes visible, then the barrier: the weight loads in flight are not waited for */
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            float tot = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) tot += s_part[wv][mt][li];
            const float minv = rsqrtf(tot / (float)p.K + p.eps);
#pragma unroll
            for (int s = 0; s < SMAX; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    ar[mt][s][e] = (gd_half)((float)ar[mt][s][e] * (float)nr[s][e] * minv);
        }
    }

    /* ---- 5. the stream: group g is read from its slot while the MFMAs of group g-1 run; the slot of g-1 is
     *         refilled behind those MFMAs, which could not issue before its reads had returned ---- */
    gd_float4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[mt][j] = (gd_float4){0.f, 0.f, 0.f, 0.f};
    {
        const uint32_t li8 = (uint32_t)li % 8u, half_rows = ((uint32_t)li / 8u) * 1024u;
        const uint32_t rd0 = half_rows + (li8 * 8u + ((uint32_t)lg ^ li8)) * 16u;
        const uint32_t rd1 = half_rows + (li8 * 8u + ((4u + (uint32_t)lg) ^ li8)) * 16u;
        const unsigned char *ring = &s_mem[0] + (size_t)wave * (RING * 2048);
        gd_half8 f0 = zero8, f1 = zero8, pf0 = zero8, pf1 = zero8;
#pragma unroll
        for (int g = 0; g <= NGMAX; ++g) {
            if (g < NGMAX && g < ng) {
                /* loads return in order: group g has landed once only the groups requested after it are outstanding.
                 * Requested so far: the first RING, plus one behind the MFMAs of every group up to g - 2. */
                const int issued = g < 2 ? RING - 1 : g - 2 + RING;
                const int last = issued < ng - 1 ? issued : ng - 1;
                gd_wide_wait_groups(last - g);
                const unsigned char *slot = ring + (g % RING) * 2048;
                f0 = *reinterpret_cast<const gd_half8 *>(slot + rd0);
                f1 = *reinterpret_cast<const gd_half8 *>(slot + rd1);
            }
            if (g >= 1 && g - 1 < ng) {
                const int q = g - 1, pair = q / NT, j = q % NT;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[mt][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar[mt][2 * pair], pf0, acc[mt][j], 0, 0, 0);
                    acc[mt][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar[mt][2 * pair + 1], pf1, acc[mt][j], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (q + RING < NGMAX && q + RING < ng) issue_group(q + RING);
            }
            pf0 = f0;
            pf1 = f1;
        }
    }

    /* ---- 6. sum of the wavefronts through LDS (the ring's memory: every wavefront is done reading it) ---- */
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    float *sm = reinterpret_cast<float *>(&s_mem[0]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < NT; ++j)
            *reinterpret_cast<gd_float4 *>(sm + (((wave * MT + mt) * NT + j) * 64 + lane) * 4) = acc[mt][j];
    __syncthreads();
    auto total = [&](int mt, int j, int rl, int rr) __attribute__((always_inline)) -> float {
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) v += sm[(((wv * MT + mt) * NT + j) * 64 + rl) * 4 + rr];
        return v;
    };
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
        const int idx = (int)threadIdx.x + 512 * i;
        const int jj = idx >> 8, mt = jj / NTO, j = jj % NTO, rl = idx & 63, rr = (idx >> 6) & 3;
        if (jj >= NTO * MT) continue;
        const uint32_t col = n0 + 16u * j + (rl & 15);
        const uint32_t row = m0 + 16u * mt + 4u * (rl >> 4) + rr;
        const float v1 = total(mt, j, rl, rr);
        const float v2 = PAIRED ? total(mt, j + NT / 2, rl, rr) : 0.f;
        if (row >= p.M || col >= p.N) continue;
        gd_half h1, h2 = (gd_half)0.f;
        if (p.epilogue == GD_HIP_EPI_BIAS_F32) {
            h1 = (gd_half)(v1 + (float)pf_b1[i]);
            if (PAIRED) h2 = (gd_half)(v2 + (float)pf_b2[i]);
        } else if (p.epilogue == GD_HIP_EPI_BIAS_F16) {
            h1 = (gd_half)v1 + pf_b1[i];
            if (PAIRED) h2 = (gd_half)v2 + pf_b2[i];
        } else {
            h1 = (gd_half)v1;
            if (PAIRED) h2 = (gd_half)v2;
        }
        if (EPI == GD_WIDE_EPI_PLAIN) {
            if (p.has_residual) h1 = pf_res[i] + h1;
            y[(size_t)row * p.ldy + col] = h1;
        } else if (EPI == GD_WIDE_EPI_SWIGLU) {
            y[(size_t)row * p.ldy + col] = (gd_half)((float)h1 * gd_lin_silu((float)h2));
        } else {
            /* col = (section * heads + head) * head_dim + pair: q is rotated into its own tensor, k rotated and v
             * copied into row cache_pos of the sequence's caches (skipped when that row does not exist) */
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

/*
 * The plain projection (no prologue; bias, optional residual) for outputs so NARROW that 16 columns per workgroup
 * leave compute units without one (N = 2048: 128 workgroups on 256 units): 8 columns per workgroup.  A weight group
 * is still 2 KB in two instructions of 8 rows x 128 bytes, but both cover the same 8 weight rows, at consecutive
 * 64-wide pieces of K; the matrix instruction takes weight row l % 8 in lanes l % 16 = 0..7 and again in 8..15, so
 * its output columns 8..15 repeat 0..7 and are dropped (the matrix cores have time to spare: the kernel is bound by
 * the weight stream).  One row tile of 16 per workgroup (blockIdx.y walks further ones), a wavefront's K range is
 * at most QMAX pieces of 128.  Host guarantees: K % 128 == 0, ceil(K / 128 / 8) <= QMAX, N % 8 == 0, byte offsets
 * below 2^31, 16-byte aligned rows.
 */
template <int QMAX, int RING>
__global__ void __launch_bounds__(512)
gd_linear_wide_half_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w, const gd_half *__restrict__ bias,
                           const gd_half *__restrict__ residual, gd_half *__restrict__ y, gd_hip_linear_params p,
                           uint32_t n_tiles)
{
    constexpr int WAVES = 8;
    constexpr int SMAX = 4 * QMAX; /* K steps of 32 per wavefront */
    static_assert(RING >= 2 && RING <= 8, "ring depth");
    constexpr int RING_BYTES = WAVES * RING * 2048, SUM_BYTES = WAVES * 1024;
    __shared__ __align__(16) unsigned char s_mem[RING_BYTES > SUM_BYTES ? RING_BYTES : SUM_BYTES];

    asm volatile("" ::"s"(x), "s"(w), "s"(bias), "s"(residual), "s"(y), "s"(p.M), "s"(p.N), "s"(p.K), "s"(p.ldx),
                 "s"(p.ldw), "s"(p.ldy), "s"(p.epilogue), "s"(p.has_residual), "s"(p.ldr), "s"(n_tiles));
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15, lg = lane >> 4;
    uint32_t tile = blockIdx.x;
    if ((n_tiles & 7u) == 0u) tile = (blockIdx.x & 7u) * (n_tiles >> 3) + (blockIdx.x >> 3);
    const uint32_t n0 = tile * 8u, m0 = blockIdx.y * 16u;

    /* what the epilogue will need, requested first: thread t < 128 owns output (row 4*(t/32) + (t/8)%4, column t%8) */
    const uint32_t e_col = n0 + (threadIdx.x & 7u), e_row = m0 + 4u * (threadIdx.x >> 5) + ((threadIdx.x >> 3) & 3u);
    gd_half pf_b = (gd_half)0.f, pf_res = (gd_half)0.f;
    if (threadIdx.x < 128u) {
        if (p.epilogue != GD_HIP_EPI_NONE) pf_b = bias[e_col];
        if (p.has_residual) pf_res = residual[(size_t)min(e_row, p.M - 1u) * p.ldr + e_col];
    }

    /* the wavefront's K range in pieces of 128: the first kq % 8 wavefronts take one piece more */
    const uint32_t kq = p.K / 128u, base = kq / WAVES, rem = kq % WAVES;
    const uint32_t q_begin = (uint32_t)wave * base + min((uint32_t)wave, rem);
    const int nq = (int)(base + ((uint32_t)wave < rem ? 1u : 0u)); /* 0..QMAX: groups of this wavefront */
    const unsigned char *wb = reinterpret_cast<const unsigned char *>(w) + (size_t)q_begin * 256u;
    /* (a wavefront without a K range requests the first piece of the row instead of one past its end) */
    const unsigned char *xb = reinterpret_cast<const unsigned char *>(x) + (size_t)(nq > 0 ? q_begin : 0u) * 256u;
    const gd_half8 zero8 = (gd_half8)(gd_half)0.f;

    /* lane's 16 bytes of an instruction: weight row n0 + lane/8, chunk (lane%8 ^ lane/8) of the 128-byte piece */
    const uint32_t goff = ((n0 + (uint32_t)lane / 8u) * p.ldw + ((((uint32_t)lane % 8u) ^ ((uint32_t)lane / 8u)) * 8u)) * 2u;
    const uint32_t ring_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)s_mem +
                               (uint32_t)wave * (RING * 2048u);
    auto issue_group = [&](int g) __attribute__((always_inline)) {
        const uint32_t slot = ring_base + (uint32_t)(g % RING) * 2048u;
        const uint64_t sp = (uint64_t)(uintptr_t)(wb + (size_t)g * 256u);
        const unsigned char *src = reinterpret_cast<const unsigned char *>(
            ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(sp >> 32)) << 32) |
            (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)sp));
        gd_lin_load_lds16(src, goff, slot);
        gd_lin_load_lds16(src + 128, goff, slot + 1024u);
    };
    /* the activation slice of the wavefront, resident: requested in front of the ring and counted by hand (see
     * gd_wide_request16), so that the first weight group can be multiplied as soon as it lands */
    gd_half8 ar[SMAX];
    {
        const uint32_t mrow = min(m0 + (uint32_t)li, p.M - 1u);
        const uint32_t xoff = (mrow * p.ldx + (uint32_t)lg * 8u) * 2u;
#pragma unroll
        for (int s = 0; s < SMAX; ++s) ar[s] = gd_wide_request16(xb, (s < 4 * nq ? (uint32_t)s * 64u : 0u) + xoff);
    }
    int first_groups = 0;
#pragma unroll
    for (int g = 0; g < RING && g < QMAX; ++g) {
        if (g < nq) {
            issue_group(g);
            first_groups = g + 1;
        }
    }
    gd_wide_wait_groups(first_groups);
#pragma unroll
    for (int s = 0; s < SMAX; ++s) gd_wide_arrived(ar[s]);

    /* the stream: group g is read from its slot while the matrix instructions of group g-1 run; the slot of g-1 is
     * refilled behind them */
    gd_float4 acc = (gd_float4){0.f, 0.f, 0.f, 0.f};
    {
        const uint32_t li8 = (uint32_t)li % 8u;
        const uint32_t rd0 = (li8 * 8u + ((uint32_t)lg ^ li8)) * 16u;
        const uint32_t rd1 = (li8 * 8u + ((4u + (uint32_t)lg) ^ li8)) * 16u;
        const unsigned char *ring = &s_mem[0] + (size_t)wave * (RING * 2048);
        gd_half8 f[4] = {zero8, zero8, zero8, zero8}, pf[4] = {zero8, zero8, zero8, zero8};
#pragma unroll
        for (int g = 0; g <= QMAX; ++g) {
            if (g < QMAX && g < nq) {
                const int issued = g < 2 ? RING - 1 : g - 2 + RING;
                const int last = issued < nq - 1 ? issued : nq - 1;
                gd_wide_wait_groups(last - g);
                const unsigned char *slot = ring + (g % RING) * 2048;
                f[0] = *reinterpret_cast<const gd_half8 *>(slot + rd0);
                f[1] = *reinterpret_cast<const gd_half8 *>(slot + rd1);
                f[2] = *reinterpret_cast<const gd_half8 *>(slot + 1024 + rd0);
                f[3] = *reinterpret_cast<const gd_half8 *>(slot + 1024 + rd1);
            }
            if (g >= 1 && g - 1 < nq) {
                const int q = g - 1;
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar[4 * q + t], pf[t], acc, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (q + RING < QMAX && q + RING < nq) issue_group(q + RING);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) pf[t] = f[t];
        }
    }

    /* sum of the wavefronts through LDS (the ring's memory: every wavefront is done reading it) */
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    float *sm = reinterpret_cast<float *>(&s_mem[0]);
    if (li < 8) *reinterpret_cast<gd_float4 *>(sm + ((wave * 4 + lg) * 8 + li) * 4) = acc;
    __syncthreads();
    if (threadIdx.x < 128u) {
        /* lane (li, lg) of the matrix instruction holds column li, rows 4*lg + 0..3 */
        const int c = threadIdx.x & 7, r = (threadIdx.x >> 3) & 3, g4 = threadIdx.x >> 5;
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) v += sm[((wv * 4 + g4) * 8 + c) * 4 + r];
        if (e_row < p.M) {
            gd_half h;
            if (p.epilogue == GD_HIP_EPI_BIAS_F32) h = (gd_half)(v + (float)pf_b);
            else if (p.epilogue == GD_HIP_EPI_BIAS_F16) h = (gd_half)v + pf_b;
            else h = (gd_half)v;
            if (p.has_residual) h = pf_res + h;
            y[(size_t)e_row * p.ldy + e_col] = h;
        }
    }
}

/*
 * The same projection for matrices with MANY column tiles (rms_norm prologue, K = 512 * PMAX: every wavefront owns
 * exactly PMAX pairs of steps): persistent workgroups.  gridDim.x workgroups share the n_tiles column tiles in
 * contiguous runs; a workgroup loads and normalises its activation slice ONCE and then walks its tiles with the
 * weight ring running on across tile ends (the first groups of the next tile are in flight while the sums of the
 * current one go through LDS and out), so the stream of a compute unit is interrupted neither by a launch nor by a
 * prologue.  Bias values and positions of all its tiles are copied to LDS up front: the steady state issues no
 * register loads, whose waits would also wait for the ring.  At most TPW tiles per workgroup (host).
 */
template <int NT, int MT, int PMAX, int RING, int EPI, int TPW>
__global__ void __launch_bounds__(512)
gd_linear_wide_persistent_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w,
                                 const gd_half *__restrict__ bias, const gd_half *__restrict__ residual,
                                 const gd_half *__restrict__ norm_w, gd_half *__restrict__ y, gd_hip_linear_params p,
                                 uint32_t n_tiles, uint32_t tile_w, gd_hip_rope_epilogue rope)
{
    constexpr int WAVES = 8;
    constexpr int SMAX = 2 * PMAX;
    constexpr int NG = PMAX * NT; /* weight groups per wavefront and tile */
    constexpr bool PAIRED = EPI != GD_WIDE_EPI_PLAIN;
    constexpr int NTO = PAIRED ? NT / 2 : NT;
    constexpr int EPT = (NTO * MT * 256 + 511) / 512;
    constexpr uint32_t COLS = 16u * NT, OUT_COLS = 16u * NTO;
    static_assert(!PAIRED || NT >= 2, "paired epilogues need two column tiles");
    static_assert(RING >= 3 && RING <= 8 && RING <= NG, "ring depth");
    __shared__ __align__(16) unsigned char s_ring[WAVES * RING * 2048];
    __shared__ __align__(16) float s_sum[WAVES * MT * NT * 256];
    __shared__ float s_part[WAVES][MT][16];
    __shared__ gd_half s_bias[2][TPW * OUT_COLS];
    __shared__ int32_t s_pos[2][16 * MT];

    asm volatile("" ::"s"(x), "s"(w), "s"(bias), "s"(residual), "s"(norm_w), "s"(y), "s"(p.M), "s"(p.N), "s"(p.K),
                 "s"(p.ldx), "s"(p.ldw), "s"(p.ldy), "s"(p.epilogue), "s"(p.has_residual), "s"(p.ldr), "s"(p.eps),
                 "s"(p.swiglu_cols), "s"(p.rope_head_dim), "s"(n_tiles));
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15, lg = lane >> 4;
    /* contiguous runs of tiles; workgroup ids are dealt round-robin to the 8 XCDs, so neighbouring runs (which share
     * nothing but DRAM pages) go to different XCDs */
    const uint32_t t_begin = (uint32_t)(((uint64_t)blockIdx.x * n_tiles) / gridDim.x);
    const uint32_t t_end = (uint32_t)(((uint64_t)(blockIdx.x + 1u) * n_tiles) / gridDim.x);
    const int tiles = (int)(t_end - t_begin);
    const uint32_t pair_offset = EPI == GD_WIDE_EPI_ROPE ? p.rope_head_dim / 2u : (EPI == GD_WIDE_EPI_SWIGLU ? p.swiglu_cols : 0u);
    /* Outputs are numbered 0 .. outs-1: output columns (plain), gated columns (swiglu: value row o, gate row
     * swiglu_cols + o) or rotation pairs (rope: pair o of the q, k, v sections lies in weight rows first_row(o) and
     * first_row(o) + D/2).  Tile t covers outputs t * tile_w .. + tile_w - 1.  tile_w is OUT_COLS, or, when that would
     * give fewer tiles than compute units, what the host makes it (ceil(outs / units)), so that every unit streams its
     * share of the weights: a narrow tile uses the first tile_w of its OUT_COLS columns; the others repeat the last
     * used weight row (same cache lines: no traffic) and are not stored.  Narrow rope tiles may straddle heads, so
     * the row of a pair is computed per lane (the host narrows them only when D/2 is a power of two). */
    const uint32_t outs = EPI == GD_WIDE_EPI_ROPE ? p.N / 2u : (EPI == GD_WIDE_EPI_SWIGLU ? p.swiglu_cols : p.N);
    const uint32_t hd2 = EPI == GD_WIDE_EPI_ROPE ? p.rope_head_dim / 2u : 1u;
    const bool hd2_pow2 = (hd2 & (hd2 - 1u)) == 0u;
    const uint32_t hd2_shift = 31u - (uint32_t)__builtin_clz(hd2);
    auto first_row = [&](uint32_t o) __attribute__((always_inline)) -> uint32_t {
        if (EPI != GD_WIDE_EPI_ROPE) return o;
        if (hd2_pow2) return ((o >> hd2_shift) << (hd2_shift + 1u)) | (o & (hd2 - 1u));
        return (o / hd2) * p.rope_head_dim + o % hd2;
    };
    auto tile_o0 = [&](uint32_t tile) __attribute__((always_inline)) -> uint32_t { return tile * tile_w; };
    auto tile_valid = [&](uint32_t o0) __attribute__((always_inline)) -> uint32_t { return min(tile_w, outs - o0); };
    const uint32_t m0 = blockIdx.y * (16u * MT);

    /* ---- the weight stream: group = (tile, pair, column tile), two instructions of 8 rows x 128 bytes ---- */
    const uint32_t p_begin = (uint32_t)wave * PMAX;
    const unsigned char *wb = reinterpret_cast<const unsigned char *>(w) + (size_t)p_begin * 128u;
    uint32_t lrow[2]; /* the lane's weight row within a 16-row tile, and its swizzled 16-byte chunk */
    lrow[0] = (uint32_t)lane / 8u;
    lrow[1] = 8u + (uint32_t)lane / 8u;
    const uint32_t lchunk = ((((uint32_t)lane % 8u) ^ ((uint32_t)lane / 8u)) * 16u);
    const uint32_t ring_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)s_ring +
                               (uint32_t)wave * (RING * 2048u);
    const int total_groups = tiles * NG;
    /* requests group number `gi` of the wavefront's stream (gi = tile_index * NG + pair * NT + j) into ring slot */
    auto issue_group = [&](int gi, int slot) __attribute__((always_inline)) {
        const int ti = gi / NG, g = gi % NG, pair = g / NT, j = g % NT;
        const uint32_t o0 = tile_o0(t_begin + (uint32_t)ti);
        const uint32_t nbase = (PAIRED && j >= NT / 2) ? pair_offset : 0u;
        const uint32_t jc = 16u * (uint32_t)((PAIRED && j >= NT / 2) ? j - NT / 2 : j); /* first column of the column tile */
        const uint32_t last = tile_valid(o0) - 1u;
        /* the base is the same in every lane; said explicitly, it stays in scalar registers inside the tile loop */
        const uint64_t sp = (uint64_t)(uintptr_t)(wb + (size_t)pair * 128u);
        /* (the builtin returns a signed int: through uint32_t, or a low half with its top bit set would sign-extend
         * over the high half) */
        const unsigned char *src = reinterpret_cast<const unsigned char *>(
            ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(sp >> 32)) << 32) |
            (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)sp));
        const uint32_t a = __builtin_amdgcn_readfirstlane(ring_base + (uint32_t)slot * 2048u);
        gd_lin_load_lds16(src, (nbase + first_row(o0 + min(jc + lrow[0], last))) * p.ldw * 2u + lchunk, a);
        gd_lin_load_lds16(src, (nbase + first_row(o0 + min(jc + lrow[1], last))) * p.ldw * 2u + lchunk, a + 1024u);
    };
    /* ---- requested in front of the ring and counted by hand (gd_wide_request16): the bias values and positions of
     *      all tiles of this workgroup (TPW * OUT_COLS <= 512: at most one column per thread) and the activation
     *      slice with its norm weights.  They are usable while the ring's first groups are still crossing the chip,
     *      so the row sums, their barrier and the scaling pass behind the weight stream, not in front of it ---- */
    static_assert(TPW * OUT_COLS <= 512, "one bias column per thread");
    uint32_t rq_b1 = 0u, rq_b2 = 0u, rq_pos = 0u, rq_cpos = 0u;
    const bool has_col = (int)threadIdx.x < tiles * (int)OUT_COLS;
    const uint32_t b_o0 = tile_o0(t_begin + (has_col ? threadIdx.x / OUT_COLS : 0u));
    const uint32_t b_col = first_row(b_o0 + min(threadIdx.x % OUT_COLS, tile_valid(b_o0) - 1u));
    if (p.epilogue != GD_HIP_EPI_NONE) {
        rq_b1 = gd_wide_request2(bias, b_col * 2u);
        if (PAIRED) rq_b2 = gd_wide_request2(bias, (pair_offset + b_col) * 2u);
    }
    if (EPI == GD_WIDE_EPI_ROPE) {
        const uint32_t row = min(m0 + (threadIdx.x & (16u * MT - 1u)), p.M - 1u);
        rq_pos = gd_wide_request4(rope.rope_pos, row * 4u);
        rq_cpos = gd_wide_request4(rope.cache_pos, row * 4u);
    }
    const unsigned char *xb = reinterpret_cast<const unsigned char *>(x) + (size_t)p_begin * 128u;
    const unsigned char *nb = reinterpret_cast<const unsigned char *>(norm_w) + (size_t)p_begin * 128u;
    gd_half8 ar[MT][SMAX];
    {
        gd_half8 nr[SMAX];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const uint32_t mrow = min(m0 + 16u * mt + (uint32_t)li, p.M - 1u);
            const uint32_t xoff = (mrow * p.ldx + (uint32_t)lg * 8u) * 2u;
#pragma unroll
            for (int s = 0; s < SMAX; ++s) ar[mt][s] = gd_wide_request16(xb, (uint32_t)s * 64u + xoff);
        }
#pragma unroll
        for (int s = 0; s < SMAX; ++s) nr[s] = gd_wide_request16(nb, (uint32_t)s * 64u + (uint32_t)lg * 16u);
    int first_groups = 0;
#pragma unroll
        for (int g = 0; g < RING; ++g) {
            if (g < total_groups) {
                issue_group(g, g);
                first_groups = g + 1;
            }
        }
        gd_wide_wait_groups(first_groups);
        gd_wide_arrived(rq_b1);
        gd_wide_arrived(rq_b2);
        gd_wide_arrived(rq_pos);
        gd_wide_arrived(rq_cpos);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int s = 0; s < SMAX; ++s) gd_wide_arrived(ar[mt][s]);
#pragma unroll
        for (int s = 0; s < SMAX; ++s) gd_wide_arrived(nr[s]);
        if (has_col) {
            s_bias[0][threadIdx.x] = gd_wide_half_of(rq_b1);
            s_bias[1][threadIdx.x] = gd_wide_half_of(rq_b2);
        }
        if (EPI == GD_WIDE_EPI_ROPE && threadIdx.x < 16u * MT) {
            s_pos[0][threadIdx.x] = (int32_t)rq_pos;
            s_pos[1][threadIdx.x] = (int32_t)rq_cpos;
        }
        float ss[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            ss[mt] = 0.f;
#pragma unroll
            for (int s = 0; s < SMAX; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e) ss[mt] = fmaf((float)ar[mt][s][e], (float)ar[mt][s][e], ss[mt]);
            ss[mt] += __shfl_xor(ss[mt], 16, 64);
            ss[mt] += __shfl_xor(ss[mt], 32, 64);
            if (lg == 0) s_part[wave][mt][li] = ss[mt];
        }
        /* LDS writes visible (row sums, bias, positions), then the barrier; the ring loads are not waited for */
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            float tot = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) tot += s_part[wv][mt][li];
            const float minv = rsqrtf(tot / (float)p.K + p.eps);
#pragma unroll
            for (int s = 0; s < SMAX; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    ar[mt][s][e] = (gd_half)((float)ar[mt][s][e] * (float)nr[s][e] * minv);
        }
    }

    const uint32_t li8 = (uint32_t)li % 8u, half_rows = ((uint32_t)li / 8u) * 1024u;
    const uint32_t rd0 = half_rows + (li8 * 8u + ((uint32_t)lg ^ li8)) * 16u;
    const uint32_t rd1 = half_rows + (li8 * 8u + ((4u + (uint32_t)lg) ^ li8)) * 16u;
    const unsigned char *ring = &s_ring[0] + (size_t)wave * (RING * 2048);
    const gd_half8 zero8 = (gd_half8)(gd_half)0.f;
    int gbase = 0; /* stream index of the tile's first group */
    int slot = 0;  /* ring slot of the group read next */
    for (int ti = 0; ti < tiles; ++ti) {
        gd_float4 acc[MT][NT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[mt][j] = (gd_float4){0.f, 0.f, 0.f, 0.f};
        gd_half8 f0 = zero8, f1 = zero8, pf0 = zero8, pf1 = zero8;
        int pslot = 0;
#pragma unroll
        for (int g = 0; g <= NG; ++g) {
            if (g < NG) {
                /* requested so far: the first RING groups of the stream, plus one behind the MFMAs of every group
                 * up to the one before the previous */
                const int gi = gbase + g;
                int issued = gi - 2 + RING;
                if (issued < RING - 1) issued = RING - 1;
                const int last = issued < total_groups - 1 ? issued : total_groups - 1;
                gd_wide_wait_groups(__builtin_amdgcn_readfirstlane(last - gi));
                const unsigned char *sl = ring + __builtin_amdgcn_readfirstlane(slot) * 2048;
                f0 = *reinterpret_cast<const gd_half8 *>(sl + rd0);
                f1 = *reinterpret_cast<const gd_half8 *>(sl + rd1);
            }
            if (g >= 1) {
                const int q = g - 1, pair = q / NT, j = q % NT;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[mt][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar[mt][2 * pair], pf0, acc[mt][j], 0, 0, 0);
                    acc[mt][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar[mt][2 * pair + 1], pf1, acc[mt][j], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                /* the slot just multiplied is free: the group RING further down the stream goes there */
                if (gbase + q + RING < total_groups) issue_group(gbase + q + RING, pslot);
            }
            pf0 = f0;
            pf1 = f1;
            if (g < NG) {
                pslot = slot;
                slot = slot + 1 == RING ? 0 : slot + 1;
            }
        }
        gbase += NG;

        /* sums of the wavefronts through LDS, epilogue; the ring keeps filling meanwhile */
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int j = 0; j < NT; ++j)
                *reinterpret_cast<gd_float4 *>(s_sum + (((wave * MT + mt) * NT + j) * 64 + lane) * 4) = acc[mt][j];
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        const uint32_t o0 = tile_o0(t_begin + (uint32_t)ti);
        const uint32_t valid = tile_valid(o0);
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
            const int idx = (int)threadIdx.x + 512 * i;
            const int jj = idx >> 8, mt = jj / NTO, j = jj % NTO, rl = idx & 63, rr = (idx >> 6) & 3;
            if (jj >= NTO * MT) continue;
            const bool col_used = 16u * (uint32_t)j + (uint32_t)(rl & 15) < valid;
            const uint32_t col = first_row(o0 + 16u * j + (rl & 15));
            const uint32_t lrow_i = 16u * mt + 4u * (rl >> 4) + rr, row = m0 + lrow_i;
            float v1 = 0.f, v2 = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) {
                v1 += s_sum[(((wv * MT + mt) * NT + j) * 64 + rl) * 4 + rr];
                if (PAIRED) v2 += s_sum[(((wv * MT + mt) * NT + j + NT / 2) * 64 + rl) * 4 + rr];
            }
            if (row >= p.M || !col_used) continue;
            const gd_half b1 = s_bias[0][ti * (int)OUT_COLS + 16 * j + (rl & 15)];
            const gd_half b2 = s_bias[1][ti * (int)OUT_COLS + 16 * j + (rl & 15)];
            gd_half h1, h2 = (gd_half)0.f;
            if (p.epilogue == GD_HIP_EPI_BIAS_F32) {
                h1 = (gd_half)(v1 + (float)b1);
                if (PAIRED) h2 = (gd_half)(v2 + (float)b2);
            } else if (p.epilogue == GD_HIP_EPI_BIAS_F16) {
                h1 = (gd_half)v1 + b1;
                if (PAIRED) h2 = (gd_half)v2 + b2;
            } else {
                h1 = (gd_half)v1;
                if (PAIRED) h2 = (gd_half)v2;
            }
            if (EPI == GD_WIDE_EPI_PLAIN) {
                if (p.has_residual) h1 = residual[(size_t)row * p.ldr + col] + h1;
                y[(size_t)row * p.ldy + col] = h1;
            } else if (EPI == GD_WIDE_EPI_SWIGLU) {
                y[(size_t)row * p.ldy + col] = (gd_half)((float)h1 * gd_lin_silu((float)h2));
            } else {
                const uint32_t D = p.rope_head_dim, area = p.rope_heads * D;
                const uint32_t section = col / area, within = col % area, pair = within % D;
                gd_half o1 = h1, o2 = h2;
                if (section < 2u) {
                    float c, sn;
                    gd_rope_cos_sin((float)s_pos[0][lrow_i], pair, p.rope_freq_scale, &c, &sn);
                    gd_rope_rotate((float)h1, (float)h2, c, sn, &o1, &o2);
                }
                if (section == 0u) {
                    gd_half *dst = (gd_half *)rope.q + (size_t)row * area + within;
                    dst[0] = o1;
                    dst[D / 2u] = o2;
                } else {
                    const int32_t cp = s_pos[1][lrow_i];
                    if (cp >= 0 && (uint32_t)cp < p.rope_tmax) {
                        gd_half *dst = (gd_half *)(section == 1u ? rope.k_cache : rope.v_cache) +
                                       ((size_t)row * p.rope_tmax + (size_t)cp) * area + within;
                        dst[0] = o1;
                        dst[D / 2u] = o2;
                    }
                }
            }
        }
        /* the sums have been read: the next tile may overwrite them */
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
}

#endif
