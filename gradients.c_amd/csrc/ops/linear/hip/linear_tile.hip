/*
 * F16 projections with F32 accumulation for many rows (prefill): LDS-tiled MFMA kernel for gfx950.
 *
 * Same contract and rounding points as the weight-streaming kernel in linear.hip (reference GEMMs
 * src/ops/_shared/gemm/metal_gemm_common.h:54-135 and :161-237); this one is for M >= 128 where the
 * work is bound by the matrix cores, not by weight traffic.
 *
 * Tiling.  A workgroup of 4 wavefronts (2 x 2) owns a BM x BN output tile, BM = BN = 256 or 128; a
 * wavefront owns (BM/2) x (BN/2) as WM x WN tiles of v_mfma_f32_32x32x16_f16 (4 x 4 tiles = 256
 * accumulator registers per lane for the 256 tile, one wavefront per SIMD).  Every MFMA fragment
 * (row l%32, 8 consecutive k starting at 8*(l/32)) is one 16-byte LDS read; a 4 x 4 wavefront tile reads
 * 8 fragments for 16 MFMAs.
 *
 * Two ways of staging the operand tiles in LDS:
 *  - direct (no prologue, whole tiles, K % 32 == 0): global -> LDS loads that bypass the registers, K in
 *    tiles of 32 through four LDS stages with three tiles in flight; serves both weight layouts (a [K,N]
 *    weight is staged as it lies and transposed by ds_read_b64_tr_b16).  Described at the code.
 *  - through registers (prologues, ragged tiles): K in tiles of 64, two LDS stages; the next tile's global
 *    loads are issued before the matrix instructions of the current one and stored to the other stage
 *    during its last two steps.  Chunk c of row r sits at r*8 + (c ^ (r & 7) ^ ((r >> 3) & 7)): the first
 *    xor makes the fragment reads of 8 neighbouring rows hit 8 different bank groups, the second does the
 *    same for the transposing store of a [K,N] weight (a thread gathers an 8(k) x 8(n) block with eight
 *    16-byte row loads, transposes it in registers and stores eight k-contiguous chunks).
 *
 * What bounds the direct path on MI355X (8192^3, measured by leaving out one side): matrix instructions
 * plus fragment reads alone 1.55 PFLOP/s, operand staging alone (8.6 GB through L2 -> LDS at about
 * 12-13 TB/s, 90 % L2 hits) 1.5 PFLOP/s-equivalent, both together 1.05 PFLOP/s: the two sides are balanced
 * and share the LDS, so neither hides completely behind the other.
 *
 * Prologues are applied while the activation tile moves from registers to LDS (rounded to F16 there,
 * like the reference's separate kernels): the swiglu gate reads the second half of the row, the
 * rms_norm scale uses per-row factors computed by the workgroup before the main loop.
 *
 * Epilogue.  Accumulators (+ bias, in F32 or after the F16 rounding, by mode) are rounded to F16 into
 * the now idle LDS, then written with 16-byte row-contiguous stores, adding the residual in F16.
 *
 * Workgroup order: ids are dealt round-robin to the 8 XCDs, so the id is first remapped to give
 * each XCD a contiguous run of tiles, and runs walk 8 tile rows by column so that the 32 workgroups
 * resident on one XCD share a few activation and weight panels in its L2.
 *
 * MFMA result layout (32x32 tile): lane l holds column l%32; register 4q+r holds row 8q + 4*(l/32) + r.
 */
#include "../../_shared/hip_device.h"
#include "hip_linear_types.h"
#include <type_traits>

#define GD_TILE_BK 64u

__device__ __forceinline__ uint32_t gd_tile_slot(uint32_t row, uint32_t c)
{
    return row * 8u + (c ^ (row & 7u) ^ ((row >> 3) & 7u));
}

__device__ __forceinline__ float gd_tile_silu(float z)
{
    const float e = __expf(-fabsf(z));
    const float inv = 1.0f / (1.0f + e);
    return z * (z >= 0.0f ? inv : e * inv);
}

/* 16 bytes per lane from global memory straight into LDS: lane l's data lands at lds_base + 16*l.
 * Written as assembly because the compiler, not knowing which LDS stage a load fills, would otherwise
 * wait for ALL outstanding loads before every LDS read; the kernel counts them itself (s_waitcnt vmcnt). */
__device__ __forceinline__ void gd_tile_load_lds16(const gd_half *uniform_base, uint32_t lane_byte_offset,
                                                   uint32_t lds_byte_address)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_byte_address), "v"(lane_byte_offset), "s"(uniform_base)
                 : "memory");
}

template <int WM, int WN, bool W_NK, int PRO>
__global__ void __launch_bounds__(256)
gd_linear_tile_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w, const gd_half *__restrict__ bias,
                      const gd_half *__restrict__ residual, const gd_half *__restrict__ norm_w,
                      gd_half *__restrict__ y, gd_hip_linear_params p, uint32_t tiles_m, uint32_t tiles_n,
                      uint32_t vector_store)
{
    constexpr uint32_t BM = 64u * WM, BN = 64u * WN;
    constexpr int A_PER = BM / 32;                 /* 16-byte chunks of the activation tile per thread */
    constexpr int B_PER = W_NK ? (int)(BN / 32) : 8; /* weight chunks per thread */
    extern __shared__ __align__(16) unsigned char gd_tile_smem[];
    __shared__ float s_inv[PRO == GD_HIP_PRO_RMS_NORM ? BM : 1];
    gd_half8 *sA = reinterpret_cast<gd_half8 *>(gd_tile_smem); /* [2][BM*8] */
    gd_half8 *sB = sA + 2u * BM * 8u;                          /* [2][BN*8] */

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1u;

    /* tile of this workgroup */
    uint32_t pid = blockIdx.x;
    const uint32_t total = tiles_m * tiles_n;
    if ((total & 7u) == 0u) pid = (pid & 7u) * (total >> 3) + (pid >> 3);
    const uint32_t width = 8u * tiles_n;
    const uint32_t first_m = (pid / width) * 8u;
    const uint32_t gsz = min(tiles_m - first_m, 8u);
    const uint32_t tile_m = first_m + (pid % width) % gsz;
    const uint32_t tile_n = (pid % width) / gsz;
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    if (PRO == GD_HIP_PRO_RMS_NORM) {
        for (uint32_t r = wave; r < BM; r += 4u) {
            const uint32_t row = min(m0 + r, p.M - 1u);
            const gd_half *xr = x + (size_t)row * p.ldx;
            float ss = 0.f;
            for (uint32_t k = lane * 8u; k < p.K; k += 512u) {
                const gd_half8 v = *reinterpret_cast<const gd_half8 *>(xr + k);
#pragma unroll
                for (int e = 0; e < 8; ++e) ss = fmaf((float)v[e], (float)v[e], ss);
            }
            ss = gd_wave_sum(ss);
            if (lane == 0u) s_inv[r] = rsqrtf(ss / (float)p.K + p.eps);
        }
        __syncthreads();
    }

    /* staging coordinates */
    const uint32_t a_c = tid & 7u, a_r = tid >> 3; /* activation: chunk a_c of rows a_r + 32*i */
    /* weight [K,N]: thread owns the 8(k) x 8(n) block (kb_j, kb_nc) of the tile */
    const uint32_t kb_per_row = BN / 8u;
    const uint32_t kb_j = tid / kb_per_row, kb_nc = tid % kb_per_row;
    constexpr bool KB_ALL = BN >= 256u; /* every thread owns a block */
    const bool kb_active = W_NK ? false : (tid < BN);

    gd_half8 ra[A_PER], rz[PRO == GD_HIP_PRO_SWIGLU ? A_PER : 1], rb[B_PER], rn;
    const gd_half8 zero8 = (gd_half8)(gd_half)0.f;
    const uint32_t ktiles = (p.K + GD_TILE_BK - 1u) / GD_TILE_BK;
    /* interior tile: every staged chunk is in range, so the main loop carries no guards (one basic
     * block, which lets the scheduler interleave memory operations with the matrix instructions) */
    const bool interior = m0 + BM <= p.M && n0 + BN <= p.N && (p.K % GD_TILE_BK) == 0u;
    const bool interior_direct = m0 + BM <= p.M && n0 + BN <= p.N && (p.K % 32u) == 0u && p.K >= 96u;

    /* ---- staging through registers (any prologue, either weight layout, ragged tiles) ---------------- */
    auto load_tile = [&](uint32_t kt, auto guarded_tag) __attribute__((always_inline)) {
        constexpr bool GUARDED = decltype(guarded_tag)::value;
        const uint32_t k = kt * GD_TILE_BK + a_c * 8u;
        const bool kok = !GUARDED || k < p.K;
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const uint32_t gm = m0 + a_r + 32u * i;
            if (GUARDED) {
                ra[i] = zero8;
                if (PRO == GD_HIP_PRO_SWIGLU) rz[i] = zero8;
            }
            if (!GUARDED || (kok && gm < p.M)) {
                const gd_half *xr = x + (size_t)gm * p.ldx + k;
                ra[i] = *reinterpret_cast<const gd_half8 *>(xr);
                if (PRO == GD_HIP_PRO_SWIGLU) rz[i] = *reinterpret_cast<const gd_half8 *>(xr + p.K);
            }
        }
        if (PRO == GD_HIP_PRO_RMS_NORM) rn = kok ? *reinterpret_cast<const gd_half8 *>(norm_w + k) : zero8;
        if (W_NK) {
#pragma unroll
            for (int i = 0; i < B_PER; ++i) {
                const uint32_t gn = n0 + a_r + 32u * i;
                if (GUARDED) rb[i] = zero8;
                if (!GUARDED || (kok && gn < p.N)) rb[i] = *reinterpret_cast<const gd_half8 *>(w + (size_t)gn * p.ldw + k);
            }
        } else {
            const uint32_t gn = n0 + kb_nc * 8u;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t gk = kt * GD_TILE_BK + kb_j * 8u + i;
                if (GUARDED || !KB_ALL) rb[i] = zero8;
                if ((KB_ALL || kb_active) && (!GUARDED || (gk < p.K && gn < p.N)))
                    rb[i] = *reinterpret_cast<const gd_half8 *>(w + (size_t)gk * p.ldw + gn);
            }
        }
    };
    auto store_a = [&](uint32_t stage, int i) __attribute__((always_inline)) {
        gd_half8 *dA = sA + stage * BM * 8u;
        const uint32_t r = a_r + 32u * i;
        gd_half8 a = ra[i];
        if (PRO == GD_HIP_PRO_SWIGLU) {
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = (gd_half)((float)a[e] * gd_tile_silu((float)rz[i][e]));
        }
        if (PRO == GD_HIP_PRO_RMS_NORM) {
            const float inv = s_inv[r];
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = (gd_half)((float)a[e] * (float)rn[e] * inv);
        }
        dA[gd_tile_slot(r, a_c)] = a;
    };
    auto store_b = [&](uint32_t stage, int i) __attribute__((always_inline)) {
        gd_half8 *dB = sB + stage * BN * 8u;
        if (W_NK) {
            dB[gd_tile_slot(a_r + 32u * i, a_c)] = rb[i];
        } else if (KB_ALL || kb_active) {
            gd_half8 t; /* column i of the 8 x 8 block becomes one k-contiguous chunk */
#pragma unroll
            for (int r = 0; r < 8; ++r) t[r] = rb[r][i];
            dB[gd_tile_slot(kb_nc * 8u + i, kb_j)] = t;
        }
    };
    auto store_tile = [&](uint32_t stage) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < A_PER; ++i) store_a(stage, i);
#pragma unroll
        for (int i = 0; i < B_PER; ++i) store_b(stage, i);
    };

    /* ---- staging straight into LDS (plain activation, interior tiles) -----------------------------
     * Global -> LDS loads that bypass the registers.  What limits this kernel is the round trip of the
     * operand tiles through the vector memory path (about 64 KB per compute unit and 64 k), so this path
     * keeps three K tiles in flight: K advances in tiles of 32 (rows of 4 chunks) through 4 LDS stages.
     * A wavefront-wide 16-byte load writes 64 consecutive chunks = 16 rows of an LDS tile; lane L fills
     * position L%4 of row L/4 and therefore fetches the global chunk that the swizzle puts there
     * (chunk c of row r sits at r*4 + (c ^ ((r >> 2) & 3))).  Wavefront w stages rows
     * [w*BM/4, (w+1)*BM/4) of the activation tile and the same share of the weight tile.
     *
     * A weight stored [K,N] is staged as it lies: 32 k-rows of BN halfs per stage, a wavefront load
     * filling 1024 / (2*BN) whole rows, with chunk p of k-row r at position p ^ ((r & 3) << 2).  Its
     * fragments come from ds_read_b64_tr_b16, which hands lane i of a 16-lane group element i%4 of the
     * 8-byte words addressed by lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12: lane q + 4e addresses k-row e,
     * columns 4q..4q+3, so lane i receives four consecutive k of column i.  Two such reads (k 0-3, 4-7)
     * make one MFMA operand; the xor spreads the four k-rows of a read over all banks. */
    constexpr bool DIRECT = PRO == GD_HIP_PRO_NONE;
    constexpr uint32_t DBK = 32u, DSTAGES = 4u;
    constexpr int A_DIRECT = BM / 64, B_DIRECT = BN / 64; /* loads per wavefront, K tile and operand */
    const uint32_t d_off_a = ((lane >> 2) * p.ldx + ((lane & 3u) ^ ((lane >> 4) & 3u)) * 8u) * 2u; /* bytes */
    constexpr uint32_t CPR = BN / 8u, RPL = 64u / CPR; /* [K,N] stage: chunks per k-row, k-rows per wavefront load */
    const uint32_t d_off_b = W_NK ? ((lane >> 2) * p.ldw + ((lane & 3u) ^ ((lane >> 4) & 3u)) * 8u) * 2u
                                  : ((lane / CPR) * p.ldw) * 2u;
    gd_half8 *dA = reinterpret_cast<gd_half8 *>(gd_tile_smem); /* [4][BM*4] */
    gd_half8 *dB = dA + DSTAGES * BM * 4u;                     /* [4][BN*4] */
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)gd_tile_smem;
    auto direct_loads = [&](uint32_t kt) __attribute__((always_inline)) {
        const uint32_t stage = kt & (DSTAGES - 1u);
#pragma unroll
        for (int t = 0; t < A_DIRECT; ++t) {
            const uint32_t row0 = wave_u * (BM / 4u) + (uint32_t)t * 16u;
            gd_tile_load_lds16(x + (size_t)(m0 + row0) * p.ldx + kt * DBK, d_off_a,
                               lds_base + (stage * BM * 4u + row0 * 4u) * 16u);
        }
#pragma unroll
        for (int t = 0; t < B_DIRECT; ++t) {
            if (W_NK) {
                const uint32_t row0 = wave_u * (BN / 4u) + (uint32_t)t * 16u;
                gd_tile_load_lds16(w + (size_t)(n0 + row0) * p.ldw + kt * DBK, d_off_b,
                                   lds_base + ((DSTAGES * BM + stage * BN) * 4u + row0 * 4u) * 16u);
            } else {
                /* k-rows kr0 .. kr0+RPL-1 of the tile; lane L fills position L%CPR of row kr0 + L/CPR */
                const uint32_t kr0 = (wave_u * (uint32_t)B_DIRECT + (uint32_t)t) * RPL;
                const uint32_t row = (RPL >= 4u ? 0u : (((uint32_t)t * RPL) & 3u)) + lane / CPR; /* row & 3 */
                const uint32_t chunk = (lane % CPR) ^ ((row & 3u) << 2);
                gd_tile_load_lds16(w + (size_t)(kt * DBK + kr0) * p.ldw + n0, d_off_b + chunk * 16u,
                                   lds_base + ((DSTAGES * BM + stage * BN) * 4u + kr0 * CPR) * 16u);
            }
        }
    };

    gd_float16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const uint32_t frag_row = lane & 31u, frag_c = lane >> 5;
    const uint32_t a_frag_row = wm * (WM * 32u) + frag_row, b_frag_row = wn * (WN * 32u) + frag_row;

    auto load_frags = [&](const gd_half8 *cA, const gd_half8 *cB, uint32_t ks, gd_half8 (&fa)[WM], gd_half8 (&fb)[WN])
        __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < WM; ++i) fa[i] = cA[gd_tile_slot(a_frag_row + i * 32u, ks * 2u + frag_c)];
#pragma unroll
        for (int j = 0; j < WN; ++j) fb[j] = cB[gd_tile_slot(b_frag_row + j * 32u, ks * 2u + frag_c)];
    };
    auto multiply = [&](const gd_half8 (&fa)[WM], const gd_half8 (&fb)[WN]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };

    constexpr uint32_t STEPS = GD_TILE_BK / 16u;
    /* One K tile, 4 steps of 16: the fragments of step s+1 are read while the matrix cores work on step s.
     * Register path: the next tile's global loads are issued first and stored to the other LDS stage
     * during the last two steps. */
    auto k_tile_regs = [&](uint32_t kt, auto guarded_tag, auto more_tag) __attribute__((always_inline)) {
        constexpr bool MORE = decltype(more_tag)::value;
        const uint32_t stage = kt & 1u;
        const gd_half8 *cA = sA + stage * BM * 8u, *cB = sB + stage * BN * 8u;
        gd_half8 fa[2][WM], fb[2][WN];
        load_frags(cA, cB, 0u, fa[0], fb[0]);
        if (MORE) load_tile(kt + 1u, guarded_tag);
#pragma unroll
        for (uint32_t ks = 0; ks < STEPS; ++ks) {
            if (ks + 1u < STEPS) load_frags(cA, cB, ks + 1u, fa[(ks + 1u) & 1u], fb[(ks + 1u) & 1u]);
            multiply(fa[ks & 1u], fb[ks & 1u]);
            if (MORE && ks >= STEPS - 2u) {
                const int half = (int)(ks - (STEPS - 2u));
#pragma unroll
                for (int i = half * (A_PER / 2); i < (half + 1) * (A_PER / 2); ++i) store_a(stage ^ 1u, i);
#pragma unroll
                for (int i = half * (B_PER / 2); i < (half + 1) * (B_PER / 2); ++i) store_b(stage ^ 1u, i);
            }
        }
        __syncthreads();
    };
    /* Direct path, K tile kt of 32 (2 steps of 16) in stage kt % 4.  On entry the loads of tiles kt .. kt+2
     * are in flight; the wait leaves the newer ones outstanding, the barrier makes every wavefront's share
     * of tile kt visible and proves that stage (kt+3) % 4, read during tile kt-1, is free again. */
    auto direct_frags = [&](const gd_half8 *cA, const gd_half8 *cB, uint32_t ks, gd_half8 (&fa)[WM], gd_half8 (&fb)[WN])
        __attribute__((always_inline)) {
        const uint32_t c = ks * 2u + frag_c;
#pragma unroll
        for (int i = 0; i < WM; ++i) {
            const uint32_t r = a_frag_row + i * 32u;
            fa[i] = cA[r * 4u + (c ^ ((r >> 2) & 3u))];
        }
#pragma unroll
        for (int j = 0; j < WN; ++j) {
            if (W_NK) {
                const uint32_t r = b_frag_row + j * 32u;
                fb[j] = cB[r * 4u + (c ^ ((r >> 2) & 3u))];
            } else {
                /* lane l = 16g + (q + 4e): k-rows ks*16 + 8*(g/2) + e (+4 for the second read), columns
                 * 16*(g%2) + 4q .. +3 of this 32-column block */
                const uint32_t g = lane >> 4, q = lane & 3u, e = (lane >> 2) & 3u;
                const uint32_t col = wn * (WN * 32u) + (uint32_t)j * 32u + 16u * (g & 1u) + 4u * q;
                const uint32_t krow = ks * 16u + 8u * (g >> 1) + e; /* krow & 3 == e for both reads */
                const uint32_t byte0 = krow * (BN * 2u) + (((col >> 3) ^ (e << 2)) << 4) + (q & 1u) * 8u;
                const unsigned char *base = reinterpret_cast<const unsigned char *>(cB);
                typedef short gd_short4 __attribute__((ext_vector_type(4)));
                const gd_short4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) gd_short4 *)(base + byte0));
                const gd_short4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) gd_short4 *)(base + byte0 + 4u * (BN * 2u)));
                union { gd_short4 s[2]; gd_half8 h; } u;
                u.s[0] = lo;
                u.s[1] = hi;
                fb[j] = u.h;
            }
        }
    };
    auto k_tile_direct = [&](uint32_t kt, auto newer_tag) __attribute__((always_inline)) {
        constexpr int TAG = decltype(newer_tag)::value; /* 2: steady state (requests tile kt+3); 3, 1, 0: tail */
        constexpr int NEWER = TAG == 3 ? 2 : TAG;          /* tiles requested after kt that may stay in flight */
        constexpr int PER_TILE = A_DIRECT + B_DIRECT;
        /* s_waitcnt vmcnt(NEWER * PER_TILE), other counters unconstrained */
        constexpr int VM = NEWER * PER_TILE;
        __builtin_amdgcn_s_waitcnt(0x0F70 | (VM & 15) | ((VM >> 4) << 14));
        __syncthreads();
        if (TAG == 2) direct_loads(kt + 3u);
        const uint32_t stage = kt & (DSTAGES - 1u);
        const gd_half8 *cA = dA + stage * BM * 4u, *cB = dB + stage * BN * 4u;
        gd_half8 fa[2][WM], fb[2][WN];
        direct_frags(cA, cB, 0u, fa[0], fb[0]);
        direct_frags(cA, cB, 1u, fa[1], fb[1]);
        multiply(fa[0], fb[0]);
        multiply(fa[1], fb[1]);
    };
    using gd_t = std::true_type;
    using gd_f = std::false_type;

    if (DIRECT && interior_direct) {
        const uint32_t dtiles = p.K / DBK; /* >= 3 */
        direct_loads(0u);
        direct_loads(1u);
        direct_loads(2u);
        uint32_t kt = 0;
        for (; kt + 3u < dtiles; ++kt) k_tile_direct(kt, std::integral_constant<int, 2>{});
        /* the last three tiles request nothing new; the newer loads are 2, 1, 0 tiles' worth */
        k_tile_direct(kt, std::integral_constant<int, 3>{});
        k_tile_direct(kt + 1u, std::integral_constant<int, 1>{});
        k_tile_direct(kt + 2u, std::integral_constant<int, 0>{});
        __syncthreads(); /* every wavefront has read its fragments before the epilogue reuses the LDS */
    } else {
        load_tile(0u, gd_t{});
        store_tile(0u);
        __syncthreads();
        if (interior) {
            for (uint32_t kt = 0; kt + 1u < ktiles; ++kt) k_tile_regs(kt, gd_f{}, gd_t{});
            k_tile_regs(ktiles - 1u, gd_f{}, gd_f{});
        } else {
            for (uint32_t kt = 0; kt + 1u < ktiles; ++kt) k_tile_regs(kt, gd_t{}, gd_t{});
            k_tile_regs(ktiles - 1u, gd_t{}, gd_f{});
        }
    }

    /* epilogue: bias and F16 rounding in registers, then through LDS for row-contiguous stores */
    gd_half *sC = reinterpret_cast<gd_half *>(gd_tile_smem); /* [BM][BN] halfs = the staging buffers' size */
    auto round_tiles = [&](auto mode_tag) __attribute__((always_inline)) {
        constexpr uint32_t MODE = decltype(mode_tag)::value;
#pragma unroll
        for (int j = 0; j < WN; ++j) {
            const uint32_t lc = b_frag_row + j * 32u;
            const gd_half bh = MODE != GD_HIP_EPI_NONE ? bias[min(n0 + lc, p.N - 1u)] : (gd_half)0.f;
#pragma unroll
            for (int i = 0; i < WM; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t lr = wm * (WM * 32u) + i * 32u + 8u * (e >> 2) + 4u * frag_c + (e & 3);
                    const float v = acc[i][j][e];
                    gd_half h;
                    if (MODE == GD_HIP_EPI_BIAS_F32) h = (gd_half)(v + (float)bh);
                    else if (MODE == GD_HIP_EPI_BIAS_F16) h = (gd_half)v + bh;
                    else h = (gd_half)v;
                    sC[lr * BN + lc] = h;
                }
            }
        }
    };
    if (p.epilogue == GD_HIP_EPI_BIAS_F32) round_tiles(std::integral_constant<uint32_t, GD_HIP_EPI_BIAS_F32>{});
    else if (p.epilogue == GD_HIP_EPI_BIAS_F16) round_tiles(std::integral_constant<uint32_t, GD_HIP_EPI_BIAS_F16>{});
    else round_tiles(std::integral_constant<uint32_t, GD_HIP_EPI_NONE>{});
    __syncthreads();
    constexpr uint32_t CHUNKS = BM * BN / 8u;
    for (uint32_t idx = tid; idx < CHUNKS; idx += 256u) {
        const uint32_t lr = idx / (BN / 8u), lc = (idx % (BN / 8u)) * 8u;
        const uint32_t gr = m0 + lr, gc = n0 + lc;
        if (gr >= p.M || gc >= p.N) continue;
        gd_half8 h = *reinterpret_cast<const gd_half8 *>(sC + lr * BN + lc);
        gd_half *yr = y + (size_t)gr * p.ldy + gc;
        if (vector_store && gc + 8u <= p.N) {
            if (p.has_residual) {
                const gd_half8 r = *reinterpret_cast<const gd_half8 *>(residual + (size_t)gr * p.ldr + gc);
#pragma unroll
                for (int e = 0; e < 8; ++e) h[e] = r[e] + h[e];
            }
            *reinterpret_cast<gd_half8 *>(yr) = h;
        } else {
            for (uint32_t e = 0; e < 8u && gc + e < p.N; ++e) {
                gd_half v = h[e];
                if (p.has_residual) v = residual[(size_t)gr * p.ldr + gc + e] + v;
                yr[e] = v;
            }
        }
    }
}

template <int WM, int WN, bool W_NK, int PRO>
static int launch_tile_one(hipStream_t stream, const gd_half *x, const gd_half *w, const gd_half *bias,
                           const gd_half *residual, const gd_half *norm_w, gd_half *y, const gd_hip_linear_params &p,
                           uint32_t vector_store)
{
    constexpr uint32_t BM = 64u * WM, BN = 64u * WN;
    constexpr size_t lds = (size_t)2u * (BM + BN) * 8u * 16u;
    static_assert(lds >= (size_t)BM * BN * 2u, "the epilogue reuses the staging buffers");
    static bool configured = false;
    auto kernel = gd_linear_tile_kernel<WM, WN, W_NK, PRO>;
    if (!configured) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const uint32_t tiles_m = (p.M + BM - 1u) / BM, tiles_n = (p.N + BN - 1u) / BN;
    kernel<<<tiles_m * tiles_n, 256, lds, stream>>>(x, w, bias, residual, norm_w, y, p, tiles_m, tiles_n, vector_store);
    return (int)hipGetLastError();
}

template <int WM, int WN>
static int launch_tile(hipStream_t stream, const gd_half *x, const gd_half *w, const gd_half *bias,
                       const gd_half *residual, const gd_half *norm_w, gd_half *y, const gd_hip_linear_params &p,
                       uint32_t vector_store)
{
#define GD_GO(NK, PRO) return launch_tile_one<WM, WN, NK, PRO>(stream, x, w, bias, residual, norm_w, y, p, vector_store)
    if (p.w_is_nk) {
        if (p.prologue == GD_HIP_PRO_SWIGLU) GD_GO(true, GD_HIP_PRO_SWIGLU);
        if (p.prologue == GD_HIP_PRO_RMS_NORM) GD_GO(true, GD_HIP_PRO_RMS_NORM);
        GD_GO(true, GD_HIP_PRO_NONE);
    }
    if (p.prologue == GD_HIP_PRO_SWIGLU) GD_GO(false, GD_HIP_PRO_SWIGLU);
    if (p.prologue == GD_HIP_PRO_RMS_NORM) GD_GO(false, GD_HIP_PRO_RMS_NORM);
    GD_GO(false, GD_HIP_PRO_NONE);
#undef GD_GO
}

/* Requires: K % 8 == 0, 16-byte aligned x rows (and gate half), w rows (for [K,N]: N % 8 == 0 too) and
 * norm weight; M >= 1.  big_tiles: use the 256 x 256 tile. */
extern "C" int gd_hip_launch_linear_tile(hipStream_t stream, const void *x, const void *w, const void *bias,
                                         const void *residual, const void *norm_w, void *y,
                                         const gd_hip_linear_params *params, int big_tiles, int vector_store)
{
    const gd_hip_linear_params &p = *params;
    if (big_tiles)
        return launch_tile<4, 4>(stream, (const gd_half *)x, (const gd_half *)w, (const gd_half *)bias,
                                 (const gd_half *)residual, (const gd_half *)norm_w, (gd_half *)y, p, (uint32_t)vector_store);
    return launch_tile<2, 2>(stream, (const gd_half *)x, (const gd_half *)w, (const gd_half *)bias,
                             (const gd_half *)residual, (const gd_half *)norm_w, (gd_half *)y, p, (uint32_t)vector_store);
}
