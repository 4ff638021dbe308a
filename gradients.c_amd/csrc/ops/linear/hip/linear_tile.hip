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
 * 8 fragments for 16 MFMAs.  The weight fragment is the first MFMA operand, so a lane ends up with four
 * consecutive output columns of one row per register quad (result layout of a 32x32 tile: lane l holds
 * activation row l%32; register 4q+r holds weight row 8q + 4*(l/32) + r).
 *
 * Workgroups are persistent: the grid has one workgroup per compute unit, which walks the output tiles
 * t, t + grid, ...  The operand loads of the next tile are requested before the epilogue of the current
 * one, so their latency and the epilogue's stores overlap.
 *
 * K advances in tiles of 64 through two LDS stages.  Two ways of staging:
 *  - direct (no prologue, whole tiles, K % 64 == 0): global -> LDS loads that bypass the registers, serving
 *    both weight layouts (a [K,N] weight is staged as it lies and transposed by ds_read_b64_tr_b16).  The
 *    instruction stream of a K tile is laid out by hand, see the code.
 *  - through registers (prologues, ragged tiles): the next tile's global loads are issued before the matrix
 *    instructions of the current one and stored to the other stage during its last two steps.
 * LDS has 64 banks of 4 bytes on this chip and serves 16 lanes of a 16-byte read at a time; chunk c (16
 * bytes = 8 k) of row r sits at r*8 + (c ^ swizzle(r)) with swizzles that make any 16 consecutive rows of
 * one k chunk hit all 64 banks (measured: no bank conflict cycles).
 *
 * What bounds it on MI355X: under this load the chip clocks at about 1.55 GHz (counter GRBM_GUI_ACTIVE
 * against the kernel's duration), which puts the matrix peak at about 1.6 PFLOP/s, 64 % of the published
 * 2.5 at 2.4 GHz; the vendor library reaches 1.0-1.5 PFLOP/s on the same shapes.
 *
 * Prologues are applied while the activation tile moves from registers to LDS (rounded to F16 there,
 * like the reference's separate kernels): the swiglu gate reads the second half of the row, the
 * rms_norm scale uses per-row factors computed by the workgroup before the main loop.
 *
 * Epilogue.  In WM passes of 64 rows: accumulators (+ bias, in F32 or after the F16 rounding, by mode) are
 * rounded to F16 and written as 8-byte pieces into a separate 64-row LDS buffer, then read back as 16-byte
 * row pieces and stored, adding the residual in F16.
 *
 * Tile order: workgroup ids are dealt round-robin to the 8 XCDs, so the tile index is first remapped to
 * give each XCD a contiguous run of tiles, and runs walk 8 tile rows by column so that the workgroups
 * resident on one XCD share a few activation and weight panels in its L2.
 */
#include "../../_shared/hip_device.h"
#include "hip_linear_types.h"
#include "../../qkv_split_rope/hip/rope_device.h"
#include <type_traits>

#define GD_TILE_BK 64u

/* Profiling build (make TILE_TIMELINE=1): the first wavefront of every workgroup notes, for its first 32 tiles, the
 * 100 MHz real-time counter at the start of the tile, after the K loop and after the epilogue, and the shader clock
 * ticks the K loop took (their ratio is the clock the chip ran at).  gd_hip_linear_tile_timeline copies the notes of
 * the last launch out; bench.py --probe tile_timeline prints them.  Not part of a normal build. */
#ifdef GD_TILE_TIMELINE
__device__ unsigned long long gd_tile_timeline[256 * 32 * 4];
extern "C" __attribute__((visibility("default"))) int gd_hip_linear_tile_timeline(unsigned long long *host)
{
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(gd_tile_timeline), sizeof(gd_tile_timeline));
}
#define GD_TILE_NOTE(slot, value)                                                                              \
    do {                                                                                                        \
        if (threadIdx.x == 0 && blockIdx.x < 256u && timeline_tile < 32u)                                       \
            gd_tile_timeline[(blockIdx.x * 32u + timeline_tile) * 4u + (slot)] = (value);                       \
    } while (0)
#else
#define GD_TILE_NOTE(slot, value) do { } while (0)
#endif

/* Rotation + cache append epilogue of the packed prefill's qkv projection (ROPE instantiation): the tile kernel
 * writes rotated q rows to q [M, hd], rotated k rows and v rows into cache row cache_row[m] of the K / V caches
 * (row pitch hd), and no [M, 3*hd] intermediate.  cos / sin hold, F32, the angles of row m's position for the half_d
 * pairs of a head (NeoX pairing: column c of a head with column c + half_d) in the layout of the table kernel
 * (gd_rope_table_at in ops/qkv_split_rope/hip/qkv_split_rope.hip). */
struct gd_tile_rope {
    const float *cos, *sin;
    const int32_t *cache_row; /* [M]; negative: the row's k and v go nowhere */
    gd_half *q, *k_cache, *v_cache;
    uint32_t hd;     /* heads * head_dim, a multiple of 256 */
    uint32_t half_d; /* 32 or 64 */
};

__device__ __forceinline__ uint32_t gd_tile_slot(uint32_t row, uint32_t c)
{
    return row * 8u + (c ^ (row & 7u) ^ ((row >> 3) & 7u));
}

__device__ __forceinline__ float gd_tile_silu(float z)
{
    const float e = __expf(-fabsf(z));
    /* 1 / (1 + e) with e in (0, 1]: the reciprocal instruction is good to one unit in the last place of F32, and the
     * product is rounded to F16 afterwards; the division's dozen instructions per element would make the gated
     * epilogue of a tile a quarter longer */
    const float inv = __builtin_amdgcn_rcpf(1.0f + e);
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

template <int WM, int WN, bool W_NK, int PRO, bool ROPE = false>
__global__ void __launch_bounds__(256)
gd_linear_tile_kernel(const gd_half *__restrict__ x, const gd_half *__restrict__ w, const gd_half *__restrict__ bias,
                      const gd_half *__restrict__ residual, const gd_half *__restrict__ norm_w,
                      gd_half *__restrict__ y, gd_hip_linear_params p, uint32_t tiles_m, uint32_t tiles_n,
                      uint32_t vector_store, gd_tile_rope rp)
{
    constexpr uint32_t BM = 64u * WM, BN = 64u * WN;
    constexpr int A_PER = BM / 32;                 /* 16-byte chunks of the activation tile per thread */
    constexpr int B_PER = W_NK ? (int)(BN / 32) : 8; /* weight chunks per thread */
    constexpr uint32_t STAGE_BYTES = 2u * (BM + BN) * 8u * 16u; /* both stages of both operands */
    extern __shared__ __align__(16) unsigned char gd_tile_smem[];
    gd_half8 *sA = reinterpret_cast<gd_half8 *>(gd_tile_smem); /* [2][BM*8] */
    gd_half8 *sB = sA + 2u * BM * 8u;                          /* [2][BN*8] */
    unsigned char *epi = gd_tile_smem + STAGE_BYTES;           /* [64][BN] halfs */
    float *s_inv = reinterpret_cast<float *>(epi); /* [BM] row factors of rms_norm; live during the main loop only */

    const uint32_t total = tiles_m * tiles_n;
    constexpr bool DIRECT = PRO == GD_HIP_PRO_NONE;
    uint32_t m0 = 0u, n0 = 0u; /* origin of the current tile (rows, output columns) */
    /* swiglu epilogue ([N,K] weights of 2H rows, H = p.N output columns).  The BN weight rows of a tile are two
     * wavefront columns of BN/2; each holds HW = BN/4 value rows (n0 + wc*HW ..) in its first half and the matching
     * gate rows (H + n0 + wc*HW ..) in its second half, so a lane finds value and gate of one output column in
     * its own accumulators (tiles j and j + WN/2).  The tile then owns BN/2 output columns. */
    const bool gated = p.swiglu_cols != 0u;
    const uint32_t out_bn = gated ? BN / 2u : BN;
    constexpr uint32_t HW = BN / 4u;
    auto wrow = [&](uint32_t tn0, uint32_t r) __attribute__((always_inline)) {
        const uint32_t wc = r / (BN / 2u), wr = r % (BN / 2u);
        return gated ? (wr < HW ? tn0 + wc * HW + wr : p.swiglu_cols + tn0 + wc * HW + (wr - HW)) : tn0 + r;
    };
    auto wrow_ok = [&](uint32_t tn0, uint32_t r) __attribute__((always_inline)) {
        return (gated ? tn0 + (r / (BN / 2u)) * HW + r % HW : tn0 + r) < p.N;
    };
    auto locate = [&](uint32_t t, uint32_t &tm0, uint32_t &tn0) __attribute__((always_inline)) {
        uint32_t pid = t;
        if ((total & 7u) == 0u) pid = (pid & 7u) * (total >> 3) + (pid >> 3);
        const uint32_t width = 8u * tiles_n;
        const uint32_t first_m = (pid / width) * 8u;
        const uint32_t gsz = min(tiles_m - first_m, 8u);
        tm0 = (first_m + (pid % width) % gsz) * BM;
        tn0 = ((pid % width) / gsz) * out_bn;
    };
    auto direct_ok = [&](uint32_t tm0, uint32_t tn0) __attribute__((always_inline)) {
        return DIRECT && tm0 + BM <= p.M && tn0 + out_bn <= p.N && (p.K % 64u) == 0u && p.K >= 128u;
    };

    uint32_t tid_opaque = threadIdx.x;
    bool prefetched = false; /* the first two K tiles of the current output tile are already requested */
#ifdef GD_TILE_TIMELINE
    uint32_t timeline_tile = 0xffffffffu;
#endif
    for (uint32_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
#ifdef GD_TILE_TIMELINE
    ++timeline_tile;
    const unsigned long long timeline_c0 = __builtin_amdgcn_s_memtime();
    GD_TILE_NOTE(0, __builtin_amdgcn_s_memrealtime());
#endif
    /* Everything below is derived from the thread id anew for every tile: were it loop-invariant, the
     * compiler would hoist some hundred addresses and offsets out of the tile loop and spill them. */
    asm volatile("" : "+v"(tid_opaque));
    const uint32_t tid = tid_opaque, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    locate(tile, m0, n0);

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
                const uint32_t gn = wrow(n0, a_r + 32u * (uint32_t)i);
                if (GUARDED) rb[i] = zero8;
                if (!GUARDED || (kok && wrow_ok(n0, a_r + 32u * (uint32_t)i)))
                    rb[i] = *reinterpret_cast<const gd_half8 *>(w + (size_t)gn * p.ldw + k);
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
     * A wavefront-wide 16-byte load writes 64 consecutive chunks = 8 rows of an LDS tile, whole 128-byte
     * lines per row; lane L fills position L%8 of row L/8 and therefore fetches the global chunk that the
     * swizzle puts there (chunk c of row r sits at r*8 + (c ^ (r & 7) ^ ((r >> 3) & 1))).  Wavefront w
     * stages rows [w*BM/4, (w+1)*BM/4) of the activation tile and the same share of the weight tile.
     *
     * A weight stored [K,N] is staged as it lies: 64 k-rows of BN halfs per stage, a wavefront load
     * filling 1024 / (2*BN) whole rows, with chunk p of k-row r at position p ^ ((r & 3) << 2).  Its
     * fragments come from ds_read_b64_tr_b16, which hands lane i of a 16-lane group element i%4 of the
     * 8-byte words addressed by lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12: lane q + 4e addresses k-row e,
     * columns 4q..4q+3, so lane i receives four consecutive k of column i.  Two such reads (k 0-3, 4-7)
     * make one MFMA operand; the xor spreads the four k-rows of a read over all banks. */
    constexpr uint32_t DBK = 64u, CH = 8u, RW = 8u; /* K tile, chunks per staged row, rows per wavefront load */
    constexpr int A_DIRECT = BM / 4 / RW, B_DIRECT = BN / 4 / RW; /* loads per wavefront, K tile and operand */
    constexpr int PER_TILE = A_DIRECT + B_DIRECT;
    const uint32_t d_lane_chunk = (lane & 7u) ^ ((lane >> 3) & 7u);
    /* rows 8..15 of every 16 (odd wavefront loads) use the swizzle with bit 0 flipped */
    const uint32_t d_off_a = ((lane >> 3) * p.ldx + d_lane_chunk * 8u) * 2u; /* bytes */
    const uint32_t d_off_a1 = ((lane >> 3) * p.ldx + (d_lane_chunk ^ 1u) * 8u) * 2u;
    constexpr uint32_t CPR = BN / 8u, RPL = 64u / CPR; /* [K,N] stage: chunks per k-row, k-rows per wavefront load */
    const uint32_t d_off_b = W_NK ? ((lane >> 3) * p.ldw + d_lane_chunk * 8u) * 2u : ((lane / CPR) * p.ldw) * 2u;
    const uint32_t d_off_b1 = ((lane >> 3) * p.ldw + (d_lane_chunk ^ 1u) * 8u) * 2u;
    gd_half8 *dA = reinterpret_cast<gd_half8 *>(gd_tile_smem); /* [2][BM*8] */
    gd_half8 *dB = dA + 2u * BM * CH;                          /* [2][BN*8] */
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)gd_tile_smem;
    /* item t < A_DIRECT: a wavefront load of the activation tile; A_DIRECT <= t: one of the weight tile */
    auto direct_load_item = [&](uint32_t tm0, uint32_t tn0, uint32_t kt, uint32_t t) __attribute__((always_inline)) {
        const uint32_t stage = kt & 1u;
        if (t < (uint32_t)A_DIRECT) {
            const uint32_t row0 = wave_u * (BM / 4u) + t * RW;
            gd_tile_load_lds16(x + (size_t)(tm0 + row0) * p.ldx + kt * DBK, (t & 1u) ? d_off_a1 : d_off_a,
                               lds_base + (stage * BM * CH + row0 * CH) * 16u);
        } else if (W_NK) {
            const uint32_t tb = t - (uint32_t)A_DIRECT;
            const uint32_t row0 = wave_u * (BN / 4u) + tb * RW;
            gd_tile_load_lds16(w + (size_t)wrow(tn0, row0) * p.ldw + kt * DBK, (tb & 1u) ? d_off_b1 : d_off_b,
                               lds_base + ((2u * BM + stage * BN) * CH + row0 * CH) * 16u);
        } else {
            /* k-rows kr0 .. kr0+RPL-1 of the tile; lane L fills position L%CPR of row kr0 + L/CPR */
            const uint32_t tb = t - (uint32_t)A_DIRECT;
            const uint32_t kr0 = (wave_u * (uint32_t)B_DIRECT + tb) * RPL;
            const uint32_t row = (RPL >= 4u ? 0u : ((tb * RPL) & 3u)) + lane / CPR; /* row & 3 */
            const uint32_t chunk = (lane % CPR) ^ ((row & 3u) << 2);
            gd_tile_load_lds16(w + (size_t)(kt * DBK + kr0) * p.ldw + tn0, d_off_b + chunk * 16u,
                               lds_base + ((2u * BM + stage * BN) * CH + kr0 * CPR) * 16u);
        }
    };
    auto direct_loads = [&](uint32_t tm0, uint32_t tn0, uint32_t kt) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t t = 0; t < (uint32_t)PER_TILE; ++t) direct_load_item(tm0, tn0, kt, t);
    };

    gd_float16 acc[WM][WN];

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
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    };

    constexpr uint32_t STEPS = GD_TILE_BK / 16u;
    /* Register path, one K tile of 4 steps of 16: the fragments of step s+1 are read while the matrix cores
     * work on step s; the next tile's global loads are issued first and stored to the other LDS stage
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

    auto direct_frag_a = [&](const gd_half8 *cA, uint32_t ks, uint32_t i) __attribute__((always_inline)) {
        const uint32_t c = ks * 2u + frag_c;
        const uint32_t r = a_frag_row + i * 32u;
        return cA[r * CH + (c ^ (r & 7u) ^ ((r >> 3) & 1u))];
    };
    auto direct_frag_b = [&](const gd_half8 *cB, uint32_t ks, uint32_t j) __attribute__((always_inline)) {
        if (W_NK) {
            const uint32_t c = ks * 2u + frag_c;
            const uint32_t r = b_frag_row + j * 32u;
            return cB[r * CH + (c ^ (r & 7u) ^ ((r >> 3) & 1u))];
        } else {
            /* lane l = 16g + (q + 4e): k-rows ks*16 + 8*(g/2) + e (+4 for the second read), columns
             * 16*(g%2) + 4q .. +3 of this 32-column block */
            const uint32_t g = lane >> 4, q = lane & 3u, e = (lane >> 2) & 3u;
            const uint32_t col = wn * (WN * 32u) + j * 32u + 16u * (g & 1u) + 4u * q;
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
            return u.h;
        }
    };
    /* Direct path, one wavefront's instruction stream for a K tile (4 steps of 16 matrix instructions),
     * pinned with scheduling barriers: every matrix instruction is followed by at most one fragment read or
     * one global -> LDS load, so the matrix pipe never waits for an LDS round trip.
     *   steps 0-2 of tile kt: their first matrix instructions are followed by the fragment reads of the next
     *   step (into the other register set);
     *   step 3: wait for this wavefront's loads of tile kt+1, barrier (tile kt+1 visible to all, stage kt%2
     *           read by all), then read step 0 of tile kt+1 and, behind the later matrix instructions,
     *           request the first half of tile kt+2 into the freed stage; step 0 of the next tile requests
     *           the second half.
     * TAIL 0: steady state; 1: tile kt+1 exists but not kt+2; 2: last tile. */
    gd_half8 qa[2][WM], qb[2][WN];
    constexpr uint32_t NM = WM * WN, NR = WM + WN, NL = PER_TILE / 2;
    constexpr uint32_t RPM = NM >= 2u * NR ? 1u : (2u * NR + NM - 1u) / NM; /* fragment reads per matrix instruction */
    constexpr uint32_t LPM = NM >= 2u * NL ? 1u : (2u * NL + NM - 1u) / NM; /* loads per matrix instruction */
    auto direct_step = [&](uint32_t kt, auto ks_tag, auto tail_tag) __attribute__((always_inline)) {
        constexpr uint32_t KS = decltype(ks_tag)::value;
        constexpr int TAIL = decltype(tail_tag)::value;
        constexpr uint32_t CUR = KS & 1u, NXT = CUR ^ 1u;
        constexpr bool READS = KS < 3u || TAIL < 2;
        constexpr bool LOADS = (KS == 3u && TAIL == 0) || (KS == 0u && TAIL < 2);
        const uint32_t rstage = KS < 3u ? (kt & 1u) : ((kt + 1u) & 1u);
        const gd_half8 *cA = dA + rstage * BM * CH, *cB = dB + rstage * BN * CH;
        const uint32_t rks = KS < 3u ? KS + 1u : 0u;
        const bool loads_on = KS == 3u || kt >= 1u; /* tiles 0 and 1 are requested before the loop */
        if (KS == 3u && TAIL < 2) {
            __builtin_amdgcn_s_waitcnt(0x0070); /* vmcnt(0) lgkmcnt(0) */
            __syncthreads();
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t idx = 0; idx < NM; ++idx) {
            const uint32_t i = idx / WN, j = idx % WN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qb[CUR][j], qa[CUR][i], acc[i][j], 0, 0, 0);
            if (READS) {
#pragma unroll
                for (uint32_t r = min(idx * RPM, NR); r < min((idx + 1u) * RPM, NR); ++r) {
                    /* a0 b0 a1 b1 ...: the order in which the next step consumes them; behind the shorter of the
                     * two lists the rest of the longer one */
                    constexpr uint32_t BOTH = 2u * (WM < WN ? WM : WN);
                    if (r >= BOTH) {
                        if constexpr (WM > WN) qa[NXT][r - BOTH / 2u] = direct_frag_a(cA, rks, r - BOTH / 2u);
                        else qb[NXT][r - BOTH / 2u] = direct_frag_b(cB, rks, r - BOTH / 2u);
                    } else if ((r & 1u) == 0u) qa[NXT][r >> 1] = direct_frag_a(cA, rks, r >> 1);
                    else qb[NXT][r >> 1] = direct_frag_b(cB, rks, r >> 1);
                }
            }
            constexpr uint32_t LI = (NL + LPM - 1u) / LPM; /* matrix instructions that carry loads */
            if (LOADS && loads_on && idx >= NM - LI) {
#pragma unroll
                for (uint32_t t = (idx - (NM - LI)) * LPM; t < min((idx - (NM - LI) + 1u) * LPM, NL); ++t)
                    direct_load_item(m0, n0, KS == 3u ? kt + 2u : kt + 1u, KS == 3u ? t : NL + t);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto k_tile_direct = [&](uint32_t kt, auto tail_tag) __attribute__((always_inline)) {
        direct_step(kt, std::integral_constant<uint32_t, 0>{}, tail_tag);
        direct_step(kt, std::integral_constant<uint32_t, 1>{}, tail_tag);
        direct_step(kt, std::integral_constant<uint32_t, 2>{}, tail_tag);
        direct_step(kt, std::integral_constant<uint32_t, 3>{}, tail_tag);
    };
    using gd_t = std::true_type;
    using gd_f = std::false_type;

    /* 8-byte pieces of the epilogue buffer: piece u of row e sits at e*EU + (u ^ (e & 31)), which spreads the
     * 32 rows that one wavefront store touches over all banks; a 16-byte read-back takes pieces 2v, 2v+1 */
    constexpr uint32_t EU = BN / 4u;
    typedef _Float16 gd_half4 __attribute__((ext_vector_type(4)));
    gd_half4 bq[WN][4]; /* bias of the 4 columns of every register quad, loaded once per tile */
    auto load_bias = [&]() __attribute__((always_inline)) {
        const bool vec = (reinterpret_cast<uintptr_t>(bias) & 7u) == 0u;
#pragma unroll
        for (int j = 0; j < WN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t lc = wn * (WN * 32u) + (uint32_t)j * 32u + 8u * (uint32_t)q + 4u * frag_c;
                const uint32_t gc = wrow(n0, lc); /* the four columns of a quad lie in the same half of a gated tile */
                if (vec && (gc & 3u) == 0u && wrow_ok(n0, lc + 3u)) {
                    bq[j][q] = *reinterpret_cast<const gd_half4 *>(bias + gc);
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        bq[j][q][r] = wrow_ok(n0, lc + (uint32_t)r) ? bias[gc + (uint32_t)r] : (gd_half)0.f;
                }
            }
        }
    };
    /* the four columns of register quad q of accumulator tile a, rounded to F16 with the bias of the mode */
    auto quad_f16 = [&](auto mode_tag, const gd_float16 &a, int j, int q) __attribute__((always_inline)) {
        constexpr uint32_t MODE = decltype(mode_tag)::value;
        gd_half4 h;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float v = a[4 * q + r];
            if (MODE == GD_HIP_EPI_NONE) h[r] = (gd_half)v;
            else if (MODE == GD_HIP_EPI_BIAS_F32) h[r] = (gd_half)(v + (float)bq[j][q][r]);
            else h[r] = (gd_half)v + bq[j][q][r];
        }
        return h;
    };
    auto epilogue_pass = [&](auto pass_tag, auto mode_tag) __attribute__((always_inline)) {
        constexpr int I = decltype(pass_tag)::value;
        const uint32_t e = wm * 32u + frag_row;
#pragma unroll
        for (int j = 0; j < WN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t lc = wn * (WN * 32u) + (uint32_t)j * 32u + 8u * (uint32_t)q + 4u * frag_c;
                *reinterpret_cast<gd_half4 *>(epi + (e * EU + ((lc >> 2) ^ (e & 31u))) * 8u) = quad_f16(mode_tag, acc[I][j], j, q);
            }
        }
        __syncthreads();
        constexpr uint32_t CPRW = BN / 8u; /* 16-byte chunks per row */
        auto read_chunk = [&](uint32_t er, uint32_t v) __attribute__((always_inline)) {
            const uint32_t xr = er & 31u;
            const gd_half8 raw = *reinterpret_cast<const gd_half8 *>(epi + (er * EU + 2u * (v ^ (xr >> 1))) * 8u);
            gd_half8 h = raw;
            if (xr & 1u) {
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    h[t] = raw[4 + t];
                    h[4 + t] = raw[t];
                }
            }
            return h;
        };
        if (gated) {
            /* a value chunk and the gate chunk HW/8 behind it make one output chunk */
#pragma unroll
            for (uint32_t idx0 = 0; idx0 < 32u * CPRW; idx0 += 256u) {
                const uint32_t idx = idx0 + tid;
                const uint32_t er = idx / (CPRW / 2u), v = idx % (CPRW / 2u);
                const uint32_t gr = m0 + (er >> 5) * (WM * 32u) + (uint32_t)I * 32u + (er & 31u), gc = n0 + v * 8u;
                if (gr >= p.M || gc >= p.N) continue;
                /* staged columns: wavefront column wc holds its HW value columns, then their gates */
                const uint32_t cv = (v / (HW / 8u)) * (HW / 4u) + v % (HW / 8u);
                const gd_half8 hv = read_chunk(er, cv), hg = read_chunk(er, cv + HW / 8u);
                gd_half8 h;
#pragma unroll
                for (int t = 0; t < 8; ++t) h[t] = (gd_half)((float)hv[t] * gd_tile_silu((float)hg[t]));
                gd_half *yr = y + (size_t)gr * p.ldy + gc;
                if (vector_store && gc + 8u <= p.N) {
                    *reinterpret_cast<gd_half8 *>(yr) = h;
                } else {
                    for (uint32_t t = 0; t < 8u && gc + t < p.N; ++t) yr[t] = h[t];
                }
            }
        } else {
#pragma unroll
        for (uint32_t idx0 = 0; idx0 < 64u * CPRW; idx0 += 256u) {
            const uint32_t idx = idx0 + tid;
            const uint32_t er = idx / CPRW, v = idx % CPRW;
            const uint32_t gr = m0 + (er >> 5) * (WM * 32u) + (uint32_t)I * 32u + (er & 31u), gc = n0 + v * 8u;
            if (gr >= p.M || gc >= p.N) continue;
            gd_half8 h = read_chunk(er, v);
            gd_half *yr = y + (size_t)gr * p.ldy + gc;
            if (vector_store && gc + 8u <= p.N) {
                if (p.has_residual) {
                    const gd_half8 r = *reinterpret_cast<const gd_half8 *>(residual + (size_t)gr * p.ldr + gc);
#pragma unroll
                    for (int t = 0; t < 8; ++t) h[t] = r[t] + h[t];
                }
                /* long K: the output is not read again soon and would only push operand panels out of L2 */
                if (p.K >= 1024u) __builtin_nontemporal_store(h, reinterpret_cast<gd_half8 *>(yr));
                else *reinterpret_cast<gd_half8 *>(yr) = h;
            } else {
                for (uint32_t t = 0; t < 8u && gc + t < p.N; ++t) {
                    gd_half v1 = h[t];
                    if (p.has_residual) v1 = residual[(size_t)gr * p.ldr + gc + t] + v1;
                    yr[t] = v1;
                }
            }
        }
        }
        if (I + 1 < WM) __syncthreads(); /* the next pass overwrites the buffer; after the last pass the barriers
                                            of the next tile's main loop come first */
    };
    auto epilogue = [&](auto mode_tag) __attribute__((always_inline)) {
        if (decltype(mode_tag)::value != GD_HIP_EPI_NONE) load_bias();
        epilogue_pass(std::integral_constant<int, 0>{}, mode_tag);
        epilogue_pass(std::integral_constant<int, 1>{}, mode_tag);
        if (WM > 2) epilogue_pass(std::integral_constant<int, (WM > 2 ? 2 : 0)>{}, mode_tag);
        if (WM > 3) epilogue_pass(std::integral_constant<int, (WM > 3 ? 3 : 0)>{}, mode_tag);
    };

    /* Epilogue of a whole 256-column tile whose rows can take 16-byte stores: no workgroup barriers.  A wavefront
     * rounds its own 32 x 128 block of a pass, brings the two 8-byte pieces that lanes l and l + 32 hold of one
     * 16-byte chunk into one lane (v_permlane32_swap), writes whole chunks into its own quarter of the buffer and
     * reads them back as row pieces (16 lanes x 16 bytes per row, four rows per instruction; gated tiles, whose
     * wavefront has already multiplied value and gate in registers: 8 lanes per row, eight rows).  LDS operations
     * of one wavefront are carried out in order, so the next pass overwrites the quarter without a barrier.
     * Chunk c of row e sits at e*16 + (c ^ (e & 15)) (gated: e*8 + (c ^ ((e >> 1) & 7))): 16 consecutive rows of
     * one chunk, and the lanes of one read, hit all banks.  The residual rows of a pass are requested before its
     * accumulators are rounded, so that their latency passes behind that work. */
    typedef unsigned gd_uint2v __attribute__((ext_vector_type(2)));
    auto pair_chunk = [&](gd_half4 a, gd_half4 b) __attribute__((always_inline)) {
        union { gd_half4 h; uint32_t u[2]; } ua, ub;
        ua.h = a;
        ub.h = b;
        /* lanes 32-63 of the first operand change places with lanes 0-31 of the second */
        const gd_uint2v s0 = __builtin_amdgcn_permlane32_swap(ua.u[0], ub.u[0], false, false);
        const gd_uint2v s1 = __builtin_amdgcn_permlane32_swap(ua.u[1], ub.u[1], false, false);
        union { uint32_t u[4]; gd_half8 h; } c;
        c.u[0] = s0[0];
        c.u[1] = s1[0];
        c.u[2] = s0[1];
        c.u[3] = s1[1];
        return c.h;
    };
    auto epilogue_own = [&](auto mode_tag) __attribute__((always_inline)) {
        if (decltype(mode_tag)::value != GD_HIP_EPI_NONE) load_bias();
        unsigned char *own = epi + wave * 8192u;
        const uint32_t rr = lane >> 4, v = lane & 15u;
        /* offsets of this lane's piece from the tile's first element; the pass and the row group add a uniform
         * term */
        const gd_half *rtile = residual + ((size_t)m0 * p.ldr + n0);
        gd_half *ytile = y + ((size_t)m0 * p.ldy + n0);
        const uint32_t y_lane = (wm * (WM * 32u) + rr) * p.ldy + wn * (WN * 32u) + v * 8u;
        const uint32_t r_lane = (wm * (WM * 32u) + rr) * p.ldr + wn * (WN * 32u) + v * 8u;
        auto pass = [&](auto pass_tag) __attribute__((always_inline)) {
            constexpr int I = decltype(pass_tag)::value;
            gd_half8 res[8];
            if (p.has_residual) {
#pragma unroll
                for (uint32_t it = 0; it < 8u; ++it)
                    res[it] = *reinterpret_cast<const gd_half8 *>(rtile + ((uint32_t)I * 32u + it * 4u) * p.ldr + r_lane);
            }
#pragma unroll
            for (int j = 0; j < WN; ++j) {
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    const uint32_t c = (uint32_t)j * 4u + 2u * (uint32_t)pr + frag_c;
                    *reinterpret_cast<gd_half8 *>(own + (frag_row * 16u + (c ^ (frag_row & 15u))) * 16u) =
                        pair_chunk(quad_f16(mode_tag, acc[I][j], j, 2 * pr), quad_f16(mode_tag, acc[I][j], j, 2 * pr + 1));
                }
            }
            gd_half8 h[8];
#pragma unroll
            for (uint32_t it = 0; it < 8u; ++it) {
                const uint32_t e = it * 4u + rr;
                h[it] = *reinterpret_cast<const gd_half8 *>(own + (e * 16u + (v ^ (e & 15u))) * 16u);
            }
#pragma unroll
            for (uint32_t it = 0; it < 8u; ++it) {
                if (p.has_residual) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) h[it][t] = res[it][t] + h[it][t];
                }
                *reinterpret_cast<gd_half8 *>(ytile + ((uint32_t)I * 32u + it * 4u) * p.ldy + y_lane) = h[it];
            }
        };
        pass(std::integral_constant<int, 0>{});
        pass(std::integral_constant<int, 1>{});
        if (WM > 2) pass(std::integral_constant<int, (WM > 2 ? 2 : 0)>{});
        if (WM > 3) pass(std::integral_constant<int, (WM > 3 ? 3 : 0)>{});
    };
    auto epilogue_own_gated = [&](auto mode_tag) __attribute__((always_inline)) {
        if (decltype(mode_tag)::value != GD_HIP_EPI_NONE) load_bias();
        unsigned char *own = epi + wave * 8192u;
        const uint32_t rr = lane >> 3, v = lane & 7u;
        gd_half *ytile = y + ((size_t)m0 * p.ldy + n0);
        const uint32_t y_lane = (wm * (WM * 32u) + rr) * p.ldy + wn * HW + v * 8u;
        auto pass = [&](auto pass_tag) __attribute__((always_inline)) {
            constexpr int I = decltype(pass_tag)::value;
#pragma unroll
            for (int j = 0; j < WN / 2; ++j) {
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    gd_half4 o[2];
#pragma unroll
                    for (int s2 = 0; s2 < 2; ++s2) {
                        const gd_half4 hv = quad_f16(mode_tag, acc[I][j], j, 2 * pr + s2);
                        const gd_half4 hg = quad_f16(mode_tag, acc[I][j + WN / 2], j + WN / 2, 2 * pr + s2);
#pragma unroll
                        for (int t = 0; t < 4; ++t) o[s2][t] = (gd_half)((float)hv[t] * gd_tile_silu((float)hg[t]));
                    }
                    const uint32_t c = (uint32_t)j * 4u + 2u * (uint32_t)pr + frag_c;
                    *reinterpret_cast<gd_half8 *>(own + (frag_row * 8u + (c ^ ((frag_row >> 1) & 7u))) * 16u) =
                        pair_chunk(o[0], o[1]);
                }
            }
            gd_half8 h[4];
#pragma unroll
            for (uint32_t it = 0; it < 4u; ++it) {
                const uint32_t e = it * 8u + rr;
                h[it] = *reinterpret_cast<const gd_half8 *>(own + (e * 8u + (v ^ ((e >> 1) & 7u))) * 16u);
            }
#pragma unroll
            for (uint32_t it = 0; it < 4u; ++it)
                *reinterpret_cast<gd_half8 *>(ytile + ((uint32_t)I * 32u + it * 8u) * p.ldy + y_lane) = h[it];
        };
        pass(std::integral_constant<int, 0>{});
        pass(std::integral_constant<int, 1>{});
        if (WM > 2) pass(std::integral_constant<int, (WM > 2 ? 2 : 0)>{});
        if (WM > 3) pass(std::integral_constant<int, (WM > 3 ? 3 : 0)>{});
    };

    /* ROPE instantiation (whole tiles only; the launcher sees to that): the wavefront's 128 columns lie inside q, k
     * or v (hd is a multiple of 256) and hold whole heads, so both columns of a rotation pair (c, c + half_d) are in
     * one lane's accumulators: tiles j and j + half_d / 32.  Rounding points as in the separate operators: the
     * projection is rounded to F16 (with its bias), rotated in F32 with the angles of the row's position, rounded
     * again.  Rotated quads then take the path of epilogue_own; a row piece goes to row m of q or to row
     * cache_row[m] of the K or V cache. */
    auto epilogue_own_rope = [&](auto mode_tag) __attribute__((always_inline)) {
        if (decltype(mode_tag)::value != GD_HIP_EPI_NONE) load_bias();
        unsigned char *own = epi + wave * 8192u;
        const uint32_t rr = lane >> 4, v = lane & 15u;
        const uint32_t col0 = n0 + wn * (WN * 32u);
        const uint32_t region = col0 >= 2u * rp.hd ? 2u : (col0 >= rp.hd ? 1u : 0u); /* q, k, v */
        gd_half *dst = rp.q;
        if (region == 1u) dst = rp.k_cache;
        if (region == 2u) dst = rp.v_cache;
        dst += col0 - region * rp.hd + v * 8u;
        const uint32_t row_w = m0 + wm * (WM * 32u);
        typedef float gd_float4v __attribute__((ext_vector_type(4)));
        /* What a pass needs from memory: the angles of its 32 rows (region q or k) and the destination rows of the
         * lane's 8 row pieces.  Both are requested one pass ahead so that their latency passes behind the pass in
         * front: the angles into the registers the running pass has just used them from, the rows into a second
         * set.
         * table_at: element offset of the lane's first angle of pass I in the angle tables, which are laid out for this read
         * (blocks of 32 rows, groups of 8 pairs, the low and the high 4 pairs of all 32 rows: the 64 lanes of a load
         * read 1 KB of consecutive memory; group g of the block lies 256 elements behind group g - 1); a signed
         * 32-bit number (the launcher keeps the tables below 2^31 elements), so that the loads take the table's base
         * from scalar registers and the constant steps as immediate offsets */
        auto table_at = [&](int I) __attribute__((always_inline)) {
            return (int32_t)(((row_w >> 5) + (uint32_t)I) * (rp.half_d * 32u) + frag_c * 128u + frag_row * 4u);
        };
        auto request_rows = [&](int I, int32_t (&drow)[8]) __attribute__((always_inline)) {
#pragma unroll
            for (uint32_t it = 0; it < 8u; ++it) {
                const uint32_t r = row_w + (uint32_t)I * 32u + it * 4u + rr;
                drow[it] = region == 0u ? (int32_t)r : rp.cache_row[r];
            }
        };
        auto pass = [&](auto pass_tag, auto t_tag, gd_float4v (&cs)[8], gd_float4v (&sn)[8], const int32_t (&drow)[8],
                        int32_t (&drow_next)[8]) __attribute__((always_inline)) {
            constexpr int I = decltype(pass_tag)::value;
            constexpr int T = decltype(t_tag)::value; /* accumulator tiles per half head */
            constexpr bool MORE = I + 1 < WM;
            if (MORE) request_rows(I + 1, drow_next);
            auto stage = [&](int j, int pr, gd_half4 a, gd_half4 b) __attribute__((always_inline)) {
                const uint32_t c = (uint32_t)j * 4u + 2u * (uint32_t)pr + frag_c;
                *reinterpret_cast<gd_half8 *>(own + (frag_row * 16u + (c ^ (frag_row & 15u))) * 16u) = pair_chunk(a, b);
            };
            if (region < 2u) {
                const int32_t tnext = table_at(I + 1);
#pragma unroll
                for (int t = 0; t < T; ++t) {
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr) {
                        gd_half4 olo[WN / (2 * T)][2], ohi[WN / (2 * T)][2];
#pragma unroll
                        for (int s2 = 0; s2 < 2; ++s2) {
                            const int q = 2 * pr + s2;
#pragma unroll
                            for (int g = 0; g < WN / (2 * T); ++g) {
                                const int jlo = g * 2 * T + t, jhi = jlo + T;
                                const gd_half4 lo = quad_f16(mode_tag, acc[I][jlo], jlo, q);
                                const gd_half4 hi = quad_f16(mode_tag, acc[I][jhi], jhi, q);
#pragma unroll
                                for (int r = 0; r < 4; ++r) {
                                    gd_half a, b;
                                    gd_rope_rotate((float)lo[r], (float)hi[r], cs[t * 4 + q][r], sn[t * 4 + q][r], &a, &b);
                                    olo[g][s2][r] = a;
                                    ohi[g][s2][r] = b;
                                }
                            }
                            if (MORE) {
                                cs[t * 4 + q] = *reinterpret_cast<const gd_float4v *>(rp.cos + (tnext + 256 * (t * 4 + q)));
                                sn[t * 4 + q] = *reinterpret_cast<const gd_float4v *>(rp.sin + (tnext + 256 * (t * 4 + q)));
                            }
                        }
#pragma unroll
                        for (int g = 0; g < WN / (2 * T); ++g) {
                            stage(g * 2 * T + t, pr, olo[g][0], olo[g][1]);
                            stage(g * 2 * T + t + T, pr, ohi[g][0], ohi[g][1]);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < WN; ++j)
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr)
                        stage(j, pr, quad_f16(mode_tag, acc[I][j], j, 2 * pr), quad_f16(mode_tag, acc[I][j], j, 2 * pr + 1));
            }
            gd_half8 h[8];
#pragma unroll
            for (uint32_t it = 0; it < 8u; ++it) {
                const uint32_t e = it * 4u + rr;
                h[it] = *reinterpret_cast<const gd_half8 *>(own + (e * 16u + (v ^ (e & 15u))) * 16u);
            }
#pragma unroll
            for (uint32_t it = 0; it < 8u; ++it) {
                if (drow[it] >= 0) *reinterpret_cast<gd_half8 *>(dst + (size_t)(uint32_t)drow[it] * rp.hd) = h[it];
            }
        };
        auto passes = [&](auto t_tag) __attribute__((always_inline)) {
            constexpr int T = decltype(t_tag)::value;
            gd_float4v cs[8], sn[8];
            int32_t even[8], odd[8];
            request_rows(0, even);
            if (region < 2u) {
                const int32_t t0 = table_at(0);
#pragma unroll
                for (int t = 0; t < T * 4; ++t) {
                    cs[t] = *reinterpret_cast<const gd_float4v *>(rp.cos + (t0 + 256 * t));
                    sn[t] = *reinterpret_cast<const gd_float4v *>(rp.sin + (t0 + 256 * t));
                }
            }
            pass(std::integral_constant<int, 0>{}, t_tag, cs, sn, even, odd);
            pass(std::integral_constant<int, 1>{}, t_tag, cs, sn, odd, even);
            pass(std::integral_constant<int, (WM > 2 ? 2 : 0)>{}, t_tag, cs, sn, even, odd);
            pass(std::integral_constant<int, (WM > 2 ? 3 : 0)>{}, t_tag, cs, sn, odd, even);
        };
        if (rp.half_d == 64u) passes(std::integral_constant<int, (WN >= 4 ? 2 : 1)>{});
        else passes(std::integral_constant<int, 1>{});
    };

        /* interior tile: every staged chunk is in range, so the main loop carries no guards */
        const bool interior = m0 + BM <= p.M && n0 + out_bn <= p.N && (p.K % GD_TILE_BK) == 0u;

        if (PRO == GD_HIP_PRO_RMS_NORM) {
            __syncthreads(); /* the previous tile's epilogue has left the buffer that holds the row factors */
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

#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

        if (direct_ok(m0, n0)) {
            const uint32_t dtiles = p.K / 64u; /* >= 2 */
            if (!prefetched) {
                direct_loads(m0, n0, 0u);
                direct_loads(m0, n0, 1u);
            }
            /* at most PER_TILE vector memory operations outstanding: loads complete in order, so K tile 0 has
             * landed whatever else (K tile 1, stores of the previous epilogue) is still on its way */
            __builtin_amdgcn_s_waitcnt(0x0F70 | (PER_TILE & 15) | ((PER_TILE >> 4) << 14));
            __syncthreads();
            {
#pragma unroll
                for (int i = 0; i < WM; ++i) qa[0][i] = direct_frag_a(dA, 0u, (uint32_t)i);
#pragma unroll
                for (int j = 0; j < WN; ++j) qb[0][j] = direct_frag_b(dB, 0u, (uint32_t)j);
            }
            uint32_t kt = 0;
            for (; kt + 2u < dtiles; ++kt) k_tile_direct(kt, std::integral_constant<int, 0>{});
            k_tile_direct(kt, std::integral_constant<int, 1>{});
            k_tile_direct(kt + 1u, std::integral_constant<int, 2>{});
            __syncthreads(); /* every wavefront has read its last fragments: both stages are free */
            /* request the next output tile's first two K tiles now; they land during the epilogue */
            prefetched = false;
            const uint32_t next = tile + gridDim.x;
            if (next < total) {
                uint32_t nm0, nn0;
                locate(next, nm0, nn0);
                if (direct_ok(nm0, nn0)) {
                    direct_loads(nm0, nn0, 0u);
                    direct_loads(nm0, nn0, 1u);
                    prefetched = true;
                }
            }
        } else {
            prefetched = false;
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

#ifdef GD_TILE_TIMELINE
        GD_TILE_NOTE(1, __builtin_amdgcn_s_memrealtime());
        GD_TILE_NOTE(3, __builtin_amdgcn_s_memtime() - timeline_c0);
#endif
        auto finish = [&](auto mode_tag) __attribute__((always_inline)) {
            if constexpr (ROPE) {
                epilogue_own_rope(mode_tag);
            } else if (WM >= 3 && WN == 4 && vector_store && m0 + BM <= p.M && n0 + out_bn <= p.N) {
                if (gated) epilogue_own_gated(mode_tag);
                else epilogue_own(mode_tag);
            } else {
                epilogue(mode_tag);
            }
        };
        if (p.epilogue == GD_HIP_EPI_BIAS_F32) finish(std::integral_constant<uint32_t, GD_HIP_EPI_BIAS_F32>{});
        else if (p.epilogue == GD_HIP_EPI_BIAS_F16) finish(std::integral_constant<uint32_t, GD_HIP_EPI_BIAS_F16>{});
        else finish(std::integral_constant<uint32_t, GD_HIP_EPI_NONE>{});
        GD_TILE_NOTE(2, __builtin_amdgcn_s_memrealtime());
    }
}

template <int WM, int WN, bool W_NK, int PRO>
static int launch_tile_one(hipStream_t stream, const gd_half *x, const gd_half *w, const gd_half *bias,
                           const gd_half *residual, const gd_half *norm_w, gd_half *y, const gd_hip_linear_params &p,
                           uint32_t vector_store, uint32_t workgroups)
{
    constexpr uint32_t BM = 64u * WM, BN = 64u * WN;
    constexpr size_t lds = (size_t)2u * (BM + BN) * 8u * 16u + (size_t)64u * BN * 2u; /* stages + epilogue rows */
    static bool configured = false;
    auto kernel = gd_linear_tile_kernel<WM, WN, W_NK, PRO>;
    if (!configured) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const uint32_t out_bn = p.swiglu_cols != 0u ? BN / 2u : BN; /* output columns per tile */
    const uint32_t tiles_m = (p.M + BM - 1u) / BM, tiles_n = (p.N + out_bn - 1u) / out_bn;
    /* persistent workgroups: at most `workgroups` of them (a multiple of 8 keeps the tile -> XCD relation) */
    const uint32_t grid = tiles_m * tiles_n < workgroups ? tiles_m * tiles_n : workgroups;
    kernel<<<grid, 256, lds, stream>>>(x, w, bias, residual, norm_w, y, p, tiles_m, tiles_n, vector_store,
                                       gd_tile_rope{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0u, 0u});
    return (int)hipGetLastError();
}

template <int WM, int WN>
static int launch_tile(hipStream_t stream, const gd_half *x, const gd_half *w, const gd_half *bias,
                       const gd_half *residual, const gd_half *norm_w, gd_half *y, const gd_hip_linear_params &p,
                       uint32_t vector_store, uint32_t workgroups)
{
#define GD_GO(NK, PRO) return launch_tile_one<WM, WN, NK, PRO>(stream, x, w, bias, residual, norm_w, y, p, vector_store, workgroups)
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
 * norm weight; M >= 1.  big_tiles: use the 256 x 256 tile (one workgroup per compute unit; the 128 x 128 tile
 * fits two). */
extern "C" int gd_hip_launch_linear_tile(hipStream_t stream, const void *x, const void *w, const void *bias,
                                         const void *residual, const void *norm_w, void *y,
                                         const gd_hip_linear_params *params, int big_tiles, int vector_store,
                                         int compute_units)
{
    const gd_hip_linear_params &p = *params;
    const uint32_t units = ((uint32_t)(compute_units > 0 ? compute_units : 256) + 7u) & ~7u;
    const gd_half *xp = (const gd_half *)x, *rp = (const gd_half *)residual;
    gd_half *yp = (gd_half *)y;
    if (big_tiles) {
        /* The persistent workgroups walk whole rounds of 256 x 256 tiles; a last round that fills only part of the
         * compute units costs a full tile time.  When that costs more than it would with small tiles, the rows of
         * the last, partial round are left to a second launch with 128 x 128 tiles (rows are independent; two such
         * workgroups fit a compute unit).  A small tile is priced at 0.35 of a big one (a quarter of the work, less
         * reuse of the staged operands). */
        const uint32_t out_bn = p.swiglu_cols != 0u ? 128u : 256u;
        const uint32_t tiles_m = (p.M + 255u) / 256u, tiles_n = (p.N + out_bn - 1u) / out_bn;
        const uint64_t tiles = (uint64_t)tiles_m * tiles_n, rem = tiles % units;
        const uint32_t head_m = (uint32_t)((tiles - rem) / tiles_n); /* row tiles that fill whole rounds */
        if (rem != 0u && head_m != 0u && head_m < tiles_m) {
            const uint32_t head_rows = head_m * 256u, tail_rows = p.M - head_rows;
            const uint64_t small = (uint64_t)((tail_rows + 127u) / 128u) * ((p.N + out_bn / 2u - 1u) / (out_bn / 2u));
            const double whole = (double)((tiles + units - 1u) / units);
            const double cut = (double)(((uint64_t)head_m * tiles_n + units - 1u) / units) +
                               0.35 * (double)((small + 2u * units - 1u) / (2u * units));
            /* a tail that small tiles would need more than one round for, and that fits one round of 192 x 256
             * tiles (three row tiles per wavefront instead of four): one launch of those; measured on the
             * 2048-column projections of the scaled decoder (5,653 tail rows: 720 small tiles on 512 places, or 248
             * tiles of 192 rows, or 240 when the launch is anchored at the last row, see below) */
            const uint32_t mid_rows = (tail_rows + 191u) / 192u * 192u;
            const uint64_t mid = (uint64_t)(mid_rows / 192u) * tiles_n;
            /* whole tiles only (a ragged row tile would leave the direct staging path and take twice as long as the
             * others of its round): the launch covers the LAST mid_rows rows, so its first rows, fewer than 192,
             * are rows of the head launch computed once more, to the same bits (the same products in the same
             * order, the same epilogue); that needs an output the residual does not alias */
            const bool apart = rp == nullptr || rp + (size_t)p.M * p.ldr <= yp || yp + (size_t)p.M * p.ldy <= rp;
            const bool mid_tiles = p.w_is_nk && p.prologue == GD_HIP_PRO_NONE && p.swiglu_cols == 0u &&
                                   small > 2u * units && mid <= units && mid_rows <= p.M && (p.N % 256u) == 0u &&
                                   vector_store && apart;
            if (mid_tiles || cut + 0.1 < whole) {
                gd_hip_linear_params head = p, tail = p;
                int e;
                head.M = head_rows;
                tail.M = tail_rows;
                e = launch_tile<4, 4>(stream, xp, (const gd_half *)w, (const gd_half *)bias, rp, (const gd_half *)norm_w,
                                      yp, head, (uint32_t)vector_store, units);
                if (e != (int)hipSuccess) return e;
                if (mid_tiles) {
                    const uint32_t first = p.M - mid_rows;
                    tail.M = mid_rows;
                    return launch_tile_one<3, 4, true, GD_HIP_PRO_NONE>(
                        stream, xp + (size_t)first * p.ldx, (const gd_half *)w, (const gd_half *)bias,
                        rp != nullptr ? rp + (size_t)first * p.ldr : nullptr, (const gd_half *)norm_w,
                        yp + (size_t)first * p.ldy, tail, (uint32_t)vector_store, units);
                }
                /* small tiles: whole row tiles as well when the output allows it (anchored at the last row) */
                uint32_t first = head_rows;
                const uint32_t up = (tail_rows + 127u) / 128u * 128u;
                if (apart && up <= p.M) {
                    first = p.M - up;
                    tail.M = up;
                }
                return launch_tile<2, 2>(stream, xp + (size_t)first * p.ldx, (const gd_half *)w, (const gd_half *)bias,
                                         rp != nullptr ? rp + (size_t)first * p.ldr : nullptr, (const gd_half *)norm_w,
                                         yp + (size_t)first * p.ldy, tail, (uint32_t)vector_store, 2u * units);
            }
        }
        return launch_tile<4, 4>(stream, xp, (const gd_half *)w, (const gd_half *)bias, rp, (const gd_half *)norm_w, yp, p,
                                 (uint32_t)vector_store, units);
    }
    return launch_tile<2, 2>(stream, xp, (const gd_half *)w, (const gd_half *)bias, rp, (const gd_half *)norm_w, yp, p,
                             (uint32_t)vector_store, 2u * units);
}

/* The qkv projection of a packed prefill with rotation and cache append in the epilogue (gd_tile_rope): x [M,K],
 * w [3*hd, K], whole 256 x 256 tiles only.  Requires: M % 256 == 0, hd % 256 == 0, K % 64 == 0, K >= 128, 16-byte
 * aligned rows of x, w, q and the caches, half_d 32 or 64 (head size 64 or 128). */
extern "C" int gd_hip_launch_linear_tile_rope(hipStream_t stream, const void *x, const void *w, const void *bias,
                                              const gd_hip_linear_params *params, const float *cos_rows,
                                              const float *sin_rows, const int32_t *cache_row, void *q, void *k_cache,
                                              void *v_cache, uint32_t hd, uint32_t half_d, int compute_units)
{
    const gd_hip_linear_params &p = *params;
    constexpr size_t lds = (size_t)2u * (256u + 256u) * 8u * 16u + (size_t)64u * 256u * 2u;
    static bool configured = false;
    auto kernel = gd_linear_tile_kernel<4, 4, true, GD_HIP_PRO_NONE, true>;
    if (p.M == 0u) return (int)hipSuccess;
    if ((p.M % 256u) != 0u || (hd % 256u) != 0u || p.N != 3u * hd || (p.K % 64u) != 0u || p.K < 128u || !p.w_is_nk ||
        p.prologue != GD_HIP_PRO_NONE || p.has_residual || p.swiglu_cols != 0u || (half_d != 32u && half_d != 64u))
        return (int)hipErrorInvalidValue;
    if (!configured) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const uint32_t units = ((uint32_t)(compute_units > 0 ? compute_units : 256) + 7u) & ~7u;
    const uint32_t tiles_m = p.M / 256u, tiles_n = p.N / 256u;
    const uint32_t grid = tiles_m * tiles_n < units ? tiles_m * tiles_n : units;
    kernel<<<grid, 256, lds, stream>>>((const gd_half *)x, (const gd_half *)w, (const gd_half *)bias, nullptr, nullptr,
                                       nullptr, p, tiles_m, tiles_n, 1u,
                                       gd_tile_rope{cos_rows, sin_rows, cache_row, (gd_half *)q, (gd_half *)k_cache,
                                                    (gd_half *)v_cache, hd, half_d});
    return (int)hipGetLastError();
}

/* Row tiles of 256 that fill whole rounds of `units` workgroups for an [M, N] output in 256-column tiles: the rows
 * the rope form takes; the rest (a partly filled last round, a ragged last row tile) goes through the plain
 * projection and the table-driven rotation kernel. */
extern "C" uint32_t gd_hip_linear_tile_rope_head_rows(uint32_t M, uint32_t N, int compute_units)
{
    const uint32_t units = ((uint32_t)(compute_units > 0 ? compute_units : 256) + 7u) & ~7u;
    const uint32_t tiles_n = (N + 255u) / 256u, whole_m = M / 256u;
    const uint64_t tiles = (uint64_t)whole_m * tiles_n;
    const uint64_t rounds = tiles / units;
    uint32_t head_m = rounds != 0u ? (uint32_t)(rounds * units / tiles_n) : 0u;
    /* a few tiles beyond whole rounds cost less than they would in small tiles only when the remainder is nearly a
     * round itself */
    if (tiles - (uint64_t)head_m * tiles_n >= (uint64_t)units * 3u / 4u) head_m = whole_m;
    return head_m * 256u;
}
