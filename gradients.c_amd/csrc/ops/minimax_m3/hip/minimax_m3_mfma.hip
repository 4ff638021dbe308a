/*
 * MiniMax-M3 block picker and block-sparse attention on the matrix cores (gfx950) for the reference's own
 * configuration: F16, head size 64, block size a multiple of 64 (M3 uses 128).  Same contracts as the per-row
 * kernels in minimax_m3.hip (reference metal_minimax_m3_index_topk.metal:20-137,
 * metal_minimax_m3_sparse_attention.metal:36-113); those remain for every other shape.
 *
 * Both kernels use the transposed flash-attention layout of the packed-prefill attention kernel: a workgroup of 4
 * wavefronts owns 128 consecutive query rows of one sequence and one head, a wavefront 32 of them; keys pass
 * through LDS in tiles of 64 (two stages, global -> LDS loads that bypass the registers, K swizzled for
 * conflict-free fragment reads); S^T = K Q^T by v_mfma_f32_32x32x16_f16 puts a query row into ONE lane (column
 * l % 32) with its 32 keys of a tile in that lane's registers, the other 32 in lane l ^ 32.
 *   picker     walks every key tile up to the causal limit of its rows, keeps the running maximum of the current
 *              block per lane, and at the end of a block inserts it into the lane's sorted topk registers
 *              (forced first / last blocks as in the reference).  No V, no softmax: half the flops of dense
 *              attention, bound by the matrix cores.
 *   attention  the rows of a workgroup mostly share their blocks (first, last, and a few scored ones): the union
 *              of their lists is formed in LDS, only tiles of listed blocks are walked, and a row that did not
 *              list the block is masked; a block listed k times weighs k times, as in the reference's loop over
 *              the list.
 */
#include "../../_shared/hip_device.h"

#define GD_M3F_NEG_INF (-__builtin_inff())
#define GD_M3F_MAX_BLOCKS 2048u /* blocks per sequence the union bitmap covers */
#define GD_M3F_MAX_TILES 4096u  /* 128 rows x 16 listed blocks x 2 tiles per block */

struct gd_m3f_params {
    uint32_t n_rows, batch, hq, hkv;
    uint32_t max_seqlen, block, topk, init_blocks, local_blocks;
    float scale;
};

/* 16 bytes per lane from global memory straight into LDS (lane l's data lands at lds_address + 16*l).
 * Assembly, because the compiler would otherwise wait for every outstanding load before each LDS read;
 * the kernel places its own s_waitcnt vmcnt. */
__device__ __forceinline__ void gd_m3_load_lds16(const gd_half *uniform_base, uint32_t lane_byte_offset,
                                                 uint32_t lds_byte_address)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_byte_address), "v"(lane_byte_offset), "s"(uniform_base)
                 : "memory");
}


/* MODE 1: attention over listed blocks; MODE 2: block picker (q has hkv heads, v / out unused).  SLOTS: capacity of
 * the per-row lists kept in registers (topk <= SLOTS). */
template <int MODE, int SLOTS>
__global__ void __launch_bounds__(256, 2)
gd_m3_mfma_kernel(const gd_half *__restrict__ q, const gd_half *__restrict__ k, const gd_half *__restrict__ v,
                  const int32_t *__restrict__ cu, int32_t *__restrict__ topk, gd_half *__restrict__ out,
                  gd_m3f_params p)
{
    constexpr int D = 64;
    constexpr uint32_t BQ = 128u, BKEYS = 64u;
    constexpr uint32_t CPR = D / 8u;            /* 16-byte chunks per row */
    constexpr uint32_t RPL = 64u / CPR;         /* key rows per wavefront load */
    constexpr int LOADS = (int)(BKEYS / RPL / 4u); /* wavefront loads per operand, key tile and wavefront */
    constexpr uint32_t TILE_CHUNKS = BKEYS * CPR; /* one K or V tile */
    constexpr int KSTEPS = D / 16, DTILES = D / 32;
    typedef short gd_short4 __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) unsigned char gd_m3_smem[]; /* [2 stages][K tile, V tile] */
    __shared__ uint32_t s_bits[MODE == 1 ? GD_M3F_MAX_BLOCKS / 32u : 1u];
    __shared__ int32_t s_tiles[MODE == 1 ? GD_M3F_MAX_TILES : 1u];
    __shared__ uint32_t s_ntiles;

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lq = lane & 31u, h = lane >> 5;
    const uint32_t heads = MODE == 2 ? p.hkv : p.hq;
    const uint32_t hq = blockIdx.x % heads, pair = blockIdx.x / heads;
    const uint32_t hkv = MODE == 2 ? hq : hq / (p.hq / p.hkv);

    /* (sequence, 128-row block) number `pair` */
    if (cu[0] < 0) return;
    uint32_t seen = 0u, b = 0u;
    int start = 0, end = 0;
    for (; b < p.batch; ++b) {
        start = cu[b];
        end = cu[b + 1u];
        const uint32_t nb = end > start ? ((uint32_t)(end - start) + BQ - 1u) / BQ : 0u;
        if (pair < seen + nb) break;
        seen += nb;
    }
    if (b == p.batch || end > (int)p.n_rows) return;
    const int T_len = end - start;
    const int i0 = (int)((pair - seen) * BQ);
    if (i0 >= (int)p.max_seqlen) return; /* rows at or beyond max_seqlen are not processed */
    const int block = (int)p.block;

    const int i_last = min(i0 + (int)BQ, T_len) - 1;
    const int kend = min(T_len, i_last + 1); /* causal limit of the workgroup's rows */

    /* this lane's query row */
    const int wi0 = i0 + (int)wave * 32;
    const int i = wi0 + (int)lq;
    const bool row_live = i < T_len;
    const size_t q_elem = ((size_t)(start + min(i, T_len - 1)) * heads + hq) * D;
    gd_half8 qf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        qf[ks] = (gd_half8)(gd_half)0.f;
        if (row_live) qf[ks] = *reinterpret_cast<const gd_half8 *>(q + q_elem + 16 * ks + 8 * h);
    }

    /* attention: this row's list, the union of the workgroup's lists, and the tiles of the union in ascending order */
    int32_t lst[SLOTS];
    if (MODE == 1) {
        const int32_t *mine = topk + ((size_t)hkv * p.n_rows + (size_t)(start + min(i, T_len - 1))) * p.topk;
#pragma unroll
        for (int t = 0; t < SLOTS; ++t) lst[t] = (row_live && t < (int)p.topk) ? mine[t] : -1;
        for (uint32_t w = tid; w < GD_M3F_MAX_BLOCKS / 32u; w += 256u) s_bits[w] = 0u;
        __syncthreads();
        if (h == 0u) {
#pragma unroll
            for (int t = 0; t < SLOTS; ++t) {
                const int32_t blk = lst[t];
                if (blk >= 0 && (uint32_t)blk < GD_M3F_MAX_BLOCKS && blk * block < kend) atomicOr(&s_bits[blk >> 5], 1u << (blk & 31));
            }
        }
        __syncthreads();
        if (tid == 0u) {
            uint32_t n = 0u;
            for (uint32_t w = 0; w < GD_M3F_MAX_BLOCKS / 32u; ++w) {
                uint32_t bits = s_bits[w];
                while (bits != 0u) {
                    const int blk = (int)(w * 32u) + __builtin_ctz(bits);
                    bits &= bits - 1u;
                    for (int jb = blk * block; jb < min((blk + 1) * block, kend) && n < GD_M3F_MAX_TILES; jb += (int)BKEYS)
                        s_tiles[n++] = jb;
                }
            }
            s_ntiles = n;
        }
        __syncthreads();
    }
    const uint32_t ntiles = MODE == 1 ? s_ntiles : (uint32_t)((kend + (int)BKEYS - 1) / (int)BKEYS);
    auto tile_start = [&](uint32_t it) { return MODE == 1 ? s_tiles[it] : (int)(it * BKEYS); };

    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)gd_m3_smem;
    const gd_half *k_head = k + (size_t)hkv * D, *v_head = MODE == 1 ? v + (size_t)hkv * D : k;
    const uint32_t row_pitch = p.hkv * D * 2u; /* bytes between consecutive key rows */
    auto issue_tile = [&](int jb, uint32_t stage) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < LOADS; ++t) {
            const uint32_t r0 = (wave * (uint32_t)LOADS + (uint32_t)t) * RPL;
            const uint32_t r = r0 + lane / CPR, pos = lane % CPR;
            const uint32_t grow = min((uint32_t)(start + jb) + r, p.n_rows - 1u); /* stays inside the tensor */
            const uint32_t ck = pos ^ ((r >> 1) & 7u);
            const uint32_t cv = pos ^ (((r >> 1) & 1u) << 2);
            const uint32_t dst = lds_base + (stage * 2u * TILE_CHUNKS + r0 * CPR) * 16u;
            gd_m3_load_lds16(k_head, grow * row_pitch + ck * 16u, dst);
            if (MODE == 1) gd_m3_load_lds16(v_head, grow * row_pitch + cv * 16u, dst + TILE_CHUNKS * 16u);
        }
    };

    gd_float16 o[DTILES];
#pragma unroll
    for (int t = 0; t < DTILES; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
    float m = GD_M3F_NEG_INF, l = 0.f;
    const float scale2 = p.scale * 1.4426950408889634f;
    const uint32_t tr_q = lane & 3u, tr_e = (lane >> 2) & 3u, tr_g1 = (lane >> 4) & 1u;

    /* picker state: the sorted list of this row, the running maximum of the current block */
    float score[SLOTS];
    int32_t index[SLOTS];
#pragma unroll
    for (int t = 0; t < SLOTS; ++t) {
        score[t] = GD_M3F_NEG_INF;
        index[t] = -1;
    }
    float bmax = GD_M3F_NEG_INF;
    const int valid = row_live ? (i + block) / block : 0;
    const int local_start = max(0, valid - (int)p.local_blocks);

    if (ntiles > 0u) issue_tile(tile_start(0u), 0u);
    for (uint32_t it = 0u; it < ntiles; ++it) {
        const int jb = tile_start(it);
        const uint32_t stage = it & 1u;
        __builtin_amdgcn_s_waitcnt(0x0F70); /* vmcnt(0): this wavefront's share of the tile is in LDS */
        __syncthreads();                    /* everyone's share is, and the other stage is no longer read */
        if (it + 1u < ntiles) issue_tile(tile_start(it + 1u), stage ^ 1u);
        const unsigned char *sK = gd_m3_smem + (size_t)stage * 2u * TILE_CHUNKS * 16u;
        const unsigned char *sV = sK + TILE_CHUNKS * 16u;
        if (MODE == 1 && jb + (int)BKEYS > T_len) {
            /* last, partial tile: rows past the sequence hold another sequence's values; their probabilities are
             * zero, but 0 * inf would still poison the sum, so clear those V rows */
            const uint32_t first = (uint32_t)(T_len - jb);
            for (uint32_t c = first * CPR + tid; c < TILE_CHUNKS; c += 256u)
                reinterpret_cast<gd_u128 *>(const_cast<unsigned char *>(sV))[c] = gd_u128{0u, 0u, 0u, 0u};
            __syncthreads();
        }
        /* a wavefront whose rows all precede the tile has nothing to add */
        if (jb > wi0 + 31) continue;

        /* S^T = K Q^T for the two 32-key halves */
        gd_float16 st[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int e = 0; e < 16; ++e) st[t][e] = 0.f;
            const uint32_t r = 32u * t + lq;
            const uint32_t swz = (r >> 1) & 7u;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                const gd_half8 kf = *reinterpret_cast<const gd_half8 *>(sK + (r * CPR + ((2u * ks + h) ^ swz)) * 16u);
                st[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], st[t], 0, 0, 0);
            }
        }
        const int blk = jb / block;
        if (MODE == 2) {
            /* largest visible score of the tile, folded into the block's; a tile that lies in front of all the
             * wavefront's rows and inside the sequence needs no mask (fmaxf drops a NaN score) */
            float mloc = GD_M3F_NEG_INF;
            if (jb + (int)BKEYS - 1 <= wi0 && jb + (int)BKEYS <= T_len) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int e = 0; e < 16; ++e) mloc = fmaxf(mloc, st[t][e]);
            } else {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int j = jb + 32 * t + 8 * (e >> 2) + 4 * (int)h + (e & 3);
                        if (j <= i && j < T_len) mloc = fmaxf(mloc, st[t][e]);
                    }
                }
            }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
            bmax = fmaxf(bmax, mloc);
            /* the block ends with this tile, or this is the last tile the wavefront's rows can see */
            if ((jb + (int)BKEYS) % block == 0 || jb + (int)BKEYS >= kend || jb + (int)BKEYS > wi0 + 31) {
                float cs = bmax;
                if (blk < (int)p.init_blocks) cs = 1.0e30f;
                if (p.local_blocks > 0u && blk >= local_start) cs = 1.0e29f;
                /* the last slot in use tells whether the block enters the list at all; mostly no lane's does */
                float worst = score[0];
#pragma unroll
                for (int t = 1; t < SLOTS; ++t) worst = t < (int)p.topk ? score[t] : worst;
                const bool enters = blk < valid && cs > worst;
                if (__ballot(enters) != 0ull) {
                    /* sorted insertion without branches: the candidate takes the first slot it beats; what it
                     * pushes out is carried down (it came from further up, so it wins ties) */
                    int32_t ci = blk;
                    bool carrying = false;
#pragma unroll
                    for (int t = 0; t < SLOTS; ++t) {
                        if (t < (int)p.topk) {
                            const bool take = enters && (carrying || cs > score[t]);
                            const float os = score[t];
                            const int32_t oi = index[t];
                            score[t] = take ? cs : os;
                            index[t] = take ? ci : oi;
                            cs = take ? os : cs;
                            ci = take ? oi : ci;
                            carrying = carrying || take;
                        }
                    }
                }
                bmax = GD_M3F_NEG_INF;
            }
            continue;
        }

        /* attention: how often this row lists the block (0: masked) */
        int weight = 0;
#pragma unroll
        for (int t = 0; t < SLOTS; ++t) weight += lst[t] == blk ? 1 : 0;
        float mloc = GD_M3F_NEG_INF;
        if (jb + (int)BKEYS - 1 <= wi0 && jb + (int)BKEYS <= T_len) {
            /* the tile lies in front of all the wavefront's rows: only the row's own list decides */
            const float keep = weight > 0 ? scale2 : 0.f, base = weight > 0 ? 0.f : GD_M3F_NEG_INF;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float s = weight > 0 ? st[t][e] * keep : base;
                    st[t][e] = s;
                    mloc = fmaxf(mloc, s);
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int j = jb + 32 * t + 8 * (e >> 2) + 4 * (int)h + (e & 3);
                    const float s = (weight > 0 && j <= i && j < T_len) ? st[t][e] * scale2 : GD_M3F_NEG_INF;
                    st[t][e] = s;
                    mloc = fmaxf(mloc, s);
                }
            }
        }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
        const float mnew = fmaxf(m, mloc);
        const float msafe = mnew == GD_M3F_NEG_INF ? 0.f : mnew;
        const float corr = __builtin_amdgcn_exp2f(m - msafe); /* m = -inf -> 0 */
        const float wf = (float)weight;
        float psum = 0.f;
        gd_half8 pf[4];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float pe = __builtin_amdgcn_exp2f(st[t][e] - msafe) * wf;
                psum += pe;
                pf[2 * t + (e >> 3)][e & 7] = (gd_half)pe;
            }
        }
        l = l * corr + psum;
        m = mnew;
#pragma unroll
        for (int t = 0; t < DTILES; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[t][e] *= corr;

        /* O^T += V^T P^T: four 16-key steps, DTILES channel tiles */
#pragma unroll
        for (int ts = 0; ts < 4; ++ts) {
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                const uint32_t chunk = 4u * dt + 2u * tr_g1 + (tr_q >> 1);
                const uint32_t r_lo = 16u * ts + 4u * h + tr_e;
                const uint32_t swz_lo = ((r_lo >> 1) & 1u) << 2;
                const uint32_t swz_hi = (((r_lo + 8u) >> 1) & 1u) << 2;
                const gd_short4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) gd_short4 *)(
                    sV + (r_lo * CPR + (chunk ^ swz_lo)) * 16u + (tr_q & 1u) * 8u));
                const gd_short4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) gd_short4 *)(
                    sV + ((r_lo + 8u) * CPR + (chunk ^ swz_hi)) * 16u + (tr_q & 1u) * 8u));
                union { gd_short4 s[2]; gd_half8 hv; } u;
                u.s[0] = lo;
                u.s[1] = hi;
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(u.hv, pf[ts], o[dt], 0, 0, 0);
            }
        }
    }

    if (MODE == 2) {
        if (row_live && h == 0u && i < (int)p.max_seqlen) {
            int32_t *dst = topk + ((size_t)hkv * p.n_rows + (size_t)(start + i)) * p.topk;
#pragma unroll
            for (int t = 0; t < SLOTS; ++t) {
                if (t < (int)p.topk) dst[t] = t < valid ? index[t] : -1;
            }
        }
        return;
    }

    /* normalise, then through LDS so that rows leave with 16-byte stores */
    l += __shfl_xor(l, 32, 64);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    __syncthreads(); /* all fragment reads of the last tile are done */
    gd_half *sO = reinterpret_cast<gd_half *>(gd_m3_smem) + (size_t)wave * 32u * D;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            gd_half4 hv;
#pragma unroll
            for (int r = 0; r < 4; ++r) hv[r] = (gd_half)(o[dt][4 * a + r] * inv);
            *reinterpret_cast<gd_half4 *>(sO + lq * D + 32 * dt + 8 * a + 4 * h) = hv;
        }
    }
    __syncthreads();
    for (uint32_t c = lane; c < 32u * CPR; c += 64u) {
        const uint32_t r = c / CPR, cc = c % CPR;
        const int ri = wi0 + (int)r;
        if (ri < T_len && ri < (int)p.max_seqlen)
            *reinterpret_cast<gd_half8 *>(out + ((size_t)(start + ri) * p.hq + hq) * D + cc * 8u) =
                *reinterpret_cast<const gd_half8 *>(sO + r * D + cc * 8u);
    }
}

/* F16, head size 64, block size a multiple of 64, sequences of at most 2048 blocks, tensors below 4 GiB.  One
 * workgroup per (128-row block of a sequence, head); workgroups past the last sequence exit at once. */
extern "C" int gd_hip_launch_m3_mfma(hipStream_t stream, int picker, const void *q, const void *k, const void *v,
                                     const int32_t *cu, int32_t *topk, void *out, const gd_m3f_params *p)
{
    const uint64_t pairs = (uint64_t)(p->n_rows + 127u) / 128u + p->batch; /* upper bound of sum ceil(len_b / 128) */
    const uint64_t blocks = pairs * (picker ? p->hkv : p->hq);
    const size_t lds = 2u * 2u * 64u * 8u * 16u;
    if (p->n_rows == 0u || blocks == 0u) return (int)hipSuccess;
    if (blocks > 0x7fffffffull) return (int)hipErrorInvalidValue;
#define GD_M3F_GO(SLOTS)                                                                                              \
    do {                                                                                                            \
        if (picker)                                                                                                 \
            gd_m3_mfma_kernel<2, SLOTS><<<(unsigned)blocks, 256, lds, stream>>>((const gd_half *)q, (const gd_half *)k,  \
                                                                                nullptr, cu, topk, nullptr, *p);   \
        else                                                                                                        \
            gd_m3_mfma_kernel<1, SLOTS><<<(unsigned)blocks, 256, lds, stream>>>(                                     \
                (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, cu, topk, (gd_half *)out, *p);          \
    } while (0)
    if (p->topk <= 4u) GD_M3F_GO(4);
    else if (p->topk <= 8u) GD_M3F_GO(8);
    else GD_M3F_GO(16);
#undef GD_M3F_GO
    return (int)hipGetLastError();
}
