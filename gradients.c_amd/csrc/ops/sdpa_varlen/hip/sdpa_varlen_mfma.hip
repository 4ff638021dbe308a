/*
 * sdpa_varlen forward on the matrix cores (gfx950): packed causal / windowed / prefix attention over
 * cu_seqlens for F16 tensors with head size 64 or 128 (prefill).  Same contract as the scalar kernel in
 * sdpa_varlen.hip (reference src/ops/sdpa_varlen/metal_sdpa_varlen.metal:137-228, mask :30-55).
 *
 * Work split.  A workgroup of 4 wavefronts owns 128 consecutive query rows of one segment and one query
 * head; a wavefront owns 32 of them.  Keys advance in blocks of 64, staged in LDS (K and V, two stages,
 * global -> LDS loads that bypass the registers) and shared by the four wavefronts.
 *
 * Transposed formulation.  Both products are computed transposed so that a query row lives in ONE lane
 * (column l%32 of every v_mfma_f32_32x32x16_f16 result) and its keys / channels in that lane's registers:
 *     S^T = K   Q^T    (A = K rows from LDS, B = Q kept in registers for the whole kernel)
 *     O^T = V^T P^T    (A = V^T gathered by ds_read_b64_tr_b16, B = P^T = the S^T registers, rounded to F16)
 * Row maxima and sums are then in-lane reductions plus one exchange with lane l^32, the rescale of O by
 * exp2(m_old - m_new) is a per-lane scalar, and P never moves between lanes: result register 4a+r of S^T
 * is key 8a + 4*(l/32) + r of a 32-key tile, and eight consecutive registers are exactly the eight k-slots
 * of lane l for one 16-key step of the second product, provided V^T supplies the same keys in the same
 * slots - which the transposing LDS read can do for any choice of rows.
 *
 * Softmax in the exp2 domain: s = (q.k) * scale * log2(e), F32 throughout; probabilities are rounded to F16
 * only as the operand of the second product, the row sum accumulates the unrounded values.  The scaling rides in
 * the multiply-add in front of the exp2, and the running maximum of a row moves (O and the row sum rescaled) only
 * when a block raises it by more than 8 binary orders: the result does not depend on the reference point.
 *
 * LDS layouts (16-byte chunks, CPR = D/8 per row).  K: chunk c of key row r at position c ^ (r & 15)
 * (D = 128) or c ^ ((r >> 1) & 7) (D = 64): the 16 lanes of a fragment read hit 16 different bank groups.
 * V: chunk c of key row r at c ^ ((r & 3) << 2) (D = 128) or c ^ (((r >> 1) & 1) << 2) (D = 64): the four
 * key rows of a transposing read cover all banks.
 */
#include "../../_shared/hip_device.h"

#define GD_VL_NEG_INF (-__builtin_inff())

struct gd_hip_sdpa_varlen_params {
    uint32_t n_rows, batch, hq, hkv, dh;
    uint32_t causal, window, prefix_len, max_seqlen;
    float scale;
    uint32_t kv_tmax; /* 0: k and v are packed like q; otherwise caches [batch, kv_tmax, hkv, dh], token t of
                         segment b in cache row t of sequence b */
};

__device__ __forceinline__ bool gd_vl_allowed(int i, int j, int causal, int window, int prefix_len)
{
    if (causal) {
        if (prefix_len > 0) {
            if (i < prefix_len) {
                if (j >= prefix_len) return false;
            } else if (j > i) {
                return false;
            }
        } else if (j > i) {
            return false;
        }
    }
    if (window > 0) {
        if (prefix_len > 0) {
            if (i >= prefix_len && j >= prefix_len && (i - j) >= window) return false;
        } else if ((i - j) >= window) {
            return false;
        }
    }
    return true;
}

/* 16 bytes per lane from global memory straight into LDS (lane l's data lands at lds_address + 16*l).
 * Assembly, because the compiler would otherwise wait for every outstanding load before each LDS read;
 * the kernel places its own s_waitcnt vmcnt. */
__device__ __forceinline__ void gd_vl_load_lds16(const gd_half *uniform_base, uint32_t lane_byte_offset,
                                                 uint32_t lds_byte_address)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_byte_address), "v"(lane_byte_offset), "s"(uniform_base)
                 : "memory");
}

template <int D>
__global__ void __launch_bounds__(256, 2)
gd_sdpa_varlen_mfma_kernel(const gd_half *__restrict__ q, const gd_half *__restrict__ k, const gd_half *__restrict__ v,
                           const int32_t *__restrict__ cu, gd_half *__restrict__ out, gd_hip_sdpa_varlen_params p)
{
    constexpr uint32_t BQ = 128u, BKEYS = 64u;
    constexpr uint32_t CPR = D / 8u;            /* 16-byte chunks per row */
    constexpr uint32_t RPL = 64u / CPR;         /* key rows per wavefront load */
    constexpr int LOADS = (int)(BKEYS / RPL / 4u); /* wavefront loads per operand, key block and wavefront */
    constexpr uint32_t TILE_CHUNKS = BKEYS * CPR; /* one K or V block */
    constexpr int KSTEPS = D / 16, DTILES = D / 32;
    typedef short gd_short4 __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) unsigned char gd_vl_smem[]; /* [2 stages][K block, V block] */

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lq = lane & 31u, h = lane >> 5;
    const uint32_t hq = blockIdx.x % p.hq, pair = blockIdx.x / p.hq;
    const uint32_t hkv = hq / (p.hq / p.hkv);

    /* (segment, 128-row block) number `pair`: lane t of the wavefront takes segment t of a run of 64 segments (one
     * load of cu per lane instead of a chain of dependent scalar loads, which cost a workgroup of a short prompt as
     * much as its attention), the blocks of the run are summed across the lanes, and the first lane whose running
     * count passes `pair` names the segment */
    if (cu[0] < 0) return;
    uint32_t seen = 0u, b = p.batch;
    int start = 0, end = 0;
    for (uint32_t b0 = 0u; b0 < p.batch; b0 += 64u) {
        const uint32_t bl = b0 + lane;
        int s0 = 0, e0 = 0;
        if (bl < p.batch) {
            s0 = cu[bl];
            e0 = cu[bl + 1u];
        }
        const uint32_t nb = e0 > s0 ? ((uint32_t)(e0 - s0) + BQ - 1u) / BQ : 0u;
        uint32_t incl = nb; /* inclusive sum over the lanes below and this one */
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t up = (uint32_t)__shfl_up((int)incl, off, 64);
            if ((int)lane >= off) incl += up;
        }
        const unsigned long long hit = __builtin_amdgcn_ballot_w64(seen + incl > pair);
        if (hit != 0ull) {
            const int src = __builtin_ctzll(hit);
            b = b0 + (uint32_t)src;
            start = __shfl(s0, src, 64);
            end = __shfl(e0, src, 64);
            seen += (uint32_t)__shfl((int)(incl - nb), src, 64);
            break;
        }
        seen += (uint32_t)__shfl((int)incl, 63, 64);
    }
    if (b == p.batch || end > (int)p.n_rows) return;
    const int T_len = end - start;
    if (p.kv_tmax != 0u && (uint32_t)T_len > p.kv_tmax) return; /* a segment its cache cannot hold: out stays */
    /* first and last row of K and V this workgroup may touch */
    const uint32_t kv_first = p.kv_tmax != 0u ? b * p.kv_tmax : (uint32_t)start;
    const uint32_t kv_last = p.kv_tmax != 0u ? b * p.kv_tmax + (p.kv_tmax - 1u) : p.n_rows - 1u;
    const int i0 = (int)((pair - seen) * BQ);
    const int causal = (int)p.causal, window = (int)p.window, prefix = (int)p.prefix_len;

    /* key blocks this workgroup walks */
    const int i_last = min(i0 + (int)BQ, T_len) - 1;
    int kend = T_len, kbeg = 0;
    if (causal) {
        kend = min(T_len, i_last + 1);
        if (prefix > 0 && i0 < prefix) kend = max(kend, min(T_len, prefix));
    }
    if (window > 0 && prefix == 0) kbeg = max(0, i0 - window + 1) & ~63;

    /* this lane's query row */
    const int wi0 = i0 + (int)wave * 32;          /* first row of the wavefront */
    const int i = wi0 + (int)lq;
    const bool row_live = i < T_len;
    const size_t q_elem = ((size_t)(start + min(i, T_len - 1)) * p.hq + hq) * D;
    gd_half8 qf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        qf[ks] = (gd_half8)(gd_half)0.f;
        if (row_live) qf[ks] = *reinterpret_cast<const gd_half8 *>(q + q_elem + 16 * ks + 8 * h);
    }

    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)gd_vl_smem;
    const gd_half *k_head = k + (size_t)hkv * D, *v_head = v + (size_t)hkv * D;
    const uint32_t row_pitch = p.hkv * D * 2u; /* bytes between consecutive key rows */
    auto issue_block = [&](int jb, uint32_t stage) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < LOADS; ++t) {
            const uint32_t r0 = (wave * (uint32_t)LOADS + (uint32_t)t) * RPL;
            const uint32_t r = r0 + lane / CPR, pos = lane % CPR;
            const uint32_t grow = min(kv_first + (uint32_t)jb + r, kv_last); /* stays inside the tensor */
            const uint32_t ck = pos ^ (D == 128 ? (r & 15u) : ((r >> 1) & 7u));
            const uint32_t cv = pos ^ (D == 128 ? ((r & 3u) << 2) : (((r >> 1) & 1u) << 2));
            const uint32_t dst = lds_base + (stage * 2u * TILE_CHUNKS + r0 * CPR) * 16u;
            gd_vl_load_lds16(k_head, grow * row_pitch + ck * 16u, dst);
            gd_vl_load_lds16(v_head, grow * row_pitch + cv * 16u, dst + TILE_CHUNKS * 16u);
        }
    };

    gd_float16 o[DTILES];
#pragma unroll
    for (int t = 0; t < DTILES; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
    float m = GD_VL_NEG_INF, l = 0.f;
    const float scale2 = p.scale * 1.4426950408889634f;
    const bool plain_causal = causal != 0 && window == 0 && prefix == 0;
    const int jmax = min(i, T_len - 1); /* last visible key of this lane's row under plain causal attention */

    /* transposing read coordinates of this lane: group g = lane/16 -> channel block 16*(g&1), key half g/2 == h;
     * lane q + 4e of a group addresses key row e, channels 4q .. 4q+3 */
    const uint32_t tr_q = lane & 3u, tr_e = (lane >> 2) & 3u, tr_g1 = (lane >> 4) & 1u;

    issue_block(kbeg, 0u);
    uint32_t it = 0u;
    for (int jb = kbeg; jb < kend; jb += (int)BKEYS, ++it) {
        const uint32_t stage = it & 1u;
        __builtin_amdgcn_s_waitcnt(0x0F70); /* vmcnt(0): this wavefront's share of block jb is in LDS */
        __syncthreads();                    /* everyone's share is, and the other stage is no longer read */
        if (jb + (int)BKEYS < kend) issue_block(jb + (int)BKEYS, stage ^ 1u);
        const unsigned char *sK = gd_vl_smem + (size_t)stage * 2u * TILE_CHUNKS * 16u;
        const unsigned char *sV = sK + TILE_CHUNKS * 16u;
        if (jb + (int)BKEYS > T_len) {
            /* last, partial block: rows past the segment hold another segment's values; their probabilities
             * are zero, but 0 * inf would still poison the sum, so clear those V rows */
            const uint32_t first = (uint32_t)(T_len - jb);
            for (uint32_t c = first * CPR + tid; c < TILE_CHUNKS; c += 256u)
                reinterpret_cast<gd_u128 *>(const_cast<unsigned char *>(sV))[c] = gd_u128{0u, 0u, 0u, 0u};
            __syncthreads();
        }
        /* a causal wavefront whose rows all precede the block has nothing to add */
        const bool wave_needs = !causal || jb <= wi0 + 31 || (prefix > 0 && jb < prefix);
        if (!wave_needs) continue;

        /* S^T = K Q^T for the two 32-key tiles */
        gd_float16 st[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int e = 0; e < 16; ++e) st[t][e] = 0.f;
            const uint32_t r = 32u * t + lq;
            const uint32_t swz = D == 128 ? (r & 15u) : ((r >> 1) & 7u);
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                const gd_half8 kf = *reinterpret_cast<const gd_half8 *>(sK + (r * CPR + ((2u * ks + h) ^ swz)) * 16u);
                st[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], st[t], 0, 0, 0);
            }
        }

        /* scale, mask, block maximum.  The scores stay unscaled in their registers: scale2 > 0, so the maximum of the
         * raw values is the raw value of the maximum, and the scaling rides in the multiply-add in front of the exp2. */
        const bool full = jb + (int)BKEYS <= T_len &&
                          (causal ? (prefix == 0 && jb + 63 <= wi0 && (window == 0 || wi0 + 31 - jb < window))
                                  : (window == 0));
        float mraw = GD_VL_NEG_INF;
        if (!full) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int j = jb + 32 * t + 8 * (e >> 2) + 4 * (int)h + (e & 3);
                    /* plain causal attention (no window, no prefix): one comparison against min(i, T_len - 1) */
                    if (plain_causal ? j > jmax : (j >= T_len || !gd_vl_allowed(i, j, causal, window, prefix)))
                        st[t][e] = GD_VL_NEG_INF;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) mraw = fmaxf(mraw, st[t][e]);
        float mloc = mraw * scale2; /* -inf stays -inf */
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
        /* The running maximum is only a reference point: the result does not depend on it as long as nothing
         * overflows.  It moves (and O and the row sum are rescaled) only when some row of the wavefront has found a
         * score more than 8 binary orders above its reference, or has none yet; until then the probabilities of a
         * block may reach 2^8, which F16 holds with its full precision, and 64 multiplications per block are saved. */
        const bool moves = mloc > m + 8.f || (m == GD_VL_NEG_INF && mloc != GD_VL_NEG_INF);
        if (__builtin_amdgcn_ballot_w64(moves) != 0ull) {
            const float mnew = fmaxf(m, mloc);
            const float msafe_new = mnew == GD_VL_NEG_INF ? 0.f : mnew;
            const float corr = __builtin_amdgcn_exp2f(m - msafe_new); /* m = -inf -> 0 */
            l *= corr;
            m = mnew;
#pragma unroll
            for (int t = 0; t < DTILES; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[t][e] *= corr;
        }
        const float msafe = m == GD_VL_NEG_INF ? 0.f : m;
        float psum = 0.f;
        gd_half8 pf[4];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float pe = __builtin_amdgcn_exp2f(fmaf(st[t][e], scale2, -msafe));
                psum += pe;
                pf[2 * t + (e >> 3)][e & 7] = (gd_half)pe;
            }
        }
        l += psum;

        /* O^T += V^T P^T: four 16-key steps, DTILES channel tiles */
#pragma unroll
        for (int ts = 0; ts < 4; ++ts) {
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                const uint32_t chunk = 4u * dt + 2u * tr_g1 + (tr_q >> 1);
                const uint32_t r_lo = 16u * ts + 4u * h + tr_e; /* second read: + 8; both have r & 3 == tr_e */
                const uint32_t swz_lo = D == 128 ? (tr_e << 2) : (((r_lo >> 1) & 1u) << 2);
                const uint32_t swz_hi = D == 128 ? (tr_e << 2) : ((((r_lo + 8u) >> 1) & 1u) << 2);
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

    /* normalise, then through LDS so that rows leave with 16-byte stores */
    l += __shfl_xor(l, 32, 64);
    const bool zero_row = p.max_seqlen > 0u && i >= (int)p.max_seqlen;
    const float inv = (l > 0.f && !zero_row) ? 1.f / l : 0.f;
    __syncthreads(); /* all fragment reads of the last block are done */
    gd_half *sO = reinterpret_cast<gd_half *>(gd_vl_smem) + (size_t)wave * 32u * D;
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
        if (ri < T_len)
            *reinterpret_cast<gd_half8 *>(out + ((size_t)(start + ri) * p.hq + hq) * D + cc * 8u) =
                *reinterpret_cast<const gd_half8 *>(sO + r * D + cc * 8u);
    }
}

/* F16, head size 64 or 128, every row pitch a multiple of 16 bytes, tensors below 4 GiB.  The grid has one
 * workgroup per (128-row block of a segment, query head); blocks past the last segment exit at once. */
extern "C" int gd_hip_launch_sdpa_varlen_mfma(hipStream_t stream, const void *q, const void *k, const void *v,
                                              const int32_t *cu, void *out, uint32_t n_rows, uint32_t batch,
                                              uint32_t hq, uint32_t hkv, uint32_t dh, uint32_t causal, uint32_t window,
                                              uint32_t prefix_len, uint32_t max_seqlen, float scale,
                                              uint32_t kv_tmax)
{
    gd_hip_sdpa_varlen_params p = {n_rows, batch, hq, hkv, dh, causal, window, prefix_len, max_seqlen, scale, kv_tmax};
    const uint64_t pairs = (uint64_t)(n_rows + 127u) / 128u + batch; /* upper bound of sum ceil(len_b / 128) */
    const uint64_t blocks = pairs * hq;
    if (n_rows == 0u || blocks == 0u) return (int)hipSuccess;
    if (blocks > 0x7fffffffull) return (int)hipErrorInvalidValue;
    if (dh == 128u) {
        const size_t lds = 2u * 2u * 64u * 16u * 16u;
        static bool configured = false;
        if (!configured) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(gd_sdpa_varlen_mfma_kernel<128>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            configured = true;
        }
        gd_sdpa_varlen_mfma_kernel<128><<<(unsigned)blocks, 256, lds, stream>>>(
            (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, cu, (gd_half *)out, p);
    } else {
        const size_t lds = 2u * 2u * 64u * 8u * 16u;
        gd_sdpa_varlen_mfma_kernel<64><<<(unsigned)blocks, 256, lds, stream>>>(
            (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, cu, (gd_half *)out, p);
    }
    return (int)hipGetLastError();
}
