/*
 * sdpa_decode over a ragged batch, gfx950: the PIECES form of the split-KV kernel (sdpa_decode_split_kernel.h).
 *
 * One workgroup per (row, kv head) lets the longest row decide the time of the launch: at its end a single compute
 * unit streams alone.  Here the visible keys of every row are cut into pieces of params.chunk keys, one workgroup
 * per piece (grid (Hkv, B, params.nsplit); the host never sees lengths, so pieces a row does not have leave at
 * once).  A piece stores its (max, sum, acc) partial with write-through stores and counts itself in at the row's
 * arrival counter; the piece that arrives last merges the row and stores F16.  One launch, nobody waits.  Rows of
 * about one length are not cut at params.chunk: they stay whole (or in params.even_pieces equal parts), which is
 * the one-workgroup-per-row kernel again.
 *
 * Reference semantics: src/ops/sdpa_decode/metal_sdpa_decode.metal:177-281 (per-row positions).
 */
#include "sdpa_decode_split_kernel.h"

template <int D, int G>
static int launch_pieces(hipStream_t stream, const void *q, const void *k, const void *v, const int32_t *pos,
                         void *out, float *ws, const gd_hip_sdpa_decode_params &p)
{
    constexpr int U = G == 1 ? 2 : 4;
    const dim3 grid(p.hkv, p.batch, p.nsplit);
#define GD_GO(NT, PFX)                                                                                     \
    gd_sdpa_decode_split_kernel<D, G, 4, U, NT, PFX, true><<<grid, 256, 0, stream>>>(                       \
        (const gd_half *)q, (const gd_half *)k, (const gd_half *)v, pos, (gd_half *)out, ws, p)
    if (p.prefix_len > 0u) GD_GO(false, true);
    else if (p.nontemporal) GD_GO(true, false);
    else GD_GO(false, false);
#undef GD_GO
    return (int)hipGetLastError();
}

/* Returns hipErrorInvalidValue when (D, G) has no instantiation. */
extern "C" int gd_hip_launch_sdpa_decode_pieces(hipStream_t stream, const void *q, const void *k, const void *v,
                                                const int32_t *pos, void *out, float *ws,
                                                const gd_hip_sdpa_decode_params *params)
{
    const gd_hip_sdpa_decode_params &p = *params;
    const uint32_t g = p.hq / p.hkv;
#define GD_CASE(DD, GG) if (p.dh == DD && g == GG) return launch_pieces<DD, GG>(stream, q, k, v, pos, out, ws, p)
    GD_CASE(64, 1); GD_CASE(64, 2); GD_CASE(64, 3); GD_CASE(64, 4); GD_CASE(64, 6); GD_CASE(64, 8);
    GD_CASE(128, 1); GD_CASE(128, 2); GD_CASE(128, 3); GD_CASE(128, 4); GD_CASE(128, 6); GD_CASE(128, 8);
#undef GD_CASE
    return (int)hipErrorInvalidValue;
}
