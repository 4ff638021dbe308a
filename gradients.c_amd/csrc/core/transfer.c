/*
 * Host <-> device transfers of the host core.  Contract restated from the reference's
 * src/core/transfer.c:99-270: tensors must be valid and contiguous (else GD_ERR_UNSUPPORTED), the
 * byte count must equal the logical size (else GD_ERR_INVALID_ARGUMENT), F32 <-> F16 conversion
 * rounds to nearest even (src/core/dtype_internal.h:6-88), the F32 helpers take F16/F32 tensors
 * only, and a transfer is ordered after everything already enqueued (the backend upload/download
 * synchronise on the stream).  Conversion goes through a fixed stack block: no heap allocation.
 */
#include "core_internal.h"

uint16_t gd_f32_to_f16_bits(float value)
{
    union { float f; uint32_t u; } in;
    uint32_t sign, biased, frac;
    int32_t e;
    in.f = value;
    sign = (in.u >> 16) & 0x8000U;
    biased = (in.u >> 23) & 0xffU;
    frac = in.u & 0x7fffffU;
    if (biased == 0xffU) return (uint16_t)(sign | (frac ? 0x7e00U : 0x7c00U));
    e = (int32_t)biased - 127;
    if (e > 15) return (uint16_t)(sign | 0x7c00U);
    if (e < -14) {
        const int32_t shift = -14 - e;
        uint32_t drop, kept, rest, half;
        if (shift > 11) return (uint16_t)sign; /* below half of the smallest subnormal */
        frac |= 0x800000U;
        drop = (uint32_t)shift + 13U;
        kept = frac >> drop;
        rest = frac & ((1U << drop) - 1U);
        half = 1U << (drop - 1U);
        if (rest > half || (rest == half && (kept & 1U))) kept += 1U;
        return (uint16_t)(sign | kept);
    }
    {
        uint32_t he = (uint32_t)(e + 15), hm = frac >> 13;
        const uint32_t rest = frac & 0x1fffU;
        if (rest > 0x1000U || (rest == 0x1000U && (hm & 1U))) {
            hm += 1U;
            if (hm == 0x400U) {
                hm = 0U;
                he += 1U;
                if (he >= 31U) return (uint16_t)(sign | 0x7c00U);
            }
        }
        return (uint16_t)(sign | (he << 10) | hm);
    }
}

float gd_f16_bits_to_f32(uint16_t bits)
{
    union { uint32_t u; float f; } out;
    const uint32_t sign = ((uint32_t)bits & 0x8000U) << 16;
    int32_t e = (int32_t)((bits >> 10) & 0x1fU);
    uint32_t m = (uint32_t)bits & 0x3ffU;
    if (e == 0) {
        if (m == 0U) {
            out.u = sign;
            return out.f;
        }
        e = 1;
        while (!(m & 0x400U)) {
            m <<= 1;
            e -= 1;
        }
        m &= 0x3ffU;
    } else if (e == 31) {
        out.u = sign | 0x7f800000U | (m << 13);
        return out.f;
    }
    out.u = sign | ((uint32_t)(e + 112) << 23) | (m << 13);
    return out.f;
}

gd_status gd_synchronize(gd_context *ctx)
{
    gd_status st;
    if (ctx == NULL) return GD_ERR_INVALID_ARGUMENT;
    st = gd_backend_flush(gd_context_backend(ctx));
    return st == GD_OK ? GD_OK : gd_context_set_error(ctx, st, "backend flush failed");
}

static gd_status check_transfer(gd_context *ctx, const gd_tensor *t, size_t nbytes, const char *what_contig,
                                const char *what_size)
{
    size_t logical;
    gd_status st = gd_tensor_validate(ctx, t);
    if (st != GD_OK) return st;
    if (!gd_tensor_is_contiguous(t)) return gd_context_set_error(ctx, GD_ERR_UNSUPPORTED, what_contig);
    st = gd_tensor_logical_nbytes(t, &logical);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "tensor transfer invalid shape");
    if (nbytes != logical) return gd_context_set_error(ctx, GD_ERR_INVALID_ARGUMENT, what_size);
    return GD_OK;
}

gd_status gd_tensor_write(gd_context *ctx, gd_tensor *dst, const void *src, size_t nbytes)
{
    gd_status st;
    if (ctx == NULL || src == NULL || dst == NULL || nbytes == 0U) return GD_ERR_INVALID_ARGUMENT;
    st = check_transfer(ctx, dst, nbytes, "tensor upload requires contiguous tensor", "tensor upload size mismatch");
    if (st != GD_OK) return st;
    st = gd_backend_upload(gd_context_backend(ctx), (gd_backend_buffer *)dst->storage.buffer,
                           dst->storage.offset + dst->view_offset, src, nbytes);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "backend upload failed");
    dst->version += 1U;
    if (dst->version == 0U) dst->version = 1U;
    return GD_OK;
}

gd_status gd_tensor_read(gd_context *ctx, const gd_tensor *src, void *dst, size_t nbytes)
{
    gd_status st;
    if (ctx == NULL || src == NULL || dst == NULL || nbytes == 0U) return GD_ERR_INVALID_ARGUMENT;
    st = check_transfer(ctx, src, nbytes, "tensor download requires contiguous tensor", "tensor download size mismatch");
    if (st != GD_OK) return st;
    st = gd_backend_download(gd_context_backend(ctx), (gd_backend_buffer *)src->storage.buffer,
                             src->storage.offset + src->view_offset, dst, nbytes);
    return st == GD_OK ? GD_OK : gd_context_set_error(ctx, st, "backend download failed");
}

static gd_status check_f32(gd_context *ctx, const gd_tensor *t, size_t count)
{
    int64_t n;
    gd_status st;
    if (count == 0U) return GD_ERR_INVALID_ARGUMENT;
    st = gd_tensor_validate(ctx, t);
    if (st != GD_OK) return st;
    if (t->dtype != GD_DTYPE_F16 && t->dtype != GD_DTYPE_F32)
        return gd_context_set_error(ctx, GD_ERR_UNSUPPORTED, "f32 tensor transfer supports f16 and f32 tensors");
    if (!gd_tensor_is_contiguous(t))
        return gd_context_set_error(ctx, GD_ERR_UNSUPPORTED, "f32 tensor transfer requires contiguous tensor");
    st = gd_tensor_numel(t, &n);
    if (st != GD_OK) return gd_context_set_error(ctx, st, "f32 tensor transfer invalid shape");
    if ((uint64_t)n != (uint64_t)count)
        return gd_context_set_error(ctx, GD_ERR_INVALID_ARGUMENT, "f32 tensor transfer count mismatch");
    return GD_OK;
}


gd_status gd_tensor_write_f32(gd_context *ctx, gd_tensor *dst, const float *src, size_t count)
{
    uint16_t *block;
    size_t done = 0U;
    gd_status st;
    if (ctx == NULL || dst == NULL || src == NULL) return GD_ERR_INVALID_ARGUMENT;
    st = check_f32(ctx, dst, count);
    if (st != GD_OK) return st;
    if (dst->dtype == GD_DTYPE_F32) return gd_tensor_write(ctx, dst, src, count * sizeof(float));
    block = ctx->pack;
    while (done < count) {
        const size_t n = count - done < ctx->pack_count ? count - done : ctx->pack_count;
        int64_t i;
#pragma omp parallel for schedule(static) if (n > 65536U)
        for (i = 0; i < (int64_t)n; ++i) block[i] = gd_f32_to_f16_bits(src[done + (size_t)i]);
        st = gd_backend_upload(gd_context_backend(ctx), (gd_backend_buffer *)dst->storage.buffer,
                               dst->storage.offset + dst->view_offset + done * 2U, block, n * 2U);
        if (st != GD_OK) return gd_context_set_error(ctx, st, "backend upload failed");
        done += n;
    }
    dst->version += 1U;
    if (dst->version == 0U) dst->version = 1U;
    return GD_OK;
}

gd_status gd_tensor_read_f32(gd_context *ctx, const gd_tensor *src, float *dst, size_t count)
{
    uint16_t *block;
    size_t done = 0U;
    gd_status st;
    if (ctx == NULL || src == NULL || dst == NULL) return GD_ERR_INVALID_ARGUMENT;
    st = check_f32(ctx, src, count);
    if (st != GD_OK) return st;
    if (src->dtype == GD_DTYPE_F32) return gd_tensor_read(ctx, src, dst, count * sizeof(float));
    block = ctx->pack;
    while (done < count) {
        const size_t n = count - done < ctx->pack_count ? count - done : ctx->pack_count;
        size_t i;
        st = gd_backend_download(gd_context_backend(ctx), (gd_backend_buffer *)src->storage.buffer,
                                 src->storage.offset + src->view_offset + done * 2U, block, n * 2U);
        if (st != GD_OK) return gd_context_set_error(ctx, st, "backend download failed");
        for (i = 0U; i < n; ++i) dst[done + i] = gd_f16_bits_to_f32(block[i]);
        done += n;
    }
    return GD_OK;
}
