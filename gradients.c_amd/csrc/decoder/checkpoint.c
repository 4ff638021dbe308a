/*
 * Reader of the reference's ".gdckpt" container: header, directory, metadata blob and raw
 * tensor bytes.  Restates the reading half of src/nn/module_io.c of the reference
 * (gd_ckpt_read_header :424-459, gd_ckpt_read_dir :491-561, gd_checkpoint_read_metadata
 * :942-992) with the same status codes, plus three checks the reference leaves to its writer
 * (byte count against shape, data inside the file, unique paths).
 */
#define _POSIX_C_SOURCE 200809L
#define _FILE_OFFSET_BITS 64
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/types.h>

#include "gd_checkpoint.h"

#define CKPT_VERSION 1U
#define CKPT_HEADER_BYTES 64U
#define CKPT_ENTRY_FIXED_BYTES (16U + 8U * GD_MAX_DIMS + 16U)

static const unsigned char ckpt_magic[8] = {'G', 'D', 'C', 'K', 'P', 'T', '1', '\0'};

typedef struct ckpt_header {
    uint32_t version, header_size;
    uint64_t tensor_count, dir_offset, dir_size, metadata_offset, metadata_len, data_offset;
} ckpt_header;

struct gd_checkpoint {
    FILE *file;
    uint64_t file_size;
    ckpt_header header;
    uint32_t count;
    gd_checkpoint_entry *entries;
};

static uint32_t le32(const unsigned char *p)
{
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

static uint64_t le64(const unsigned char *p) { return (uint64_t)le32(p) | ((uint64_t)le32(p + 4) << 32); }

static gd_status read_exact(FILE *f, void *dst, size_t n)
{
    if (n == 0U) return GD_OK;
    return fread(dst, 1U, n, f) == n ? GD_OK : GD_ERR_IO;
}

static gd_status seek_to(FILE *f, uint64_t offset)
{
    if (offset > (uint64_t)INT64_MAX) return GD_ERR_INVALID_ARGUMENT;
    return fseeko(f, (off_t)offset, SEEK_SET) == 0 ? GD_OK : GD_ERR_IO;
}

static gd_status read_header(FILE *f, ckpt_header *h)
{
    unsigned char raw[CKPT_HEADER_BYTES];
    gd_status st;
    memset(h, 0, sizeof(*h));
    /* the reference reads field by field, so a short file fails with GD_ERR_IO before anything is compared,
     * except that a wrong magic in a file of at least 8 bytes is GD_ERR_BAD_STATE */
    st = read_exact(f, raw, 8U);
    if (st != GD_OK) return st;
    if (memcmp(raw, ckpt_magic, 8U) != 0) return GD_ERR_BAD_STATE;
    st = read_exact(f, raw + 8U, CKPT_HEADER_BYTES - 8U);
    if (st != GD_OK) return st;
    h->version = le32(raw + 8);
    h->header_size = le32(raw + 12);
    h->tensor_count = le64(raw + 16);
    h->dir_offset = le64(raw + 24);
    h->dir_size = le64(raw + 32);
    h->metadata_offset = le64(raw + 40);
    h->metadata_len = le64(raw + 48);
    h->data_offset = le64(raw + 56);
    if (h->version != CKPT_VERSION || h->header_size != CKPT_HEADER_BYTES || h->dir_offset < h->header_size ||
        h->metadata_offset < h->dir_offset || h->data_offset < h->metadata_offset)
        return GD_ERR_BAD_STATE;
    return GD_OK;
}

gd_status gd_checkpoint_read_metadata(const char *path, char **metadata_out, size_t *metadata_len_out)
{
    ckpt_header h;
    FILE *f;
    char *blob;
    gd_status st;
    if (path == NULL || path[0] == '\0' || metadata_out == NULL || metadata_len_out == NULL)
        return GD_ERR_INVALID_ARGUMENT;
    *metadata_out = NULL;
    *metadata_len_out = 0U;
    f = fopen(path, "rb");
    if (f == NULL) return GD_ERR_IO;
    st = read_header(f, &h);
    if (st != GD_OK) {
        fclose(f);
        return st;
    }
    if (h.metadata_len > (uint64_t)SIZE_MAX - 1U) {
        fclose(f);
        return GD_ERR_OUT_OF_MEMORY;
    }
    {
        /* a length that runs past the end of the file is the short read it would end in, found before the
         * allocation: a damaged header cannot ask for more memory than the file holds */
        off_t size;
        if (fseeko(f, 0, SEEK_END) != 0 || (size = ftello(f)) < 0 || h.metadata_offset > (uint64_t)size ||
            h.metadata_len > (uint64_t)size - h.metadata_offset) {
            fclose(f);
            return GD_ERR_IO;
        }
    }
    blob = (char *)malloc((size_t)h.metadata_len + 1U);
    if (blob == NULL) {
        fclose(f);
        return GD_ERR_OUT_OF_MEMORY;
    }
    st = seek_to(f, h.metadata_offset);
    if (st == GD_OK) st = read_exact(f, blob, (size_t)h.metadata_len);
    if (fclose(f) != 0 && st == GD_OK) st = GD_ERR_IO;
    if (st != GD_OK) {
        free(blob);
        return st;
    }
    blob[(size_t)h.metadata_len] = '\0';
    *metadata_out = blob;
    *metadata_len_out = (size_t)h.metadata_len;
    return GD_OK;
}

/* numel x element size with overflow detection; false if the dtype has no size or the product overflows */
static bool entry_bytes(const gd_checkpoint_entry *e, uint64_t *out)
{
    uint64_t n = (uint64_t)gd_dtype_size(e->dtype);
    uint32_t i;
    if (n == 0U) return false;
    for (i = 0U; i < e->rank; ++i) {
        const uint64_t d = (uint64_t)e->shape[i];
        if (d != 0U && n > UINT64_MAX / d) return false;
        n *= d;
    }
    *out = n;
    return true;
}

static gd_status read_directory(gd_checkpoint *c)
{
    const ckpt_header *h = &c->header;
    uint64_t consumed = 0U;
    uint32_t i;
    gd_status st;
    if (h->tensor_count > (uint64_t)UINT32_MAX) return GD_ERR_INVALID_ARGUMENT;
    /* every entry takes at least its fixed part: a count the directory cannot hold is refused before allocating */
    if (h->tensor_count * (uint64_t)CKPT_ENTRY_FIXED_BYTES > h->dir_size) return GD_ERR_BAD_STATE;
    /* a directory that runs past the end of the file is the short read it would end in, found before allocating */
    if (h->dir_offset > c->file_size || h->dir_size > c->file_size - h->dir_offset) return GD_ERR_IO;
    c->count = (uint32_t)h->tensor_count;
    if (c->count == 0U) return h->dir_size == 0U ? GD_OK : GD_ERR_BAD_STATE;
    c->entries = (gd_checkpoint_entry *)calloc(c->count, sizeof(gd_checkpoint_entry));
    if (c->entries == NULL) return GD_ERR_OUT_OF_MEMORY;
    st = seek_to(c->file, h->dir_offset);
    if (st != GD_OK) return st;
    for (i = 0U; i < c->count; ++i) {
        gd_checkpoint_entry *e = &c->entries[i];
        unsigned char raw[CKPT_ENTRY_FIXED_BYTES];
        uint32_t path_len, j;
        uint64_t expect, end;
        st = read_exact(c->file, raw, 16U);
        if (st != GD_OK) return st;
        path_len = le32(raw);
        e->flags = le32(raw + 4);
        e->dtype = (gd_dtype)le32(raw + 8);
        e->rank = le32(raw + 12);
        if (path_len == 0U || path_len >= GD_CHECKPOINT_PATH_MAX || e->rank > GD_MAX_DIMS ||
            (e->flags != GD_CHECKPOINT_ENTRY_PARAM && e->flags != GD_CHECKPOINT_ENTRY_BUFFER))
            return GD_ERR_BAD_STATE;
        st = read_exact(c->file, raw + 16U, CKPT_ENTRY_FIXED_BYTES - 16U);
        if (st != GD_OK) return st;
        for (j = 0U; j < GD_MAX_DIMS; ++j) {
            const uint64_t dim = le64(raw + 16U + 8U * j);
            if (j < e->rank && dim > (uint64_t)INT64_MAX) return GD_ERR_BAD_STATE;
            e->shape[j] = j < e->rank ? (int64_t)dim : 0;
        }
        e->data_offset = le64(raw + 16U + 8U * GD_MAX_DIMS);
        e->nbytes = le64(raw + 24U + 8U * GD_MAX_DIMS);
        st = read_exact(c->file, e->path, path_len);
        if (st != GD_OK) return st;
        e->path[path_len] = '\0';
        consumed += (uint64_t)CKPT_ENTRY_FIXED_BYTES + path_len;
        if (consumed > h->dir_size || e->data_offset < h->data_offset) return GD_ERR_BAD_STATE;
        /* beyond the reference: size against shape, data inside the file, no repeated or cut-short path */
        if (strlen(e->path) != path_len || !entry_bytes(e, &expect) || expect != e->nbytes) return GD_ERR_BAD_STATE;
        end = e->data_offset + e->nbytes;
        if (end < e->data_offset || end > c->file_size) return GD_ERR_BAD_STATE;
        for (j = 0U; j < i; ++j) {
            if (strcmp(c->entries[j].path, e->path) == 0) return GD_ERR_BAD_STATE;
        }
    }
    return consumed == h->dir_size ? GD_OK : GD_ERR_BAD_STATE;
}

gd_status gd_checkpoint_open(const char *path, gd_checkpoint **out)
{
    gd_checkpoint *c;
    gd_status st;
    off_t size;
    if (out != NULL) *out = NULL;
    if (path == NULL || path[0] == '\0' || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    c = (gd_checkpoint *)calloc(1U, sizeof(*c));
    if (c == NULL) return GD_ERR_OUT_OF_MEMORY;
    c->file = fopen(path, "rb");
    if (c->file == NULL) {
        free(c);
        return GD_ERR_IO;
    }
    if (fseeko(c->file, 0, SEEK_END) != 0 || (size = ftello(c->file)) < 0 || fseeko(c->file, 0, SEEK_SET) != 0) {
        gd_checkpoint_close(c);
        return GD_ERR_IO;
    }
    c->file_size = (uint64_t)size;
    st = read_header(c->file, &c->header);
    if (st == GD_OK) st = read_directory(c);
    if (st != GD_OK) {
        gd_checkpoint_close(c);
        return st;
    }
    *out = c;
    return GD_OK;
}

void gd_checkpoint_close(gd_checkpoint *c)
{
    if (c == NULL) return;
    if (c->file != NULL) fclose(c->file);
    free(c->entries);
    free(c);
}

uint32_t gd_checkpoint_count(const gd_checkpoint *c) { return c != NULL ? c->count : 0U; }

const gd_checkpoint_entry *gd_checkpoint_entry_at(const gd_checkpoint *c, uint32_t index)
{
    return c != NULL && index < c->count ? &c->entries[index] : NULL;
}

const gd_checkpoint_entry *gd_checkpoint_find(const gd_checkpoint *c, const char *path)
{
    uint32_t i;
    if (c == NULL || path == NULL) return NULL;
    for (i = 0U; i < c->count; ++i) {
        if (strcmp(c->entries[i].path, path) == 0) return &c->entries[i];
    }
    return NULL;
}

gd_status gd_checkpoint_read(gd_checkpoint *c, const gd_checkpoint_entry *entry, uint64_t offset, void *dst,
                             size_t nbytes)
{
    gd_status st;
    if (c == NULL || entry == NULL || entry < c->entries || entry >= c->entries + c->count ||
        (dst == NULL && nbytes != 0U) || offset > entry->nbytes || (uint64_t)nbytes > entry->nbytes - offset)
        return GD_ERR_INVALID_ARGUMENT;
    st = seek_to(c->file, entry->data_offset + offset);
    if (st != GD_OK) return st;
    return read_exact(c->file, dst, nbytes);
}
