/*
 * Reader of the reference's checkpoint container (".gdckpt", written by gd_module_save_state,
 * reference src/nn/module_io.c:713-807).  Host-only: no device work happens here; the decoder's
 * loader (gd_gpt_decoder_load_checkpoint, gd_gpt_decoder.h) moves the bytes to the device
 * through gd_tensor_write.
 *
 * File layout, all integers little-endian (module_io.c:17-27, 399-422, 461-489, 563-604):
 *   header, 64 bytes   "GDCKPT1\0", u32 version = 1, u32 header_size = 64, u64 tensor_count,
 *                      u64 dir_offset, u64 dir_size, u64 metadata_offset, u64 metadata_len,
 *                      u64 data_offset
 *   directory          per tensor: u32 path_len, u32 flags (1 parameter, 2 buffer), u32 dtype
 *                      (gd_dtype code), u32 rank, 8 x u64 shape, u64 data_offset (absolute),
 *                      u64 nbytes, then path_len path bytes without terminator
 *   metadata           opaque bytes
 *   tensor data        raw elements, row-major
 *
 * Status codes follow the reference reader (module_io.c:424-459, 491-561): a file that cannot be
 * opened or ends early is GD_ERR_IO; wrong magic / version / header size / section order, a bad
 * directory entry or a directory that does not fill dir_size exactly is GD_ERR_BAD_STATE.  On
 * top of the reference's checks this reader also rejects (GD_ERR_BAD_STATE) an entry whose byte
 * count is not numel x element size, whose data reaches past the end of the file, or whose path
 * repeats an earlier one: the reference trusts the writer for these.
 */
#ifndef GD_CHECKPOINT_H
#define GD_CHECKPOINT_H

#include "gradients_infer.h"

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

#define GD_CHECKPOINT_PATH_MAX 256U /* reference GD_MODULE_PATH_MAX */
#define GD_CHECKPOINT_ENTRY_PARAM 1U
#define GD_CHECKPOINT_ENTRY_BUFFER 2U

typedef struct gd_checkpoint_entry {
    char path[GD_CHECKPOINT_PATH_MAX];
    uint32_t flags;
    gd_dtype dtype;
    uint32_t rank;
    int64_t shape[GD_MAX_DIMS];
    uint64_t data_offset; /* from the start of the file */
    uint64_t nbytes;
} gd_checkpoint_entry;

typedef struct gd_checkpoint gd_checkpoint;

/* Same name, arguments and results as the reference's function (include/gradients/module.h:266-270,
 * src/nn/module_io.c:942-992): the metadata blob as a NUL-terminated malloc allocation the caller
 * frees.  Only the header is validated, as in the reference. */
gd_status gd_checkpoint_read_metadata(const char *path, char **metadata_out, size_t *metadata_len_out);

/* Opens the file and reads and validates header and directory (module_io.c:424-459, 491-561). */
gd_status gd_checkpoint_open(const char *path, gd_checkpoint **out);
void gd_checkpoint_close(gd_checkpoint *ckpt);

uint32_t gd_checkpoint_count(const gd_checkpoint *ckpt);
const gd_checkpoint_entry *gd_checkpoint_entry_at(const gd_checkpoint *ckpt, uint32_t index);
/* Linear search by path like the reference (module_io.c:277-289); NULL if absent. */
const gd_checkpoint_entry *gd_checkpoint_find(const gd_checkpoint *ckpt, const char *path);

/* Copies bytes [offset, offset + nbytes) of the entry's data into dst (module_io.c:675-711 reads
 * in 4 MiB pieces the same way).  GD_ERR_INVALID_ARGUMENT if the range leaves the entry. */
gd_status gd_checkpoint_read(gd_checkpoint *ckpt, const gd_checkpoint_entry *entry, uint64_t offset, void *dst,
                             size_t nbytes);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif

#endif /* GD_CHECKPOINT_H */
