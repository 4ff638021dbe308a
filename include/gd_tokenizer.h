/*
 * Byte-level BPE tokenizer, the part of the reference's tokenizer an inference program uses: load a
 * vocabulary file the reference wrote ("gd-bpe-tokenizer-v1"), encode text to token ids, decode ids to
 * text.  Names, arguments and results are the reference's (include/gradients/tokenizer.h:17-20, 71-95;
 * src/tokenizer/tokenizer.c, tokenizer_codec.c, tokenizer_io.c), so a program written against the
 * reference's header compiles against this one.  Training and saving a vocabulary are not provided.
 * Host code only: nothing here touches a device.
 */
#ifndef GD_TOKENIZER_H
#define GD_TOKENIZER_H

#include "gradients_infer.h"

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

typedef struct gd_tokenizer gd_tokenizer;

typedef struct gd_tokenizer_config { /* tokenizer.h:17-20 */
    int split_digits;  /* every ASCII digit is a piece of its own */
    int allow_special; /* special-token texts in the input become their ids; 0: they are ordinary text */
} gd_tokenizer_config;

/* Reads a vocabulary file written by the reference's gd_bpe_tokenizer_save (tokenizer_io.c:46-88): one token per
 * line, ids contiguous from 0, kinds "byte" (ids 0-255), "special" and "merge".  cfg == NULL: split_digits as the
 * file says, specials allowed (tokenizer_io.c:238-371).  GD_ERR_IO if the file cannot be read;
 * GD_ERR_INVALID_ARGUMENT for ids out of sequence, a malformed field, an empty token, more than 64 specials or
 * fewer than 256 tokens; GD_ERR_UNSUPPORTED for an escape other than \n \r \t \" \\ in a special's text. */
gd_status gd_bpe_tokenizer_load(const char *tokenizer_path, const gd_tokenizer_config *cfg, gd_tokenizer **out);
void gd_tokenizer_destroy(gd_tokenizer *tok);

/* Text (NUL-terminated bytes, normally UTF-8) to ids (tokenizer_codec.c:66-200, pretokenizer tokenizer.c:399-526):
 * the text is cut into special tokens and pieces (a run of letters / bytes >= 0x80, of digits, of other
 * characters, each optionally led by one space; runs of white space; single digits with split_digits; at most 256
 * bytes per piece); a piece that is a token is that token, otherwise its bytes are merged pair by pair, always
 * the pair whose merged token has the lowest id, leftmost first.  *ids_out is malloc'ed (gd_tokenizer_free). */
gd_status gd_tokenizer_encode(gd_tokenizer *tok, const char *text, int32_t **ids_out, int *n_ids_out);

/* Concatenation of the tokens' bytes, NUL-terminated, malloc'ed (tokenizer_codec.c:202-238).
 * GD_ERR_INVALID_ARGUMENT for an id outside the vocabulary. */
gd_status gd_tokenizer_decode(gd_tokenizer *tok, const int32_t *ids, int n_ids, char **text_out);

/* Id of a special token by its text; GD_ERR_INVALID_ARGUMENT if there is none (tokenizer.c:550-563). */
gd_status gd_tokenizer_id(gd_tokenizer *tok, const char *special, int32_t *id_out);

int gd_tokenizer_vocab_size(const gd_tokenizer *tok);
/* FNV-style digest of split_digits and every token (tokenizer.c:151-174); equals the "hash" field of the file when
 * split_digits is what the file was written with. */
uint64_t gd_tokenizer_hash(const gd_tokenizer *tok);
void gd_tokenizer_free(void *ptr);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif

#endif /* GD_TOKENIZER_H */
