/*
 * TEST INFRASTRUCTURE ONLY.  Runs the reference's OWN byte-level BPE tokenizer (src/tokenizer/*.c,
 * linked from the reference tree; pure host code): trains a small vocabulary on a corpus with
 * gd_bpe_tokenizer_train, writes it with gd_bpe_tokenizer_save, loads it back with
 * gd_bpe_tokenizer_load under three configurations and encodes / decodes given texts.  The output
 * is the golden data of the tokenizer tests.
 *
 * usage: ref_tokenizer <corpus> <vocab_size> <tokenizer.json> <texts.bin> <out.bin> [special ...]
 * texts.bin: int32 count, then per text int32 length + bytes (no NUL inside).
 * out.bin:   uint64 hash, int32 vocab_size, int32 n_specials, int32 special_id[n_specials], then for
 *            each configuration (split_digits, allow_special) in (1,1), (1,0), (0,1) and each text:
 *            int32 n_ids, int32 ids[n_ids], int32 decoded_length (of decoding those ids again).
 */
#include <gradients/tokenizer.h>

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static void die(const char *what)
{
    fprintf(stderr, "ref_tokenizer: %s\n", what);
    exit(2);
}

#define OK(expr) do { if ((expr) != GD_OK) die(#expr); } while (0)

int main(int argc, char **argv)
{
    static const int configs[3][2] = {{1, 1}, {1, 0}, {0, 1}};
    gd_bpe_train_config cfg;
    gd_tokenizer *tok = NULL;
    const char *corpus;
    int32_t count, i, c, n_specials;
    char **texts;
    FILE *f, *out;
    uint64_t hash;
    int32_t vocab;
    if (argc < 6) die("usage: ref_tokenizer <corpus> <vocab_size> <tokenizer.json> <texts.bin> <out.bin> [special ...]");
    corpus = argv[1];
    n_specials = argc - 6;
    memset(&cfg, 0, sizeof(cfg));
    cfg.vocab_size = atoi(argv[2]);
    cfg.min_frequency = 1;
    cfg.split_digits = 1;
    cfg.n_special_tokens = n_specials;
    cfg.special_tokens = (const char **)&argv[6];
    cfg.seed = 17U;
    OK(gd_bpe_tokenizer_train(&corpus, 1, &cfg, &tok));
    OK(gd_bpe_tokenizer_save(tok, argv[3]));
    hash = gd_tokenizer_hash(tok);
    vocab = gd_tokenizer_vocab_size(tok);

    f = fopen(argv[4], "rb");
    if (f == NULL || fread(&count, sizeof(count), 1, f) != 1 || count < 0) die("cannot read the texts");
    texts = (char **)calloc((size_t)count + 1U, sizeof(char *));
    for (i = 0; i < count; ++i) {
        int32_t len;
        if (fread(&len, sizeof(len), 1, f) != 1 || len < 0) die("short texts file");
        texts[i] = (char *)calloc((size_t)len + 1U, 1U);
        if (len > 0 && fread(texts[i], 1U, (size_t)len, f) != (size_t)len) die("short text");
    }
    fclose(f);

    out = fopen(argv[5], "wb");
    if (out == NULL) die("cannot open the output");
    fwrite(&hash, sizeof(hash), 1, out);
    fwrite(&vocab, sizeof(vocab), 1, out);
    fwrite(&n_specials, sizeof(n_specials), 1, out);
    for (i = 0; i < n_specials; ++i) {
        int32_t id = -1;
        OK(gd_tokenizer_id(tok, argv[6 + i], &id));
        fwrite(&id, sizeof(id), 1, out);
    }
    gd_tokenizer_destroy(tok);
    for (c = 0; c < 3; ++c) {
        gd_tokenizer_config load;
        gd_tokenizer *loaded = NULL;
        load.split_digits = configs[c][0];
        load.allow_special = configs[c][1];
        OK(gd_bpe_tokenizer_load(argv[3], &load, &loaded));
        for (i = 0; i < count; ++i) {
            int32_t *ids = NULL;
            int n = 0;
            int32_t n32, dlen;
            char *back = NULL;
            OK(gd_tokenizer_encode(loaded, texts[i], &ids, &n));
            OK(gd_tokenizer_decode(loaded, ids, n, &back));
            n32 = (int32_t)n;
            dlen = (int32_t)strlen(back);
            fwrite(&n32, sizeof(n32), 1, out);
            fwrite(ids, sizeof(int32_t), (size_t)n, out);
            fwrite(&dlen, sizeof(dlen), 1, out);
            gd_tokenizer_free(back);
            gd_tokenizer_free(ids);
        }
        gd_tokenizer_destroy(loaded);
    }
    fclose(out);
    printf("ref_tokenizer: ok vocab=%d texts=%d\n", (int)vocab, (int)count);
    return 0;
}
