/*
 * Text in, text out with a checkpoint and a tokenizer of the reference's gpt_lm example: the counterpart of
 * the reference's examples/gpt_lm/infer.c (options :100-123, flow :434-525) on this repository's decoder.
 * The model's dimensions come from the checkpoint (directory + the trainer's metadata), the prompt is encoded
 * with the byte-level BPE tokenizer, gd_gpt_decoder_generate runs prefill, sampling and the decode loop on the
 * device, and the new tokens are decoded and printed.
 */
#include <stdio.h>
#include <unistd.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "gd_checkpoint.h"
#include "gd_gpt_decoder.h"
#include "gd_tokenizer.h"

static void usage(const char *argv0)
{
    printf("usage: %s --checkpoint PATH --tokenizer-path PATH --prompt TEXT [options]\n\n", argv0);
    printf("Options:\n");
    printf("  --checkpoint PATH      checkpoint written by the reference's gd_module_save_state\n");
    printf("  --tokenizer-path PATH  tokenizer JSON written by the reference's gd_bpe_tokenizer_save\n");
    printf("  --prompt TEXT          prompt text (alias: --generate)\n");
    printf("  --max-new-tokens N     generated tokens (default: 64)\n");
    printf("  --temperature T        sampling temperature; 0 means greedy (default: 0)\n");
    printf("  --min-p P              min-p cutoff relative to the top token; 0 disables (default: 0)\n");
    printf("  --repetition-penalty P repetition penalty; 1 disables (default: 1)\n");
    printf("  --logits-softcap C     final logits soft cap; 0 disables; the metadata value is used when available\n");
    printf("  --heads N              attention heads, if the checkpoint's metadata does not say\n");
    printf("  --context N            cache rows (default: the metadata's context_length)\n");
    printf("  --seed N               sampling seed (default: 1337)\n");
    printf("  --no-special           special-token texts in the prompt are ordinary text\n");
    printf("  --ids                  also print the token ids\n");
}

static int fail(const char *what, gd_status st, gd_context *ctx)
{
    fprintf(stderr, "gpt_lm_infer: %s failed: %s%s%s\n", what, gd_status_string(st), ctx != NULL ? " - " : "",
            ctx != NULL ? gd_context_error(ctx) : "");
    return 1;
}

/* "key=value" line of the metadata as a float; 0 if absent (the reference's metadata_value, infer.c:344-376) */
static float metadata_float(const char *blob, size_t len, const char *key)
{
    const size_t key_len = strlen(key);
    size_t at = 0U;
    while (at < len) {
        size_t end = at;
        while (end < len && blob[end] != '\n') ++end;
        if (end > at + key_len && strncmp(blob + at, key, key_len) == 0 && blob[at + key_len] == '=')
            return strtof(blob + at + key_len + 1U, NULL);
        at = end < len ? end + 1U : end;
    }
    return 0.0f;
}

int main(int argc, char **argv)
{
    const char *checkpoint = NULL, *tokenizer_path = NULL, *prompt = NULL;
    int max_new = 64, allow_special = 1, print_ids = 0, softcap_set = 0, i;
    unsigned long long seed = 1337ULL;
    gd_gpt_sampling sampling = {0.0f, 0.0f, 1.0f, 0.0f, -1, 0U};
    gd_gpt_config cfg;
    gd_tokenizer_config tok_cfg;
    gd_memory_config mem;
    gd_tokenizer *tok = NULL;
    gd_context *ctx = NULL;
    gd_gpt_decoder *dec = NULL;
    int32_t *ids = NULL, *out = NULL;
    int32_t cu[2], count = 0, stop = -1;
    int n_ids = 0;
    char *metadata = NULL, *text = NULL;
    size_t metadata_len = 0U;
    struct timespec t0, t1;
    double seconds;
    gd_status st;

    memset(&cfg, 0, sizeof(cfg));
    cfg.batch = 1;
    cfg.rms_eps = 1.0e-5f;
    cfg.rope_theta = 10000.0f;
    for (i = 1; i < argc; ++i) {
        const char *a = argv[i], *v = i + 1 < argc ? argv[i + 1] : NULL;
        if (!strcmp(a, "--help")) {
            usage(argv[0]);
            return 0;
        } else if (!strcmp(a, "--no-special")) {
            allow_special = 0;
        } else if (!strcmp(a, "--ids")) {
            print_ids = 1;
        } else if (v == NULL) {
            fprintf(stderr, "gpt_lm_infer: %s needs a value\n", a);
            return 2;
        } else {
            ++i;
            if (!strcmp(a, "--checkpoint")) checkpoint = v;
            else if (!strcmp(a, "--tokenizer-path")) tokenizer_path = v;
            else if (!strcmp(a, "--prompt") || !strcmp(a, "--generate")) prompt = v;
            else if (!strcmp(a, "--max-new-tokens")) max_new = atoi(v);
            else if (!strcmp(a, "--temperature")) sampling.temperature = strtof(v, NULL);
            else if (!strcmp(a, "--min-p")) sampling.min_p = strtof(v, NULL);
            else if (!strcmp(a, "--repetition-penalty")) sampling.repetition_penalty = strtof(v, NULL);
            else if (!strcmp(a, "--logits-softcap")) { sampling.logits_softcap = strtof(v, NULL); softcap_set = 1; }
            else if (!strcmp(a, "--heads")) cfg.n_heads = atoi(v);
            else if (!strcmp(a, "--context")) cfg.max_seq = atoi(v);
            else if (!strcmp(a, "--seed")) seed = strtoull(v, NULL, 10);
            else {
                fprintf(stderr, "gpt_lm_infer: unknown option %s\n", a);
                return 2;
            }
        }
    }
    if (checkpoint == NULL || tokenizer_path == NULL || prompt == NULL || max_new <= 0) {
        usage(argv[0]);
        return 2;
    }

    st = gd_gpt_config_from_checkpoint(checkpoint, &cfg);
    if (st != GD_OK) return fail("reading the model dimensions from the checkpoint", st, NULL);
    if (cfg.max_seq <= 0) {
        fprintf(stderr, "gpt_lm_infer: the checkpoint does not say its context length: pass --context\n");
        return 2;
    }
    if (!softcap_set && gd_checkpoint_read_metadata(checkpoint, &metadata, &metadata_len) == GD_OK)
        sampling.logits_softcap = metadata_float(metadata, metadata_len, "logits_softcap");
    free(metadata);

    tok_cfg.split_digits = 1; /* as the reference's generation code loads it (gpt_lm_shared.c:1281-1283) */
    tok_cfg.allow_special = allow_special;
    st = gd_bpe_tokenizer_load(tokenizer_path, &tok_cfg, &tok);
    if (st != GD_OK) return fail("loading the tokenizer", st, NULL);
    if (gd_tokenizer_vocab_size(tok) > cfg.vocab) {
        fprintf(stderr, "gpt_lm_infer: the tokenizer has %d tokens, the model %d\n", gd_tokenizer_vocab_size(tok), cfg.vocab);
        return 1;
    }
    if (gd_tokenizer_id(tok, "<|im_end|>", &stop) != GD_OK) stop = -1; /* :1291-1293 */
    sampling.stop_token = stop;
    sampling.rng_state = gd_gpt_generation_rng((uint64_t)seed, 1, 0U);
    st = gd_tokenizer_encode(tok, prompt, &ids, &n_ids);
    if (st != GD_OK) return fail("encoding the prompt", st, NULL);
    if (n_ids <= 0) {
        fprintf(stderr, "gpt_lm_infer: empty prompt\n");
        return 1;
    }

    mem = gd_memory_config_default();
    mem.params_bytes = gd_gpt_params_bytes(&cfg);
    mem.state_bytes = gd_gpt_state_bytes(&cfg);
    mem.scratch_slot_bytes = gd_gpt_scratch_bytes(&cfg, n_ids < cfg.max_seq ? n_ids : cfg.max_seq);
    mem.data_slot_bytes = (size_t)(16 * cfg.max_seq) + ((size_t)1 << 20);
    st = gd_context_create(&mem, &ctx);
    if (st != GD_OK) return fail("gd_context_create (no HIP device? there is no CPU fallback)", st, NULL);
    st = gd_gpt_decoder_create(ctx, &cfg, &dec);
    if (st == GD_OK) st = gd_gpt_decoder_load_checkpoint(dec, checkpoint, 1);
    if (st != GD_OK) return fail("creating the decoder from the checkpoint", st, ctx);

    out = (int32_t *)malloc((size_t)max_new * sizeof(int32_t));
    if (out == NULL) return fail("allocating the output", GD_ERR_OUT_OF_MEMORY, NULL);
    cu[0] = 0;
    cu[1] = n_ids;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    st = gd_gpt_decoder_generate(dec, ids, cu, max_new, &sampling, out, &count);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    if (st != GD_OK) return fail("gd_gpt_decoder_generate", st, ctx);
    seconds = (double)(t1.tv_sec - t0.tv_sec) + 1.0e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
    st = gd_tokenizer_decode(tok, out, count, &text);
    if (st != GD_OK) return fail("decoding the new tokens", st, NULL);

    printf("inference: checkpoint=%s layers=%d d_model=%d heads=%d vocab=%d context=%d prompt_tokens=%d "
           "temperature=%.3f min_p=%.3f repetition_penalty=%.3f logits_softcap=%.3f\n",
           checkpoint, cfg.n_layers, cfg.d_model, cfg.n_heads, cfg.vocab, cfg.max_seq, n_ids, (double)sampling.temperature,
           (double)sampling.min_p, (double)sampling.repetition_penalty, (double)sampling.logits_softcap);
    if (print_ids) {
        printf("ids:");
        for (i = 0; i < count; ++i) printf(" %d", (int)out[i]);
        printf("\n");
    }
    printf("generated_text=%s\n", text);
    printf("generate: generated=%d elapsed=%.3fs tok/s=%.1f\n", (int)count, seconds, seconds > 0.0 ? (double)count / seconds : 0.0);

    gd_tokenizer_free(text);
    gd_tokenizer_free(ids);
    free(out);
    gd_gpt_decoder_destroy(dec);
    gd_context_destroy(ctx);
    gd_tokenizer_destroy(tok);
    /* everything this program created is released; what the HIP runtime does in its exit handlers is skipped */
    fflush(stdout);
    fflush(stderr);
    _exit(0);
}
