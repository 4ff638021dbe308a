/*
 * TEST INFRASTRUCTURE ONLY.  Runs the reference's OWN host sampler on given logits: the file-static
 * functions gpt_apply_logits_softcap (examples/gpt_lm/gpt_lm_shared.c:1322-1331) and
 * gpt_sample_next_token (:1371-1442, which applies gpt_apply_repetition_penalty :1347-1369) are
 * reached by compiling gpt_lm_shared.c where it lies (the #include below).  No context, backend or
 * device is touched: the program runs on any machine.  Rows are served in order from one
 * generator, as the reference's generation loop does (:1586-1600).
 *
 * Input file:  int32 rows, vocab, hist_cap; float temperature, min_p, penalty, softcap;
 *              uint64 rng; float logits[rows][vocab]; int32 hist_len[rows];
 *              int32 history[rows][hist_cap]
 * Output file: int32 token[rows]; uint64 rng_after[rows]; float logits_after[rows][vocab]
 *              (the rows as the sampler left them: capped and penalised)
 */
#include "gpt_lm_shared.c"

static void die(const char *what)
{
    fprintf(stderr, "ref_sampler: %s\n", what);
    exit(2);
}

int main(int argc, char **argv)
{
    int32_t head[3], rows, vocab, cap, r;
    float par[4];
    uint64_t rng;
    float *logits;
    int32_t *hist_len, *history, *tokens;
    uint64_t *after;
    FILE *f;
    if (argc != 3) die("usage: ref_sampler <in> <out>");
    f = fopen(argv[1], "rb");
    if (f == NULL) die("cannot open the input file");
    if (fread(head, sizeof(int32_t), 3, f) != 3 || fread(par, sizeof(float), 4, f) != 4 ||
        fread(&rng, sizeof(rng), 1, f) != 1)
        die("short header");
    rows = head[0];
    vocab = head[1];
    cap = head[2];
    if (rows <= 0 || vocab <= 0 || cap <= 0) die("bad header");
    logits = (float *)calloc((size_t)rows * (size_t)vocab, sizeof(float));
    hist_len = (int32_t *)calloc((size_t)rows, sizeof(int32_t));
    history = (int32_t *)calloc((size_t)rows * (size_t)cap, sizeof(int32_t));
    tokens = (int32_t *)calloc((size_t)rows, sizeof(int32_t));
    after = (uint64_t *)calloc((size_t)rows, sizeof(uint64_t));
    if (fread(logits, sizeof(float), (size_t)rows * (size_t)vocab, f) != (size_t)rows * (size_t)vocab ||
        fread(hist_len, sizeof(int32_t), (size_t)rows, f) != (size_t)rows ||
        fread(history, sizeof(int32_t), (size_t)rows * (size_t)cap, f) != (size_t)rows * (size_t)cap)
        die("short body");
    fclose(f);
    for (r = 0; r < rows; ++r) {
        float *row = logits + (size_t)r * (size_t)vocab;
        gpt_apply_logits_softcap(row, vocab, par[3]);
        tokens[r] = gpt_sample_next_token(row, vocab, history + (size_t)r * (size_t)cap, hist_len[r], par[0], par[1],
                                          par[2], &rng);
        after[r] = rng;
    }
    f = fopen(argv[2], "wb");
    if (f == NULL) die("cannot open the output file");
    fwrite(tokens, sizeof(int32_t), (size_t)rows, f);
    fwrite(after, sizeof(uint64_t), (size_t)rows, f);
    fwrite(logits, sizeof(float), (size_t)rows * (size_t)vocab, f);
    fclose(f);
    printf("ref_sampler: ok rows=%d vocab=%d\n", rows, vocab);
    return 0;
}
