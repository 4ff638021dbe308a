/*
 * TEST INFRASTRUCTURE ONLY.  Drives the reference's OWN cached-generation code on whatever backend
 * the program is linked with: examples/gpt_lm/gpt_lm_shared.c is compiled where it lies (the
 * #include below, with -I pointing into the reference tree) so that its file-static functions
 * gpt_lm_prepare_generation_cache, gpt_lm_prefill_last_logits (gpt_lm_shared.c:1174-1202) and
 * gpt_lm_decode_logits (:1204-1248) are reachable without a tokenizer or a checkpoint.  The loop
 * below follows gpt_generate_prompts_loaded (:1560-1680) for temperature 0: packed prefill of
 * ragged prompts, greedy pick by gpt_sample_next_token, one cached decode step per new token.
 *
 * Input file  (int32): batch, new_tokens, n_layers, prompt_len[batch], packed prompt ids
 * Output file:         int32 ids[new_tokens][batch], then float logits[new_tokens][batch][GPT_VOCAB_SIZE]
 * (row 0 of both comes from the prefill, row s > 0 from decode step s).
 * Seed: argv[3] (decimal), the weight seed handed to gpt_lm_init.
 * Optional argv[4]: the freshly initialised model is also written there by the reference's own
 * gd_module_save_state (src/nn/module_io.c:700-800), which gives the loader tests a checkpoint that the
 * reference itself produced.  Optional argv[5]: a file whose bytes become the checkpoint's metadata blob
 * (the tests pass the "key=value" lines the reference's trainer writes, examples/gpt_lm/main.c:1836-1864).  The model dimensions are the example's compile-time macros
 * (gpt_lm_shared.h:10-28); the Makefile also builds a small-dimension variant for that fixture.
 */
#include "gpt_lm_shared.c"

static void die(const char *what)
{
    fprintf(stderr, "ref_gpt_generate: %s\n", what);
    exit(2);
}

int main(int argc, char **argv)
{
    gpt_config config;
    gd_memory_config mem;
    gd_context *ctx = NULL;
    gpt_lm model;
    gpt_kv_cache *cache = NULL;
    FILE *f;
    int32_t head[3];
    int32_t *prompt_len, *cu, *packed_ids, *packed_pos, *cache_pos, *ids, *pos, *out_ids;
    float *logits_host, *out_logits;
    uint64_t rng = 1U;
    int batch, steps, total = 0, b, i, s;
    gd_status st;
    if (argc < 4 || argc > 6) die("usage: ref_gpt_generate <in> <out> <seed> [checkpoint to write [metadata file]]");
    f = fopen(argv[1], "rb");
    if (f == NULL || fread(head, sizeof(head[0]), 3U, f) != 3U) die("cannot read the input header");
    batch = head[0];
    steps = head[1];
    if (batch <= 0 || steps <= 0 || head[2] <= 0) die("bad header");
    prompt_len = (int32_t *)calloc((size_t)batch, sizeof(int32_t));
    cu = (int32_t *)calloc((size_t)batch + 1U, sizeof(int32_t));
    if (fread(prompt_len, sizeof(int32_t), (size_t)batch, f) != (size_t)batch) die("cannot read prompt lengths");
    for (b = 0; b < batch; ++b) {
        if (prompt_len[b] <= 0 || prompt_len[b] + steps > GPT_CONTEXT_LENGTH) die("prompt does not fit the context");
        cu[b] = total;
        total += prompt_len[b];
    }
    cu[batch] = total;
    packed_ids = (int32_t *)calloc((size_t)total, sizeof(int32_t));
    packed_pos = (int32_t *)calloc((size_t)total, sizeof(int32_t));
    if (fread(packed_ids, sizeof(int32_t), (size_t)total, f) != (size_t)total) die("cannot read prompt ids");
    fclose(f);
    for (b = 0; b < batch; ++b)
        for (i = 0; i < prompt_len[b]; ++i) packed_pos[cu[b] + i] = i;

    memset(&config, 0, sizeof(config));
    config.batch_size = batch;
    config.n_layers = head[2];
    config.architecture = GPT_ARCH_GPT;
    config.minimax_m3_topk_blocks = GPT_MINIMAX_M3_TOPK_BLOCKS;
    config.minimax_m3_init_blocks = GPT_MINIMAX_M3_INIT_BLOCKS;
    config.minimax_m3_local_blocks = GPT_MINIMAX_M3_LOCAL_BLOCKS;
    config.dataloader_workers = 1;
    config.dataloader_prefetch_factor = 1;
    config.seed = strtoull(argv[3], NULL, 10);
    config.dropout_p = 0.0f;
    config.temperature = 0.0f;
    config.repetition_penalty = 1.0f;
    config.pad_token_id = -1;
    /* generate_prompt / generate_every_n_steps stay unset: the cache is then created by
     * gpt_lm_prepare_generation_cache with exactly `batch` rows (the state arena's optimizer share,
     * unused here, leaves room for it) */

    mem = gpt_memory_config(&config);
    mem.scratch_slot_bytes = 512ULL * 1024ULL * 1024ULL;
    st = gd_context_create(&mem, &ctx);
    if (st == GD_ERR_UNSUPPORTED) {
        printf("ref_gpt_generate: skipped (no backend)\n");
        return 77;
    }
    if (st != GD_OK) gpt_fail_status(ctx, st, "gd_context_create", __LINE__);
    gpt_lm_init(ctx, &model, &config);
    if (argc >= 5) {
        static const char meta[] = "{\"writer\":\"gd_module_save_state\",\"model\":\"gpt_lm\"}";
        gd_module_save_options save = gd_module_save_options_default();
        char *blob = NULL;
        save.metadata = meta;
        save.metadata_len = sizeof(meta) - 1U;
        if (argc >= 6) {
            FILE *m = fopen(argv[5], "rb");
            long n;
            if (m == NULL) die("cannot open the metadata file");
            fseek(m, 0, SEEK_END);
            n = ftell(m);
            fseek(m, 0, SEEK_SET);
            blob = (char *)calloc((size_t)n + 1U, 1U);
            if (n < 0 || blob == NULL || fread(blob, 1U, (size_t)n, m) != (size_t)n) die("cannot read the metadata file");
            fclose(m);
            save.metadata = blob;
            save.metadata_len = (size_t)n;
        }
        TRY(ctx, gd_module_save_state(ctx, &model.mod, argv[4], &save));
        free(blob);
    }
    TRY(ctx, gd_context_seal_params(ctx));
    TRY(ctx, gpt_lm_prepare_generation_cache(ctx, &model, &config, batch, GPT_CONTEXT_LENGTH, &cache));
    gd_module_set_training(&model.mod, false);

    cache_pos = (int32_t *)calloc((size_t)batch, sizeof(int32_t));
    ids = (int32_t *)calloc((size_t)batch, sizeof(int32_t));
    pos = (int32_t *)calloc((size_t)batch, sizeof(int32_t));
    logits_host = (float *)calloc((size_t)batch * GPT_VOCAB_SIZE, sizeof(float));
    out_ids = (int32_t *)calloc((size_t)steps * (size_t)batch, sizeof(int32_t));
    out_logits = (float *)calloc((size_t)steps * (size_t)batch * GPT_VOCAB_SIZE, sizeof(float));

    for (s = 0; s < steps; ++s) {
        gd_tensor ids_t, pos_t, cu_t, cache_pos_t, logits;
        TRY(ctx, gd_begin_step(ctx, GD_SCOPE_INFER, gd_batch_empty()));
        if (s == 0) {
            TRY(ctx, gpt_data_i32_tensor(ctx, packed_ids, total, &ids_t));
            TRY(ctx, gpt_data_i32_tensor(ctx, packed_pos, total, &pos_t));
            TRY(ctx, gpt_data_i32_tensor(ctx, cu, batch + 1, &cu_t));
            TRY(ctx, gpt_data_i32_tensor(ctx, cache_pos, batch, &cache_pos_t));
            TRY(ctx, gpt_lm_prefill_last_logits(ctx, &model, cache, &ids_t, &pos_t, &cu_t, cu, &cache_pos_t, &logits));
        } else {
            for (b = 0; b < batch; ++b) {
                ids[b] = out_ids[(size_t)(s - 1) * (size_t)batch + (size_t)b];
                pos[b] = cache->pos[b];
                cache_pos[b] = cache->pos[b];
            }
            TRY(ctx, gpt_data_i32_tensor(ctx, ids, batch, &ids_t));
            TRY(ctx, gpt_data_i32_tensor(ctx, pos, batch, &pos_t));
            TRY(ctx, gpt_data_i32_tensor(ctx, cache_pos, batch, &cache_pos_t));
            TRY(ctx, gpt_lm_decode_logits(ctx, &model, cache, &ids_t, &pos_t, &cache_pos_t, &logits));
        }
        TRY(ctx, gd_end_step(ctx));
        TRY(ctx, gd_tensor_read_f32(ctx, &logits, logits_host, (size_t)batch * GPT_VOCAB_SIZE));
        memcpy(out_logits + (size_t)s * (size_t)batch * GPT_VOCAB_SIZE, logits_host,
               (size_t)batch * GPT_VOCAB_SIZE * sizeof(float));
        for (b = 0; b < batch; ++b) {
            out_ids[(size_t)s * (size_t)batch + (size_t)b] = gpt_sample_next_token(
                logits_host + (size_t)b * GPT_VOCAB_SIZE, GPT_VOCAB_SIZE, NULL, 0, 0.0f, 0.0f, 1.0f, &rng);
            if (s == 0) cache->pos[b] = prompt_len[b];
        }
    }
    f = fopen(argv[2], "wb");
    if (f == NULL) die("cannot open the output file");
    fwrite(out_ids, sizeof(int32_t), (size_t)steps * (size_t)batch, f);
    fwrite(out_logits, sizeof(float), (size_t)steps * (size_t)batch * GPT_VOCAB_SIZE, f);
    fclose(f);
    printf("ref_gpt_generate: ok batch=%d new_tokens=%d layers=%d\n", batch, steps, (int)head[2]);
    gpt_lm_deinit(&model);
    gd_context_destroy(ctx);
    return 0;
}
