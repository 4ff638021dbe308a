/*
 * gd_gpt_decoder.h - the decoder-only language model of the reference's example
 * (examples/gpt_lm/gpt_lm_shared.c), inference part, with run-time dimensions: weights, K/V
 * caches, packed prefill and the batched cached decode step, written against the public gd_*
 * operators of gradients_infer.h in the reference's call order
 * (gpt_block_decode_cached :961-1071, gpt_lm_decode_logits :1204-1246,
 * gpt_block_prefill_cached :825-959, gpt_lm_prefill_last_logits :1174-1202).
 *
 * Two ways to run a decode step:
 *   gd_gpt_decoder_step          one gd_begin_step .. gd_end_step scope per token, every operator
 *                                issued through the public API, ids uploaded and results
 *                                downloaded each step (the reference generator's loop);
 *   gd_gpt_decoder_run_resident  token ids and cache positions stay on the device, the greedy
 *                                token of step t feeds step t+1 without a host round trip, and the
 *                                step is replayed from a captured graph.
 * Both produce the same tokens.
 */
#ifndef GD_GPT_DECODER_H
#define GD_GPT_DECODER_H

#include "gradients_infer.h"

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default) /* the library is built with hidden visibility: only these are exported */

typedef struct gd_gpt_config {
    int32_t vocab, d_model, n_layers, n_heads, head_dim, mlp_hidden;
    int32_t max_seq;     /* cache rows per sequence (Tmax) */
    int32_t batch;       /* sequences decoded together */
    int32_t sdpa_window; /* 0 = attend to the whole cache; the reference example uses 256 */
    int32_t tie_lm_head; /* 1: LM head shares the embedding table (reference :393-402); 0: own [V,Dm] weight */
    float rms_eps;       /* reference 1e-5 (gpt_lm_shared.h:58) */
    float rope_theta;    /* reference 10000 */
    uint64_t seed;
    /* MiniMax-M3 architecture of the reference's example (gpt_lm_shared.h:29-40, 83; gpt_lm_shared.c:588-600,
     * 918-933): with m3_block_size > 0 the packed prefill picks m3_topk_blocks key blocks per row (the first
     * m3_init_blocks and the last m3_local_blocks forced) and attends over those, provided the context is long
     * enough for that to matter (max_seq > 8 blocks and 2 x topk blocks < max_seq); the decode step is the dense
     * one either way.  All zero: the plain architecture.  The reference's values: 128, 3, 1, 1. */
    int32_t m3_block_size, m3_topk_blocks, m3_init_blocks, m3_local_blocks;
} gd_gpt_config;

typedef struct gd_gpt_decoder gd_gpt_decoder;

/* Bytes the params and state arenas need for this configuration (for gd_memory_config). */
size_t gd_gpt_params_bytes(const gd_gpt_config *cfg);
size_t gd_gpt_state_bytes(const gd_gpt_config *cfg);
/* Bytes one scratch slot needs for a packed prefill of max_prefill_tokens rows (at least batch rows: a decode step). */
size_t gd_gpt_scratch_bytes(const gd_gpt_config *cfg, int32_t max_prefill_tokens);

/* Allocates weights in the params arena and caches in the state arena and initialises the weights
 * the way the reference example does (N(0,0.02) from a splitmix64 + Box-Muller stream seeded per
 * tensor, residual projections scaled by 1/sqrt(2L), biases 0, norm weights 1; :196-218,290-402). */
gd_status gd_gpt_decoder_create(gd_context *ctx, const gd_gpt_config *cfg, gd_gpt_decoder **out);
void gd_gpt_decoder_destroy(gd_gpt_decoder *dec);

/* Weight / cache tensors by name (embed, lm_head, lm_bias, final_norm, attn_norm, mlp_norm, w_qkv,
 * b_qkv, w_attn, b_attn, w_upgate, b_upgate, w_down, b_down, k_cache, v_cache); NULL if unknown. */
gd_tensor *gd_gpt_decoder_tensor(gd_gpt_decoder *dec, const char *name, int32_t layer);

/* Replaces the weights with those of a checkpoint the reference wrote with gd_module_save_state for its
 * gpt_lm example (".gdckpt"; container described in gd_checkpoint.h).  The counterpart of the
 * reference's gd_module_load_state(ctx, &model.mod, path, {strict, load_buffers}) as its inference
 * programs call it (examples/gpt_lm/infer.c:514-516; src/nn/module_io.c:826-940): tensors are matched
 * by the paths gpt_lm_init registers ("gpt_lm.token_embedding", "gpt_lm.lm_head_bias",
 * "gpt_lm.final_norm_w", "gpt_lm.blocks.<l>.{attn_norm_w, mlp_norm_w, qkv_proj.weight, qkv_proj.bias,
 * attn_proj.weight, attn_proj.bias, up_gate.weight, up_gate.bias, down_proj.weight, down_proj.bias}")
 * and every match must agree in dtype, rank, shape and byte count (GD_ERR_BAD_STATE otherwise).
 * strict != 0: a parameter in the file the decoder does not have, or one the decoder has and the file
 * lacks, is GD_ERR_BAD_STATE; strict == 0: both are skipped.  Buffer entries are ignored (the decoder
 * registers none).  All checks run before the first byte is written, so a refused file leaves the
 * weights untouched.  The reference ties the LM head to the embedding table; a decoder created with
 * tie_lm_head = 0 receives the table in both places.  The [d_model, hidden] copy of each down
 * projection is rebuilt from the loaded [hidden, d_model] weight.  GD_ERR_BUSY while a resident
 * session is open; file errors as in gd_checkpoint_open.  Caches and positions are not touched. */
gd_status gd_gpt_decoder_load_checkpoint(gd_gpt_decoder *dec, const char *path, int32_t strict);

/* Fills the model dimensions of *cfg from a checkpoint of the reference's gpt_lm example, the way its inference
 * programs size the model before loading (examples/gpt_lm/infer.c:344-432, 464-478): vocab, d_model, mlp_hidden
 * and n_layers from the directory (shapes of "gpt_lm.token_embedding" and "gpt_lm.blocks.0.down_proj.weight",
 * highest block index); n_heads, head_dim, sdpa_window and (only if cfg->max_seq <= 0) max_seq = context_length
 * from the "key=value" lines the reference's trainer stores as metadata (examples/gpt_lm/main.c:1836-1864); a line
 * "architecture=minimax_m3" also sets m3_* from the minimax_m3_* lines (defaults 128, 3, 1, 1).
 * Fields the file does not tell keep the caller's values (n_heads / head_dim given by the caller complete each
 * other through d_model); tie_lm_head is set (the reference ties).  GD_ERR_BAD_STATE if the expected tensors are
 * absent, if metadata and directory contradict each other, or if n_heads x head_dim != d_model at the end. */
gd_status gd_gpt_config_from_checkpoint(const char *path, gd_gpt_config *cfg);

/* Host copy of the live length of every sequence ([batch]); writable (e.g. after filling caches). */
int32_t *gd_gpt_decoder_positions(gd_gpt_decoder *dec);

/* Packed prefill from position 0: ids [cu[batch]], cu [batch+1] on the host.  Outputs (each may be
 * NULL): greedy next ids [batch], top-2 gaps [batch], logits [batch, vocab] as F16 bits. */
gd_status gd_gpt_decoder_prefill(gd_gpt_decoder *dec, const int32_t *ids, const int32_t *cu, int32_t *next_ids,
                                 float *gaps, uint16_t *logits);

/* One batched decode step through the public operator API.  ids [batch] on the host. */
gd_status gd_gpt_decoder_step(gd_gpt_decoder *dec, const int32_t *ids, int32_t *next_ids, float *gaps,
                              uint16_t *logits);

/* Device-resident greedy decoding.  A session keeps token ids and cache positions on the device:
 *   begin  uploads first_ids [batch] and the positions, opens one inference step scope, runs the
 *          first step eagerly and captures the step into a graph;
 *   run    enqueues n more steps (graph replays) without waiting;
 *   sync   waits for everything enqueued;
 *   end    closes the scope and downloads the tokens of all steps run so far: out_ids
 *          [steps, batch] and (may be NULL) out_gaps; steps_done (may be NULL) = rows written.
 * At most max_steps steps can run in a session (run beyond that: GD_ERR_INVALID_ARGUMENT); run, sync and end
 * without an open session are GD_ERR_BAD_STATE.  While a session is open the decoder is busy: prefill, step,
 * generate, load_checkpoint and another begin return GD_ERR_BUSY and change nothing.  flags:
 *   GD_GPT_RESIDENT_HOLD_POSITIONS  the cache positions do not advance: every step appends at the
 *                                   same row and attends over the same number of keys (used to time
 *                                   one fixed-shape step repeatedly);
 *   GD_GPT_RESIDENT_UNFUSED         issue the step through the public operators exactly like
 *                                   gd_gpt_decoder_step (about 40 launches for 3 layers).  Without
 *                                   it the step uses the fused backend entry points
 *                                   (gd_backend_fused_linear, gd_backend_qkv_rope_append: 5 launches
 *                                   per layer), which keep every rounding point of the separate
 *                                   operators;
 *   GD_GPT_RESIDENT_KEEP_LOGITS     every step also copies its logits [batch, vocab] into the decoder's
 *                                   "last_logits" tensor (one more launch per step; greedy sessions only):
 *                                   after sync it holds the logits of the last step run. */
#define GD_GPT_RESIDENT_HOLD_POSITIONS 1
#define GD_GPT_RESIDENT_UNFUSED 2
#define GD_GPT_RESIDENT_KEEP_LOGITS 4
gd_status gd_gpt_decoder_resident_begin(gd_gpt_decoder *dec, const int32_t *first_ids, int32_t max_steps,
                                        int32_t flags);
gd_status gd_gpt_decoder_resident_run(gd_gpt_decoder *dec, int32_t n_steps);
gd_status gd_gpt_decoder_resident_sync(gd_gpt_decoder *dec);
gd_status gd_gpt_decoder_resident_end(gd_gpt_decoder *dec, int32_t *out_ids, float *out_gaps, int32_t *steps_done);

/* begin + run(n_steps - 1) + end in one call.  step_ms (may be NULL) receives the mean device time
 * per replayed step measured with stream events. */
gd_status gd_gpt_decoder_run_resident(gd_gpt_decoder *dec, const int32_t *first_ids, int32_t n_steps,
                                      int32_t *out_ids, float *out_gaps, float *step_ms);

/* Generation with the reference's sampling front end, tokens in and tokens out: what gpt_generate_prompts_loaded
 * of the reference's example does between its tokenizer calls (examples/gpt_lm/gpt_lm_shared.c:1444-1700), with
 * the logits never leaving the device (gd_backend_sample_advance after the packed prefill and after every step
 * of the resident loop).
 *   ids / cu     packed prompts of the batch rows, cu [batch+1]; a prompt longer than the room the new tokens
 *                leave (max_seq - max_new, or max_seq - 1 if max_new >= max_seq) keeps its last tokens (:1514-1533)
 *   max_new      at most this many tokens per row
 *   sampling     temperature <= 0 picks greedily; min_p, repetition_penalty (> 1 acts, over prompt + generated
 *                tokens) and logits_softcap (> 0 acts) as in :1322-1442; a row ends when it picks stop_token
 *                (>= 0; the token is not part of its output) or its sequence reaches max_seq; rng_state is the
 *                generator state before the first draw: gd_gpt_generation_rng(seed, batch, step) gives the
 *                reference's (:1565)
 *   out_tokens   [batch, max_new]: row b's new tokens in its first out_counts[b] places
 * The caches are rewritten from position 0.  GD_ERR_BUSY while a resident session is open. */
typedef struct gd_gpt_sampling {
    float temperature, min_p, repetition_penalty, logits_softcap;
    int32_t stop_token; /* < 0: none */
    uint64_t rng_state;
} gd_gpt_sampling;

/* The sampled form of gd_gpt_decoder_resident_begin, for callers that drive the session themselves
 * (gd_gpt_decoder_generate is prefill + this + run + end).  It starts from the logits the last
 * gd_gpt_decoder_prefill left on the device: ids / cu are the rows' histories so far (normally that prefill's
 * prompts; the repetition penalty looks at them), max_picks counts picks, the first of which is made on those
 * logits, so at most max_picks - 1 decode steps can run.  run / sync / end as for a greedy session; end returns
 * one record per pick and row: the token appended to the row's history, or -1 for a row that has ended.  flags:
 * GD_GPT_RESIDENT_HOLD_POSITIONS, GD_GPT_RESIDENT_UNFUSED. */
gd_status gd_gpt_decoder_resident_begin_sampled(gd_gpt_decoder *dec, const int32_t *ids, const int32_t *cu,
                                                int32_t max_picks, int32_t flags, const gd_gpt_sampling *sampling);

uint64_t gd_gpt_generation_rng(uint64_t seed, int32_t n_prompts, uint64_t step);
gd_status gd_gpt_decoder_generate(gd_gpt_decoder *dec, const int32_t *ids, const int32_t *cu, int32_t max_new,
                                  const gd_gpt_sampling *sampling, int32_t *out_tokens, int32_t *out_counts);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif

#endif /* GD_GPT_DECODER_H */
