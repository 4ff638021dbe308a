/*
 * Decoder-only language model of the reference's example, inference part, with run-time
 * dimensions.  The operator order, residual wiring and cache bookkeeping restate
 * examples/gpt_lm/gpt_lm_shared.c of the reference: gpt_block_decode_cached (:961-1071),
 * gpt_lm_decode_logits (:1204-1246), gpt_block_prefill_cached (:825-959),
 * gpt_lm_prefill_last_logits (:1174-1202), gpt_kv_cache_init (:480-538) and the weight
 * initialisation (:196-218, 290-402).  Everything goes through the public gd_* operators.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <stdio.h>

#include "gd_checkpoint.h"
#include "gd_gpt_decoder.h"

#define TRY(expr)                       \
    do {                                \
        gd_status st__ = (expr);        \
        if (st__ != GD_OK) return st__; \
    } while (0)

typedef struct gpt_linear {
    gd_tensor weight, bias;
    bool transposed; /* weight stored [out, in] */
} gpt_linear;

typedef struct gpt_block {
    gd_tensor attn_norm_w, mlp_norm_w;
    gpt_linear qkv_proj, attn_proj, up_gate, down_proj;
    /* the down projection's weight once more as [d_model, hidden] (the reference keeps it [hidden, d_model]): with
     * few rows the projection streams the weight once, and rows that are contiguous along the summed dimension
     * come in whole cache lines per workgroup; a 16-column slice of the [K,N] layout uses a quarter of every line */
    gd_tensor down_t;
} gpt_block;

struct gd_gpt_decoder {
    gd_context *ctx;
    gd_gpt_config cfg;
    gd_tensor token_embedding, lm_head, lm_head_bias, final_norm_w;
    gpt_block *blocks;
    gd_tensor *k_cache, *v_cache;
    int32_t *pos; /* host copy of the live lengths */
    /* device-resident decode state (state arena) */
    gd_tensor ids_dev, pos_dev, step_dev, step_rows_dev; /* step counters: one for the whole batch / one per row */
    gd_tensor x0_dev;     /* [B, Dm]: embedding rows of the tokens the fused resident step starts from */
    bool resident_x0;     /* x0_dev is kept current by the greedy-pick kernel */
    /* open resident session */
    bool resident_open;
    int32_t resident_max_steps, resident_steps, resident_hold, resident_unfused, resident_keep_logits;
    gd_backend_graph *resident_graph;
    gd_tensor resident_out_ids, resident_out_gaps;
    /* sampling front end (state arena): what the reference's generation loop keeps on the host */
    gd_tensor last_logits;                 /* [B, V] F16: logits of the last packed prefill */
    gd_tensor history, hist_len, finished; /* [B, max_seq], [B], [B] I32 */
    gd_tensor sample_state, sample_work;   /* generator + per-row records; [B*V] F32 */
    bool resident_sampling;
    gd_gpt_sampling sampling;
};

/* ---- deterministic initialisation (reference :32-48, 196-218) ----------------------- */

static uint64_t mix64(uint64_t x)
{
    x = (x ^ (x >> 30)) * UINT64_C(0xbf58476d1ce4e5b9);
    x = (x ^ (x >> 27)) * UINT64_C(0x94d049bb133111eb);
    return x ^ (x >> 31);
}

static uint64_t splitmix64(uint64_t x) { return mix64(x + UINT64_C(0x9e3779b97f4a7c15)); }

/* Draw number n (1-based) of the stream started at `seed`: the state advances by a constant, so any draw
 * is addressable and the fill below can run in parallel and still equal the reference's sequential loop. */
static double uniform_open_closed_at(uint64_t seed, uint64_t n)
{
    return ((double)(mix64(seed + n * UINT64_C(0x9e3779b97f4a7c15)) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
}

/* twin != NULL: t is [rows, cols]; the same values also go to twin as [cols, rows] */
static gd_status init_normal_twin(gd_context *ctx, gd_tensor *t, uint64_t seed, float stddev, gd_tensor *twin,
                                  int64_t rows, int64_t cols)
{
    int64_t n, pairs, pi;
    float *values;
    gd_status st;
    TRY(gd_tensor_numel(t, &n));
    values = (float *)malloc((size_t)n * sizeof(float));
    if (values == NULL) return GD_ERR_OUT_OF_MEMORY;
    pairs = (n + 1) / 2;
#pragma omp parallel for schedule(static)
    for (pi = 0; pi < pairs; ++pi) {
        const double u1 = uniform_open_closed_at(seed, 2U * (uint64_t)pi + 1U);
        const double u2 = uniform_open_closed_at(seed, 2U * (uint64_t)pi + 2U);
        const double radius = sqrt(-2.0 * log(u1)), angle = 6.283185307179586476925286766559 * u2;
        values[2 * pi] = (float)(radius * cos(angle) * (double)stddev);
        if (2 * pi + 1 < n) values[2 * pi + 1] = (float)(radius * sin(angle) * (double)stddev);
    }
    st = gd_tensor_write_f32(ctx, t, values, (size_t)n);
    if (st == GD_OK && twin != NULL) {
        float *turned = (float *)malloc((size_t)n * sizeof(float));
        int64_t r;
        if (turned == NULL) {
            free(values);
            return GD_ERR_OUT_OF_MEMORY;
        }
#pragma omp parallel for schedule(static)
        for (r = 0; r < cols; ++r) {
            int64_t c;
            for (c = 0; c < rows; ++c) turned[r * rows + c] = values[c * cols + r];
        }
        st = gd_tensor_write_f32(ctx, twin, turned, (size_t)n);
        free(turned);
    }
    free(values);
    return st;
}

static gd_status init_normal(gd_context *ctx, gd_tensor *t, uint64_t seed, float stddev)
{
    return init_normal_twin(ctx, t, seed, stddev, NULL, 0, 0);
}

static gd_status param(gd_context *ctx, gd_dtype dtype, uint32_t rank, int64_t d0, int64_t d1, gd_tensor *out)
{
    int64_t dims[2] = {d0, d1};
    return gd_tensor_empty(ctx, GD_ARENA_PARAMS, dtype, gd_shape_make(rank, dims), 256U, out);
}

static gd_status linear_init(gd_context *ctx, gpt_linear *l, int64_t in, int64_t out, bool transposed, uint64_t seed,
                             float stddev)
{
    l->transposed = transposed;
    TRY(param(ctx, GD_DTYPE_F16, 2U, transposed ? out : in, transposed ? in : out, &l->weight));
    TRY(init_normal(ctx, &l->weight, seed, stddev));
    TRY(param(ctx, GD_DTYPE_F16, 1U, out, 0, &l->bias));
    return gd_tensor_zero_(ctx, &l->bias);
}

static gd_status ones_param(gd_context *ctx, int64_t n, gd_tensor *out)
{
    int64_t dims[1] = {n};
    return gd_tensor_ones(ctx, GD_ARENA_PARAMS, GD_DTYPE_F16, gd_shape_make(1U, dims), 256U, out);
}

static size_t pad256(size_t n) { return (n + 255U) & ~(size_t)255U; }

size_t gd_gpt_params_bytes(const gd_gpt_config *c)
{
    const size_t Dm = (size_t)c->d_model, Hm = (size_t)c->mlp_hidden, V = (size_t)c->vocab;
    size_t per_layer = 2U * pad256(Dm * 2U) + pad256(3U * Dm * Dm * 2U) + pad256(3U * Dm * 2U) + pad256(Dm * Dm * 2U) +
                       pad256(Dm * 2U) + pad256(2U * Hm * Dm * 2U) + pad256(2U * Hm * 2U) + 2U * pad256(Hm * Dm * 2U) +
                       pad256(Dm * 2U);
    size_t total = pad256(V * Dm * 2U) * (c->tie_lm_head ? 1U : 2U) + pad256(V * 2U) + pad256(Dm * 2U);
    return total + per_layer * (size_t)c->n_layers + 4096U;
}

size_t gd_gpt_state_bytes(const gd_gpt_config *c)
{
    const size_t cache = pad256((size_t)c->batch * (size_t)c->max_seq * (size_t)c->n_heads * (size_t)c->head_dim * 2U);
    const size_t B = (size_t)c->batch, V = (size_t)c->vocab;
    const size_t sampling = pad256(B * V * 2U) + pad256(gd_backend_sample_work_count((uint32_t)B, (uint32_t)V) * 4U) +
                            pad256(B * (size_t)c->max_seq * 4U) +
                            2U * pad256(B * 4U) + pad256(gd_backend_sample_state_count((uint32_t)B) * 4U);
    return cache * 2U * (size_t)c->n_layers + 4U * pad256((size_t)c->batch * 4U) +
           pad256((size_t)c->batch * (size_t)c->d_model * 2U) + sampling + 4096U;
}

size_t gd_gpt_scratch_bytes(const gd_gpt_config *c, int32_t max_prefill_tokens)
{
    /* every operator output of every layer lives until the step ends (bump allocation): 13 d_model-wide and one
     * 2 x hidden-wide F16 tensor per layer and row, each padded to 256 bytes; 10 % slack; one transient activation of
     * the many-row swiglu path; logits, picks and records; 64 MiB for everything small */
    const size_t rows = (size_t)(max_prefill_tokens > c->batch ? max_prefill_tokens : c->batch);
    const size_t picked = c->m3_block_size > 0 ? (size_t)c->n_heads * 16U * 4U + 256U : 0U; /* block ids of a row */
    const size_t per_row = 2U * (13U * (size_t)c->d_model + 2U * (size_t)c->mlp_hidden) + 14U * 256U + picked;
    const size_t layers = rows * per_row * (size_t)c->n_layers;
    const size_t angles = (rows + 32U) * ((size_t)c->head_dim * 4U + 4U) + 3U * 256U; /* cos, sin and cache row per prompt row */
    return layers + layers / 10U + rows * ((size_t)c->d_model * 4U + (size_t)c->mlp_hidden * 2U) + angles +
           (size_t)c->batch * (size_t)c->vocab * 4U + ((size_t)64 << 20);
}

gd_status gd_gpt_decoder_create(gd_context *ctx, const gd_gpt_config *cfg, gd_gpt_decoder **out)
{
    gd_gpt_decoder *d;
    const float std = 0.02f;
    float resid;
    int32_t l;
    int64_t cache_dims[4], bdim[1], one[1] = {1};
    gd_status st = GD_OK;
    if (out != NULL) *out = NULL;
    if (ctx == NULL || cfg == NULL || out == NULL || cfg->vocab <= 0 || cfg->d_model <= 0 || cfg->n_layers <= 0 ||
        cfg->n_heads <= 0 || cfg->head_dim <= 0 || cfg->mlp_hidden <= 0 || cfg->max_seq <= 0 || cfg->batch <= 0 ||
        cfg->n_heads * cfg->head_dim != cfg->d_model || cfg->sdpa_window < 0 || cfg->m3_block_size < 0 ||
        cfg->m3_block_size > 128 || cfg->m3_topk_blocks < 0 || cfg->m3_topk_blocks > 16 || cfg->m3_init_blocks < 0 ||
        cfg->m3_local_blocks < 0 || (cfg->m3_block_size > 0 && cfg->head_dim > 64))
        return GD_ERR_INVALID_ARGUMENT;
    d = (gd_gpt_decoder *)calloc(1, sizeof(*d));
    if (d == NULL) return GD_ERR_OUT_OF_MEMORY;
    d->ctx = ctx;
    d->cfg = *cfg;
    if (!(d->cfg.rms_eps > 0.0f)) d->cfg.rms_eps = 1.0e-5f;
    if (!(d->cfg.rope_theta > 0.0f)) d->cfg.rope_theta = 10000.0f;
    d->blocks = (gpt_block *)calloc((size_t)cfg->n_layers, sizeof(gpt_block));
    d->k_cache = (gd_tensor *)calloc((size_t)cfg->n_layers, sizeof(gd_tensor));
    d->v_cache = (gd_tensor *)calloc((size_t)cfg->n_layers, sizeof(gd_tensor));
    d->pos = (int32_t *)calloc((size_t)cfg->batch, sizeof(int32_t));
    if (d->blocks == NULL || d->k_cache == NULL || d->v_cache == NULL || d->pos == NULL) {
        gd_gpt_decoder_destroy(d);
        return GD_ERR_OUT_OF_MEMORY;
    }
    resid = std / sqrtf(2.0f * (float)cfg->n_layers);
#define STEP(expr) do { if (st == GD_OK) st = (expr); } while (0)
    STEP(param(ctx, GD_DTYPE_F16, 2U, cfg->vocab, cfg->d_model, &d->token_embedding));
    STEP(init_normal(ctx, &d->token_embedding, splitmix64(cfg->seed ^ UINT64_C(0xabc001)), std));
    if (cfg->tie_lm_head) {
        d->lm_head = d->token_embedding;
    } else {
        STEP(param(ctx, GD_DTYPE_F16, 2U, cfg->vocab, cfg->d_model, &d->lm_head));
        STEP(init_normal(ctx, &d->lm_head, splitmix64(cfg->seed ^ UINT64_C(0xabc002)), std));
    }
    STEP(param(ctx, GD_DTYPE_F16, 1U, cfg->vocab, 0, &d->lm_head_bias));
    STEP(gd_tensor_zero_(ctx, &d->lm_head_bias));
    STEP(ones_param(ctx, cfg->d_model, &d->final_norm_w));
    cache_dims[0] = cfg->batch;
    cache_dims[1] = cfg->max_seq;
    cache_dims[2] = cfg->n_heads;
    cache_dims[3] = cfg->head_dim;
    for (l = 0; l < cfg->n_layers && st == GD_OK; ++l) {
        gpt_block *b = &d->blocks[l];
        const uint64_t bs = cfg->seed ^ ((uint64_t)l << 8);
        STEP(ones_param(ctx, cfg->d_model, &b->attn_norm_w));
        STEP(ones_param(ctx, cfg->d_model, &b->mlp_norm_w));
        STEP(linear_init(ctx, &b->qkv_proj, cfg->d_model, 3 * (int64_t)cfg->d_model, true, splitmix64(bs ^ 1U), std));
        STEP(linear_init(ctx, &b->attn_proj, cfg->d_model, cfg->d_model, true, splitmix64(bs ^ 2U), resid));
        STEP(linear_init(ctx, &b->up_gate, cfg->d_model, 2 * (int64_t)cfg->mlp_hidden, true, splitmix64(bs ^ 3U), std));
        b->down_proj.transposed = false;
        STEP(param(ctx, GD_DTYPE_F16, 2U, cfg->mlp_hidden, cfg->d_model, &b->down_proj.weight));
        STEP(param(ctx, GD_DTYPE_F16, 2U, cfg->d_model, cfg->mlp_hidden, &b->down_t));
        STEP(init_normal_twin(ctx, &b->down_proj.weight, splitmix64(bs ^ 4U), resid, &b->down_t, cfg->mlp_hidden,
                              cfg->d_model));
        STEP(param(ctx, GD_DTYPE_F16, 1U, cfg->d_model, 0, &b->down_proj.bias));
        STEP(gd_tensor_zero_(ctx, &b->down_proj.bias));
        STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_F16, gd_shape_make(4U, cache_dims), 256U, &d->k_cache[l]));
        STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_F16, gd_shape_make(4U, cache_dims), 256U, &d->v_cache[l]));
    }
    bdim[0] = cfg->batch;
    STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_I32, gd_shape_make(1U, bdim), 256U, &d->ids_dev));
    STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_I32, gd_shape_make(1U, bdim), 256U, &d->pos_dev));
    STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_I32, gd_shape_make(1U, one), 256U, &d->step_dev));
    STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_I32, gd_shape_make(1U, bdim), 256U, &d->step_rows_dev));
    {
        int64_t xdim[2] = {cfg->batch, cfg->d_model};
        STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_F16, gd_shape_make(2U, xdim), 256U, &d->x0_dev));
    }
    {
        int64_t ldim[2] = {cfg->batch, cfg->vocab}, hdim[2] = {cfg->batch, cfg->max_seq};
        int64_t sdim[1] = {(int64_t)gd_backend_sample_state_count((uint32_t)cfg->batch)};
        int64_t wdim[1] = {(int64_t)gd_backend_sample_work_count((uint32_t)cfg->batch, (uint32_t)cfg->vocab)};
        STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_F16, gd_shape_make(2U, ldim), 256U, &d->last_logits));
        STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_I32, gd_shape_make(2U, hdim), 256U, &d->history));
        STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_I32, gd_shape_make(1U, bdim), 256U, &d->hist_len));
        STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_I32, gd_shape_make(1U, bdim), 256U, &d->finished));
        STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_I32, gd_shape_make(1U, sdim), 256U, &d->sample_state));
        STEP(gd_tensor_zeros(ctx, GD_ARENA_STATE, GD_DTYPE_F32, gd_shape_make(1U, wdim), 256U, &d->sample_work));
    }
#undef STEP
    if (st != GD_OK) {
        gd_gpt_decoder_destroy(d);
        return st;
    }
    *out = d;
    return GD_OK;
}

void gd_gpt_decoder_destroy(gd_gpt_decoder *d)
{
    if (d == NULL) return;
    free(d->blocks);
    free(d->k_cache);
    free(d->v_cache);
    free(d->pos);
    free(d);
}

gd_tensor *gd_gpt_decoder_tensor(gd_gpt_decoder *d, const char *name, int32_t layer)
{
    gpt_block *b;
    if (d == NULL || name == NULL) return NULL;
    if (!strcmp(name, "embed")) return &d->token_embedding;
    if (!strcmp(name, "lm_head")) return &d->lm_head;
    if (!strcmp(name, "lm_bias")) return &d->lm_head_bias;
    if (!strcmp(name, "final_norm")) return &d->final_norm_w;
    if (layer < 0 || layer >= d->cfg.n_layers) return NULL;
    b = &d->blocks[layer];
    if (!strcmp(name, "attn_norm")) return &b->attn_norm_w;
    if (!strcmp(name, "mlp_norm")) return &b->mlp_norm_w;
    if (!strcmp(name, "w_qkv")) return &b->qkv_proj.weight;
    if (!strcmp(name, "b_qkv")) return &b->qkv_proj.bias;
    if (!strcmp(name, "w_attn")) return &b->attn_proj.weight;
    if (!strcmp(name, "b_attn")) return &b->attn_proj.bias;
    if (!strcmp(name, "w_upgate")) return &b->up_gate.weight;
    if (!strcmp(name, "b_upgate")) return &b->up_gate.bias;
    if (!strcmp(name, "w_down")) return &b->down_proj.weight;
    if (!strcmp(name, "w_down_t")) return &b->down_t;
    if (!strcmp(name, "b_down")) return &b->down_proj.bias;
    if (!strcmp(name, "last_logits")) return &d->last_logits;
    if (!strcmp(name, "k_cache")) return &d->k_cache[layer];
    if (!strcmp(name, "v_cache")) return &d->v_cache[layer];
    return NULL;
}

int32_t *gd_gpt_decoder_positions(gd_gpt_decoder *d) { return d != NULL ? d->pos : NULL; }

/* ---- weights from a checkpoint of the reference ------------------------------------------ */

typedef struct ckpt_slot {
    char path[GD_CHECKPOINT_PATH_MAX];
    gd_tensor *dst, *second; /* second: another tensor that receives the same values (untied LM head) */
    gd_tensor *turned;       /* [cols, rows] copy of a [rows, cols] weight */
    const gd_checkpoint_entry *entry;
} ckpt_slot;

static void slot_set(ckpt_slot *s, gd_tensor *dst, const char *fmt, int32_t layer)
{
    memset(s, 0, sizeof(*s));
    (void)snprintf(s->path, sizeof(s->path), fmt, (int)layer);
    s->dst = dst;
}

/* same test as the reference's gd_ckpt_file_entry_matches_tensor (src/nn/module_io.c:809-824) */
static bool entry_fits(const gd_checkpoint_entry *e, const gd_tensor *t)
{
    size_t nbytes = 0U;
    uint32_t i;
    if (gd_tensor_logical_nbytes(t, &nbytes) != GD_OK || e->dtype != t->dtype || e->rank != t->rank ||
        e->nbytes != (uint64_t)nbytes)
        return false;
    for (i = 0U; i < t->rank; ++i) {
        if (e->shape[i] != t->shape[i]) return false;
    }
    return true;
}

gd_status gd_gpt_decoder_load_checkpoint(gd_gpt_decoder *d, const char *path, int32_t strict)
{
    gd_checkpoint *ck = NULL;
    ckpt_slot *slots;
    unsigned char *bytes = NULL, *flipped = NULL;
    size_t n_slots, capacity = 0U, si;
    uint32_t fi;
    int32_t l;
    gd_status st;
    if (d == NULL || path == NULL || path[0] == '\0') return GD_ERR_INVALID_ARGUMENT;
    if (d->resident_open) return GD_ERR_BUSY;
    /* the names gpt_lm_init gives its parameters (gpt_lm_shared.c:272-279, 303-338, 382-413) */
    n_slots = 3U + 10U * (size_t)d->cfg.n_layers;
    slots = (ckpt_slot *)calloc(n_slots, sizeof(*slots));
    if (slots == NULL) return GD_ERR_OUT_OF_MEMORY;
    slot_set(&slots[0], &d->token_embedding, "gpt_lm.token_embedding", 0);
    if (!d->cfg.tie_lm_head) slots[0].second = &d->lm_head; /* the reference's head is the embedding table */
    slot_set(&slots[1], &d->lm_head_bias, "gpt_lm.lm_head_bias", 0);
    slot_set(&slots[2], &d->final_norm_w, "gpt_lm.final_norm_w", 0);
    for (l = 0; l < d->cfg.n_layers; ++l) {
        gpt_block *b = &d->blocks[l];
        ckpt_slot *s = &slots[3U + 10U * (size_t)l];
        slot_set(&s[0], &b->attn_norm_w, "gpt_lm.blocks.%d.attn_norm_w", l);
        slot_set(&s[1], &b->mlp_norm_w, "gpt_lm.blocks.%d.mlp_norm_w", l);
        slot_set(&s[2], &b->qkv_proj.weight, "gpt_lm.blocks.%d.qkv_proj.weight", l);
        slot_set(&s[3], &b->qkv_proj.bias, "gpt_lm.blocks.%d.qkv_proj.bias", l);
        slot_set(&s[4], &b->attn_proj.weight, "gpt_lm.blocks.%d.attn_proj.weight", l);
        slot_set(&s[5], &b->attn_proj.bias, "gpt_lm.blocks.%d.attn_proj.bias", l);
        slot_set(&s[6], &b->up_gate.weight, "gpt_lm.blocks.%d.up_gate.weight", l);
        slot_set(&s[7], &b->up_gate.bias, "gpt_lm.blocks.%d.up_gate.bias", l);
        slot_set(&s[8], &b->down_proj.weight, "gpt_lm.blocks.%d.down_proj.weight", l);
        s[8].turned = &b->down_t;
        slot_set(&s[9], &b->down_proj.bias, "gpt_lm.blocks.%d.down_proj.bias", l);
    }
    st = gd_checkpoint_open(path, &ck);
    /* everything is checked before the first byte is written (module_io.c:868-899): a refused file leaves the
     * decoder's weights as they were */
    for (fi = 0U; st == GD_OK && fi < gd_checkpoint_count(ck); ++fi) {
        const gd_checkpoint_entry *e = gd_checkpoint_entry_at(ck, fi);
        ckpt_slot *hit = NULL;
        if (e->flags == GD_CHECKPOINT_ENTRY_BUFFER) continue; /* the decoder registers no buffers */
        for (si = 0U; si < n_slots; ++si) {
            if (strcmp(slots[si].path, e->path) == 0) {
                hit = &slots[si];
                break;
            }
        }
        if (hit == NULL) {
            if (strict) st = GD_ERR_BAD_STATE; /* unexpected tensor */
            continue;
        }
        if (!entry_fits(e, hit->dst)) {
            st = GD_ERR_BAD_STATE; /* dtype, rank, shape or size differ */
            break;
        }
        hit->entry = e;
        if ((size_t)e->nbytes > capacity) capacity = (size_t)e->nbytes;
    }
    for (si = 0U; st == GD_OK && strict && si < n_slots; ++si) {
        if (slots[si].entry == NULL) st = GD_ERR_BAD_STATE; /* missing tensor */
    }
    if (st == GD_OK && capacity > 0U) {
        bytes = (unsigned char *)malloc(capacity);
        flipped = (unsigned char *)malloc(capacity);
        if (bytes == NULL || flipped == NULL) st = GD_ERR_OUT_OF_MEMORY;
    }
    for (si = 0U; st == GD_OK && si < n_slots; ++si) {
        const ckpt_slot *s = &slots[si];
        size_t nbytes;
        if (s->entry == NULL) continue;
        nbytes = (size_t)s->entry->nbytes;
        st = gd_checkpoint_read(ck, s->entry, 0U, bytes, nbytes);
        if (st == GD_OK) st = gd_tensor_write(d->ctx, s->dst, bytes, nbytes);
        if (st == GD_OK && s->second != NULL) st = gd_tensor_write(d->ctx, s->second, bytes, nbytes);
        if (st == GD_OK && s->turned != NULL) {
            const int64_t rows = s->dst->shape[0], cols = s->dst->shape[1];
            const uint16_t *src = (const uint16_t *)bytes;
            uint16_t *out = (uint16_t *)flipped;
            int64_t c;
#pragma omp parallel for schedule(static)
            for (c = 0; c < cols; ++c) {
                int64_t r;
                for (r = 0; r < rows; ++r) out[c * rows + r] = src[r * cols + c];
            }
            st = gd_tensor_write(d->ctx, s->turned, flipped, nbytes);
        }
    }
    free(bytes);
    free(flipped);
    gd_checkpoint_close(ck);
    free(slots);
    return st;
}

/* value of "key=value" on a line of its own in the metadata blob, as the reference's inference programs look it
 * up (examples/gpt_lm/infer.c:344-376); false if absent or not a whole non-negative number that fits an int32 */
static bool metadata_i32(const char *blob, size_t len, const char *key, int32_t *out)
{
    const size_t key_len = strlen(key);
    size_t at = 0U;
    while (at < len) {
        size_t end = at;
        while (end < len && blob[end] != '\n') ++end;
        if (end > at + key_len && strncmp(blob + at, key, key_len) == 0 && blob[at + key_len] == '=') {
            int64_t v = 0;
            size_t i = at + key_len + 1U;
            if (i == end) return false;
            for (; i < end; ++i) {
                if (blob[i] < '0' || blob[i] > '9') return false;
                v = v * 10 + (blob[i] - '0');
                if (v > INT32_MAX) return false;
            }
            *out = (int32_t)v;
            return true;
        }
        at = end < len ? end + 1U : end;
    }
    return false;
}

gd_status gd_gpt_config_from_checkpoint(const char *path, gd_gpt_config *cfg)
{
    gd_checkpoint *ck = NULL;
    const gd_checkpoint_entry *embed, *down;
    char *blob = NULL;
    size_t blob_len = 0U;
    int32_t layers = 0, v;
    uint32_t i;
    gd_status st;
    if (path == NULL || cfg == NULL) return GD_ERR_INVALID_ARGUMENT;
    st = gd_checkpoint_open(path, &ck);
    if (st != GD_OK) return st;
    /* the directory fixes vocabulary, width, MLP width and depth */
    embed = gd_checkpoint_find(ck, "gpt_lm.token_embedding");
    down = gd_checkpoint_find(ck, "gpt_lm.blocks.0.down_proj.weight");
    for (i = 0U; i < gd_checkpoint_count(ck); ++i) {
        const char *p = gd_checkpoint_entry_at(ck, i)->path;
        int n = -1, used = 0;
        if (sscanf(p, "gpt_lm.blocks.%d.attn_norm_w%n", &n, &used) == 1 && used > 0 && p[used] == '\0' && n >= layers)
            layers = n + 1;
    }
    if (embed == NULL || down == NULL || embed->rank != 2U || down->rank != 2U || layers <= 0 ||
        embed->shape[0] > INT32_MAX || embed->shape[1] > INT32_MAX || down->shape[0] > INT32_MAX ||
        down->shape[1] != embed->shape[1]) {
        gd_checkpoint_close(ck);
        return GD_ERR_BAD_STATE;
    }
    cfg->vocab = (int32_t)embed->shape[0];
    cfg->d_model = (int32_t)embed->shape[1];
    cfg->mlp_hidden = (int32_t)down->shape[0];
    cfg->n_layers = layers;
    gd_checkpoint_close(ck); /* embed and down point into ck: nothing reads them past this line */
    cfg->tie_lm_head = 1;
    /* the metadata the reference's trainer writes (examples/gpt_lm/main.c:1836-1864) carries what shapes cannot
     * tell; where it repeats what the directory fixes, the two must agree */
    st = gd_checkpoint_read_metadata(path, &blob, &blob_len);
    if (st != GD_OK) return st;
    if ((metadata_i32(blob, blob_len, "vocab_size", &v) && v != cfg->vocab) ||
        (metadata_i32(blob, blob_len, "d_model", &v) && v != cfg->d_model) ||
        (metadata_i32(blob, blob_len, "mlp_hidden", &v) && v != cfg->mlp_hidden) ||
        (metadata_i32(blob, blob_len, "n_layers", &v) && v != cfg->n_layers)) {
        free(blob);
        return GD_ERR_BAD_STATE;
    }
    if (metadata_i32(blob, blob_len, "n_heads", &v)) cfg->n_heads = v;
    if (metadata_i32(blob, blob_len, "head_dim", &v)) cfg->head_dim = v;
    if (metadata_i32(blob, blob_len, "sdpa_window", &v)) cfg->sdpa_window = v;
    if (cfg->max_seq <= 0 && metadata_i32(blob, blob_len, "context_length", &v)) cfg->max_seq = v;
    /* "architecture=minimax_m3" switches the packed prefill to picked blocks (the reference's inference programs
     * read the same keys, infer.c:407-421); the other lines give the block size and counts */
    {
        static const char key[] = "architecture=minimax_m3";
        size_t at = 0U;
        bool m3 = false;
        while (at < blob_len && !m3) {
            size_t end = at;
            while (end < blob_len && blob[end] != '\n') ++end;
            m3 = end - at == sizeof(key) - 1U && strncmp(blob + at, key, sizeof(key) - 1U) == 0;
            at = end < blob_len ? end + 1U : end;
        }
        if (m3) {
            cfg->m3_block_size = metadata_i32(blob, blob_len, "minimax_m3_block_size", &v) && v > 0 ? v : 128;
            cfg->m3_topk_blocks = metadata_i32(blob, blob_len, "minimax_m3_topk_blocks", &v) && v > 0 ? v : 3;
            cfg->m3_init_blocks = metadata_i32(blob, blob_len, "minimax_m3_init_blocks", &v) ? v : 1;
            cfg->m3_local_blocks = metadata_i32(blob, blob_len, "minimax_m3_local_blocks", &v) ? v : 1;
        }
    }
    free(blob);
    if (cfg->n_heads > 0 && cfg->head_dim <= 0 && cfg->d_model % cfg->n_heads == 0) cfg->head_dim = cfg->d_model / cfg->n_heads;
    if (cfg->head_dim > 0 && cfg->n_heads <= 0 && cfg->d_model % cfg->head_dim == 0) cfg->n_heads = cfg->d_model / cfg->head_dim;
    if (cfg->n_heads <= 0 || cfg->head_dim <= 0 || (int64_t)cfg->n_heads * cfg->head_dim != cfg->d_model)
        return GD_ERR_BAD_STATE;
    return GD_OK;
}

/* ---- forward pieces -------------------------------------------------------------------- */

/* reference src/nn/module.c:1012-1028 */
static gd_status linear_forward(gd_context *ctx, const gpt_linear *l, const gd_tensor *x, gd_tensor *out)
{
    if (l->transposed) return gd_linear_transposed_weight(ctx, x, &l->weight, &l->bias, out);
    return gd_linear(ctx, x, &l->weight, &l->bias, out);
}

static void tview(const gd_tensor *t, gd_backend_tensor_view *v);
static gd_status fused_project_rows(gd_gpt_decoder *d, int64_t B, const gd_tensor *x, int64_t x_cols,
                                    const gpt_linear *lin, const gd_tensor *w_override, const gd_tensor *bias,
                                    const gd_tensor *residual, const gd_tensor *norm_w, uint32_t prologue,
                                    uint32_t epilogue, int64_t n_out, gd_tensor *y);

/* attention input -> block output of the packed prefill: the two residual additions ride in the epilogues of the
 * projections in front of them (same F16 rounding points as the separate gd_add), everything else as block_tail */
static gd_status block_tail_prefill(gd_gpt_decoder *d, const gpt_block *b, const gd_tensor *residual,
                                    const gd_tensor *attn_flat, gd_tensor *out)
{
    gd_context *ctx = d->ctx;
    const int64_t rows = attn_flat->shape[0], Dm = d->cfg.d_model, Hm = d->cfg.mlp_hidden;
    gd_tensor attn_resid, mlp_normed, up_gate, gated;
    TRY(fused_project_rows(d, rows, attn_flat, Dm, &b->attn_proj, NULL, &b->attn_proj.bias, residual, NULL, 0U, 0U, Dm,
                           &attn_resid));
    TRY(gd_rms_norm(ctx, &attn_resid, &b->mlp_norm_w, d->cfg.rms_eps, &mlp_normed));
    if (b->up_gate.transposed && (Dm % 8) == 0) {
        /* swiglu in the epilogue of the up/gate projection: the [rows, 2H] intermediate is never written */
        TRY(fused_project_rows(d, rows, &mlp_normed, Dm, &b->up_gate, NULL, &b->up_gate.bias, NULL, NULL, 0U, 1U, Hm,
                               &gated));
    } else {
        TRY(linear_forward(ctx, &b->up_gate, &mlp_normed, &up_gate));
        TRY(gd_swiglu_split(ctx, &up_gate, &gated));
    }
    /* through the [N,K] twin of the down projection's [K,N] weight, as the decode step does: the same products and
     * sums, and the kernel's small tiles (the rows of the last, partly filled round) are a third faster on [N,K] */
    return fused_project_rows(d, rows, &gated, Hm, &b->down_proj, &b->down_t, &b->down_proj.bias, &attn_resid, NULL, 0U,
                              0U, Dm, out);
}

/* attention input -> block output, shared by decode and prefill (reference :1052-1070, 941-958) */
static gd_status block_tail(gd_gpt_decoder *d, const gpt_block *b, const gd_tensor *residual, const gd_tensor *attn_flat,
                            gd_tensor *out)
{
    gd_context *ctx = d->ctx;
    gd_tensor attn_proj, attn_resid, mlp_normed, up_gate, mlp_proj;
    TRY(linear_forward(ctx, &b->attn_proj, attn_flat, &attn_proj));
    TRY(gd_add(ctx, residual, &attn_proj, &attn_resid));
    TRY(gd_rms_norm(ctx, &attn_resid, &b->mlp_norm_w, d->cfg.rms_eps, &mlp_normed));
    TRY(linear_forward(ctx, &b->up_gate, &mlp_normed, &up_gate));
    TRY(gd_swiglu_split_linear(ctx, &up_gate, &b->down_proj.weight, &b->down_proj.bias, &mlp_proj));
    return gd_add(ctx, &attn_resid, &mlp_proj, out);
}

static gd_status block_decode(gd_gpt_decoder *d, int32_t l, const gd_tensor *x, const gd_tensor *positions,
                              const gd_tensor *cache_positions, gd_tensor *out)
{
    gd_context *ctx = d->ctx;
    const gpt_block *b = &d->blocks[l];
    const gd_gpt_config *c = &d->cfg;
    const gd_rope_config rope = {c->rope_theta, c->head_dim, false};
    const gd_sdpa_decode_config sdpa = {0.0f, c->sdpa_window, 0};
    gd_tensor normed, qkv, q3, k3, v3, q, k, v, attn, attn_flat;
    int64_t q_shape[4] = {x->shape[0], 1, c->n_heads, c->head_dim};
    int64_t flat_shape[2] = {x->shape[0], c->d_model};
    TRY(gd_rms_norm(ctx, x, &b->attn_norm_w, c->rms_eps, &normed));
    TRY(linear_forward(ctx, &b->qkv_proj, &normed, &qkv));
    TRY(gd_qkv_split_rope(ctx, &qkv, positions, c->n_heads, c->head_dim, &rope, &q3, &k3, &v3));
    TRY(gd_reshape(ctx, &q3, gd_shape_make(4U, q_shape), &q));
    TRY(gd_reshape(ctx, &k3, gd_shape_make(4U, q_shape), &k));
    TRY(gd_reshape(ctx, &v3, gd_shape_make(4U, q_shape), &v));
    TRY(gd_kv_cache_append_positions(ctx, &d->k_cache[l], &d->v_cache[l], cache_positions, &k, &v));
    TRY(gd_sdpa_decode_positions(ctx, &q, &d->k_cache[l], &d->v_cache[l], cache_positions, &sdpa, &attn));
    TRY(gd_reshape(ctx, &attn, gd_shape_make(2U, flat_shape), &attn_flat));
    return block_tail(d, b, x, &attn_flat, out);
}

/* angles and cache rows of the packed prompt rows (gd_backend_rope_table_packed), shared by the layers of a prefill */
typedef struct prefill_rope_rows {
    gd_tensor cos_rows, sin_rows, cache_rows;
} prefill_rope_rows;

static bool mview(const gd_tensor *t, int64_t rows, int64_t cols, gd_backend_matrix_view *m);
static void vview(const gd_tensor *t, gd_backend_vector_view *v);
static gd_status scratch_f16(gd_context *ctx, int64_t rows, int64_t cols, gd_tensor *out);

/* the qkv projection can carry rotation, split and cache append in its epilogue (gd_backend_linear_qkv_rope_packed) */
static bool prefill_rope_in_projection(const gd_gpt_decoder *d)
{
    const gd_gpt_config *c = &d->cfg;
    const bool m3 = c->m3_block_size > 0 && c->m3_topk_blocks > 0 &&
                    (int64_t)c->max_seq > (int64_t)c->m3_block_size * 8 &&
                    (int64_t)c->m3_block_size * c->m3_topk_blocks * 2 < (int64_t)c->max_seq;
    return !m3 && (c->head_dim == 64 || c->head_dim == 128) && (c->d_model % 256) == 0 &&
           d->blocks[0].qkv_proj.transposed && d->blocks[0].qkv_proj.weight.dtype == GD_DTYPE_F16 &&
           (uint64_t)c->batch * (uint64_t)c->max_seq * (uint64_t)c->d_model * 2U < 0xffffffffULL;
}

static gd_status block_prefill(gd_gpt_decoder *d, int32_t l, const gd_tensor *x, const gd_tensor *positions,
                               const gd_tensor *cu, const gd_tensor *cache_positions, const prefill_rope_rows *rows,
                               gd_tensor *out)
{
    gd_context *ctx = d->ctx;
    const gpt_block *b = &d->blocks[l];
    const gd_gpt_config *c = &d->cfg;
    const gd_rope_config rope = {c->rope_theta, c->head_dim, false};
    const gd_sdpa_varlen_config sdpa = {0.0f, true, c->sdpa_window, 0, c->max_seq};
    const bool m3 = c->m3_block_size > 0 && c->m3_topk_blocks > 0 &&
                    (int64_t)c->max_seq > (int64_t)c->m3_block_size * 8 &&
                    (int64_t)c->m3_block_size * c->m3_topk_blocks * 2 < (int64_t)c->max_seq;
    /* the prefill appends every sequence at cache position 0 (gd_gpt_decoder_prefill), so the attention can read the
     * keys and values of a sequence where the append has just put them, and the packed k / v are never written */
    const bool from_caches = !m3 && (c->head_dim == 64 || c->head_dim == 128) &&
                             (uint64_t)c->batch * (uint64_t)c->max_seq * (uint64_t)c->n_heads * (uint64_t)c->head_dim * 2U <
                                 0xffffffffULL;
    gd_tensor normed, qkv, q, k, v, attn, attn_flat;
    int64_t flat_shape[2] = {x->shape[0], c->d_model};
    bool attended = false;
    TRY(gd_rms_norm(ctx, x, &b->attn_norm_w, c->rms_eps, &normed));
    if (rows != NULL && from_caches && x->shape[0] >= 256) {
        /* rotation, split and cache append in the epilogue of the projection's tiles; attention from the caches */
        const gd_backend_sdpa_varlen_args va = {(float)(1.0 / sqrt((double)c->head_dim)), 1U, (uint32_t)c->sdpa_window, 0U,
                                                (uint32_t)c->max_seq, 0U};
        const int64_t N = x->shape[0];
        int64_t dims[3] = {N, c->n_heads, c->head_dim};
        gd_backend_matrix_view xm, wm, workm;
        gd_backend_vector_view bv;
        gd_backend_tensor_view vcos, vsin, vrows, vq, vkc, vvc, vcu, vo;
        gd_status st;
        TRY(gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F16, gd_shape_make(3U, dims), 256U, &q));
        TRY(scratch_f16(ctx, N, 3 * (int64_t)c->d_model, &qkv));
        mview(&normed, N, c->d_model, &xm);
        mview(&b->qkv_proj.weight, b->qkv_proj.weight.shape[0], b->qkv_proj.weight.shape[1], &wm);
        mview(&qkv, N, 3 * (int64_t)c->d_model, &workm);
        vview(&b->qkv_proj.bias, &bv);
        tview(&rows->cos_rows, &vcos);
        tview(&rows->sin_rows, &vsin);
        tview(&rows->cache_rows, &vrows);
        tview(&q, &vq);
        tview(&d->k_cache[l], &vkc);
        tview(&d->v_cache[l], &vvc);
        tview(cu, &vcu);
        /* bias mode 2: gd_linear_transposed_weight is matmul_nt + add, two roundings */
        st = gd_backend_linear_qkv_rope_packed(gd_context_backend(ctx), &xm, &wm, &bv, &vcos, &vsin, &vrows, &vq, &vkc, &vvc,
                                               &workm, (uint32_t)c->n_heads, (uint32_t)c->head_dim, 2U);
        if (st == GD_OK) {
            TRY(gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F16, gd_shape_make(3U, dims), 256U, &attn));
            tview(&attn, &vo);
            TRY(gd_backend_sdpa_varlen_cached(gd_context_backend(ctx), &vq, &vkc, &vvc, &vcu, &vo, &va));
            TRY(gd_reshape(ctx, &attn, gd_shape_make(2U, flat_shape), &attn_flat));
            return block_tail_prefill(d, b, x, &attn_flat, out);
        }
        if (st != GD_ERR_UNSUPPORTED) return st;
    }
    TRY(linear_forward(ctx, &b->qkv_proj, &normed, &qkv));
    if ((c->head_dim % 16) == 0 && qkv.dtype == GD_DTYPE_F16) {
        /* rotation, split and cache append in one pass over the projection: the appended rows are not read back */
        const gd_backend_rope_args ra = {c->rope_theta, (uint32_t)c->head_dim, 0U};
        int64_t dims[3] = {x->shape[0], c->n_heads, c->head_dim};
        gd_backend_tensor_view vqkv, vpos, vcp, vcu, vq, vk, vv, vkc, vvc;
        TRY(gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F16, gd_shape_make(3U, dims), 256U, &q));
        if (!from_caches) {
            TRY(gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F16, gd_shape_make(3U, dims), 256U, &k));
            TRY(gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F16, gd_shape_make(3U, dims), 256U, &v));
            tview(&k, &vk);
            tview(&v, &vv);
        }
        tview(&qkv, &vqkv);
        tview(positions, &vpos);
        tview(cache_positions, &vcp);
        tview(cu, &vcu);
        tview(&q, &vq);
        tview(&d->k_cache[l], &vkc);
        tview(&d->v_cache[l], &vvc);
        TRY(gd_backend_qkv_rope_append_packed(gd_context_backend(ctx), &vqkv, &vpos, &vcp, &vcu, &vq,
                                              from_caches ? NULL : &vk, from_caches ? NULL : &vv, &vkc, &vvc,
                                              (uint32_t)c->n_heads, (uint32_t)c->head_dim, &ra));
        if (from_caches) {
            const gd_backend_sdpa_varlen_args va = {(float)(1.0 / sqrt((double)c->head_dim)), 1U, (uint32_t)c->sdpa_window,
                                                    0U, (uint32_t)c->max_seq, 0U};
            gd_backend_tensor_view vo;
            TRY(gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F16, gd_shape_make(3U, dims), 256U, &attn));
            tview(&attn, &vo);
            TRY(gd_backend_sdpa_varlen_cached(gd_context_backend(ctx), &vq, &vkc, &vvc, &vcu, &vo, &va));
            attended = true;
        }
    } else {
        TRY(gd_qkv_split_rope(ctx, &qkv, positions, c->n_heads, c->head_dim, &rope, &q, &k, &v));
        TRY(gd_kv_cache_append_packed(ctx, &d->k_cache[l], &d->v_cache[l], cache_positions, cu, &k, &v));
    }
    /* MiniMax-M3: picked blocks when the context is long enough for that to matter (reference :588-600, 918-933) */
    if (attended) {
        /* done above, from the caches */
    } else if (m3) {
        const gd_minimax_m3_sparse_config m3 = {0.0f, c->m3_block_size, c->m3_topk_blocks, c->m3_init_blocks,
                                                c->m3_local_blocks, c->max_seq};
        gd_tensor picked;
        TRY(gd_minimax_m3_index_topk(ctx, &q, &k, cu, &m3, &picked));
        TRY(gd_minimax_m3_sparse_attention(ctx, &q, &k, &v, cu, &picked, &m3, &attn));
    } else {
        TRY(gd_sdpa_varlen(ctx, &q, &k, &v, cu, &sdpa, &attn));
    }
    TRY(gd_reshape(ctx, &attn, gd_shape_make(2U, flat_shape), &attn_flat));
    if (x->shape[0] >= 128) return block_tail_prefill(d, b, x, &attn_flat, out);
    return block_tail(d, b, x, &attn_flat, out);
}

static gd_status data_i32(gd_context *ctx, const int32_t *values, int64_t n, gd_tensor *out)
{
    int64_t dims[1] = {n};
    TRY(gd_tensor_empty(ctx, GD_ARENA_DATA, GD_DTYPE_I32, gd_shape_make(1U, dims), 256U, out));
    return gd_tensor_write(ctx, out, values, (size_t)n * sizeof(int32_t));
}

static gd_status head(gd_gpt_decoder *d, const gd_tensor *x, gd_tensor *logits, gd_tensor *ids, gd_tensor *gaps)
{
    gd_tensor normed;
    TRY(gd_rms_norm(d->ctx, x, &d->final_norm_w, d->cfg.rms_eps, &normed));
    TRY(gd_linear_transposed_weight(d->ctx, &normed, &d->lm_head, &d->lm_head_bias, logits));
    return gd_argmax_rows(d->ctx, logits, ids, gaps);
}

static gd_status fetch(gd_gpt_decoder *d, const gd_tensor *logits, const gd_tensor *ids, const gd_tensor *gaps,
                       int32_t *next_ids, float *out_gaps, uint16_t *out_logits)
{
    const size_t B = (size_t)d->cfg.batch;
    if (next_ids != NULL) TRY(gd_tensor_read(d->ctx, ids, next_ids, B * sizeof(int32_t)));
    if (out_gaps != NULL) TRY(gd_tensor_read(d->ctx, gaps, out_gaps, B * sizeof(float)));
    if (out_logits != NULL) TRY(gd_tensor_read(d->ctx, logits, out_logits, B * (size_t)d->cfg.vocab * 2U));
    return GD_OK;
}

gd_status gd_gpt_decoder_step(gd_gpt_decoder *d, const int32_t *ids, int32_t *next_ids, float *gaps, uint16_t *logits)
{
    gd_context *ctx;
    gd_tensor t_ids, t_pos, t_cache_pos, x, y, t_logits, t_next, t_gaps;
    gd_status st;
    int32_t l, b;
    if (d == NULL || ids == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (d->resident_open) return GD_ERR_BUSY;
    ctx = d->ctx;
    TRY(gd_begin_step(ctx, GD_SCOPE_INFER, gd_batch_empty()));
    st = data_i32(ctx, ids, d->cfg.batch, &t_ids);
    if (st == GD_OK) st = data_i32(ctx, d->pos, d->cfg.batch, &t_pos);
    if (st == GD_OK) st = data_i32(ctx, d->pos, d->cfg.batch, &t_cache_pos);
    if (st == GD_OK) st = gd_embedding(ctx, &d->token_embedding, &t_ids, &x);
    for (l = 0; l < d->cfg.n_layers && st == GD_OK; ++l) {
        st = block_decode(d, l, &x, &t_pos, &t_cache_pos, &y);
        x = y;
    }
    if (st == GD_OK) st = head(d, &x, &t_logits, &t_next, &t_gaps);
    if (st != GD_OK) {
        (void)gd_end_step(ctx);
        return st;
    }
    for (b = 0; b < d->cfg.batch; ++b) d->pos[b] += 1;
    TRY(gd_end_step(ctx));
    return fetch(d, &t_logits, &t_next, &t_gaps, next_ids, gaps, logits);
}

gd_status gd_gpt_decoder_prefill(gd_gpt_decoder *d, const int32_t *ids, const int32_t *cu, int32_t *next_ids,
                                 float *gaps, uint16_t *logits)
{
    gd_context *ctx;
    gd_tensor t_ids, t_pos, t_cu, t_cache_pos, t_last, x, y, last_hidden, t_logits, t_next, t_gaps;
    prefill_rope_rows rope_rows;
    bool have_rows = false;
    gd_status st = GD_OK;
    int32_t *positions, *zero, *last_rows;
    int32_t B, N, b, r, l;
    if (d == NULL || ids == NULL || cu == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (d->resident_open) return GD_ERR_BUSY;
    ctx = d->ctx;
    B = d->cfg.batch;
    N = cu[B];
    if (cu[0] != 0 || N <= 0) return GD_ERR_INVALID_ARGUMENT;
    for (b = 0; b < B; ++b) {
        if (cu[b + 1] <= cu[b] || cu[b + 1] - cu[b] > d->cfg.max_seq) return GD_ERR_INVALID_ARGUMENT;
    }
    positions = (int32_t *)malloc((size_t)N * sizeof(int32_t));
    zero = (int32_t *)calloc((size_t)B, sizeof(int32_t));
    last_rows = (int32_t *)malloc((size_t)B * sizeof(int32_t));
    if (positions == NULL || zero == NULL || last_rows == NULL) {
        free(positions); free(zero); free(last_rows);
        return GD_ERR_OUT_OF_MEMORY;
    }
    for (b = 0; b < B; ++b) {
        for (r = cu[b]; r < cu[b + 1]; ++r) positions[r] = r - cu[b];
        last_rows[b] = cu[b + 1] - 1;
    }
    st = gd_begin_step(ctx, GD_SCOPE_INFER, gd_batch_empty());
    if (st == GD_OK) {
        st = data_i32(ctx, ids, N, &t_ids);
        if (st == GD_OK) st = data_i32(ctx, positions, N, &t_pos);
        if (st == GD_OK) st = data_i32(ctx, cu, (int64_t)B + 1, &t_cu);
        if (st == GD_OK) st = data_i32(ctx, zero, B, &t_cache_pos);
        if (st == GD_OK) st = data_i32(ctx, last_rows, B, &t_last);
        if (st == GD_OK) st = gd_embedding(ctx, &d->token_embedding, &t_ids, &x);
        if (st == GD_OK && N >= 256 && prefill_rope_in_projection(d)) {
            /* once for all layers: the angles of every row's position and the cache row its k and v go to */
            const gd_backend_rope_args ra = {d->cfg.rope_theta, (uint32_t)d->cfg.head_dim, 0U};
            int64_t tdims[2] = {((int64_t)N + 31) / 32 * 32, d->cfg.head_dim / 2}, rdims[1] = {N};
            gd_backend_tensor_view vpos, vcp, vcu, vcos, vsin, vrows;
            st = gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F32, gd_shape_make(2U, tdims), 256U, &rope_rows.cos_rows);
            if (st == GD_OK)
                st = gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F32, gd_shape_make(2U, tdims), 256U, &rope_rows.sin_rows);
            if (st == GD_OK)
                st = gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_I32, gd_shape_make(1U, rdims), 256U, &rope_rows.cache_rows);
            if (st == GD_OK) {
                tview(&t_pos, &vpos);
                tview(&t_cache_pos, &vcp);
                tview(&t_cu, &vcu);
                tview(&rope_rows.cos_rows, &vcos);
                tview(&rope_rows.sin_rows, &vsin);
                tview(&rope_rows.cache_rows, &vrows);
                st = gd_backend_rope_table_packed(gd_context_backend(ctx), &vpos, &vcp, &vcu, &vcos, &vsin, &vrows,
                                                  (uint32_t)d->cfg.head_dim, (uint32_t)d->cfg.max_seq, &ra);
                have_rows = st == GD_OK;
                if (st == GD_ERR_UNSUPPORTED) st = GD_OK;
            }
        }
        for (l = 0; l < d->cfg.n_layers && st == GD_OK; ++l) {
            st = block_prefill(d, l, &x, &t_pos, &t_cu, &t_cache_pos, have_rows ? &rope_rows : NULL, &y);
            x = y;
        }
        if (st == GD_OK) st = gd_gather_rows(ctx, &x, &t_last, &last_hidden);
        if (st == GD_OK) st = head(d, &last_hidden, &t_logits, &t_next, &t_gaps);
        /* the sampling front end starts from these logits without a round trip through the host */
        if (st == GD_OK)
            st = gd_backend_copy(gd_context_backend(ctx), (gd_backend_buffer *)d->last_logits.storage.buffer,
                                 d->last_logits.storage.offset + d->last_logits.view_offset,
                                 (gd_backend_buffer *)t_logits.storage.buffer,
                                 t_logits.storage.offset + t_logits.view_offset, (size_t)B * (size_t)d->cfg.vocab * 2U);
        if (st == GD_OK) {
            for (b = 0; b < B; ++b) d->pos[b] = cu[b + 1] - cu[b];
            st = gd_end_step(ctx);
        } else {
            (void)gd_end_step(ctx);
        }
    }
    free(positions); free(zero); free(last_rows);
    if (st != GD_OK) return st;
    return fetch(d, &t_logits, &t_next, &t_gaps, next_ids, gaps, logits);
}

/* ---- device-resident decode -------------------------------------------------------------- */

/* One step with ids / positions read from device tensors; enqueues only (no host transfer). */
static void view1(const gd_tensor *t, gd_backend_tensor_view *v)
{
    memset(v, 0, sizeof(*v));
    v->buffer = (gd_backend_buffer *)t->storage.buffer;
    v->offset = t->storage.offset + t->view_offset;
    v->count = (size_t)t->shape[0];
    v->dtype = (uint32_t)t->dtype;
    v->rank = 1U;
    v->shape[0] = t->shape[0];
    v->strides[0] = 1;
}

static bool mview(const gd_tensor *t, int64_t rows, int64_t cols, gd_backend_matrix_view *m)
{
    m->buffer = (gd_backend_buffer *)t->storage.buffer;
    m->offset = t->storage.offset + t->view_offset;
    m->rows = (uint32_t)rows;
    m->cols = (uint32_t)cols;
    m->row_bytes = (size_t)cols * 2U;
    m->dtype = (uint32_t)t->dtype;
    return m->buffer != NULL;
}

static void vview(const gd_tensor *t, gd_backend_vector_view *v)
{
    v->buffer = (gd_backend_buffer *)t->storage.buffer;
    v->offset = t->storage.offset + t->view_offset;
    v->length = (uint32_t)t->shape[0];
    v->dtype = (uint32_t)t->dtype;
}

static void tview(const gd_tensor *t, gd_backend_tensor_view *v)
{
    int64_t stride = 1;
    uint32_t i;
    memset(v, 0, sizeof(*v));
    v->buffer = (gd_backend_buffer *)t->storage.buffer;
    v->offset = t->storage.offset + t->view_offset;
    v->dtype = (uint32_t)t->dtype;
    v->rank = t->rank;
    for (i = t->rank; i > 0U; --i) {
        v->shape[i - 1U] = t->shape[i - 1U];
        v->strides[i - 1U] = stride;
        stride *= t->shape[i - 1U];
    }
    v->count = (size_t)stride;
}

static gd_status scratch_f16(gd_context *ctx, int64_t rows, int64_t cols, gd_tensor *out)
{
    int64_t dims[2] = {rows, cols};
    return gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F16, gd_shape_make(2U, dims), 256U, out);
}

/* y = [residual +] bias_mode(prologue(x) @ w) through gd_backend_fused_linear */
static gd_status fused_project_rows(gd_gpt_decoder *d, int64_t B, const gd_tensor *x, int64_t x_cols,
                                    const gpt_linear *lin, const gd_tensor *w_override, const gd_tensor *bias,
                                    const gd_tensor *residual, const gd_tensor *norm_w, uint32_t prologue,
                                    uint32_t epilogue, int64_t n_out, gd_tensor *y)
{
    gd_backend_matrix_view xm, wm, rm, ym;
    gd_backend_vector_view bv, nv;
    gd_backend_fused_linear_args a;
    const gd_tensor *w = w_override != NULL ? w_override : &lin->weight;
    gd_status st;
    TRY(scratch_f16(d->ctx, B, n_out, y));
    mview(x, B, x_cols, &xm);
    mview(w, w->shape[0], w->shape[1], &wm);
    mview(y, B, n_out, &ym);
    if (residual != NULL) mview(residual, B, n_out, &rm);
    if (norm_w != NULL) vview(norm_w, &nv);
    vview(bias, &bv);
    a.w_is_nk = (lin->transposed || w_override != NULL) ? 1U : 0U; /* an override is the [N,K] twin of a [K,N] weight */
    a.bias_mode = lin->transposed ? 2U : 1U; /* gd_linear_transposed_weight: matmul_nt + add (two roundings);
                                                gd_linear: F32 bias in front of the single rounding */
    a.prologue = prologue;
    a.eps = d->cfg.rms_eps;
    a.epilogue = epilogue;
    st = gd_backend_fused_linear(gd_context_backend(d->ctx), &xm, &wm, &bv, residual != NULL ? &rm : NULL,
                                 norm_w != NULL ? &nv : NULL, &ym, &a);
    return st;
}

static gd_status fused_project(gd_gpt_decoder *d, const gd_tensor *x, int64_t x_cols, const gpt_linear *lin,
                               const gd_tensor *w_override, const gd_tensor *bias, const gd_tensor *residual,
                               const gd_tensor *norm_w, uint32_t prologue, uint32_t epilogue, int64_t n_out, gd_tensor *y)
{
    return fused_project_rows(d, d->cfg.batch, x, x_cols, lin, w_override, bias, residual, norm_w, prologue, epilogue,
                              n_out, y);
}

/* The decode step with the fused backend entry points: same operators, same rounding points as
 * block_decode, 6 launches per layer. */
static gd_status enqueue_fused_step(gd_gpt_decoder *d, gd_tensor *logits)
{
    gd_context *ctx = d->ctx;
    gd_backend *be = gd_context_backend(ctx);
    const gd_gpt_config *c = &d->cfg;
    const gd_backend_rope_args rope = {c->rope_theta, (uint32_t)c->head_dim, 0U};
    const gd_sdpa_decode_config sdpa = {0.0f, c->sdpa_window, 0};
    const int64_t B = c->batch, Dm = c->d_model, Hm = c->mlp_hidden;
    gd_tensor x, qkv, q, q4, attn, x1, ug, x2;
    gd_backend_tensor_view vqkv, vpos, vq, vk, vv;
    int64_t q_shape[4] = {B, 1, c->n_heads, c->head_dim};
    int32_t l;
    if (d->resident_x0) x = d->x0_dev;
    else TRY(gd_embedding(ctx, &d->token_embedding, &d->ids_dev, &x));
    for (l = 0; l < c->n_layers; ++l) {
        const gpt_block *b = &d->blocks[l];
        TRY(scratch_f16(ctx, B, Dm, &q));
        tview(&d->pos_dev, &vpos);
        tview(&d->k_cache[l], &vk);
        tview(&d->v_cache[l], &vv);
        memset(&vq, 0, sizeof(vq));
        vq.buffer = (gd_backend_buffer *)q.storage.buffer;
        vq.offset = q.storage.offset;
        vq.count = (size_t)(B * Dm);
        vq.dtype = (uint32_t)GD_DTYPE_F16;
        vq.rank = 3U;
        vq.shape[0] = B; vq.shape[1] = c->n_heads; vq.shape[2] = c->head_dim;
        vq.strides[0] = Dm; vq.strides[1] = c->head_dim; vq.strides[2] = 1;
        if (B < 128 && (c->head_dim % 32) == 0) {
            /* qkv projection with rotation and cache append in its epilogue: the [B,3Dm] intermediate is never stored */
            gd_backend_matrix_view xm, wm;
            gd_backend_vector_view bv, nv;
            gd_backend_fused_linear_args fa;
            mview(&x, B, Dm, &xm);
            mview(&b->qkv_proj.weight, 3 * Dm, Dm, &wm);
            vview(&b->qkv_proj.bias, &bv);
            vview(&b->attn_norm_w, &nv);
            fa.w_is_nk = 1U;
            fa.bias_mode = 2U;
            fa.prologue = 2U;
            fa.eps = c->rms_eps;
            fa.epilogue = 0U;
            TRY(gd_backend_fused_qkv_rope_append(be, &xm, &wm, &bv, &nv, &vpos, &vpos, &vq, &vk, &vv, (uint32_t)c->n_heads,
                                                 (uint32_t)c->head_dim, &rope, &fa));
        } else {
            TRY(fused_project(d, &x, Dm, &b->qkv_proj, NULL, &b->qkv_proj.bias, NULL, &b->attn_norm_w, 2U, 0U, 3 * Dm, &qkv));
            tview(&qkv, &vqkv);
            TRY(gd_backend_qkv_rope_append(be, &vqkv, &vpos, &vpos, &vq, &vk, &vv, (uint32_t)c->n_heads,
                                           (uint32_t)c->head_dim, &rope));
        }
        TRY(gd_reshape(ctx, &q, gd_shape_make(4U, q_shape), &q4));
        TRY(gd_sdpa_decode_positions(ctx, &q4, &d->k_cache[l], &d->v_cache[l], &d->pos_dev, &sdpa, &attn));
        TRY(fused_project(d, &attn, Dm, &b->attn_proj, NULL, &b->attn_proj.bias, &x, NULL, 0U, 0U, Dm, &x1));
        if (B < 128) {
            /* the gate is applied in the up/gate projection's epilogue: the [B,2Hm] intermediate is never stored */
            TRY(fused_project(d, &x1, Dm, &b->up_gate, NULL, &b->up_gate.bias, NULL, &b->mlp_norm_w, 2U, 1U, Hm, &ug));
            TRY(fused_project(d, &ug, Hm, &b->down_proj, &b->down_t, &b->down_proj.bias, &x1, NULL, 0U, 0U, Dm, &x2));
        } else {
            TRY(fused_project(d, &x1, Dm, &b->up_gate, NULL, &b->up_gate.bias, NULL, &b->mlp_norm_w, 2U, 0U, 2 * Hm, &ug));
            TRY(fused_project(d, &ug, 2 * Hm, &b->down_proj, &b->down_t, &b->down_proj.bias, &x1, NULL, 1U, 0U, Dm, &x2));
        }
        x = x2;
    }
    {
        gpt_linear head_lin;
        head_lin.weight = d->lm_head;
        head_lin.bias = d->lm_head_bias;
        head_lin.transposed = true;
        TRY(fused_project(d, &x, Dm, &head_lin, NULL, &d->lm_head_bias, NULL, &d->final_norm_w, 2U, 0U, c->vocab, logits));
    }
    return GD_OK;
}

/* sampled pick instead of the greedy one: token, history, finished flags, feedback and records in two launches */
static gd_status enqueue_sample(gd_gpt_decoder *d, const gd_tensor *logits, int32_t pos_delta)
{
    gd_backend_tensor_view vl, vh, vhl, vf, vst, vw, vi, vp, vs, vo, vt, vx;
    gd_backend_sample_tensors t;
    gd_backend_sample_args a;
    tview(logits, &vl);
    tview(&d->history, &vh);
    view1(&d->hist_len, &vhl);
    view1(&d->finished, &vf);
    view1(&d->sample_state, &vst);
    view1(&d->sample_work, &vw);
    view1(&d->ids_dev, &vi);
    view1(&d->pos_dev, &vp);
    view1(&d->step_rows_dev, &vs);
    view1(&d->resident_out_ids, &vo);
    memset(&t, 0, sizeof(t));
    t.history = &vh;
    t.hist_len = &vhl;
    t.finished = &vf;
    t.state = &vst;
    t.work = &vw;
    t.ids = &vi;
    t.positions = &vp;
    t.step_counters = &vs;
    t.out_ids = &vo;
    if (d->resident_x0) {
        tview(&d->token_embedding, &vt);
        tview(&d->x0_dev, &vx);
        t.table = &vt;
        t.next_x = &vx;
    }
    a.temperature = d->sampling.temperature;
    a.min_p = d->sampling.min_p;
    a.repetition_penalty = d->sampling.repetition_penalty;
    a.logits_softcap = d->sampling.logits_softcap;
    a.stop_token = d->sampling.stop_token;
    a.pos_delta = pos_delta;
    return gd_backend_sample_advance(gd_context_backend(d->ctx), &vl, &t, &a);
}

/* GD_GPT_RESIDENT_KEEP_LOGITS: the step's logits into the state tensor that outlives the step scope */
static gd_status keep_logits(gd_gpt_decoder *d, const gd_tensor *logits)
{
    return gd_backend_copy(gd_context_backend(d->ctx), (gd_backend_buffer *)d->last_logits.storage.buffer,
                           d->last_logits.storage.offset + d->last_logits.view_offset,
                           (gd_backend_buffer *)logits->storage.buffer, logits->storage.offset + logits->view_offset,
                           (size_t)d->cfg.batch * (size_t)d->cfg.vocab * 2U);
}

static gd_status enqueue_resident_step(gd_gpt_decoder *d)
{
    gd_context *ctx = d->ctx;
    gd_tensor x, y, logits, next, gaps;
    gd_backend_tensor_view vn, vg, vi, vp, vs, vo, vog;
    int32_t l;
    if (d->resident_sampling) {
        if (d->resident_unfused) {
            TRY(gd_embedding(ctx, &d->token_embedding, &d->ids_dev, &x));
            for (l = 0; l < d->cfg.n_layers; ++l) {
                TRY(block_decode(d, l, &x, &d->pos_dev, &d->pos_dev, &y));
                x = y;
            }
            TRY(head(d, &x, &logits, &next, &gaps));
        } else {
            TRY(enqueue_fused_step(d, &logits));
        }
        return enqueue_sample(d, &logits, d->resident_hold ? 0 : 1);
    }
    if (d->resident_unfused) {
        TRY(gd_embedding(ctx, &d->token_embedding, &d->ids_dev, &x));
        for (l = 0; l < d->cfg.n_layers; ++l) {
            TRY(block_decode(d, l, &x, &d->pos_dev, &d->pos_dev, &y));
            x = y;
        }
        TRY(head(d, &x, &logits, &next, &gaps));
    } else {
        /* greedy pick, token feedback, position and record keeping in one launch */
        gd_backend_tensor_view vl;
        TRY(enqueue_fused_step(d, &logits));
        if (d->resident_keep_logits) TRY(keep_logits(d, &logits));
        tview(&logits, &vl);
        view1(&d->ids_dev, &vi);
        view1(&d->pos_dev, &vp);
        view1(&d->step_rows_dev, &vs);
        view1(&d->resident_out_ids, &vo);
        view1(&d->resident_out_gaps, &vog);
        if (d->resident_x0) {
            gd_backend_tensor_view vt, vx;
            tview(&d->token_embedding, &vt);
            tview(&d->x0_dev, &vx);
            return gd_backend_argmax_advance(gd_context_backend(ctx), &vl, &vi, &vp, &vs, &vo, &vog,
                                             d->resident_hold ? 0 : 1, &vt, &vx);
        }
        return gd_backend_argmax_advance(gd_context_backend(ctx), &vl, &vi, &vp, &vs, &vo, &vog, d->resident_hold ? 0 : 1,
                                         NULL, NULL);
    }
    if (d->resident_keep_logits) TRY(keep_logits(d, &logits));
    view1(&next, &vn);
    view1(&gaps, &vg);
    view1(&d->ids_dev, &vi);
    view1(&d->pos_dev, &vp);
    view1(&d->step_dev, &vs);
    view1(&d->resident_out_ids, &vo);
    view1(&d->resident_out_gaps, &vog);
    return gd_backend_decode_advance(gd_context_backend(ctx), &vn, &vg, &vi, &vp, &vs, &vo, &vog,
                                     d->resident_hold ? 0 : 1);
}

static void resident_abort(gd_gpt_decoder *d)
{
    (void)gd_end_step(d->ctx);
    if (d->resident_graph != NULL) gd_backend_graph_destroy(d->resident_graph);
    d->resident_graph = NULL;
    d->resident_open = false;
    d->resident_sampling = false;
}

/* sampling == NULL: greedy session that starts from first_ids.  Otherwise: the session starts from the logits the
 * last prefill left in last_logits; max_steps counts picks (the one on those logits included), so at most
 * max_steps - 1 decode steps run; history / hist_len / finished / sample_state were set by the caller. */
static gd_status resident_begin_impl(gd_gpt_decoder *d, const int32_t *first_ids, int32_t max_steps, int32_t flags,
                                     const gd_gpt_sampling *sampling)
{
    const int32_t hold_positions = flags & GD_GPT_RESIDENT_HOLD_POSITIONS;
    gd_context *ctx;
    gd_backend *be;
    gd_status st;
    int64_t dims[1];
    int32_t b, zero = 0;
    if (d == NULL || (first_ids == NULL && sampling == NULL) || max_steps <= 0) return GD_ERR_INVALID_ARGUMENT;
    if (d->resident_open) return GD_ERR_BUSY;
    ctx = d->ctx;
    be = gd_context_backend(ctx);
    for (b = 0; b < d->cfg.batch; ++b) {
        /* a sampled session may run past the end of a cache: such rows have ended (their history is full), their
         * appends are skipped and their results ignored, as in the reference's loop */
        if (d->pos[b] < 0 || (sampling == NULL && d->pos[b] + (hold_positions ? 1 : max_steps) > d->cfg.max_seq))
            return GD_ERR_INVALID_ARGUMENT;
    }
    if (sampling == NULL) TRY(gd_tensor_write(ctx, &d->ids_dev, first_ids, (size_t)d->cfg.batch * sizeof(int32_t)));
    TRY(gd_tensor_write(ctx, &d->pos_dev, d->pos, (size_t)d->cfg.batch * sizeof(int32_t)));
    TRY(gd_tensor_write(ctx, &d->step_dev, &zero, sizeof(zero)));
    TRY(gd_tensor_zero_(ctx, &d->step_rows_dev));
    TRY(gd_begin_step(ctx, GD_SCOPE_INFER, gd_batch_empty()));
    d->resident_open = true;
    d->resident_graph = NULL;
    d->resident_max_steps = max_steps;
    d->resident_steps = 0;
    d->resident_hold = hold_positions != 0;
    d->resident_sampling = sampling != NULL;
    if (sampling != NULL) d->sampling = *sampling;
    /* the fused rope + append kernel needs NeoX pairs of a head size that is a multiple of 16 */
    d->resident_unfused = (flags & GD_GPT_RESIDENT_UNFUSED) != 0 || (d->cfg.head_dim % 16) != 0;
    d->resident_keep_logits = sampling == NULL && (flags & GD_GPT_RESIDENT_KEEP_LOGITS) != 0;
    dims[0] = (int64_t)max_steps * d->cfg.batch;
    st = gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_I32, gd_shape_make(1U, dims), 256U, &d->resident_out_ids);
    if (st == GD_OK) st = gd_tensor_empty(ctx, GD_ARENA_SCRATCH, GD_DTYPE_F32, gd_shape_make(1U, dims), 256U, &d->resident_out_gaps);
    /* fused step: the pick kernel leaves the next input rows in x0_dev; the first ones are gathered here */
    d->resident_x0 = !d->resident_unfused && (d->cfg.d_model % 8) == 0;
    if (sampling != NULL) {
        /* pick number 0, on the prefill's logits: positions stay, the token becomes the first step's input */
        if (st == GD_OK) st = enqueue_sample(d, &d->last_logits, 0);
        max_steps -= 1; /* decode steps from here on */
    } else if (st == GD_OK && d->resident_x0) {
        gd_backend_tensor_view vt, vi, vx;
        gd_backend_embedding_args ea;
        tview(&d->token_embedding, &vt);
        tview(&d->ids_dev, &vi);
        tview(&d->x0_dev, &vx);
        ea.ids_count = (uint64_t)d->cfg.batch;
        ea.vocab = (uint64_t)d->cfg.vocab;
        ea.dim = (uint64_t)d->cfg.d_model;
        st = gd_backend_embedding_forward(be, &vt, &vi, &vx, &ea);
    }
    /* the first step runs eagerly (it also sizes the attention workspace); later steps replay a graph */
    if (st == GD_OK && max_steps > 0) {
        st = enqueue_resident_step(d);
        if (st == GD_OK) d->resident_steps = 1;
    }
    if (st == GD_OK && max_steps > 1) {
        st = gd_backend_graph_begin_capture(be);
        if (st == GD_OK) {
            st = enqueue_resident_step(d);
            if (st == GD_OK) st = gd_backend_graph_end_capture(be, &d->resident_graph);
            else (void)gd_backend_graph_end_capture(be, &d->resident_graph);
        }
    }
    if (st != GD_OK) resident_abort(d);
    return st;
}

gd_status gd_gpt_decoder_resident_begin(gd_gpt_decoder *d, const int32_t *first_ids, int32_t max_steps,
                                        int32_t flags)
{
    if (first_ids == NULL) return GD_ERR_INVALID_ARGUMENT;
    return resident_begin_impl(d, first_ids, max_steps, flags, NULL);
}

gd_status gd_gpt_decoder_resident_run(gd_gpt_decoder *d, int32_t n_steps)
{
    gd_backend *be;
    int32_t s;
    if (d == NULL || n_steps < 0) return GD_ERR_INVALID_ARGUMENT;
    if (!d->resident_open) return GD_ERR_BAD_STATE;
    if (d->resident_steps + n_steps > d->resident_max_steps - (d->resident_sampling ? 1 : 0)) return GD_ERR_INVALID_ARGUMENT;
    if (n_steps > 0 && d->resident_graph == NULL) return GD_ERR_BAD_STATE;
    be = gd_context_backend(d->ctx);
    for (s = 0; s < n_steps; ++s) {
        TRY(gd_backend_graph_launch(be, d->resident_graph));
        d->resident_steps += 1;
    }
    return GD_OK;
}

gd_status gd_gpt_decoder_resident_sync(gd_gpt_decoder *d)
{
    if (d == NULL) return GD_ERR_INVALID_ARGUMENT;
    return gd_synchronize(d->ctx);
}

gd_status gd_gpt_decoder_resident_end(gd_gpt_decoder *d, int32_t *out_ids, float *out_gaps, int32_t *steps_done)
{
    gd_context *ctx;
    gd_status st;
    gd_tensor ids_view, gaps_view;
    int32_t b, records;
    if (d == NULL) return GD_ERR_INVALID_ARGUMENT;
    if (!d->resident_open) return GD_ERR_BAD_STATE;
    ctx = d->ctx;
    st = gd_end_step(ctx);
    /* a sampled session has one record more than decode steps: the pick on the prefill's logits */
    records = d->resident_steps + (d->resident_sampling ? 1 : 0);
    if (st == GD_OK && out_ids != NULL) {
        st = gd_tensor_slice(ctx, &d->resident_out_ids, 0U, 0, (int64_t)records * d->cfg.batch, &ids_view);
        if (st == GD_OK) st = gd_tensor_read(ctx, &ids_view, out_ids, (size_t)records * (size_t)d->cfg.batch * sizeof(int32_t));
    }
    if (st == GD_OK && out_gaps != NULL && !d->resident_sampling) {
        st = gd_tensor_slice(ctx, &d->resident_out_gaps, 0U, 0, (int64_t)d->resident_steps * d->cfg.batch, &gaps_view);
        if (st == GD_OK) st = gd_tensor_read(ctx, &gaps_view, out_gaps, (size_t)d->resident_steps * (size_t)d->cfg.batch * sizeof(float));
    }
    if (d->resident_graph != NULL) gd_backend_graph_destroy(d->resident_graph);
    d->resident_graph = NULL;
    d->resident_open = false;
    d->resident_sampling = false;
    if (steps_done != NULL) *steps_done = records;
    if (st == GD_OK && !d->resident_hold) {
        for (b = 0; b < d->cfg.batch; ++b) d->pos[b] += d->resident_steps;
    }
    return st;
}

gd_status gd_gpt_decoder_resident_begin_sampled(gd_gpt_decoder *d, const int32_t *ids, const int32_t *cu,
                                                int32_t max_picks, int32_t flags, const gd_gpt_sampling *sampling)
{
    gd_context *ctx;
    gd_tensor head_words;
    int32_t *hist, *lens;
    int32_t state_words[8];
    int32_t B, b;
    gd_status st;
    if (d == NULL || ids == NULL || cu == NULL || sampling == NULL || max_picks <= 0 || cu[0] != 0 ||
        sampling->stop_token >= d->cfg.vocab)
        return GD_ERR_INVALID_ARGUMENT;
    if (d->resident_open) return GD_ERR_BAD_STATE;
    ctx = d->ctx;
    B = d->cfg.batch;
    if (B <= 0) return GD_ERR_BAD_STATE;
    for (b = 0; b < B; ++b) {
        if (cu[b + 1] < cu[b] || cu[b + 1] - cu[b] > d->cfg.max_seq) return GD_ERR_INVALID_ARGUMENT;
    }
    hist = (int32_t *)calloc((size_t)B * (size_t)d->cfg.max_seq, sizeof(int32_t));
    lens = (int32_t *)calloc((size_t)B, sizeof(int32_t));
    if (hist == NULL || lens == NULL) {
        free(hist); free(lens);
        return GD_ERR_OUT_OF_MEMORY;
    }
    for (b = 0; b < B; ++b) {
        lens[b] = cu[b + 1] - cu[b];
        memcpy(hist + (size_t)b * (size_t)d->cfg.max_seq, ids + cu[b], (size_t)lens[b] * sizeof(int32_t));
    }
    memset(state_words, 0, sizeof(state_words));
    memcpy(&state_words[0], &sampling->rng_state, sizeof(uint64_t));
    memcpy(&state_words[2], &sampling->rng_state, sizeof(uint64_t));
    st = gd_tensor_slice(ctx, &d->sample_state, 0U, 0, 8, &head_words);
    if (st == GD_OK) st = gd_tensor_write(ctx, &head_words, state_words, sizeof(state_words));
    if (st == GD_OK) st = gd_tensor_write(ctx, &d->history, hist, (size_t)B * (size_t)d->cfg.max_seq * sizeof(int32_t));
    if (st == GD_OK) st = gd_tensor_write(ctx, &d->hist_len, lens, (size_t)B * sizeof(int32_t));
    if (st == GD_OK) st = gd_tensor_zero_(ctx, &d->finished);
    free(hist); free(lens);
    if (st != GD_OK) return st;
    return resident_begin_impl(d, NULL, max_picks, flags, sampling);
}

/* ---- generation with the sampling front end ---------------------------------------------- */

uint64_t gd_gpt_generation_rng(uint64_t seed, int32_t n_prompts, uint64_t step)
{
    return splitmix64(seed ^ UINT64_C(0xdec0de1234567890) ^ (uint64_t)n_prompts ^ step);
}

gd_status gd_gpt_decoder_generate(gd_gpt_decoder *d, const int32_t *ids, const int32_t *cu, int32_t max_new,
                                  const gd_gpt_sampling *sampling, int32_t *out_tokens, int32_t *out_counts)
{
    const int32_t check_every = 32; /* decode steps between two looks at the finished flags */
    gd_context *ctx;
    int32_t *packed = NULL, *pcu = NULL, *lens = NULL, *records = NULL, *flags = NULL;
    int32_t B, ctx_len, room, b, total = 0, done = 0, decode_steps;
    gd_status st;
    if (d == NULL || ids == NULL || cu == NULL || sampling == NULL || out_tokens == NULL || out_counts == NULL ||
        max_new <= 0)
        return GD_ERR_INVALID_ARGUMENT;
    if (d->resident_open) return GD_ERR_BUSY;
    ctx = d->ctx;
    B = d->cfg.batch;
    ctx_len = d->cfg.max_seq;
    if (sampling->stop_token >= d->cfg.vocab || cu[0] != 0) return GD_ERR_INVALID_ARGUMENT;
    /* reference :1514-1518: the prompt may use what the new tokens leave of the context, at least one row short of it */
    room = max_new >= ctx_len ? ctx_len - 1 : ctx_len - max_new;
    if (room <= 0) return GD_ERR_INVALID_ARGUMENT;
    for (b = 0; b < B; ++b) {
        if (cu[b + 1] <= cu[b]) return GD_ERR_INVALID_ARGUMENT; /* empty prompt (:1520-1522) */
    }
    pcu = (int32_t *)calloc((size_t)B + 1U, sizeof(int32_t));
    lens = (int32_t *)calloc((size_t)B, sizeof(int32_t));
    flags = (int32_t *)calloc((size_t)B, sizeof(int32_t));
    records = (int32_t *)malloc((size_t)max_new * (size_t)B * sizeof(int32_t));
    if (pcu == NULL || lens == NULL || flags == NULL || records == NULL) {
        st = GD_ERR_OUT_OF_MEMORY;
        goto out;
    }
    /* a prompt longer than the room keeps its last tokens (:1523-1533) */
    for (b = 0; b < B; ++b) {
        const int32_t n = cu[b + 1] - cu[b];
        lens[b] = n > room ? room : n;
        pcu[b + 1] = pcu[b] + lens[b];
    }
    total = pcu[B];
    packed = (int32_t *)malloc((size_t)total * sizeof(int32_t));
    if (packed == NULL) {
        st = GD_ERR_OUT_OF_MEMORY;
        goto out;
    }
    for (b = 0; b < B; ++b) {
        const int32_t *src = ids + cu[b + 1] - lens[b];
        memcpy(packed + pcu[b], src, (size_t)lens[b] * sizeof(int32_t));
    }
    st = gd_gpt_decoder_prefill(d, packed, pcu, NULL, NULL, NULL); /* leaves the logits in last_logits */
    if (st == GD_OK) st = gd_gpt_decoder_resident_begin_sampled(d, packed, pcu, max_new, 0, sampling);
    if (st != GD_OK) goto out;
    /* the reference leaves its loop when every row has ended (:1607, 1634-1636): look at the flags now and then */
    decode_steps = max_new - 1;
    while (d->resident_steps < decode_steps) {
        int32_t n = decode_steps - d->resident_steps, alive = 0;
        if (n > check_every) n = check_every;
        st = gd_gpt_decoder_resident_run(d, n);
        if (st == GD_OK && d->resident_steps < decode_steps) {
            st = gd_tensor_read(ctx, &d->finished, flags, (size_t)B * sizeof(int32_t));
            for (b = 0; b < B; ++b) alive += flags[b] == 0;
        } else {
            alive = 1;
        }
        if (st != GD_OK) {
            resident_abort(d);
            goto out;
        }
        if (alive == 0) break;
    }
    st = gd_gpt_decoder_resident_end(d, records, NULL, &done);
    if (st != GD_OK) goto out;
    for (b = 0; b < B; ++b) {
        int32_t s, n = 0;
        for (s = 0; s < done; ++s) {
            const int32_t token = records[(size_t)s * (size_t)B + (size_t)b];
            if (token >= 0) out_tokens[(size_t)b * (size_t)max_new + (size_t)n++] = token;
        }
        out_counts[b] = n;
    }
out:
    free(packed); free(pcu); free(lens); free(records); free(flags);
    return st;
}

gd_status gd_gpt_decoder_run_resident(gd_gpt_decoder *d, const int32_t *first_ids, int32_t n_steps, int32_t *out_ids,
                                      float *out_gaps, float *step_ms)
{
    gd_backend_timer *timer = NULL;
    gd_status st;
    float ms = 0.0f;
    if (d == NULL || n_steps <= 0 || out_ids == NULL) return GD_ERR_INVALID_ARGUMENT;
    TRY(gd_gpt_decoder_resident_begin(d, first_ids, n_steps, 0));
    st = GD_OK;
    if (step_ms != NULL) st = gd_backend_timer_create(gd_context_backend(d->ctx), &timer);
    if (st == GD_OK && timer != NULL) st = gd_backend_timer_start(timer);
    if (st == GD_OK) st = gd_gpt_decoder_resident_run(d, n_steps - 1);
    if (st == GD_OK && timer != NULL) st = gd_backend_timer_stop(timer);
    if (st != GD_OK) {
        resident_abort(d);
    } else {
        st = gd_gpt_decoder_resident_end(d, out_ids, out_gaps, NULL);
        if (st == GD_OK && timer != NULL) st = gd_backend_timer_elapsed_ms(timer, &ms);
    }
    if (timer != NULL) gd_backend_timer_destroy(timer);
    if (step_ms != NULL) *step_ms = n_steps > 1 ? ms / (float)(n_steps - 1) : 0.0f;
    return st;
}
