/* Host dispatch of gd_backend_sample_advance (no counterpart in the reference's backend: the reference samples on
 * the host, examples/gpt_lm/gpt_lm_shared.c:1322-1442, 1586-1600, 1660-1680). */
#include <math.h>

#include "../../../backends/hip/backend_hip_internal.h"

#define GD_HIP_SAMPLE_MAX_COLS 262144u

/* mirrors of the kernel-side structs in sample.hip */
typedef struct gd_hip_sample_cfg {
    float temperature, min_p, penalty, softcap;
    int32_t stop_token;
    uint32_t cols, hist_cap;
    uint32_t parts; /* filled in by the launcher */
} gd_hip_sample_cfg;

typedef struct gd_hip_sample_advance {
    int32_t *history, *hist_len, *finished;
    int32_t *ids, *positions, *step_counters, *out_ids;
    uint32_t max_steps;
    int32_t pos_delta;
    const unsigned char *table;
    unsigned char *next_x;
    uint32_t row_bytes;
} gd_hip_sample_advance;

int gd_hip_launch_sample_advance(hipStream_t stream, const void *logits, int is_f16, float *work, void *state,
                                 uint32_t rows, const gd_hip_sample_cfg *cfg, const gd_hip_sample_advance *adv);

static int i32_rows(const gd_backend_tensor_view *v, uint64_t rows)
{
    return gd_hip_view_ok(v) && v->dtype == GD_BACKEND_DTYPE_I32 && v->count == (size_t)rows && (v->offset & 3u) == 0u;
}

size_t gd_backend_sample_state_count(uint32_t rows) { return 8u + 10u * (size_t)rows; }

/* F32 values [rows * cols] (rounded up to an even count), then per row and part of 2048 tokens 258 8-byte cells
 * (256 segment masses, the part's mass, the part's leader) */
size_t gd_backend_sample_work_count(uint32_t rows, uint32_t cols)
{
    const size_t values = ((size_t)rows * cols + 1u) & ~(size_t)1u, parts = ((size_t)cols + 2047u) / 2048u;
    return values + 2u * (size_t)rows * parts * 258u;
}

gd_status gd_backend_sample_advance(gd_backend *backend, const gd_backend_tensor_view *logits,
                                    const gd_backend_sample_tensors *t, const gd_backend_sample_args *args)
{
    gd_hip_sample_cfg cfg;
    gd_hip_sample_advance adv;
    uint64_t rows, cols, hist_cap, max_steps, row_bytes = 0u;
    if (backend == NULL || t == NULL || args == NULL || !gd_hip_view_ok(logits) || logits->rank != 2u ||
        !gd_hip_view_ok(t->history) || !gd_hip_view_ok(t->state) || !gd_hip_view_ok(t->work) ||
        !gd_hip_view_ok(t->out_ids))
        return GD_ERR_INVALID_ARGUMENT;
    if ((logits->dtype != GD_BACKEND_DTYPE_F16 && logits->dtype != GD_BACKEND_DTYPE_F32) ||
        t->history->dtype != GD_BACKEND_DTYPE_I32 || t->state->dtype != GD_BACKEND_DTYPE_I32 ||
        t->work->dtype != GD_BACKEND_DTYPE_F32 || t->out_ids->dtype != GD_BACKEND_DTYPE_I32)
        return GD_ERR_UNSUPPORTED;
    rows = (uint64_t)logits->shape[0];
    cols = (uint64_t)logits->shape[1];
    if (rows == 0u || rows > 65535u || cols == 0u) return GD_ERR_INVALID_ARGUMENT;
    if (cols > GD_HIP_SAMPLE_MAX_COLS) return GD_ERR_UNSUPPORTED;
    if (t->history->rank != 2u || (uint64_t)t->history->shape[0] != rows || t->history->shape[1] <= 0 ||
        t->history->shape[1] > (int64_t)INT32_MAX || (t->history->offset & 3u) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    hist_cap = (uint64_t)t->history->shape[1];
    if (!i32_rows(t->hist_len, rows) || !i32_rows(t->finished, rows) || !i32_rows(t->ids, rows) ||
        !i32_rows(t->positions, rows) || !i32_rows(t->step_counters, rows) ||
        t->state->count < gd_backend_sample_state_count((uint32_t)rows) || (t->state->offset & 7u) != 0u ||
        t->work->count < gd_backend_sample_work_count((uint32_t)rows, (uint32_t)cols) || (t->work->offset & 7u) != 0u || (t->out_ids->count % rows) != 0u ||
        (t->out_ids->offset & 3u) != 0u)
        return GD_ERR_INVALID_ARGUMENT;
    max_steps = t->out_ids->count / rows;
    if (max_steps > 0xffffffffu || (t->table == NULL) != (t->next_x == NULL)) return GD_ERR_INVALID_ARGUMENT;
    if (t->table != NULL) {
        if (!gd_hip_view_ok(t->table) || !gd_hip_view_ok(t->next_x) || t->table->rank != 2u || t->next_x->rank != 2u ||
            (uint64_t)t->table->shape[0] != cols || (uint64_t)t->next_x->shape[0] != rows ||
            t->next_x->shape[1] != t->table->shape[1])
            return GD_ERR_INVALID_ARGUMENT;
        if (t->table->dtype != t->next_x->dtype || gd_hip_dtype_size(t->table->dtype) == 0u) return GD_ERR_UNSUPPORTED;
        row_bytes = (uint64_t)t->table->shape[1] * gd_hip_dtype_size(t->table->dtype);
        if ((row_bytes & 15u) != 0u || row_bytes > 0xffffffffu || ((t->table->offset | t->next_x->offset) & 15u) != 0u)
            return GD_ERR_UNSUPPORTED;
    }
    /* the stop token doubles as the input of rows that have ended: it must be a row of the table */
    if (args->stop_token >= 0 && (uint64_t)args->stop_token >= cols) return GD_ERR_INVALID_ARGUMENT;
    cfg.temperature = args->temperature;
    cfg.min_p = args->min_p;
    cfg.penalty = args->repetition_penalty;
    cfg.softcap = args->logits_softcap;
    cfg.stop_token = args->stop_token;
    cfg.cols = (uint32_t)cols;
    cfg.hist_cap = (uint32_t)hist_cap;
    cfg.parts = 0u;
    adv.history = (int32_t *)gd_hip_view_ptr(t->history);
    adv.hist_len = (int32_t *)gd_hip_view_ptr(t->hist_len);
    adv.finished = (int32_t *)gd_hip_view_ptr(t->finished);
    adv.ids = (int32_t *)gd_hip_view_ptr(t->ids);
    adv.positions = (int32_t *)gd_hip_view_ptr(t->positions);
    adv.step_counters = (int32_t *)gd_hip_view_ptr(t->step_counters);
    adv.out_ids = (int32_t *)gd_hip_view_ptr(t->out_ids);
    adv.max_steps = (uint32_t)max_steps;
    adv.pos_delta = args->pos_delta;
    adv.table = t->table != NULL ? (const unsigned char *)gd_hip_view_ptr(t->table) : NULL;
    adv.next_x = t->next_x != NULL ? (unsigned char *)gd_hip_view_ptr(t->next_x) : NULL;
    adv.row_bytes = (uint32_t)row_bytes;
    return gd_hip_finish_op(backend, gd_hip_launch_sample_advance(
        backend->stream, gd_hip_view_ptr(logits), logits->dtype == GD_BACKEND_DTYPE_F16,
        (float *)gd_hip_view_ptr(t->work), gd_hip_view_ptr(t->state), (uint32_t)rows, &cfg, &adv));
}
