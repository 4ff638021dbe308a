/*
 * Byte-level BPE tokenizer for inference: vocabulary loader, encoder, decoder.  Behaviour restates the
 * reference's src/tokenizer/tokenizer_io.c:238-371 (loader), tokenizer.c:113-149, 348-526 (piece cutting),
 * tokenizer_codec.c:66-238 (merging, decoding) and tokenizer.c:151-174 (digest); the data structures are
 * this file's own: one token table, two open-addressing tables built once after loading (pair -> merged id,
 * bytes -> id), and a cursor-style piece cutter instead of callbacks.
 */
#include <errno.h>
#include <limits.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "gd_tokenizer.h"

#define MAX_SPECIALS 64
#define MAX_PIECE 256
#define FNV_OFFSET UINT64_C(14695981039346656037)
#define FNV_PRIME UINT64_C(1099511628211)
#define NO_PAIR UINT64_MAX

typedef struct bpe_token {
    uint8_t *bytes;
    size_t len;
    int32_t left, right; /* -1: not a merge */
    int special;
} bpe_token;

struct gd_tokenizer {
    int split_digits, allow_special;
    bpe_token *tokens;
    int32_t n_tokens, cap;
    int32_t special_ids[MAX_SPECIALS];
    int n_specials;
    uint8_t special_first[256]; /* some special text starts with this byte */
    uint64_t *pair_keys;        /* (left << 32 | right), NO_PAIR = free */
    int32_t *pair_ids;
    size_t pair_cap;
    int32_t *byte_slots; /* token ids keyed by their bytes, -1 = free */
    size_t byte_cap;
    uint64_t hash;
};

/* ---- tables ------------------------------------------------------------------------------- */

static uint64_t fnv_bytes(const uint8_t *p, size_t n)
{
    uint64_t h = FNV_OFFSET;
    size_t i;
    for (i = 0; i < n; ++i) h = (h ^ p[i]) * FNV_PRIME;
    return h;
}

static uint64_t pair_key(int32_t left, int32_t right) { return ((uint64_t)(uint32_t)left << 32) | (uint32_t)right; }

static size_t pair_slot(const gd_tokenizer *t, uint64_t key)
{
    size_t i = (size_t)((key * UINT64_C(0x9e3779b97f4a7c15)) >> 20) & (t->pair_cap - 1U);
    while (t->pair_keys[i] != NO_PAIR && t->pair_keys[i] != key) i = (i + 1U) & (t->pair_cap - 1U);
    return i;
}

/* merged token of a pair, or -1 */
static int32_t pair_lookup(const gd_tokenizer *t, int32_t left, int32_t right)
{
    const size_t i = pair_slot(t, pair_key(left, right));
    return t->pair_keys[i] == NO_PAIR ? -1 : t->pair_ids[i];
}

static size_t bytes_slot(const gd_tokenizer *t, const uint8_t *p, size_t n)
{
    size_t i = (size_t)fnv_bytes(p, n) & (t->byte_cap - 1U);
    while (t->byte_slots[i] >= 0) {
        const bpe_token *k = &t->tokens[t->byte_slots[i]];
        if (k->len == n && memcmp(k->bytes, p, n) == 0) break;
        i = (i + 1U) & (t->byte_cap - 1U);
    }
    return i;
}

/* Both tables from the token list.  Later tokens replace earlier ones with the same key, as repeated insertion
 * does in the reference (tokenizer_maps.c:82-87, 191-196); specials are in neither table (tokenizer.c:295-325). */
static gd_status build_tables(gd_tokenizer *t)
{
    size_t cap = 1024U, i;
    int32_t id;
    while (cap < (size_t)t->n_tokens * 2U) cap *= 2U;
    t->pair_cap = t->byte_cap = cap;
    t->pair_keys = (uint64_t *)malloc(cap * sizeof(uint64_t));
    t->pair_ids = (int32_t *)malloc(cap * sizeof(int32_t));
    t->byte_slots = (int32_t *)malloc(cap * sizeof(int32_t));
    if (t->pair_keys == NULL || t->pair_ids == NULL || t->byte_slots == NULL) return GD_ERR_OUT_OF_MEMORY;
    for (i = 0; i < cap; ++i) {
        t->pair_keys[i] = NO_PAIR;
        t->byte_slots[i] = -1;
    }
    memset(t->special_first, 0, sizeof(t->special_first));
    for (id = 0; id < t->n_tokens; ++id) {
        const bpe_token *k = &t->tokens[id];
        if (k->special) {
            t->special_first[k->bytes[0]] = 1U;
            continue;
        }
        t->byte_slots[bytes_slot(t, k->bytes, k->len)] = id;
        if (k->left >= 0 && k->right >= 0) {
            const uint64_t key = pair_key(k->left, k->right);
            const size_t s = pair_slot(t, key);
            t->pair_keys[s] = key;
            t->pair_ids[s] = id;
        }
    }
    return GD_OK;
}

static void digest(gd_tokenizer *t)
{
    uint64_t h = FNV_OFFSET;
    int32_t i;
#define MIX(v) (h = (h ^ (uint64_t)(v)) * FNV_PRIME)
    MIX((uint32_t)t->split_digits);
    MIX((uint32_t)t->n_tokens);
    for (i = 0; i < t->n_tokens; ++i) {
        const bpe_token *k = &t->tokens[i];
        size_t j;
        MIX((uint32_t)i);
        MIX((uint32_t)k->special);
        MIX((uint32_t)k->left);
        MIX((uint32_t)k->right);
        MIX(k->len);
        for (j = 0; j < k->len; ++j) MIX(k->bytes[j]);
    }
#undef MIX
    t->hash = h;
}

/* ---- loader ------------------------------------------------------------------------------- */

static gd_status append_token(gd_tokenizer *t, const uint8_t *bytes, size_t len, int special, int32_t left,
                              int32_t right)
{
    bpe_token *k;
    if (len == 0U) return GD_ERR_INVALID_ARGUMENT;
    if (special && t->n_specials == MAX_SPECIALS) return GD_ERR_INVALID_ARGUMENT;
    if (t->n_tokens == t->cap) {
        const int32_t cap = t->cap > 0 ? t->cap * 2 : 1024;
        bpe_token *grown = (bpe_token *)realloc(t->tokens, (size_t)cap * sizeof(bpe_token));
        if (grown == NULL) return GD_ERR_OUT_OF_MEMORY;
        t->tokens = grown;
        t->cap = cap;
    }
    k = &t->tokens[t->n_tokens];
    k->bytes = (uint8_t *)malloc(len + 1U);
    if (k->bytes == NULL) return GD_ERR_OUT_OF_MEMORY;
    memcpy(k->bytes, bytes, len);
    k->bytes[len] = 0U;
    k->len = len;
    k->left = left;
    k->right = right;
    k->special = special;
    if (special) t->special_ids[t->n_specials++] = t->n_tokens;
    t->n_tokens += 1;
    return GD_OK;
}

/* integer right after `field` in `line` */
static gd_status field_int(const char *line, const char *field, int *out)
{
    const char *p = strstr(line, field);
    char *end = NULL;
    long v;
    if (p == NULL) return GD_ERR_INVALID_ARGUMENT;
    p += strlen(field);
    errno = 0;
    v = strtol(p, &end, 10);
    if (errno != 0 || end == p || v < INT_MIN || v > INT_MAX) return GD_ERR_INVALID_ARGUMENT;
    *out = (int)v;
    return GD_OK;
}

static int hex_digit(char c)
{
    if (c >= '0' && c <= '9') return c - '0';
    if (c >= 'a' && c <= 'f') return c - 'a' + 10;
    if (c >= 'A' && c <= 'F') return c - 'A' + 10;
    return -1;
}

/* bytes of the hex string that follows `field` up to the closing quote, into buf (at most cap) */
static gd_status field_hex(const char *line, const char *field, uint8_t *buf, size_t cap, size_t *len_out)
{
    const char *p = strstr(line, field), *q;
    size_t n, i;
    if (p == NULL) return GD_ERR_INVALID_ARGUMENT;
    p += strlen(field);
    q = strchr(p, '"');
    if (q == NULL || ((size_t)(q - p) % 2U) != 0U) return GD_ERR_INVALID_ARGUMENT;
    n = (size_t)(q - p) / 2U;
    if (n > cap) return GD_ERR_OUT_OF_MEMORY;
    for (i = 0; i < n; ++i) {
        const int hi = hex_digit(p[2U * i]), lo = hex_digit(p[2U * i + 1U]);
        if (hi < 0 || lo < 0) return GD_ERR_INVALID_ARGUMENT;
        buf[i] = (uint8_t)((hi << 4) | lo);
    }
    *len_out = n;
    return GD_OK;
}

/* JSON string that follows `field` (which ends with the opening quote), unescaped into buf */
static gd_status field_text(const char *line, const char *field, uint8_t *buf, size_t cap, size_t *len_out)
{
    const char *p = strstr(line, field);
    size_t n = 0U;
    if (p == NULL) return GD_ERR_INVALID_ARGUMENT;
    for (p += strlen(field); *p != '\0' && *p != '"'; ++p) {
        char c = *p;
        if (c == '\\') {
            ++p;
            if (*p == '\0') return GD_ERR_INVALID_ARGUMENT;
            if (*p == 'n') c = '\n';
            else if (*p == 'r') c = '\r';
            else if (*p == 't') c = '\t';
            else if (*p == '"' || *p == '\\') c = *p;
            else return GD_ERR_UNSUPPORTED;
        }
        if (n == cap) return GD_ERR_OUT_OF_MEMORY;
        buf[n++] = (uint8_t)c;
    }
    if (*p != '"') return GD_ERR_INVALID_ARGUMENT;
    *len_out = n;
    return GD_OK;
}

gd_status gd_bpe_tokenizer_load(const char *path, const gd_tokenizer_config *cfg, gd_tokenizer **out)
{
    char line[4096];
    uint8_t buf[4096];
    gd_tokenizer *t;
    FILE *f;
    gd_status st = GD_OK;
    if (out != NULL) *out = NULL;
    if (path == NULL || out == NULL) return GD_ERR_INVALID_ARGUMENT;
    f = fopen(path, "rb");
    if (f == NULL) return GD_ERR_IO;
    t = (gd_tokenizer *)calloc(1U, sizeof(*t));
    if (t == NULL) {
        fclose(f);
        return GD_ERR_OUT_OF_MEMORY;
    }
    t->split_digits = cfg != NULL ? (cfg->split_digits != 0) : 1;
    t->allow_special = cfg != NULL ? (cfg->allow_special != 0) : 1;
    while (st == GD_OK && fgets(line, sizeof(line), f) != NULL) {
        size_t len = 0U;
        int id = -1, left = -1, right = -1;
        if (cfg == NULL && strstr(line, "\"split_digits\": true") != NULL) t->split_digits = 1;
        else if (cfg == NULL && strstr(line, "\"split_digits\": false") != NULL) t->split_digits = 0;
        if (strstr(line, "{\"id\":") == NULL) continue;
        st = field_int(line, "\"id\":", &id);
        if (st == GD_OK && id != t->n_tokens) st = GD_ERR_INVALID_ARGUMENT; /* ids count up from 0 */
        if (st != GD_OK) break;
        if (strstr(line, "\"kind\":\"special\"") != NULL) {
            st = field_text(line, "\"text\":\"", buf, sizeof(buf), &len);
            /* the reference keeps a special's text as a C string: it ends at a NUL */
            if (st == GD_OK) st = append_token(t, buf, strnlen((const char *)buf, len), 1, -1, -1);
        } else if (strstr(line, "\"kind\":\"merge\"") != NULL) {
            st = field_int(line, "\"left\":", &left);
            if (st == GD_OK) st = field_int(line, "\"right\":", &right);
            if (st == GD_OK) st = field_hex(line, "\"hex\":\"", buf, sizeof(buf), &len);
            if (st == GD_OK) st = append_token(t, buf, len, 0, left, right);
        } else if (strstr(line, "\"kind\":\"byte\"") != NULL) {
            st = field_hex(line, "\"hex\":\"", buf, sizeof(buf), &len);
            if (st == GD_OK && len != 1U) st = GD_ERR_INVALID_ARGUMENT;
            if (st == GD_OK) st = append_token(t, buf, len, 0, -1, -1);
        }
    }
    if (st == GD_OK && ferror(f) != 0) st = GD_ERR_IO;
    if (fclose(f) != 0 && st == GD_OK) st = GD_ERR_IO;
    if (st == GD_OK && t->n_tokens < 256) st = GD_ERR_INVALID_ARGUMENT; /* the byte vocabulary is missing */
    if (st == GD_OK) st = build_tables(t);
    if (st != GD_OK) {
        gd_tokenizer_destroy(t);
        return st;
    }
    digest(t);
    *out = t;
    return GD_OK;
}

void gd_tokenizer_destroy(gd_tokenizer *t)
{
    int32_t i;
    if (t == NULL) return;
    for (i = 0; i < t->n_tokens; ++i) free(t->tokens[i].bytes);
    free(t->tokens);
    free(t->pair_keys);
    free(t->pair_ids);
    free(t->byte_slots);
    free(t);
}

/* ---- cutting the text into pieces --------------------------------------------------------- */

enum { CLASS_SPACE, CLASS_DIGIT, CLASS_ALPHA, CLASS_OTHER };

static int is_digit(uint8_t c) { return c >= '0' && c <= '9'; }
static int is_space(uint8_t c) { return c == ' ' || c == '\n' || c == '\r' || c == '\t' || c == '\v' || c == '\f'; }

static int char_class(uint8_t c)
{
    if (is_space(c)) return CLASS_SPACE;
    if (is_digit(c)) return CLASS_DIGIT;
    if ((c >= 'A' && c <= 'Z') || (c >= 'a' && c <= 'z') || c >= 0x80U) return CLASS_ALPHA;
    return CLASS_OTHER;
}

typedef struct cutter {
    const gd_tokenizer *tok;
    const uint8_t *data;
    size_t len, at;
    int specials; /* special texts are looked for */
} cutter;

/* longest special text that starts at `pos` (the first listed among equally long ones); 0 if none */
static size_t special_at(const cutter *c, size_t pos, int32_t *id_out)
{
    size_t best = 0U;
    int s;
    if (!c->specials || !c->tok->special_first[c->data[pos]]) return 0U;
    for (s = 0; s < c->tok->n_specials; ++s) {
        const bpe_token *k = &c->tok->tokens[c->tok->special_ids[s]];
        if (k->len > best && pos + k->len <= c->len && memcmp(c->data + pos, k->bytes, k->len) == 0) {
            best = k->len;
            if (id_out != NULL) *id_out = c->tok->special_ids[s];
        }
    }
    return best;
}

/* a run of `cls` stops at its end, at a digit when digits stand alone, and where a special text starts */
static size_t run_end(const cutter *c, size_t i, int cls)
{
    while (i < c->len && char_class(c->data[i]) == cls && !(c->tok->split_digits && is_digit(c->data[i])) &&
           special_at(c, i, NULL) == 0U)
        ++i;
    return i;
}

/* Next stretch of the text: a special token (*special >= 0, nothing to merge) or ordinary bytes [*start, *end).
 * Returns 0 at the end of the text. */
static int next_stretch(cutter *c, size_t *start, size_t *end, int32_t *special)
{
    const int split = c->tok->split_digits;
    size_t i = c->at, m;
    if (i >= c->len) return 0;
    *special = -1;
    *start = i;
    m = special_at(c, i, special);
    if (m > 0U) {
        i += m;
    } else if (split && is_digit(c->data[i])) {
        i += 1U;
        *special = -1;
    } else if (is_space(c->data[i])) {
        /* one space in front of a word belongs to the word; other white space forms runs of its own */
        if (c->data[i] == ' ' && i + 1U < c->len && !is_space(c->data[i + 1U]) && !(split && is_digit(c->data[i + 1U])) &&
            special_at(c, i + 1U, NULL) == 0U) {
            i += 1U;
            i = run_end(c, i, char_class(c->data[i]));
        } else {
            i += 1U;
            while (i < c->len && is_space(c->data[i]) && special_at(c, i, NULL) == 0U) ++i;
        }
    } else {
        i = run_end(c, i + 1U, char_class(c->data[i]));
    }
    *end = i;
    c->at = i;
    return 1;
}

/* ---- encoding ----------------------------------------------------------------------------- */

typedef struct id_list {
    int32_t *ids;
    int len, cap;
} id_list;

static gd_status push_id(id_list *l, int32_t id)
{
    if (l->len == l->cap) {
        int32_t *grown;
        if (l->cap > INT_MAX / 2) return GD_ERR_OUT_OF_MEMORY;
        grown = (int32_t *)realloc(l->ids, (size_t)(l->cap > 0 ? l->cap * 2 : 64) * sizeof(int32_t));
        if (grown == NULL) return GD_ERR_OUT_OF_MEMORY;
        l->ids = grown;
        l->cap = l->cap > 0 ? l->cap * 2 : 64;
    }
    l->ids[l->len++] = id;
    return GD_OK;
}

/* One piece of at most MAX_PIECE bytes: the piece's own token if it has one, else its bytes merged pair by pair,
 * lowest merged id first, leftmost among equals (tokenizer_codec.c:66-142).  The parts form a linked list over
 * the byte positions; `rank[i]` is the merged id of part i with its successor. */
static gd_status encode_piece(const gd_tokenizer *t, const uint8_t *p, size_t n, id_list *out)
{
    int32_t part[MAX_PIECE], rank[MAX_PIECE];
    int next[MAX_PIECE], prev[MAX_PIECE];
    int i, count = (int)n;
    const size_t direct = bytes_slot(t, p, n);
    if (t->byte_slots[direct] >= 0) return push_id(out, t->byte_slots[direct]);
    for (i = 0; i < count; ++i) {
        part[i] = (int32_t)p[i];
        next[i] = i + 1 < count ? i + 1 : -1;
        prev[i] = i - 1;
    }
    for (i = 0; i < count; ++i) rank[i] = next[i] >= 0 ? pair_lookup(t, part[i], part[next[i]]) : -1;
    for (;;) {
        int best = -1, gone;
        for (i = 0; i >= 0; i = next[i]) {
            if (rank[i] >= 0 && (best < 0 || rank[i] < rank[best])) best = i;
        }
        if (best < 0) break;
        gone = next[best];
        part[best] = rank[best];
        next[best] = next[gone];
        if (next[gone] >= 0) prev[next[gone]] = best;
        rank[best] = next[best] >= 0 ? pair_lookup(t, part[best], part[next[best]]) : -1;
        if (prev[best] >= 0) rank[prev[best]] = pair_lookup(t, part[prev[best]], part[best]);
    }
    for (i = 0; i >= 0; i = next[i]) {
        const gd_status st = push_id(out, part[i]);
        if (st != GD_OK) return st;
    }
    return GD_OK;
}

gd_status gd_tokenizer_encode(gd_tokenizer *t, const char *text, int32_t **ids_out, int *n_ids_out)
{
    id_list list = {NULL, 0, 0};
    cutter c;
    size_t start, end;
    int32_t special;
    gd_status st = GD_OK;
    if (t == NULL || text == NULL || ids_out == NULL || n_ids_out == NULL) return GD_ERR_INVALID_ARGUMENT;
    *ids_out = NULL;
    *n_ids_out = 0;
    c.tok = t;
    c.data = (const uint8_t *)text;
    c.len = strlen(text);
    c.at = 0U;
    c.specials = t->allow_special && t->n_specials > 0;
    /* the reference hands back an allocation even for an empty text */
    list.ids = (int32_t *)malloc(64U * sizeof(int32_t));
    if (list.ids == NULL) return GD_ERR_OUT_OF_MEMORY;
    list.cap = 64;
    while (st == GD_OK && next_stretch(&c, &start, &end, &special)) {
        if (special >= 0) {
            st = push_id(&list, special);
            continue;
        }
        for (; st == GD_OK && start < end; start += MAX_PIECE)
            st = encode_piece(t, c.data + start, end - start < MAX_PIECE ? end - start : MAX_PIECE, &list);
    }
    if (st != GD_OK) {
        free(list.ids);
        return st;
    }
    *ids_out = list.ids;
    *n_ids_out = list.len;
    return GD_OK;
}

/* ---- decoding and queries ----------------------------------------------------------------- */

gd_status gd_tokenizer_decode(gd_tokenizer *t, const int32_t *ids, int n_ids, char **text_out)
{
    size_t total = 0U, at = 0U;
    char *text;
    int i;
    if (t == NULL || text_out == NULL || n_ids < 0 || (n_ids > 0 && ids == NULL)) return GD_ERR_INVALID_ARGUMENT;
    *text_out = NULL;
    for (i = 0; i < n_ids; ++i) {
        if (ids[i] < 0 || ids[i] >= t->n_tokens) return GD_ERR_INVALID_ARGUMENT;
        if (t->tokens[ids[i]].len > SIZE_MAX - total - 1U) return GD_ERR_OUT_OF_MEMORY;
        total += t->tokens[ids[i]].len;
    }
    text = (char *)malloc(total + 1U);
    if (text == NULL) return GD_ERR_OUT_OF_MEMORY;
    for (i = 0; i < n_ids; ++i) {
        memcpy(text + at, t->tokens[ids[i]].bytes, t->tokens[ids[i]].len);
        at += t->tokens[ids[i]].len;
    }
    text[at] = '\0';
    *text_out = text;
    return GD_OK;
}

gd_status gd_tokenizer_id(gd_tokenizer *t, const char *special, int32_t *id_out)
{
    int s;
    if (t == NULL || special == NULL || id_out == NULL) return GD_ERR_INVALID_ARGUMENT;
    for (s = 0; s < t->n_specials; ++s) {
        if (strcmp((const char *)t->tokens[t->special_ids[s]].bytes, special) == 0) {
            *id_out = t->special_ids[s];
            return GD_OK;
        }
    }
    return GD_ERR_INVALID_ARGUMENT;
}

int gd_tokenizer_vocab_size(const gd_tokenizer *t) { return t != NULL ? t->n_tokens : 0; }
uint64_t gd_tokenizer_hash(const gd_tokenizer *t) { return t != NULL ? t->hash : 0U; }
void gd_tokenizer_free(void *ptr) { free(ptr); }
