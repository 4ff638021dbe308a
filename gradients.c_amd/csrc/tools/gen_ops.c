/*
 * Operator registry generator of the HIP backend tree: the counterpart of the reference's tools/gen_ops.c for a tree
 * that builds the inference subset of the operators.
 *
 * What it keeps from the reference's generator (tools/gen_ops.c:170-271):
 *   - the scan rule: a directory ops/<name>/ is an operator iff it holds core_<name>.c or autograd_<name>.c;
 *   - the grammar of ops/<name>/op_<name>.def: key = value lines, '#' starts a comment, the keys
 *     api = unary | binary | dropout and backend = unary | binary; everything else is ignored (operators with
 *     hand-declared signatures have comment-only files);
 *   - identifiers never move: an operator that already has a number in ops/op_kind.h keeps it, new operators are
 *     appended behind the largest number in name order (reference: src/ops/op_kind.h:5-41 holds 1..33).
 * What differs: this tree builds only some of the operators the enumeration names, so a number whose operator has no
 * directory here stays RESERVED (the reference's generator renumbers when a directory disappears, which would
 * break the identifiers the two trees share); and in place of the Metal pipeline table it writes the table of
 * backend entry points this backend answers with GD_ERR_UNSUPPORTED.
 *
 * Outputs (written only when their text changes):
 *   ops/op_kind.h                             the enumeration
 *   ops/op_registry.c                         name / built / api / backend table behind gd_op_kind_* lookups
 *   backends/hip/backend_hip_unsupported.c    one GD_ERR_UNSUPPORTED entry for every symbol of
 *                                             backends/hip/backend_symbols.def that no source file of the
 *                                             backend defines
 *
 * Usage: gen_ops <csrc directory> [--check]      (--check: write nothing, exit 3 if an output would change)
 */
#include <ctype.h>
#include <dirent.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>

#define MAX_OPS 256
#define MAX_SYMS 512
#define NAME_LEN 96

typedef struct op_entry {
    char name[NAME_LEN];
    unsigned id;      /* 0 until assigned */
    int built;        /* has a directory with a core_ / autograd_ source in this tree */
    int api, backend; /* 0 custom, 1 unary, 2 binary, 3 dropout (api only) */
} op_entry;

static op_entry ops[MAX_OPS];
static int n_ops;
static int check_only, would_change;

static char *slurp(const char *path)
{
    FILE *f = fopen(path, "rb");
    char *buf;
    long n;
    if (f == NULL) return NULL;
    fseek(f, 0, SEEK_END);
    n = ftell(f);
    fseek(f, 0, SEEK_SET);
    buf = (char *)malloc((size_t)n + 1);
    if (buf != NULL) {
        if (fread(buf, 1, (size_t)n, f) != (size_t)n) n = 0;
        buf[n] = '\0';
    }
    fclose(f);
    return buf;
}

static int is_file(const char *path)
{
    struct stat st;
    return stat(path, &st) == 0 && S_ISREG(st.st_mode);
}

static int is_dir(const char *path)
{
    struct stat st;
    return stat(path, &st) == 0 && S_ISDIR(st.st_mode);
}

static op_entry *find_op(const char *name)
{
    int i;
    for (i = 0; i < n_ops; ++i)
        if (strcmp(ops[i].name, name) == 0) return &ops[i];
    return NULL;
}

static op_entry *add_op(const char *name)
{
    op_entry *op = find_op(name);
    if (op != NULL) return op;
    if (n_ops == MAX_OPS || strlen(name) >= NAME_LEN) return NULL;
    op = &ops[n_ops++];
    memset(op, 0, sizeof(*op));
    strcpy(op->name, name);
    return op;
}

/* lower-case letters, digits and '_' after a leading letter: what the reference accepts as an operator directory */
static int valid_name(const char *s)
{
    if (!islower((unsigned char)s[0])) return 0;
    for (; *s; ++s)
        if (!islower((unsigned char)*s) && !isdigit((unsigned char)*s) && *s != '_') return 0;
    return 1;
}

static void trim(char **s)
{
    char *e;
    while (isspace((unsigned char)**s)) ++*s;
    e = *s + strlen(*s);
    while (e > *s && isspace((unsigned char)e[-1])) *--e = '\0';
}

static void read_def(op_entry *op, const char *path)
{
    char line[256];
    FILE *f = fopen(path, "r");
    if (f == NULL) return;
    while (fgets(line, sizeof(line), f) != NULL) {
        char *key = line, *value, *hash = strchr(line, '#'), *eq;
        if (hash != NULL) *hash = '\0';
        eq = strchr(line, '=');
        if (eq == NULL) continue;
        *eq = '\0';
        value = eq + 1;
        trim(&key);
        trim(&value);
        if (strcmp(key, "api") == 0)
            op->api = strcmp(value, "unary") == 0 ? 1 : strcmp(value, "binary") == 0 ? 2 : strcmp(value, "dropout") == 0 ? 3 : op->api;
        else if (strcmp(key, "backend") == 0)
            op->backend = strcmp(value, "unary") == 0 ? 1 : strcmp(value, "binary") == 0 ? 2 : op->backend;
    }
    fclose(f);
}

/* numbers already given out: every GD_OP_<NAME> = <n> of the existing enumeration */
static void read_existing_ids(const char *path)
{
    char *text = slurp(path), *p;
    if (text == NULL) return;
    for (p = strstr(text, "GD_OP_"); p != NULL; p = strstr(p + 1, "GD_OP_")) {
        char name[NAME_LEN];
        size_t n = 0;
        const char *q = p + 6, *eq;
        while ((isupper((unsigned char)q[n]) || isdigit((unsigned char)q[n]) || q[n] == '_') && n + 1 < NAME_LEN) {
            name[n] = (char)tolower((unsigned char)q[n]);
            ++n;
        }
        name[n] = '\0';
        eq = q + n;
        while (*eq == ' ') ++eq;
        if (n == 0 || *eq != '=' || strcmp(name, "invalid") == 0 || strcmp(name, "count") == 0) continue;
        {
            unsigned long v = strtoul(eq + 1, NULL, 10);
            op_entry *op = v > 0 ? add_op(name) : NULL;
            if (op != NULL) op->id = (unsigned)v;
        }
    }
    free(text);
}

static int scan_ops(const char *ops_dir)
{
    DIR *d = opendir(ops_dir);
    struct dirent *e;
    if (d == NULL) {
        fprintf(stderr, "gen_ops: cannot open %s\n", ops_dir);
        return 1;
    }
    while ((e = readdir(d)) != NULL) {
        char dir[4400], a[4800], b[4800], def[4800];
        op_entry *op;
        if (e->d_name[0] == '.' || !valid_name(e->d_name)) continue;
        snprintf(dir, sizeof(dir), "%.4096s/%.255s", ops_dir, e->d_name);
        if (!is_dir(dir)) continue;
        snprintf(a, sizeof(a), "%s/core_%.255s.c", dir, e->d_name);
        snprintf(b, sizeof(b), "%s/autograd_%.255s.c", dir, e->d_name);
        if (!is_file(a) && !is_file(b)) continue; /* kernels or shared headers only: not an operator */
        op = add_op(e->d_name);
        if (op == NULL) {
            fprintf(stderr, "gen_ops: too many operators\n");
            closedir(d);
            return 1;
        }
        op->built = 1;
        snprintf(def, sizeof(def), "%s/op_%.255s.def", dir, e->d_name);
        read_def(op, def);
    }
    closedir(d);
    return 0;
}

static int by_name(const void *a, const void *b) { return strcmp(((const op_entry *)a)->name, ((const op_entry *)b)->name); }
static int by_id(const void *a, const void *b)
{
    const op_entry *x = (const op_entry *)a, *y = (const op_entry *)b;
    return x->id < y->id ? -1 : x->id > y->id;
}

static void assign_ids(void)
{
    unsigned next = 0;
    int i;
    for (i = 0; i < n_ops; ++i)
        if (ops[i].id > next) next = ops[i].id;
    qsort(ops, (size_t)n_ops, sizeof(ops[0]), by_name); /* new operators take their numbers in name order */
    for (i = 0; i < n_ops; ++i)
        if (ops[i].id == 0) ops[i].id = ++next;
    qsort(ops, (size_t)n_ops, sizeof(ops[0]), by_id);
}

/* ---- output ---------------------------------------------------------------------------------------------- */

typedef struct text {
    char *s;
    size_t len, cap;
} text;

static void put(text *t, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
#include <stdarg.h>
static void put(text *t, const char *fmt, ...)
{
    char tmp[1024];
    va_list ap;
    int n;
    va_start(ap, fmt);
    n = vsnprintf(tmp, sizeof(tmp), fmt, ap);
    va_end(ap);
    if (n < 0 || (size_t)n >= sizeof(tmp)) {
        fprintf(stderr, "gen_ops: line too long\n");
        exit(1);
    }
    if (t->len + (size_t)n + 1 > t->cap) {
        t->cap = (t->cap + (size_t)n + 1) * 2;
        t->s = (char *)realloc(t->s, t->cap);
        if (t->s == NULL) exit(1);
    }
    memcpy(t->s + t->len, tmp, (size_t)n + 1);
    t->len += (size_t)n;
}

static int write_if_changed(const char *path, const text *t)
{
    char *old = slurp(path);
    FILE *f;
    if (old != NULL && strcmp(old, t->s) == 0) {
        free(old);
        return 0;
    }
    free(old);
    would_change = 1;
    if (check_only) {
        fprintf(stderr, "gen_ops: %s is out of date\n", path);
        return 0;
    }
    f = fopen(path, "wb");
    if (f == NULL || fwrite(t->s, 1, t->len, f) != t->len) {
        fprintf(stderr, "gen_ops: cannot write %s\n", path);
        return 1;
    }
    fclose(f);
    printf("gen_ops: wrote %s\n", path);
    return 0;
}

static void upper(const char *name, char *out)
{
    for (; *name; ++name) *out++ = (char)toupper((unsigned char)*name);
    *out = '\0';
}

static int emit_kind(const char *csrc)
{
    text t = {NULL, 0, 0};
    char path[4096], up[NAME_LEN];
    unsigned last = 0;
    int i, rc;
    put(&t, "#ifndef GD_OP_KIND_H\n#define GD_OP_KIND_H\n\n");
    put(&t, "/* @generated by tools/gen_ops.c; do not edit.  Numbers 1..33 are the reference's (src/ops/op_kind.h:5-41) and\n"
            " * never move; operators this tree adds follow.  gd_op_kind_built() tells which ones this build implements. */\n");
    put(&t, "typedef enum gd_op_kind {\n    GD_OP_INVALID = 0,\n");
    for (i = 0; i < n_ops; ++i) {
        upper(ops[i].name, up);
        put(&t, "    GD_OP_%s = %u,\n", up, ops[i].id);
        last = ops[i].id;
    }
    put(&t, "    GD_OP_COUNT = %u,\n} gd_op_kind;\n\n", last + 1);
    put(&t, "#pragma GCC visibility push(default)\n");
    put(&t, "/* name of an operator (\"sdpa_decode\"), NULL for a number nobody holds */\n");
    put(&t, "const char *gd_op_kind_name(gd_op_kind kind);\n");
    put(&t, "/* GD_OP_INVALID for an unknown name */\n");
    put(&t, "gd_op_kind gd_op_kind_from_name(const char *name);\n");
    put(&t, "/* 1 when this build holds the operator's front end (ops/<name>/core_<name>.c), 0 for a reserved number */\n");
    put(&t, "int gd_op_kind_built(gd_op_kind kind);\n");
    put(&t, "#pragma GCC visibility pop\n\n#endif /* GD_OP_KIND_H */\n");
    snprintf(path, sizeof(path), "%s/ops/op_kind.h", csrc);
    rc = write_if_changed(path, &t);
    free(t.s);
    return rc;
}

static int emit_registry(const char *csrc)
{
    static const char *shape[] = {"custom", "unary", "binary", "dropout"};
    text t = {NULL, 0, 0};
    char path[4096], up[NAME_LEN];
    int i, rc;
    put(&t, "/* @generated by tools/gen_ops.c; do not edit. */\n#include <stddef.h>\n#include <string.h>\n\n#include \"op_kind.h\"\n\n");
    put(&t, "typedef struct gd_op_info {\n    gd_op_kind kind;\n    const char *name;\n    int built;\n"
            "    const char *api, *backend; /* signature shape of op_<name>.def: custom, unary, binary, dropout */\n} gd_op_info;\n\n");
    put(&t, "static const gd_op_info gd_op_table[] = {\n");
    for (i = 0; i < n_ops; ++i) {
        upper(ops[i].name, up);
        put(&t, "    {GD_OP_%s, \"%s\", %d, \"%s\", \"%s\"},\n", up, ops[i].name, ops[i].built, shape[ops[i].api], shape[ops[i].backend]);
    }
    put(&t, "};\n\nstatic const gd_op_info *gd_op_find(gd_op_kind kind)\n{\n    size_t i;\n"
            "    for (i = 0; i < sizeof(gd_op_table) / sizeof(gd_op_table[0]); ++i)\n"
            "        if (gd_op_table[i].kind == kind) return &gd_op_table[i];\n    return NULL;\n}\n\n");
    put(&t, "const char *gd_op_kind_name(gd_op_kind kind)\n{\n    const gd_op_info *e = gd_op_find(kind);\n    return e != NULL ? e->name : NULL;\n}\n\n");
    put(&t, "int gd_op_kind_built(gd_op_kind kind)\n{\n    const gd_op_info *e = gd_op_find(kind);\n    return e != NULL && e->built;\n}\n\n");
    put(&t, "gd_op_kind gd_op_kind_from_name(const char *name)\n{\n    size_t i;\n    if (name == NULL) return GD_OP_INVALID;\n"
            "    for (i = 0; i < sizeof(gd_op_table) / sizeof(gd_op_table[0]); ++i)\n"
            "        if (strcmp(gd_op_table[i].name, name) == 0) return gd_op_table[i].kind;\n    return GD_OP_INVALID;\n}\n");
    snprintf(path, sizeof(path), "%s/ops/op_registry.c", csrc);
    rc = write_if_changed(path, &t);
    free(t.s);
    return rc;
}

/* ---- the table of entry points this backend does not implement ---------------------------------------------- */

static char syms[MAX_SYMS][NAME_LEN];
static int sym_defined[MAX_SYMS];
static int n_syms;

static int read_symbols(const char *path)
{
    char line[256];
    FILE *f = fopen(path, "r");
    if (f == NULL) {
        fprintf(stderr, "gen_ops: cannot open %s\n", path);
        return 1;
    }
    while (fgets(line, sizeof(line), f) != NULL) {
        char *s = line, *hash = strchr(line, '#');
        if (hash != NULL) *hash = '\0';
        trim(&s);
        if (*s == '\0') continue;
        if (n_syms == MAX_SYMS || strlen(s) >= NAME_LEN) {
            fclose(f);
            return 1;
        }
        strcpy(syms[n_syms++], s);
    }
    fclose(f);
    return 0;
}

/* a definition: the name at the start of a declarator on a line that begins in column 0 with a type and is not a
 * prototype of a file's own forward declarations (those end in ';' before any '{') */
static void mark_definitions(const char *file)
{
    char *text = slurp(file), *p;
    int i;
    if (text == NULL) return;
    for (i = 0; i < n_syms; ++i) {
        size_t n = strlen(syms[i]);
        if (sym_defined[i]) continue;
        for (p = strstr(text, syms[i]); p != NULL; p = strstr(p + 1, syms[i])) {
            const char *line = p, *q;
            if (p[n] != '(' || (p > text && (isalnum((unsigned char)p[-1]) || p[-1] == '_'))) continue;
            while (line > text && line[-1] != '\n') --line;
            if (!isalpha((unsigned char)*line) || strncmp(line, "return", 6) == 0) continue; /* a call, indented or not */
            for (q = p + n; *q && *q != ';' && *q != '{'; ++q) {}
            if (*q == '{') {
                sym_defined[i] = 1;
                break;
            }
        }
    }
    free(text);
}

static void scan_sources(const char *dir, int depth)
{
    DIR *d = opendir(dir);
    struct dirent *e;
    if (d == NULL) return;
    while ((e = readdir(d)) != NULL) {
        char path[4400];
        size_t n;
        if (e->d_name[0] == '.' || strlen(dir) > 4096) continue;
        snprintf(path, sizeof(path), "%.4096s/%.255s", dir, e->d_name);
        if (is_dir(path)) {
            if (depth < 3) scan_sources(path, depth + 1);
            continue;
        }
        n = strlen(e->d_name);
        if (strcmp(e->d_name, "backend_hip_unsupported.c") == 0) continue; /* the generated file itself */
        if ((n > 2 && strcmp(e->d_name + n - 2, ".c") == 0) || (n > 4 && strcmp(e->d_name + n - 4, ".hip") == 0)) mark_definitions(path);
    }
    closedir(d);
}

static int by_str(const void *a, const void *b) { return strcmp((const char *)a, (const char *)b); }

static int emit_unsupported(const char *csrc)
{
    text t = {NULL, 0, 0};
    char path[4096];
    int i, rc, count = 0;
    snprintf(path, sizeof(path), "%s/backends/hip/backend_symbols.def", csrc);
    if (read_symbols(path) != 0) return 1;
    snprintf(path, sizeof(path), "%s/backends/hip", csrc);
    scan_sources(path, 0);
    snprintf(path, sizeof(path), "%s/ops", csrc);
    scan_sources(path, 0);
    put(&t, "/* @generated by tools/gen_ops.c from backends/hip/backend_symbols.def; do not edit.\n *\n");
    put(&t, " * Entry points of the reference's backend boundary (src/core/backend.h, src/core/backend_generated.h) that this\n"
            " * backend does not implement: training kernels (backward passes, losses, optimizer, AMP, dropout), unary / binary\n"
            " * operators the decoder does not call, batched matmuls, reductions, permute / split.  The reference's core\n"
            " * references all of them, so a drop-in backend has to define them; like the reference's null backend\n"
            " * (src/backends/null/backend_null.c, src/backends/null/backend_generated.c) each one reports\n"
            " * GD_ERR_UNSUPPORTED and touches nothing.  The definitions take no named parameters (the arguments the caller\n"
            " * passes are ignored), which keeps this file independent of the argument structs of those operators.\n */\n");
    put(&t, "#include \"gd_backend_hip.h\"\n\n#pragma GCC visibility push(default)\n\n");
    put(&t, "#define GD_UNSUPPORTED_ENTRY(name) \\\n    gd_status name();              \\\n    gd_status name() { return GD_ERR_UNSUPPORTED; }\n\n");
    {
        static char list[MAX_SYMS][NAME_LEN];
        for (i = 0; i < n_syms; ++i)
            if (!sym_defined[i]) strcpy(list[count++], syms[i]);
        qsort(list, (size_t)count, NAME_LEN, by_str);
        for (i = 0; i < count; ++i) put(&t, "GD_UNSUPPORTED_ENTRY(%s)\n", list[i]);
    }
    put(&t, "\n#pragma GCC visibility pop\n");
    snprintf(path, sizeof(path), "%s/backends/hip/backend_hip_unsupported.c", csrc);
    rc = write_if_changed(path, &t);
    free(t.s);
    return rc;
}

int main(int argc, char **argv)
{
    char path[4096];
    const char *csrc;
    if (argc < 2 || argc > 3 || (argc == 3 && strcmp(argv[2], "--check") != 0)) {
        fprintf(stderr, "usage: gen_ops <csrc directory> [--check]\n");
        return 2;
    }
    csrc = argv[1];
    check_only = argc == 3;
    snprintf(path, sizeof(path), "%s/ops/op_kind.h", csrc);
    read_existing_ids(path);
    snprintf(path, sizeof(path), "%s/ops", csrc);
    if (scan_ops(path) != 0) return 1;
    assign_ids();
    if (emit_kind(csrc) != 0 || emit_registry(csrc) != 0 || emit_unsupported(csrc) != 0) return 1;
    return check_only && would_change ? 3 : 0;
}
