/*
 * Shared pieces of the operator front ends (core_<op>.c): the call pattern of the reference's
 * op capsules (docs/guides/register_op.md:99-146) is validate -> allocate the output in scratch
 * -> build backend views -> call gd_backend_<op>; the autograd record of the reference is a
 * no-op in inference scopes (src/autograd/autograd.c:146-149) and has no counterpart here.
 */
#ifndef GD_OPS_OP_COMMON_H
#define GD_OPS_OP_COMMON_H

#include <math.h>

#include "../core/core_internal.h"

#define GD_TRY(expr)                 \
    do {                             \
        gd_status st__ = (expr);     \
        if (st__ != GD_OK) return st__; \
    } while (0)

#define GD_FAIL(ctx, status, msg) return gd_context_set_error((ctx), (status), (msg))

static inline gd_status gd_op_backend_result(gd_context *ctx, gd_status st, const char *msg)
{
    return st == GD_OK ? GD_OK : gd_context_set_error(ctx, st, msg);
}

static inline void gd_op_bump_version(gd_tensor *t)
{
    t->version += 1U;
    if (t->version == 0U) t->version = 1U;
}

#endif
