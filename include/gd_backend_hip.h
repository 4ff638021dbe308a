/*
 * gd_backend_hip.h - C-ABI of the MI355X (gfx950) backend for the gradients.c
 * inference decode path.
 *
 * Every `gd_backend_*` symbol declared in part 1-3 has the name, argument order,
 * struct layout and status behaviour of the symbol of the same name in the
 * reference's backend boundary, reference file `src/core/backend.h` (one backend
 * is linked per build there; this library is that backend for HIP).  Each
 * declaration cites the reference lines it replaces.  Part 4 holds entry points
 * that have no counterpart in the reference (device argmax, fused operators,
 * stream timing, graph capture); they use the same view structs.
 *
 * Conventions (reference src/core/backend.h:132-140, src/ops/op_common.h:60-94):
 *   - tensors are borrowed `gd_backend_tensor_view`s: buffer + BYTE offset,
 *     element count, dtype code, rank, shape, strides in ELEMENTS; all views the
 *     decode path passes are contiguous;
 *   - matrices are `gd_backend_matrix_view`s with a row pitch in bytes;
 *   - outputs are pre-allocated by the caller, the backend writes in place;
 *   - argument structs are read during the call only;
 *   - between gd_backend_scope_begin and gd_backend_record_fence operators are
 *     enqueued asynchronously in order on one HIP stream; outside a scope each
 *     operator returns after its work has completed;
 *   - device-side invalid cache positions are skipped silently, never trap.
 */
#ifndef GD_BACKEND_HIP_H
#define GD_BACKEND_HIP_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default) /* the library is built with hidden visibility: only these are exported */

/* ---- part 1: status, dtype codes, handles, views ------------------------- */

/* reference include/gradients/status.h:8-19 (same numeric values). */
#ifndef GRADIENTS_STATUS_H
typedef enum gd_status {
    GD_OK = 0,
    GD_ERR_INVALID_ARGUMENT = -1,
    GD_ERR_OUT_OF_MEMORY = -2,
    GD_ERR_FROZEN = -3,
    GD_ERR_BUSY = -4,
    GD_ERR_BAD_STATE = -5,
    GD_ERR_UNSUPPORTED = -6,
    GD_ERR_INTERNAL = -7,
    GD_ERR_NOT_IMPLEMENTED = -8,
    GD_ERR_IO = -9
} gd_status;
#endif

/* dtype codes carried in view.dtype: reference include/gradients/tensor.h:49-57. */
#define GD_BACKEND_DTYPE_F16 1u
#define GD_BACKEND_DTYPE_BF16 2u
#define GD_BACKEND_DTYPE_F32 3u
#define GD_BACKEND_DTYPE_I32 4u
#define GD_BACKEND_DTYPE_U8 5u
#define GD_BACKEND_DTYPE_U16 6u

#define GD_BACKEND_MAX_DIMS 8u

typedef struct gd_backend gd_backend;               /* backend.h:10 */
typedef struct gd_backend_buffer gd_backend_buffer; /* backend.h:11 */

/* backend.h:13-15 */
typedef struct gd_backend_fence {
    void *handle;
} gd_backend_fence;

/* backend.h:17-19; the reference defines only METAL = 1. */
typedef enum gd_backend_kind {
    GD_BACKEND_METAL = 1,
    GD_BACKEND_HIP = 2
} gd_backend_kind;

/* backend.h:21-28 */
typedef struct gd_backend_matrix_view {
    gd_backend_buffer *buffer;
    size_t offset;    /* bytes */
    uint32_t rows;
    uint32_t cols;
    size_t row_bytes; /* pitch */
    uint32_t dtype;
} gd_backend_matrix_view;

/* backend.h:45-50 */
typedef struct gd_backend_vector_view {
    gd_backend_buffer *buffer;
    size_t offset;
    uint32_t length;
    uint32_t dtype;
} gd_backend_vector_view;

/* backend.h:132-140 */
typedef struct gd_backend_tensor_view {
    gd_backend_buffer *buffer;
    size_t offset; /* bytes */
    size_t count;  /* elements */
    uint32_t dtype;
    uint32_t rank;
    int64_t shape[8];
    int64_t strides[8]; /* elements */
} gd_backend_tensor_view;

/* ---- part 2: lifecycle, buffers, scope, transfers ------------------------ */

/* backend.h:144-148.  GD_ERR_UNSUPPORTED when no HIP device is present. */
gd_status gd_backend_create_default(gd_backend **out_backend);
void gd_backend_destroy(gd_backend *backend);
gd_backend_kind gd_backend_kind_query(const gd_backend *backend);
const char *gd_backend_name(const gd_backend *backend);

/* backend.h:150-156.  Buffers are HBM allocations; host_ptr is NULL and
 * is_host_visible false unless the backend was created with the environment
 * variable GD_HIP_HOST_VISIBLE=1 (pinned host memory mapped into the device,
 * for running an unmodified reference core; not for performance). */
gd_status gd_backend_buffer_create(gd_backend *backend, size_t nbytes, gd_backend_buffer **out_buffer);
void gd_backend_buffer_destroy(gd_backend_buffer *buffer);
size_t gd_backend_buffer_nbytes(const gd_backend_buffer *buffer);
void *gd_backend_buffer_host_ptr(gd_backend_buffer *buffer);
bool gd_backend_buffer_is_host_visible(const gd_backend_buffer *buffer);

/* backend.h:158-159.  scope_begin: GD_ERR_BAD_STATE when nested (reference
 * src/backends/metal/backend_metal.m:541-544).  flush = submit + block. */
gd_status gd_backend_scope_begin(gd_backend *backend);
gd_status gd_backend_flush(gd_backend *backend);

/* backend.h:161-170; synchronous, ordered after all enqueued work. */
gd_status gd_backend_upload(gd_backend *backend, gd_backend_buffer *buffer, size_t offset,
                            const void *src, size_t nbytes);
gd_status gd_backend_download(gd_backend *backend, gd_backend_buffer *buffer, size_t offset,
                              void *dst, size_t nbytes);

/* backend.h:172-177; elem_size in {1,2,4}, pattern's low bytes repeated. */
gd_status gd_backend_fill(gd_backend *backend, gd_backend_buffer *buffer, size_t offset,
                          size_t count, size_t elem_size, uint32_t pattern);

/* backend.h:178-185.  Element i = low + (high - low) * u_i with u_i the 24 bits [40,64) of
 * splitmix64(seed + i) scaled by 2^-24; F16 / BF16 / F32 destinations, anything else UNSUPPORTED. */
gd_status gd_backend_rand_uniform(gd_backend *backend, gd_backend_buffer *buffer, size_t offset, size_t count,
                                  uint32_t dtype, uint64_t seed, float low, float high);

/* backend.h:788-791.  record_fence closes the scope opened by scope_begin. */
gd_status gd_backend_record_fence(gd_backend *backend, gd_backend_fence *out_fence);
void gd_backend_fence_destroy(gd_backend_fence *fence);
bool gd_backend_fence_is_complete(gd_backend_fence *fence);
gd_status gd_backend_fence_wait(gd_backend_fence *fence);

/* ---- part 3: operators on the decode path -------------------------------- */

/* backend.h:301-312.  out[i,:] = table[ids[i],:]; id out of range -> NaN row
 * (reference src/ops/embedding/metal_embedding.metal:26-30). */
typedef struct gd_backend_embedding_args {
    uint64_t ids_count;
    uint64_t vocab;
    uint64_t dim;
} gd_backend_embedding_args;
gd_status gd_backend_embedding_forward(gd_backend *backend, const gd_backend_tensor_view *table,
                                       const gd_backend_tensor_view *ids,
                                       const gd_backend_tensor_view *out,
                                       const gd_backend_embedding_args *args);

/* backend.h:528-544.  Only rows, cols, eps are read by the forward. */
typedef struct gd_backend_rms_norm_args {
    uint64_t rows;
    uint64_t cols;
    uint64_t row_blocks;
    float eps;
    uint32_t simdgroups;
    uint32_t wgrad_simdgroups;
    uint32_t wgrad_row_block;
    uint32_t reserved0;
} gd_backend_rms_norm_args;
gd_status gd_backend_rms_norm_forward(gd_backend *backend, const gd_backend_tensor_view *x,
                                      const gd_backend_tensor_view *weight,
                                      const gd_backend_tensor_view *out,
                                      const gd_backend_rms_norm_args *args);

/* backend.h:187-195.  F16 operands, F32 accumulate, one F16 rounding.
 * matmul: y[M,N] = x[M,K] w[K,N].  matmul_nt: y = x w^T with w stored [N,K]. */
gd_status gd_backend_matmul(gd_backend *backend, const gd_backend_matrix_view *x,
                            const gd_backend_matrix_view *w, const gd_backend_matrix_view *y);
gd_status gd_backend_matmul_nt(gd_backend *backend, const gd_backend_matrix_view *x,
                               const gd_backend_matrix_view *w, const gd_backend_matrix_view *y);
/* backend.h:215-219.  y = x w + bias, bias added in F32 before the rounding
 * (reference src/ops/_shared/gemm/metal_gemm_common.h:125-132). */
gd_status gd_backend_linear(gd_backend *backend, const gd_backend_matrix_view *x,
                            const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                            const gd_backend_matrix_view *y);

/* reference src/core/backend_generated.h:14-17.  F16 add with NumPy-style
 * right-aligned broadcasting of contiguous operands; residual adds (same shape)
 * and bias adds ([rows,N] + [N]) are the shapes the decode path uses. */
gd_status gd_backend_add(gd_backend *backend, const gd_backend_tensor_view *x,
                         const gd_backend_tensor_view *y, const gd_backend_tensor_view *out);

/* backend.h:321-325, 341-349.  qkv [N, 3*H*D] -> q,k rotated, v copied, each
 * [N,H,D]; full-head rotation only (n_dims == head_dim). */
typedef struct gd_backend_rope_args {
    float theta;
    uint32_t n_dims;
    uint32_t interleaved;
} gd_backend_rope_args;
gd_status gd_backend_qkv_split_rope_forward(gd_backend *backend, const gd_backend_tensor_view *qkv,
                                            const gd_backend_tensor_view *pos_ids,
                                            const gd_backend_tensor_view *q,
                                            const gd_backend_tensor_view *k,
                                            const gd_backend_tensor_view *v, uint32_t n_heads,
                                            uint32_t head_dim, const gd_backend_rope_args *args);

/* backend.h:520-522.  out[r,c] = x12[r,c] * silu(x12[r,H+c]). */
gd_status gd_backend_swiglu_split_forward(gd_backend *backend, const gd_backend_tensor_view *x12,
                                          const gd_backend_tensor_view *out);

/* backend.h:579-591.  Copies a contiguous slice into its place inside the contiguous concatenated
 * tensor: dst[outer, axis_offset + a, inner] = src[outer, a, inner] with a < slice_axis.  The
 * reference's generator concatenates the last prompt rows with it. */
typedef struct gd_backend_concat_args {
    uint64_t count;
    uint64_t inner;
    uint64_t slice_axis;
    uint64_t full_axis;
    uint64_t axis_offset;
} gd_backend_concat_args;
gd_status gd_backend_concat_to_full(gd_backend *backend, const gd_backend_tensor_view *src,
                                    const gd_backend_tensor_view *dst, const gd_backend_concat_args *args);

/* backend.h:671-698.  Packed causal attention over cu_seqlens; stats may be
 * NULL (inference).  Head dim up to 128 (the reference stops at 64). */
typedef struct gd_backend_sdpa_varlen_args {
    float scale;
    uint32_t causal;
    uint32_t sliding_window;
    uint32_t prefix_len;
    uint32_t max_seqlen;
    uint32_t use_forward_stats;
} gd_backend_sdpa_varlen_args;
gd_status gd_backend_sdpa_varlen(gd_backend *backend, const gd_backend_tensor_view *q,
                                 const gd_backend_tensor_view *k, const gd_backend_tensor_view *v,
                                 const gd_backend_tensor_view *cu_seqlens,
                                 const gd_backend_tensor_view *out,
                                 const gd_backend_tensor_view *stats,
                                 const gd_backend_sdpa_varlen_args *args);

/* gd_backend_sdpa_varlen whose keys and values are read from the caches the packed prefill has just appended them
 * to: k_cache / v_cache [B,Tmax,Hkv,D] with B = number of segments, token t of segment b in cache row t of sequence
 * b (the prefill appends at position 0).  Same kernel, same arithmetic and masks as gd_backend_sdpa_varlen on packed
 * k / v holding the same rows; what it saves is writing the packed k / v and reading them back.  A segment longer
 * than Tmax leaves its rows of `out` untouched.  F16, head size 64 or 128, caches below 4 GiB
 * (GD_ERR_UNSUPPORTED otherwise: use gd_backend_sdpa_varlen on packed rows).  No reference counterpart (the
 * reference's prefill reads the packed rows: examples/gpt_lm/gpt_lm_shared.c:896-940). */
gd_status gd_backend_sdpa_varlen_cached(gd_backend *backend, const gd_backend_tensor_view *q,
                                        const gd_backend_tensor_view *k_cache,
                                        const gd_backend_tensor_view *v_cache,
                                        const gd_backend_tensor_view *cu_seqlens,
                                        const gd_backend_tensor_view *out,
                                        const gd_backend_sdpa_varlen_args *args);

/* backend.h:680-685, 710-729.  q/out [B,Tq,Hq,D], caches [B,Tmax,Hkv,D].
 * `sdpa_decode` takes a rank-0 I32 position tensor, `_at` a host scalar in
 * args->cache_pos, `_positions` an I32 [B] tensor.  A negative position leaves
 * that batch row of `out` untouched. */
typedef struct gd_backend_sdpa_decode_args {
    float scale;
    uint32_t sliding_window;
    uint32_t prefix_len;
    int32_t cache_pos;
} gd_backend_sdpa_decode_args;
gd_status gd_backend_sdpa_decode(gd_backend *backend, const gd_backend_tensor_view *q,
                                 const gd_backend_tensor_view *k_cache,
                                 const gd_backend_tensor_view *v_cache,
                                 const gd_backend_tensor_view *cache_pos,
                                 const gd_backend_tensor_view *out,
                                 const gd_backend_sdpa_decode_args *args);
gd_status gd_backend_sdpa_decode_at(gd_backend *backend, const gd_backend_tensor_view *q,
                                    const gd_backend_tensor_view *k_cache,
                                    const gd_backend_tensor_view *v_cache,
                                    const gd_backend_tensor_view *out,
                                    const gd_backend_sdpa_decode_args *args);
gd_status gd_backend_sdpa_decode_positions(gd_backend *backend, const gd_backend_tensor_view *q,
                                           const gd_backend_tensor_view *k_cache,
                                           const gd_backend_tensor_view *v_cache,
                                           const gd_backend_tensor_view *cache_pos,
                                           const gd_backend_tensor_view *out,
                                           const gd_backend_sdpa_decode_args *args);

/* backend.h:687-689, 730-750.  cache[b, pos_b + t] = new[b, t]; rows whose
 * position is negative or whose span would pass Tmax are skipped on the device
 * (reference src/ops/kv_cache_append/metal_kv_cache_append.metal:52-54,102-113). */
typedef struct gd_backend_kv_cache_append_args {
    int32_t cache_pos;
} gd_backend_kv_cache_append_args;
gd_status gd_backend_kv_cache_append_at(gd_backend *backend, const gd_backend_tensor_view *k_cache,
                                        const gd_backend_tensor_view *v_cache,
                                        const gd_backend_tensor_view *k_new,
                                        const gd_backend_tensor_view *v_new,
                                        const gd_backend_kv_cache_append_args *args);
gd_status gd_backend_kv_cache_append_positions(gd_backend *backend,
                                               const gd_backend_tensor_view *k_cache,
                                               const gd_backend_tensor_view *v_cache,
                                               const gd_backend_tensor_view *cache_pos,
                                               const gd_backend_tensor_view *k_new,
                                               const gd_backend_tensor_view *v_new,
                                               const gd_backend_kv_cache_append_args *args);
gd_status gd_backend_kv_cache_append_packed(gd_backend *backend,
                                            const gd_backend_tensor_view *k_cache,
                                            const gd_backend_tensor_view *v_cache,
                                            const gd_backend_tensor_view *cache_pos,
                                            const gd_backend_tensor_view *cu_seqlens,
                                            const gd_backend_tensor_view *k_new,
                                            const gd_backend_tensor_view *v_new,
                                            const gd_backend_kv_cache_append_args *args);

/* MiniMax-M3 block-sparse attention over packed sequences, forward (reference src/core/backend.h:632-655; Metal
 * kernels metal_minimax_m3_index_topk.metal, metal_minimax_m3_sparse_attention.metal under src/ops).  All tensors
 * contiguous; q / k / v / out F16 [N, H, Dh] (Dh <= 64 as in the reference, odd sizes included; Dh = 64 with a block
 * size of 64 or 128 on 16-byte aligned views runs on the matrix cores, Dh in {4, 8, 16, 32, 64} on aligned views
 * with vector loads, everything else half by half), cu_seqlens
 * I32 [B+1], topk_idx I32 [Hkv, N, topk]; block_size <= 128,
 * topk <= 16; rows at or beyond max_seqlen inside their sequence are not processed.
 *   index_topk        index_q and index_k have the same number of heads.  Row i of a sequence sees blocks
 *                     0 .. i / block_size; a block's score is the largest q_i . k_j over its keys j <= i (NaN
 *                     counts as -inf); the first init_blocks blocks rank highest, the last local_blocks visible
 *                     ones next; the topk best are stored in descending order, an equal score never displaces
 *                     an earlier block; unused slots hold -1
 *   sparse_attention  softmax(scale q_i . k_j) v_j over the keys j <= i of the row's listed blocks, query head
 *                     hq using the list and the K / V of kv head hq / (Hq / Hkv); zeros when nothing is visible */
typedef struct gd_backend_minimax_m3_sparse_args {
    float scale;
    uint32_t block_size, topk, init_blocks, local_blocks, max_seqlen;
} gd_backend_minimax_m3_sparse_args;

gd_status gd_backend_minimax_m3_index_topk(gd_backend *backend, const gd_backend_tensor_view *index_q,
                                           const gd_backend_tensor_view *index_k,
                                           const gd_backend_tensor_view *cu_seqlens,
                                           const gd_backend_tensor_view *topk_idx,
                                           const gd_backend_minimax_m3_sparse_args *args);
gd_status gd_backend_minimax_m3_sparse_attention(gd_backend *backend, const gd_backend_tensor_view *q,
                                                 const gd_backend_tensor_view *k, const gd_backend_tensor_view *v,
                                                 const gd_backend_tensor_view *cu_seqlens,
                                                 const gd_backend_tensor_view *topk_idx,
                                                 const gd_backend_tensor_view *out,
                                                 const gd_backend_minimax_m3_sparse_args *args);

/* ---- part 4: entry points without a counterpart in the reference --------- */

/* Greedy next token on the device.  The reference downloads the logits and
 * scans them on the host (examples/gpt_lm/gpt_lm_shared.c:1388-1400): index of
 * the largest finite value, first occurrence wins, 0 when no value is finite.
 * logits F16 or F32 [rows, cols]; ids I32 [rows]; gap (optional, may be NULL)
 * F32 [rows] = best - second best finite value (+inf when fewer than two). */
gd_status gd_backend_argmax_rows(gd_backend *backend, const gd_backend_tensor_view *logits,
                                 const gd_backend_tensor_view *ids,
                                 const gd_backend_tensor_view *gap);

/* Fused form of the reference's two-step gd_swiglu_split + gd_linear
 * (src/ops/swiglu_split_linear/core_swiglu_split_linear.c:260-263):
 * y = half(half(x12[:, :H] * silu(x12[:, H:])) @ w[H,N] + bias).  The F16
 * rounding of the activation is kept.  bias may be NULL. */
gd_status gd_backend_swiglu_split_linear(gd_backend *backend, const gd_backend_matrix_view *x12,
                                         const gd_backend_matrix_view *w,
                                         const gd_backend_vector_view *bias,
                                         const gd_backend_matrix_view *y);

/* y = half(half(x w^T) + bias): matmul_nt followed by the bias add in one
 * launch, keeping both F16 roundings of the reference's two-kernel sequence
 * (src/ops/linear_transposed_weight/core_linear_transposed_weight.c:51,76).
 * bias may be NULL (then identical to gd_backend_matmul_nt). */
gd_status gd_backend_linear_nt(gd_backend *backend, const gd_backend_matrix_view *x,
                               const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                               const gd_backend_matrix_view *y);

/* One launch for a projection together with the elementwise operators the reference issues
 * around it in the decoder block (examples/gpt_lm/gpt_lm_shared.c:1017-1070), with the same
 * rounding points as the separate operators:
 *   a = x                                            prologue 0
 *     | half(x[:, :K] * silu(x[:, K:2K]))            prologue 1 (gd_swiglu_split)
 *     | half(x * norm_weight * rsqrt(mean(x^2)+eps)) prologue 2 (gd_rms_norm)
 *   t = a @ w  (w [K,N])  or  a @ w^T  (w [N,K], w_is_nk = 1), F32 accumulate
 *   u = half(t)                                      bias_mode 0 (bias must be NULL)
 *     | half(t + bias)                               bias_mode 1 (gd_linear)
 *     | half(half(t) + bias)                         bias_mode 2 (gd_linear_transposed_weight)
 *   y = u, or half(residual + u) when residual != NULL (gd_add)                      epilogue 0
 *     | half(u[:, :H] * silu(u[:, H:])), w [2H,K], bias [2H], y [M,H]                epilogue 1 (the gd_swiglu_split
 *       that follows the up/gate projection; w_is_nk only, no residual, else UNSUPPORTED) */
typedef struct gd_backend_fused_linear_args {
    uint32_t w_is_nk;
    uint32_t bias_mode;
    uint32_t prologue;
    float eps;
    uint32_t epilogue;
} gd_backend_fused_linear_args;
gd_status gd_backend_fused_linear(gd_backend *backend, const gd_backend_matrix_view *x,
                                  const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                                  const gd_backend_matrix_view *residual,
                                  const gd_backend_vector_view *norm_weight,
                                  const gd_backend_matrix_view *y, const gd_backend_fused_linear_args *args);

/* Decode-step form of qkv_split_rope + kv_cache_append_positions in one launch: qkv [B, 3*H*D]
 * (one new token per sequence), q [B,H,D] receives the rotated queries, the rotated keys and the
 * copied values are written to row cache_pos[b] of k_cache / v_cache [B,Tmax,H,D].  Same
 * arithmetic and the same bytes as the two separate operators; a sequence whose cache position is
 * negative or >= Tmax keeps its caches untouched.  NeoX pairing, head_dim % 16 == 0, F16 only
 * (GD_ERR_UNSUPPORTED otherwise: use the separate operators). */
gd_status gd_backend_qkv_rope_append(gd_backend *backend, const gd_backend_tensor_view *qkv,
                                     const gd_backend_tensor_view *pos_ids,
                                     const gd_backend_tensor_view *cache_pos, const gd_backend_tensor_view *q,
                                     const gd_backend_tensor_view *k_cache, const gd_backend_tensor_view *v_cache,
                                     uint32_t n_heads, uint32_t head_dim, const gd_backend_rope_args *args);

/* Packed-prefill form of qkv_split_rope + kv_cache_append_packed in one launch: qkv [N, 3*H*D] of N packed tokens,
 * q, k, v [N,H,D] as gd_backend_qkv_split_rope_forward writes them, and the rotated keys and copied values of token
 * t of sequence b (rows cu_seqlens[b] .. cu_seqlens[b+1]) also into row cache_pos[b] + t of k_cache / v_cache
 * [B,Tmax,H,D], under the rules of gd_backend_kv_cache_append_packed (nothing is appended unless cu_seqlens starts at
 * 0; a sequence with a negative position or whose rows do not fit behind it keeps its caches).  Same arithmetic as
 * the two separate operators (values bit for bit; rotated elements within one F16 unit in the last place of theirs);
 * the appended rows are the rows written to k / v and are not read back from memory.  k and v may both be NULL: then
 * the rows only go into the caches (for a caller that reads them there: gd_backend_sdpa_varlen_cached).  NeoX pairing,
 * head_dim % 16 == 0, F16 only (GD_ERR_UNSUPPORTED otherwise: use the separate operators).  No reference counterpart
 * (reference order of the two operators: examples/gpt_lm/gpt_lm_shared.c:896-917). */
gd_status gd_backend_qkv_rope_append_packed(gd_backend *backend, const gd_backend_tensor_view *qkv,
                                            const gd_backend_tensor_view *pos_ids,
                                            const gd_backend_tensor_view *cache_pos,
                                            const gd_backend_tensor_view *cu_seqlens, const gd_backend_tensor_view *q,
                                            const gd_backend_tensor_view *k, const gd_backend_tensor_view *v,
                                            const gd_backend_tensor_view *k_cache,
                                            const gd_backend_tensor_view *v_cache, uint32_t n_heads, uint32_t head_dim,
                                            const gd_backend_rope_args *args);

/* The packed prefill's rotation and cache append inside the qkv projection, in two calls.
 *
 * gd_backend_rope_table_packed, once per prefill: for the N packed prompt rows the angles of their positions,
 * cos_rows / sin_rows [ceil(N/32)*32, head_dim/2] F32 (pair p of row n: angle = float(pos_ids[n]) * exp2(p *
 * -2*log2(theta) / head_dim), as gd_backend_qkv_split_rope_forward computes them; stored for the reads of the
 * projection's epilogue, not row by row: element (n, p) sits at (((n/32) * (head_dim/16) + p/8) * 2 + (p/4)%2) * 128 +
 * (n%32) * 4 + p%4; the rows behind N are not written), and cache_rows [N] I32: the row of a
 * [B,Tmax,H,D] cache seen as [B*Tmax, H*D] that token t of sequence b goes to, b*tmax + cache_pos[b] + t, under the
 * rules of gd_backend_kv_cache_append_packed (nothing unless cu_seqlens starts at 0; a sequence with a negative
 * position or whose rows do not fit behind it is skipped), -1 for a row that is not appended.  NeoX pairing only.
 *
 * gd_backend_linear_qkv_rope_packed, once per layer: x [N,K] times w [3*H*D, K] (plus bias; bias_mode 0 none,
 * 1 added in F32 before the rounding as gd_backend_linear does, 2 added in F16 to the rounded product), the
 * projection rounded to F16, q and k rotated in F32 with the table's angles and rounded again, then rotated q to
 * q [N,H,D] and rotated k and copied v to row cache_rows[n] of k_cache / v_cache: the results of
 * gd_backend_linear + gd_backend_qkv_split_rope_forward + gd_backend_kv_cache_append_packed (values bit for bit,
 * rotated elements within one F16 unit in the last place), with no [N, 3*H*D] intermediate written and read back:
 * the rotation rides in the epilogue of the 256 x 256 tiles.  The rows of a last, partly filled round of tiles go
 * through the plain projection into `work` [N, 3*H*D] (only those rows of it are written) and a rotation kernel
 * driven by the same table.  Packed k / v rows are not produced: read them from the caches
 * (gd_backend_sdpa_varlen_cached).  F16, [N,K] weights, head size 64 or 128, H*D a multiple of 256, K a multiple
 * of 64, 16-byte aligned rows (GD_ERR_UNSUPPORTED otherwise: use the separate operators).  No reference counterpart
 * (reference order of the operators: examples/gpt_lm/gpt_lm_shared.c:880-917). */
gd_status gd_backend_rope_table_packed(gd_backend *backend, const gd_backend_tensor_view *pos_ids,
                                       const gd_backend_tensor_view *cache_pos,
                                       const gd_backend_tensor_view *cu_seqlens,
                                       const gd_backend_tensor_view *cos_rows, const gd_backend_tensor_view *sin_rows,
                                       const gd_backend_tensor_view *cache_rows, uint32_t head_dim, uint32_t tmax,
                                       const gd_backend_rope_args *args);
gd_status gd_backend_linear_qkv_rope_packed(gd_backend *backend, const gd_backend_matrix_view *x,
                                            const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                                            const gd_backend_tensor_view *cos_rows,
                                            const gd_backend_tensor_view *sin_rows,
                                            const gd_backend_tensor_view *cache_rows, const gd_backend_tensor_view *q,
                                            const gd_backend_tensor_view *k_cache,
                                            const gd_backend_tensor_view *v_cache,
                                            const gd_backend_matrix_view *work, uint32_t n_heads, uint32_t head_dim,
                                            uint32_t bias_mode);

/* out[i,:] = src[rows[i],:]; replaces the reference's per-sequence slice +
 * concat when the last prompt rows are selected
 * (examples/gpt_lm/gpt_lm_shared.c:1117-1169).  Row index out of range -> row
 * left untouched. */
gd_status gd_backend_gather_rows(gd_backend *backend, const gd_backend_tensor_view *src,
                                 const gd_backend_tensor_view *rows,
                                 const gd_backend_tensor_view *out);

/* dst[i] = src[i] + delta for contiguous I32 tensors (device-resident cache
 * positions advance without a host round trip). */
gd_status gd_backend_add_scalar_i32(gd_backend *backend, const gd_backend_tensor_view *src,
                                    const gd_backend_tensor_view *dst, int32_t delta);

/* End of a device-resident greedy decode step, one launch: ids[b] = next_ids[b];
 * positions[b] += pos_delta; s = *step_counter; when s < max_steps, out_ids[s*B + b] = next_ids[b] and
 * (out_gaps != NULL) out_gaps[s*B + b] = gaps[b]; then *step_counter = s + 1.  All tensors
 * contiguous; next_ids/ids/positions I32 [B], step_counter I32 [1], out_ids I32 [max_steps*B],
 * gaps / out_gaps F32 (both NULL or both given). */
gd_status gd_backend_decode_advance(gd_backend *backend, const gd_backend_tensor_view *next_ids,
                                    const gd_backend_tensor_view *gaps, const gd_backend_tensor_view *ids,
                                    const gd_backend_tensor_view *positions,
                                    const gd_backend_tensor_view *step_counter,
                                    const gd_backend_tensor_view *out_ids,
                                    const gd_backend_tensor_view *out_gaps, int32_t pos_delta);

/* gd_backend_fused_linear (prologue 0 or 2, w [3*H*D, K] with w_is_nk = 1, any bias mode) followed by
 * gd_backend_qkv_rope_append on its result, in one launch: the [B, 3*H*D] projection is never stored; its q
 * columns are rotated into q [B,H,D], its k columns rotated and its v columns copied into row cache_pos[b] of the
 * caches [B,Tmax,H,D] (sequences whose position is negative or >= Tmax keep their caches).  Same rounding points
 * as the separate operators.  NeoX pairing, head_dim % 32 == 0, fewer than 128 rows, else UNSUPPORTED. */
gd_status gd_backend_fused_qkv_rope_append(gd_backend *backend, const gd_backend_matrix_view *x,
                                           const gd_backend_matrix_view *w, const gd_backend_vector_view *bias,
                                           const gd_backend_vector_view *norm_weight,
                                           const gd_backend_tensor_view *pos_ids, const gd_backend_tensor_view *cache_pos,
                                           const gd_backend_tensor_view *q, const gd_backend_tensor_view *k_cache,
                                           const gd_backend_tensor_view *v_cache, uint32_t n_heads, uint32_t head_dim,
                                           const gd_backend_rope_args *rope_args,
                                           const gd_backend_fused_linear_args *args);

/* gd_backend_argmax_rows and the bookkeeping of gd_backend_decode_advance in one launch, for a loop that
 * feeds its own tokens: ids[b] = greedy token of logits row b; positions[b] += pos_delta;
 * s = step_counters[b]; when s < max_steps (= out_ids count / rows), out_ids[s*B + b] = token and
 * (out_gaps != NULL) out_gaps[s*B + b] = best - runner-up; step_counters[b] = s + 1.  Every row keeps its
 * own counter (I32 [B]) because every row is handled by its own workgroup.  With table [V, Dm] and next_x
 * [B, Dm] (both or neither; V = logits columns, rows of 16-byte multiples) the token's embedding row is also
 * copied to next_x[b], which makes the next step's gd_backend_embedding_forward unnecessary. */
gd_status gd_backend_argmax_advance(gd_backend *backend, const gd_backend_tensor_view *logits,
                                    const gd_backend_tensor_view *ids, const gd_backend_tensor_view *positions,
                                    const gd_backend_tensor_view *step_counters,
                                    const gd_backend_tensor_view *out_ids, const gd_backend_tensor_view *out_gaps,
                                    int32_t pos_delta, const gd_backend_tensor_view *table,
                                    const gd_backend_tensor_view *next_x);

/* Next-token sampling and the bookkeeping of a generation loop on the device, two launches.  What the
 * reference's example does on the host with the downloaded logits (examples/gpt_lm/gpt_lm_shared.c):
 * soft cap (:1322-1331), repetition penalty over the row's history (:1347-1369), the temperature / min-p draw
 * (:1371-1442) and the loop's handling of the result (:1586-1600, 1606-1680).  Per row b of logits [B, V]
 * (F16 or F32, V <= 262144), rows whose finished flag is set skipped:
 *   v = logits; softcap > 0: v = softcap * tanhf(v / softcap) (F32); every distinct token of
 *   history[b][0 .. hist_len[b]) inside [0, V): v > 0 ? v / penalty : v * penalty, if penalty is finite and > 1;
 *   leader = first largest finite v (token 0 if none).  temperature finite and > 0: tokens with
 *   v >= leader + temperature * log(min_p) (all finite ones if min_p <= 0) have mass exp((v - leader) /
 *   temperature) (F64); the row draws u from the generator and takes the first token whose running mass
 *   reaches u * total.  Otherwise, or if the total is not a positive finite number, the leader is taken and
 *   no draw is made.
 * The generator is the reference's: one 64-bit state for all rows, state = splitmix64(state) per draw, u =
 * (state >> 11) / 2^53, rows served in ascending order, only rows that draw advance it.
 * Then, per row: a row that was not finished ends (finished[b] = 1) if the token is stop_token (>= 0) or its
 * history is full (hist_len[b] == H); else the token is appended to history[b] and hist_len[b] += 1.
 * ids[b] = the token, or for an ended row stop_token (0 if there is none); positions[b] += pos_delta;
 * s = step_counters[b]; if s < max_steps (= out_ids count / B): out_ids[s*B + b] = the appended token, or -1
 * if nothing was appended; step_counters[b] = s + 1.  table / next_x as in gd_backend_argmax_advance (the
 * row of ids[b]).
 * state: I32 [>= gd_backend_sample_state_count(B)], 8-byte aligned, owned by the loop: words 0-1 and 2-3
 * hold the generator state (little-endian 64-bit, write the same start value to both), word 4 a launch
 * counter (start 0), the rest is scratch.  work: F32 [>= gd_backend_sample_work_count(B, V)], 8-byte aligned,
 * scratch (the rows after cap and penalty, then masses of runs of consecutive tokens).  Sums are formed in another order
 * than the reference's left-to-right loops: the token can differ from the reference's only when u * total
 * lies within rounding distance (~1e-13 of the total) of the boundary between two tokens.  Calls on one
 * state must not overlap. */
typedef struct gd_backend_sample_args {
    float temperature, min_p, repetition_penalty, logits_softcap;
    int32_t stop_token; /* < 0: none */
    int32_t pos_delta;
} gd_backend_sample_args;

typedef struct gd_backend_sample_tensors {
    const gd_backend_tensor_view *history;       /* I32 [B, H] */
    const gd_backend_tensor_view *hist_len;      /* I32 [B] */
    const gd_backend_tensor_view *finished;      /* I32 [B] */
    const gd_backend_tensor_view *state;         /* I32, see above */
    const gd_backend_tensor_view *work;          /* F32, see above */
    const gd_backend_tensor_view *ids;           /* I32 [B] */
    const gd_backend_tensor_view *positions;     /* I32 [B] */
    const gd_backend_tensor_view *step_counters; /* I32 [B] */
    const gd_backend_tensor_view *out_ids;       /* I32 [max_steps * B] */
    const gd_backend_tensor_view *table;         /* [V, Dm] or NULL */
    const gd_backend_tensor_view *next_x;        /* [B, Dm] or NULL */
} gd_backend_sample_tensors;

size_t gd_backend_sample_state_count(uint32_t rows);
size_t gd_backend_sample_work_count(uint32_t rows, uint32_t cols);
gd_status gd_backend_sample_advance(gd_backend *backend, const gd_backend_tensor_view *logits,
                                    const gd_backend_sample_tensors *tensors, const gd_backend_sample_args *args);

/* Device copy between buffers, enqueued like an operator. */
gd_status gd_backend_copy(gd_backend *backend, gd_backend_buffer *dst, size_t dst_offset,
                          gd_backend_buffer *src, size_t src_offset, size_t nbytes);

/* Stream timers: events recorded on the backend's own stream. */
typedef struct gd_backend_timer gd_backend_timer;
gd_status gd_backend_timer_create(gd_backend *backend, gd_backend_timer **out_timer);
void gd_backend_timer_destroy(gd_backend_timer *timer);
gd_status gd_backend_timer_start(gd_backend_timer *timer);
gd_status gd_backend_timer_stop(gd_backend_timer *timer);
/* Blocks until the stop event has completed. */
gd_status gd_backend_timer_elapsed_ms(gd_backend_timer *timer, float *out_ms);

/* Graph capture of the operators enqueued between begin and end (must be
 * inside a scope); launch replays them on the backend stream. */
typedef struct gd_backend_graph gd_backend_graph;
gd_status gd_backend_graph_begin_capture(gd_backend *backend);
gd_status gd_backend_graph_end_capture(gd_backend *backend, gd_backend_graph **out_graph);
gd_status gd_backend_graph_launch(gd_backend *backend, gd_backend_graph *graph);
void gd_backend_graph_destroy(gd_backend_graph *graph);

/* Device facts for benchmarks: name, compute units, total global memory. */
gd_status gd_backend_device_info(const gd_backend *backend, char *name, size_t name_len,
                                 int32_t *compute_units, uint64_t *global_mem_bytes);

/* Kernel tunables, normally left at 0 = automatic.  name "sdpa_chunk": keys per workgroup of
 * the split-KV decode kernel (also read once from the environment variable
 * GD_HIP_SDPA_CHUNK); "sdpa_waves" (4 or 8 wavefronts per workgroup) and "sdpa_unroll" (2, 4 or 8
 * key-row loads per lane and trip) of the same kernel; "sdpa_nontemporal" (GD_HIP_SDPA_NONTEMPORAL): 1 = mark its
 * K/V loads streaming, 0 = never, -1 (default) = when the caches of the call exceed 128 MiB; "sdpa_merge"
 * (GD_HIP_SDPA_MERGE): the per-row-positions form over at most 256 rows can cut the rows into pieces of 256 keys
 * (or "sdpa_chunk"), one workgroup each, and let the last piece of a row to arrive merge it, so that a ragged batch
 * spreads over the compute units; rows of about one length stay whole: 1 (default) = where there is a (row, kv head)
 * pair per compute unit and caches of 1024 rows or more, 0 = never, 2 = wherever the form applies.  "linear_tiles" (1, 2 or 4 column tiles of 16
 * per workgroup) and "linear_waves" (4 or 8 wavefronts sharing the K range) of the few-row projection
 * kernel (environment: GD_HIP_LINEAR_TILES, GD_HIP_LINEAR_WAVES).  "m3_simple" = 1: the MiniMax-M3 operators
 * take their per-row kernels also where the matrix-core kernels apply (head size 64, block size a multiple of 64).
 * "linear_wide" (GD_HIP_LINEAR_WIDE): the kernel built around the weight stream for few-row projections over [N,K]
 * weights (whole-line loads through an LDS ring, every row tile of up to 64 rows in one workgroup): 1 = wherever it
 * covers the call, 0 = never, -1 (default) = from 4 MiB of weights on.
 * "linear_tiles" = 4 also keeps the persistent form of those kernels on full-width column tiles where it would
 * otherwise deal an output with fewer full tiles than compute units out in narrower ones (same results to the bit).
 * "linear_no_lds_stream" = 1: the few-row projection always loads its weight fragments straight into registers,
 * also where it would stage the weight stream through LDS (same results to the bit; for comparing the two).
 * "prefill_rope_epilogue" = 0: gd_backend_linear_qkv_rope_packed answers GD_ERR_UNSUPPORTED, so that a caller (the
 * decoder's prefill) stays with the separate projection and rotation + append launches (for comparing the two).
 * Unknown name -> GD_ERR_INVALID_ARGUMENT. */
gd_status gd_backend_set_tunable(gd_backend *backend, const char *name, int64_t value);

/* Name of the kernel instantiation the most recent gd_backend_sdpa_decode{,_at,_positions} call on this backend
 * launched, as a kernel trace prints it (e.g. "gd_sdpa_decode_split_kernel<64,1,4,2,false>"), followed by its
 * grid in brackets; written to out as a NUL-terminated string of at most capacity bytes.  No counterpart in the
 * reference (measurement aid: bench.py labels its roofline with it).  GD_ERR_BAD_STATE before the first call. */
gd_status gd_backend_sdpa_decode_last_kernel(gd_backend *backend, char *out, size_t capacity);
/* Kernel family the last projection call (matmul / linear / fused_linear / fused_qkv_rope_append) took: "stream" (few
 * rows, fragments from global memory), "wide" (few rows over large [N,K] weights, weight stream through LDS), "tile"
 * (128 rows and more) or "scalar" (unaligned operands).  No reference counterpart. */
gd_status gd_backend_linear_last_kernel(gd_backend *backend, char *out, size_t capacity);

/* gd_backend_sdpa_decode_positions for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments, validation, kernels and result bits as gd_backend_sdpa_decode_positions; what the kernels keep beside
 * inputs and outputs (64 KiB of arrival counters, then the partial results of rows that are cut: batch * q heads *
 * pieces * (head size + 2) * 4 bytes; needed when batch * kv heads is below the number of compute units and the key
 * range is split, and when the rows of a ragged batch are cut into pieces) goes to a fixed device array of
 * GD_BACKEND_SDPA_DECODE_NOALLOC_SCRATCH_BYTES that the library holds on every GPU it runs on until the process
 * ends, instead of the backend's workspace that grows by hipMalloc.  A ragged batch whose pieces would not fit is
 * run with one workgroup per (row, kv head) instead; a split of the key range that does not fit returns
 * GD_ERR_OUT_OF_MEMORY and prints the two sizes on stderr; nothing is launched.  The call makes no hipMalloc /
 * hipFree and may be captured into a graph.  All calls on one GPU share the array: calls that overlap on one GPU
 * (two backends, two streams, a graph replay next to an eager call on another stream) race; calls on one backend
 * are ordered by its stream. */
#define GD_BACKEND_SDPA_DECODE_NOALLOC_SCRATCH_BYTES (8u << 20)
gd_status gd_backend_sdpa_decode_positions_noalloc(gd_backend *backend, const gd_backend_tensor_view *q,
                                                   const gd_backend_tensor_view *k_cache,
                                                   const gd_backend_tensor_view *v_cache,
                                                   const gd_backend_tensor_view *cache_pos,
                                                   const gd_backend_tensor_view *out,
                                                   const gd_backend_sdpa_decode_args *args);

/* Raw device address of a buffer (base of the allocation). */
void *gd_backend_buffer_device_ptr(gd_backend_buffer *buffer);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif

#endif /* GD_BACKEND_HIP_H */
