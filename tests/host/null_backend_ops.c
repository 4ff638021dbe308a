/*
 * TEST INFRASTRUCTURE ONLY: the operator entry points of the device-less backend (null_backend.c).  Each one
 * counts the call, records its name and returns GD_OK (or the status set with gd_null_backend_fail_ops) without
 * touching its arguments: declared without a parameter list on purpose, the callers pass what the header says.
 */
#include <stdint.h>

int gd_null_backend_note(const char *name);

#define GD_NULL_OP(name) \
    __attribute__((visibility("default"))) int name() { return gd_null_backend_note(#name); }

GD_NULL_OP(gd_backend_add)
GD_NULL_OP(gd_backend_add_scalar_i32)
GD_NULL_OP(gd_backend_argmax_advance)
GD_NULL_OP(gd_backend_argmax_rows)
GD_NULL_OP(gd_backend_concat_to_full)
GD_NULL_OP(gd_backend_decode_advance)
GD_NULL_OP(gd_backend_embedding_forward)
GD_NULL_OP(gd_backend_fused_linear)
GD_NULL_OP(gd_backend_fused_qkv_rope_append)
GD_NULL_OP(gd_backend_gather_rows)
GD_NULL_OP(gd_backend_kv_cache_append_at)
GD_NULL_OP(gd_backend_kv_cache_append_packed)
GD_NULL_OP(gd_backend_kv_cache_append_positions)
GD_NULL_OP(gd_backend_linear)
GD_NULL_OP(gd_backend_linear_last_kernel)
GD_NULL_OP(gd_backend_linear_nt)
GD_NULL_OP(gd_backend_linear_qkv_rope_packed)
GD_NULL_OP(gd_backend_matmul)
GD_NULL_OP(gd_backend_matmul_nt)
GD_NULL_OP(gd_backend_minimax_m3_index_topk)
GD_NULL_OP(gd_backend_minimax_m3_sparse_attention)
GD_NULL_OP(gd_backend_qkv_rope_append)
GD_NULL_OP(gd_backend_qkv_rope_append_packed)
GD_NULL_OP(gd_backend_qkv_split_rope_forward)
GD_NULL_OP(gd_backend_rand_uniform)
GD_NULL_OP(gd_backend_rms_norm_forward)
GD_NULL_OP(gd_backend_rope_table_packed)
GD_NULL_OP(gd_backend_sample_advance)
GD_NULL_OP(gd_backend_sdpa_decode)
GD_NULL_OP(gd_backend_sdpa_decode_at)
GD_NULL_OP(gd_backend_sdpa_decode_last_kernel)
GD_NULL_OP(gd_backend_sdpa_decode_positions)
GD_NULL_OP(gd_backend_sdpa_decode_positions_noalloc)
GD_NULL_OP(gd_backend_sdpa_varlen)
GD_NULL_OP(gd_backend_sdpa_varlen_cached)
GD_NULL_OP(gd_backend_swiglu_split_forward)
GD_NULL_OP(gd_backend_swiglu_split_linear)
